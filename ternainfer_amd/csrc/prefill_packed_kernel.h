// Large-M TernaSpMM kernel on the P2 layout (see packed_common.h): a bf16 MFMA GEMM whose weight
// operand goes global memory -> registers -> matrix core, expanded by v_perm_b32, and never
// touches LDS.
//
//   out[m][n] = epilogue( 2 * sum_k X[m][k] * Whalf[n][k] ),   Whalf = W / 2 in {-0.5, 0, +0.5}
//
// Tiling.  One workgroup (4 waves) owns 256 output features x BM = 32*MB batch rows and walks K in
// steps of 64.  The waves split the output features only: wave w owns rows 64w .. 64w+63 and ALL
// BM batch rows, i.e. 2 x MB accumulator tiles of v_mfma_f32_32x32x16_bf16 with W as the A
// operand -- so every weight is expanded exactly once per workgroup, and one expansion (ten VALU
// ops) feeds MB matrix instructions.  A-operand lane (row = L%32, kb = L/32) of row-tile a needs,
// for 16-column group g, the eight weights of byte pair t = kb of packed word (band, gk, i, g): the
// four words g = 0..3 of a row are adjacent, so one 16-byte load per row-tile and k-step brings
// everything the lane needs.  Only the activation tile goes through LDS (two stages, chunk order
// [g][sm][row], see the reference-format kernel), staged one k-step ahead; B operands are read one
// group ahead of the MFMAs that use them; weight registers are refilled two k-steps ahead.
#pragma once

#include "packed_common.h"
#include "prefill_kernel.h"

namespace terna {

template <int MB>
struct PackedPrefillSmem {
    static constexpr int BM = 32 * MB;
    static constexpr int PX = BM * 16 + 16;           // bytes between chunk rows of the X tile (padded)
    static constexpr int kStage = 8 * PX;
    static constexpr int kBytes = 2 * kStage;
};

template <typename Act, int MB>
__global__ __launch_bounds__(256, MB == 8 ? 1 : 2) void terna_prefill_packed_kernel(
    const Act* __restrict__ x, const uint32_t* __restrict__ packed, uint16_t* __restrict__ out,
    Epilogue ep, int M, int N, int K)
{
    using T = ActTraits<Act>;
    using S = PackedPrefillSmem<MB>;
    constexpr int BN = kPrefillBN, BM = S::BM, PX = S::PX;
    constexpr int XI = BM / 64;                       // (row, group) activation items per thread and k-step
    static_assert(MB == 2 || MB == 4 || MB == 8, "batch tile of 64, 128 or 256 rows");

    extern __shared__ __align__(16) uint8_t smem[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n0 = blockIdx.x * BN, m0 = blockIdx.y * BM;
    const int ktiles = K >> 6;
    const int last_band = (N >> 4) - 1;
    const int kb = lane >> 5, l32 = lane & 31;

    // ---- weight words of this lane: row-tile a -> band (n0/16 + 4*wave + 2a + l32/16), row i = l32 % 16
    const u32x4* w_ptr[2];                             // running: advanced one k-step per fetch
#pragma unroll
    for (int a = 0; a < 2; ++a) {
        int band = (n0 >> 4) + 4 * wave + 2 * a + (l32 >> 4);
        band = band < last_band ? band : last_band;   // a tile hanging over N re-reads the last band; never stored
        w_ptr[a] = reinterpret_cast<const u32x4*>(packed + (static_cast<size_t>(band) * ktiles) * 64 + (l32 & 15) * 4);
    }
    // ---- activation items of this thread: item = tid + 256*it -> (row = item / 4, group = item % 4)
    int x_lds[XI];
    const Act* x_ptr[XI];
#pragma unroll
    for (int it = 0; it < XI; ++it) {
        const int item = tid + 256 * it;
        const int row = item >> 2, g = item & 3;
        x_lds[it] = (g * 2) * PX + row * 16;
        int m = m0 + row;
        m = m < M ? m : M - 1;
        x_ptr[it] = x + static_cast<size_t>(m) * K + g * 16;
    }

    struct RawW { u32x4 w[2]; };                      // [a] -> words g = 0..3
    struct RawX { u32x4 x[XI][T::kXVecs]; };
    // Both fetches walk running pointers: one k-step is 16 u32x4 of weights and 64 activations.
    auto fetch_w = [&](RawW& r) {
#pragma unroll
        for (int a = 0; a < 2; ++a) {
            r.w[a] = *w_ptr[a];
            w_ptr[a] += 16;
        }
    };
    auto fetch_x = [&](RawX& r) {
#pragma unroll
        for (int it = 0; it < XI; ++it) {
            const u32x4* p = reinterpret_cast<const u32x4*>(x_ptr[it]);
#pragma unroll
            for (int v = 0; v < T::kXVecs; ++v) r.x[it][v] = p[v];
            x_ptr[it] += 64;
        }
    };
    auto stage_x = [&](const RawX& r, int st) {
#pragma unroll
        for (int it = 0; it < XI; ++it) {
            u32x4 c0, c1;
            if constexpr (sizeof(Act) == 2) {
                const u32x4 a = r.x[it][0], b = r.x[it][1];
                c0 = u32x4{a.x, a.z, b.x, b.z};
                c1 = u32x4{a.y, a.w, b.y, b.w};
            } else {
                int8_group_to_chunks(r.x[it][0], c0, c1);
            }
            uint8_t* dst = smem + st * S::kStage + x_lds[it];
            *reinterpret_cast<u32x4*>(dst) = c0;
            *reinterpret_cast<u32x4*>(dst + PX) = c1;
        }
    };

    f32x16 acc[2][MB];
    {
        const f32x16 zero = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int b = 0; b < MB; ++b) acc[a][b] = zero;
    }

    const int b_off = kb * PX + l32 * 16;                    // + g*2*PX + b*512
    const int wshift = 4 * kb;                               // byte pair t = kb of every word

    struct BOps { bf16x8 b[MB]; };
    auto load_b = [&](int st, int g, BOps& r) {
        const uint8_t* xs = smem + st * S::kStage + b_off + g * 2 * PX;
#pragma unroll
        for (int b = 0; b < MB; ++b) r.b[b] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(xs + b * 512));
    };
    // One k-step: for each 16-column group g, expand the two A operands from registers and issue
    // 2*MB MFMAs against B operands that were read from LDS one group earlier.
    auto mma_step = [&](const RawW& rw, int st) {
        BOps bcur;
        load_b(st, 0, bcur);
        static_for<0, 4>([&](auto gc) {
            constexpr int g = decltype(gc)::value;
            BOps bnxt;
            if constexpr (g < 3) load_b(st, g + 1, bnxt);
#pragma unroll
            for (int a = 0; a < 2; ++a) {
                const bf16x8 af = __builtin_bit_cast(bf16x8, expand_chunk_bf16(rw.w[a][g] >> wshift));
#pragma unroll
                for (int b = 0; b < MB; ++b)
                    acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af, bcur.b[b], acc[a][b], 0, 0, 0);
            }
            if constexpr (g < 3) bcur = bnxt;
        });
    };

    // ---- pipeline.  Two weight buffers: w0 serves even k-steps, w1 odd ones; each is refilled
    // for k + 2 as soon as step k has consumed it, so its loads have a whole k-step to land.
    // Activations: raw registers hold step k + 1 while LDS stage (k & 1) feeds the MFMAs of step k.
    RawW w0, w1;
    RawX x_raw;
    fetch_w(w0);
    fetch_x(x_raw);
    stage_x(x_raw, 0);
    if (ktiles > 1) {
        fetch_w(w1);
        fetch_x(x_raw);
    }
    __syncthreads();
    // k-step k with both look-aheads in range (k + 2 < ktiles)
    auto body_full = [&](int k, RawW& w) {
        stage_x(x_raw, (k + 1) & 1);
        fetch_x(x_raw);
        mma_step(w, k & 1);
        fetch_w(w);
        __syncthreads();
    };
    auto body_tail = [&](int k, RawW& w) {
        if (k + 1 < ktiles) stage_x(x_raw, (k + 1) & 1);
        if (k + 2 < ktiles) fetch_x(x_raw);
        mma_step(w, k & 1);
        if (k + 2 < ktiles) fetch_w(w);
        __syncthreads();
    };
    int k = 0;
    for (; k + 3 < ktiles; k += 2) {
        body_full(k, w0);
        body_full(k + 1, w1);
    }
    if (k < ktiles) body_tail(k++, w0);
    if (k < ktiles) body_tail(k++, w1);
    if (k < ktiles) body_tail(k++, w0);

    // ---- epilogue: lane holds, per accumulator tile, column m = l32 and rows n = (v&3) + 8(v>>2) + 4kb.
    // The accumulator is half the true sum (weights were +-0.5); x2 is exact.
    EpilogueRegs e[MB];
    int m_of[MB];
    static_for<0, MB>([&](auto bc) {
        constexpr int b = decltype(bc)::value;
        m_of[b] = m0 + 32 * b + l32;
        e[b].s = ep.kind == EP_BF16 ? 1.0f : bf16_bits_to_float(ep.s[m_of[b] < M ? m_of[b] : M - 1]);
    });
    static_for<0, 8>([&](auto tc) {
        constexpr int a = decltype(tc)::value >> 2, vq = decltype(tc)::value & 3;
        const int n = n0 + 64 * wave + 32 * a + 8 * vq + 4 * kb;
        float wv[4];
        load_col_scales(ep, n < N ? n : N - 4, N, wv);
        static_for<0, MB>([&](auto bc) {
            constexpr int b = decltype(bc)::value;
            EpilogueRegs eb = e[b];
#pragma unroll
            for (int v = 0; v < 4; ++v) eb.w[v] = wv[v];
            uint16_t o[4];
#pragma unroll
            for (int v = 0; v < 4; ++v) o[v] = apply_epilogue<float>(ep.kind, eb, v, acc[a][b][4 * vq + v] * 2.0f);
            const u32x2 pk = {o[0] | (static_cast<uint32_t>(o[1]) << 16), o[2] | (static_cast<uint32_t>(o[3]) << 16)};
            if (m_of[b] < M && n < N) *reinterpret_cast<u32x2*>(out + static_cast<size_t>(m_of[b]) * N + n) = pk;
        });
    });
}

}  // namespace terna
