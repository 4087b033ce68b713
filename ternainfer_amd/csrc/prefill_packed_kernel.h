// Large-M TernaSpMM kernel on the P2 layout (see packed_common.h): a bf16 MFMA GEMM whose weight
// operand goes global memory -> registers -> matrix core, expanded by v_perm_b32, and never
// touches LDS.
//
//   out[m][n] = epilogue( 2 * sum_k X[m][k] * Whalf[n][k] ),   Whalf = W / 2 in {-0.5, 0, +0.5}
//
// Tiling.  One workgroup (4 waves, 2 (n) x 2 (m)) owns 256 output features x 64*MT batch rows and
// walks K in steps of 64.  A wave owns 128 x 32*MT outputs as 4 x MT accumulator tiles of
// v_mfma_f32_32x32x16_bf16, W as the A operand.  A-operand lane (row = L%32, kb = L/32) of
// accumulator row-tile a needs, for 16-column group g, the eight weights of byte pair t = kb of
// packed word (band, gk, i, g): the four words g = 0..3 of a row are adjacent, so one 16-byte
// load per row-tile and k-step brings everything the lane needs, and ten VALU ops turn each word
// into an operand.  Only the activation tile goes through LDS (two stages, chunk order
// [g][sm][row], see the reference-format kernel), staged one k-step ahead; global loads of both
// operands run two k-steps ahead.
#pragma once

#include "packed_common.h"
#include "prefill_kernel.h"

namespace terna {

template <int MT>
struct PackedPrefillSmem {
    static constexpr int BM = 64 * MT;
    static constexpr int PX = BM * 16 + 16;           // bytes between chunk rows of the X tile (padded)
    static constexpr int kStage = 8 * PX;
    static constexpr int kBytes = 2 * kStage;
};

template <typename Act, int MT>
__global__ __launch_bounds__(256, MT == 4 ? 1 : 2) void terna_prefill_packed_kernel(
    const Act* __restrict__ x, const uint32_t* __restrict__ packed, uint16_t* __restrict__ out,
    Epilogue ep, int M, int N, int K)
{
    using T = ActTraits<Act>;
    using S = PackedPrefillSmem<MT>;
    constexpr int BN = kPrefillBN, BM = S::BM, PX = S::PX;
    constexpr int XI = MT;                            // (row, group) activation items per thread and k-step

    extern __shared__ __align__(16) uint8_t smem[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wn = wave & 1, wm = wave >> 1;
    const int n0 = blockIdx.x * BN, m0 = blockIdx.y * BM;
    const int ktiles = K >> 6;
    const int last_band = (N >> 4) - 1;
    const int kb = lane >> 5, l32 = lane & 31;

    // ---- weight words of this lane: row-tile a -> band (n0/16 + 8*wn + 2a + l32/16), row i = l32 % 16
    const u32x4* w_ptr[4];
#pragma unroll
    for (int a = 0; a < 4; ++a) {
        int band = (n0 >> 4) + 8 * wn + 2 * a + (l32 >> 4);
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

    struct RawW { u32x4 w[4]; };                      // [a] -> words g = 0..3
    struct RawX { u32x4 x[XI][T::kXVecs]; };
    auto fetch_w = [&](int gk, RawW& r) {
#pragma unroll
        for (int a = 0; a < 4; ++a) r.w[a] = w_ptr[a][static_cast<size_t>(gk) * 16];
    };
    auto fetch_x = [&](int gk, RawX& r) {
#pragma unroll
        for (int it = 0; it < XI; ++it) {
            const u32x4* p = reinterpret_cast<const u32x4*>(x_ptr[it] + gk * 64);
#pragma unroll
            for (int v = 0; v < T::kXVecs; ++v) r.x[it][v] = p[v];
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

    f32x16 acc[4][MT];
    {
        const f32x16 zero = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
            for (int b = 0; b < MT; ++b) acc[a][b] = zero;
    }

    const int b_off = kb * PX + (32 * MT * wm + l32) * 16;   // + g*2*PX + b*512
    const int wshift = 4 * kb;                               // byte pair t = kb of every word

    // One k-step: for each 16-column group g, expand the four A operands from registers, read the
    // MT B operands from the current X stage, and issue 4*MT MFMAs.
    auto mma_step = [&](const RawW& rw, int st) {
        const uint8_t* xs = smem + st * S::kStage;
        static_for<0, 4>([&](auto gc) {
            constexpr int g = decltype(gc)::value;
            bf16x8 bfr[MT];
#pragma unroll
            for (int b = 0; b < MT; ++b)
                bfr[b] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(xs + b_off + g * 2 * PX + b * 512));
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                const bf16x8 af = __builtin_bit_cast(bf16x8, expand_chunk_bf16(rw.w[a][g] >> wshift));
#pragma unroll
                for (int b = 0; b < MT; ++b)
                    acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af, bfr[b], acc[a][b], 0, 0, 0);
            }
        });
    };

    // ---- pipeline: global loads two k-steps ahead; X staged one k-step ahead (double-buffered LDS)
    RawW w_cur, w_nxt;
    RawX x_raw;
    fetch_w(0, w_cur);
    fetch_x(0, x_raw);
    stage_x(x_raw, 0);
    if (ktiles > 1) {
        fetch_w(1, w_nxt);
        fetch_x(1, x_raw);
    }
    __syncthreads();
    for (int k = 0; k < ktiles; ++k) {
        const int st = k & 1;
        if (k + 1 < ktiles) stage_x(x_raw, st ^ 1);       // k+1 activations -> other stage
        RawW w_nn;
        if (k + 2 < ktiles) {
            fetch_w(k + 2, w_nn);
            fetch_x(k + 2, x_raw);
        }
        mma_step(w_cur, st);
        w_cur = w_nxt;
        w_nxt = w_nn;
        __syncthreads();
    }

    // ---- epilogue: lane holds, per accumulator tile, column m = l32 and rows n = (v&3) + 8(v>>2) + 4kb.
    // The accumulator is half the true sum (weights were +-0.5); x2 is exact.
    EpilogueRegs e[MT];
    int m_of[MT];
    static_for<0, MT>([&](auto bc) {
        constexpr int b = decltype(bc)::value;
        m_of[b] = m0 + 32 * MT * wm + 32 * b + l32;
        e[b].s = ep.kind == EP_BF16 ? 1.0f : bf16_bits_to_float(ep.s[m_of[b] < M ? m_of[b] : M - 1]);
    });
    static_for<0, 16>([&](auto tc) {
        constexpr int a = decltype(tc)::value >> 2, vq = decltype(tc)::value & 3;
        const int n = n0 + 128 * wn + 32 * a + 8 * vq + 4 * kb;
        float wv[4];
        load_col_scales(ep, n < N ? n : N - 4, N, wv);
        static_for<0, MT>([&](auto bc) {
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
