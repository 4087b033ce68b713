// Small-M TernaSpMM kernel on the P2 layout (see packed_common.h).
//
// Same work split as the reference-format kernel -- one workgroup per 16-row band over the whole
// K, waves take the band's 64-column tiles round robin, sum through LDS in wave order, fused
// epilogue -- but a band-tile is one coalesced 256-byte line (one word per lane), its address is
// pure arithmetic, and the expansion to MFMA operands is a handful of v_perm_b32: the per-tile
// offset fetch, sign window, prefix popcounts, cross-lane gathers and LDS table of the
// reference-format kernel are all gone.  Every load of a wave is independent of every other, so
// they are all in flight after one round trip for the kernel arguments.
#pragma once

#include "packed_common.h"

namespace terna {

template <typename Act, int MB>
struct PackedRaw {
    uint32_t word;                          // 16 weights: row (L & 15), 16-column group (L >> 4)
    u32x4    x[MB][ActTraits<Act>::kXVecs]; // activation bytes of (batch row L & 15, group L >> 4)
};

template <typename Act, int WAVES, int MB, int DEPTH>
__global__ __launch_bounds__(WAVES * 64) void terna_decode_packed_kernel(
    const Act* __restrict__ x, const uint32_t* __restrict__ packed, uint16_t* __restrict__ out,
    Epilogue ep, int M, int N, int K)
{
    using T = ActTraits<Act>;
    using Acc = typename T::Acc;
    using Raw = PackedRaw<Act, MB>;
    constexpr int NBUF = DEPTH + 1;
    static_assert(DEPTH >= 1 && DEPTH <= 3, "prefetch distance");

    __shared__ Acc red[WAVES][MB][64];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int band = blockIdx.x;
    const int m_base = blockIdx.y * (16 * MB);
    const int ktiles = K >> 6;
    const int i = lane & 15, g = lane >> 4;

    const uint32_t* wp = packed + (static_cast<size_t>(band) * ktiles + wave) * 64 + i * 4 + g;
    const Act* xp[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        const int m = m_base + mb * 16 + i;
        xp[mb] = x + static_cast<size_t>(m < M ? m : M - 1) * K + wave * 64 + g * 16;   // rows past M repeat the last
    }

    const int cnt = ktiles > wave ? (ktiles - wave + WAVES - 1) / WAVES : 0;   // this wave's band-tiles
    auto fetch = [&](int j, Raw& raw) {
        raw.word = wp[static_cast<size_t>(j) * (WAVES * 64)];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            const u32x4* p = reinterpret_cast<const u32x4*>(xp[mb] + static_cast<size_t>(j) * (WAVES * 64));
#pragma unroll
            for (int v = 0; v < T::kXVecs; ++v) raw.x[mb][v] = p[v];
        }
    };

    Acc acc[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[mb] = Acc{0, 0, 0, 0};

    // Wave w finishes m-block w (and w + WAVES, ...): fetch that block's scale factors now.
    const int n0 = band * 16 + 4 * g;
    EpilogueRegs eregs[(MB + WAVES - 1) / WAVES];
#pragma unroll
    for (int e = 0; e < (MB + WAVES - 1) / WAVES; ++e) {
        const int m = m_base + (wave + e * WAVES) * 16 + i;
        eregs[e] = load_epilogue(ep, m < M ? m : M - 1, n0, N);
    }

    auto process = [&](const Raw& cur) {
        if constexpr (sizeof(Act) == 2) {
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const bf16x8 a = __builtin_bit_cast(bf16x8, expand_chunk_bf16(cur.word >> (4 * t)));
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
                    const u32x4 x0 = cur.x[mb][0], x1 = cur.x[mb][1];
                    const u32x4 b_bits = t == 0 ? u32x4{x0.x, x0.z, x1.x, x1.z} : u32x4{x0.y, x0.w, x1.y, x1.w};
                    acc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, __builtin_bit_cast(bf16x8, b_bits), acc[mb], 0, 0, 0);
                }
            }
        } else {
            const i32x4 a = expand_word_i8(cur.word);
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                const u32x4 xv = cur.x[mb][0];       // dword j = columns 4j .. 4j+3
                const i32x4 b = {
                    static_cast<int>(__builtin_amdgcn_perm(xv.y, xv.x, 0x05040100u)),   // t=0, c=0..3
                    static_cast<int>(__builtin_amdgcn_perm(xv.w, xv.z, 0x05040100u)),   // t=0, c=4..7
                    static_cast<int>(__builtin_amdgcn_perm(xv.y, xv.x, 0x07060302u)),   // t=1, c=0..3
                    static_cast<int>(__builtin_amdgcn_perm(xv.w, xv.z, 0x07060302u))};  // t=1, c=4..7
                acc[mb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, acc[mb], 0, 0, 0);
            }
        }
    };

    // Ring of DEPTH + 1 named register buffers; loads run DEPTH band-tiles ahead.
    Raw ring0, ring1, ring2, ring3;
    auto slot = [&](int j, const Raw& cur, Raw& pre) {
        if (j < cnt) {
            if (j + DEPTH < cnt) fetch(j + DEPTH, pre);
            process(cur);
        }
    };
    if (0 < cnt) fetch(0, ring0);
    if (DEPTH >= 2 && 1 < cnt) fetch(1, ring1);
    if (DEPTH >= 3 && 2 < cnt) fetch(2, ring2);
    for (int j0 = 0; j0 < cnt; j0 += NBUF) {
        if constexpr (DEPTH == 3) {
            slot(j0, ring0, ring3);
            slot(j0 + 1, ring1, ring0);
            slot(j0 + 2, ring2, ring1);
            slot(j0 + 3, ring3, ring2);
        } else if constexpr (DEPTH == 2) {
            slot(j0, ring0, ring2);
            slot(j0 + 1, ring1, ring0);
            slot(j0 + 2, ring2, ring1);
        } else {
            slot(j0, ring0, ring1);
            slot(j0 + 1, ring1, ring0);
        }
    }

    // Cross-wave sum in wave order, then the fused epilogue (accumulator layout: lane L holds
    // output rows 4*(L>>4) .. +3 of column L & 15).  bf16 weights were +-0.5: undo with an exact x2.
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) red[wave][mb][lane] = acc[mb];
    __syncthreads();
#pragma unroll
    for (int e = 0; e < (MB + WAVES - 1) / WAVES; ++e) {
        const int mb = wave + e * WAVES;
        if (mb >= MB) break;
        Acc sum = red[0][mb][lane];
#pragma unroll
        for (int w = 1; w < WAVES; ++w) sum += red[w][mb][lane];
        const int m = m_base + mb * 16 + i;
        if (m < M) {
            uint16_t o[4];
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                if constexpr (sizeof(Act) == 2) o[v] = apply_epilogue<float>(ep.kind, eregs[e], v, sum[v] * 2.0f);
                else o[v] = apply_epilogue<int>(ep.kind, eregs[e], v, sum[v]);
            }
            const u32x2 pk = {o[0] | (static_cast<uint32_t>(o[1]) << 16), o[2] | (static_cast<uint32_t>(o[3]) << 16)};
            *reinterpret_cast<u32x2*>(out + static_cast<size_t>(m) * N + n0) = pk;
        }
    }
}

}  // namespace terna
