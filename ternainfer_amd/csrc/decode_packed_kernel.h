// Small-M TernaSpMM kernel on the P2 layout (see packed_common.h).
//
// Same work split as the reference-format kernel -- one workgroup per 16-row band over the whole
// K, waves take the band's 64-column tiles round robin, sum through LDS in wave order, fused
// epilogue -- but a band-tile is one coalesced 256-byte line (one word per lane), its address is
// pure arithmetic, and the expansion to MFMA operands is a handful of v_perm_b32: the per-tile
// offset fetch, sign window, prefix popcounts, cross-lane gathers and LDS table of the
// reference-format kernel are all gone.  Every load of a wave is independent of every other, so
// they are all in flight after one round trip for the kernel arguments.
//
// NB = bands per workgroup.  Every workgroup stages the same M x K activations; with more bands than
// the chip has CUs (gate+up: 864) a CU would pull them from L2 once per round of workgroups -- at
// M = 8 four times the bytes of a band's weights.  NB bands per workgroup share one staging.
#pragma once

#include "packed_common.h"

namespace terna {

template <typename Act, int MB, int NB>
struct PackedRaw {
    uint32_t word[NB];                       // per band, 16 weights: row (L & 15), 16-column group (L >> 4)
    u32x4    x[MB][XSlab<Act>::kLoads];      // coalesced pieces of the activation slab
};

// GUARD: the launch runs on a cached P2 copy and checks it (below).  A variant of its own: the branch at the top costs
// every workgroup 0.3 us (nothing can start before all arguments are in), which launches on a caller's own P2
// buffer do not have to pay.
// Argument order: pointers and integers first, the structures last -- the first sixteen dwords of the arguments
// arrive preloaded in scalar registers, but only up to the first structure passed by value, and everything the first
// global loads depend on should be among them.
// RES: the launch is also the producer for the next one (int8 activations, one m-block): instead of its own output
// it stores h' = bf16(residual[m][n] + out[m][n]), the residual stream after this linear (model.py:330, :334), and leaves
// per row and 16-row band the partial (sum of h'^2, max |h' * next_w|) that the consumer's norm and quantisation need
// (decode_fused_kernel.h has the consumer).
struct PackedProducer {
    const uint16_t* residual;        // bf16 [M][N]
    const uint16_t* next_w;          // bf16 [N]: weights of the norm that follows
    float2* stats_out;               // [M][N/16]
    uint16_t* raw_out;               // optional: the linear's own output as well
};

template <typename Act, int WAVES, int MB, int DEPTH, int NB = 1, bool GUARD = false, bool RES = false>
__global__ __launch_bounds__(WAVES * 64) void terna_decode_packed_kernel(
    const Act* __restrict__ x, const uint32_t* __restrict__ packed, uint16_t* __restrict__ out,
    int M, int N, int K, Epilogue ep, RepackGuard guard, PackedProducer prod)
{
    static_assert(!RES || (MB == 1 && sizeof(Act) == 1), "the producing epilogue: int8 activations, up to 16 rows");
    // A launch on a cached P2 copy carries one extra workgroup in x that checks, next to the others, that the copy still
    // belongs to the caller's tensors.  It is the FIRST workgroup of the grid: the check is two dependent memory round trips
    // (the stream's total, then the samples), longer than a band's work at small M, and as the last workgroup it started
    // behind the dispatch of all the others and ended the launch (the 2B layer set through the reference symbols: 0.541 ms
    // per step with the check last, 0.504 with it first, 0.500 without a check).
    if constexpr (GUARD) {
        if (blockIdx.x == 0) {
            if (blockIdx.y == 0 && threadIdx.x < 64) repack_guard_role(guard, threadIdx.x);
            return;
        }
    }
    using T = ActTraits<Act>;
    using Acc = typename T::Acc;
    using Raw = PackedRaw<Act, MB, NB>;
    using XS = XSlab<Act>;
    constexpr int NBUF = DEPTH + 1;
    static_assert(DEPTH >= 1 && DEPTH <= 3, "prefetch distance");

    constexpr int UNITS = NB * MB;           // (band, m-block) accumulators per wave
    __shared__ Acc red[WAVES][UNITS][64];
    __shared__ __align__(16) uint8_t xslab_all[WAVES][MB][16 * XS::kPitch];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int band0 = (static_cast<int>(blockIdx.x) - (GUARD ? 1 : 0)) * NB;
    const int m_base = blockIdx.y * (16 * MB);
    const int ktiles = K >> 6;
    const int i = lane & 15, g = lane >> 4;

    // lane L loads word L of a band-tile -- consecutive lanes, consecutive words: the memory pipeline takes such a load in a
    // quarter of the steps of the operand order (word (L & 15) * 4 + (L >> 4)), which one LDS-crossbar permutation restores
    const uint32_t* wp = packed + (static_cast<size_t>(band0) * ktiles + wave) * 64 + lane;
    const int operand_src = (i * 4 + g) * 4;
    const size_t band_pitch = static_cast<size_t>(ktiles) * 64;          // words from one band to the next
    // Coalesced activation pieces of this lane; rows past M are not loaded (their operand is zero
    // and their output column is never stored).
    const Act* xp[MB][XS::kLoads];
    bool x_ok[MB][XS::kLoads];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int h = 0; h < XS::kLoads; ++h) {
            const int m = m_base + mb * 16 + XS::row_of(lane, h);
            x_ok[mb][h] = m < M;
            xp[mb][h] = x + static_cast<size_t>(x_ok[mb][h] ? m : 0) * K + wave * 64 + XS::col_of(lane);
        }

    const int cnt = ktiles > wave ? (ktiles - wave + WAVES - 1) / WAVES : 0;   // this wave's band-tiles
    auto fetch = [&](int j, Raw& raw) {
#pragma unroll
        for (int b = 0; b < NB; ++b) raw.word[b] = wp[b * band_pitch + static_cast<size_t>(j) * (WAVES * 64)];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int h = 0; h < XS::kLoads; ++h) {
                const u32x4* p = reinterpret_cast<const u32x4*>(xp[mb][h] + static_cast<size_t>(j) * (WAVES * 64));
                raw.x[mb][h] = x_ok[mb][h] ? *p : u32x4{0u, 0u, 0u, 0u};
            }
    };

    Acc acc[NB][MB];
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) acc[b][mb] = Acc{0, 0, 0, 0};

    uint8_t* slab = xslab_all[wave][0];
    auto process = [&](const Raw& cur) {
        // slab in (coalesced order), operands out (MFMA order); same wave, so LDS ordering suffices
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int h = 0; h < XS::kLoads; ++h)
                *reinterpret_cast<u32x4*>(slab + mb * (16 * XS::kPitch) + XS::write_off(lane, h)) = cur.x[mb][h];
        if constexpr (sizeof(Act) == 2) {
            bf16x8 a0[NB], a1[NB];
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const uint32_t w = static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(operand_src, static_cast<int>(cur.word[b])));
                a0[b] = __builtin_bit_cast(bf16x8, expand_chunk_bf16(w << 4));
                a1[b] = __builtin_bit_cast(bf16x8, expand_chunk_bf16(w));
            }
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                const uint8_t* src = slab + mb * (16 * XS::kPitch) + i * XS::kPitch + g * 32;
                const u32x4 b0 = *reinterpret_cast<const u32x4*>(src);        // columns 16g .. 16g+7
                const u32x4 b1 = *reinterpret_cast<const u32x4*>(src + 16);   // columns 16g+8 .. 16g+15
#pragma unroll
                for (int b = 0; b < NB; ++b) {
                    acc[b][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0[b], __builtin_bit_cast(bf16x8, b0), acc[b][mb], 0, 0, 0);
                    acc[b][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1[b], __builtin_bit_cast(bf16x8, b1), acc[b][mb], 0, 0, 0);
                }
            }
        } else {
            i32x4 a[NB];
#pragma unroll
            for (int b = 0; b < NB; ++b)
                a[b] = expand_word_i8(static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(operand_src, static_cast<int>(cur.word[b]))));
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                const i32x4 bx = __builtin_bit_cast(
                    i32x4, *reinterpret_cast<const u32x4*>(slab + mb * (16 * XS::kPitch) + i * XS::kPitch + g * 16));
#pragma unroll
                for (int b = 0; b < NB; ++b) acc[b][mb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[b], bx, acc[b][mb], 0, 0, 0);
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

    // Wave w finishes unit w (and w + WAVES, ...), unit = band * MB + m-block: with the data loads in
    // flight, fetch that unit's scale factors so that no global load sits between the last MFMA and the store.
    constexpr int FIN = (UNITS + WAVES - 1) / WAVES;
    EpilogueRaw eraw[FIN];
#pragma unroll
    for (int e = 0; e < FIN; ++e) {
        const int unit = wave + e * WAVES < UNITS ? wave + e * WAVES : 0;
        const int m = m_base + (unit % MB) * 16 + i;
        eraw[e] = load_epilogue_raw(ep, m < M ? m : M - 1, (band0 + unit / MB) * 16 + 4 * g, N);
    }
    // the producing epilogue's own operands -- four stream values, four weights of the next norm -- by the finishing
    // waves (the others read one address: no traffic); requested with everything else, used at the very end
    u32x2 eres[FIN], enw[FIN];
    if constexpr (RES) {
#pragma unroll
        for (int e = 0; e < FIN; ++e) {
            const int unit = wave + e * WAVES;
            const bool fin = unit < UNITS;
            const int n0 = (band0 + (fin ? unit : 0)) * 16 + 4 * g;
            const int m = m_base + i;
            enw[e] = *reinterpret_cast<const u32x2*>(prod.next_w + (fin ? n0 : 0));
            eres[e] = *reinterpret_cast<const u32x2*>(prod.residual + (fin ? static_cast<size_t>(m < M ? m : 0) * N + n0 : 0));
        }
    }

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
    // output rows 4*(L>>4) .. +3 of column L & 15).  bf16 weights were +-2: undo with an exact x0.5.
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) red[wave][b * MB + mb][lane] = acc[b][mb];
    __syncthreads();
#pragma unroll
    for (int e = 0; e < FIN; ++e) {
        const int unit = wave + e * WAVES;
        if (unit >= UNITS) break;
        Acc sum = red[0][unit][lane];
#pragma unroll
        for (int w = 1; w < WAVES; ++w) sum += red[w][unit][lane];
        const int m = m_base + (unit % MB) * 16 + i;
        const int n0 = (band0 + unit / MB) * 16 + 4 * g;
        if constexpr (RES) {
            // every lane takes part in the cross-lane sums; rows the batch does not have contribute zeros
            const EpilogueRegs eregs = finish_epilogue(ep, eraw[e]);
            uint16_t o[4];
            float hv[4], ssq_o = 0.0f, pmax_o = 0.0f;
            const uint32_t rbits[2] = {eres[e].x, eres[e].y}, wbits[2] = {enw[e].x, enw[e].y};
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                o[v] = apply_epilogue<int>(ep.kind, eregs, v, sum[v] >> kI8WeightShift);
                const float rv = (v & 1) ? __uint_as_float(rbits[v >> 1] & 0xffff0000u) : __uint_as_float(rbits[v >> 1] << 16);
                const float wv = (v & 1) ? __uint_as_float(wbits[v >> 1] & 0xffff0000u) : __uint_as_float(wbits[v >> 1] << 16);
                hv[v] = m < M ? bf16_bits_to_float(float_to_bf16_bits(rv + bf16_bits_to_float(o[v]))) : 0.0f;
                ssq_o = fmaf(hv[v], hv[v], ssq_o);
                pmax_o = fmaxf(pmax_o, fabsf(__fmul_rn(hv[v], wv)));
            }
            ssq_o = cross_row_reduce<false>(ssq_o);              // the four lanes (g = 0 .. 3) of a batch row: the band's sixteen features
            pmax_o = cross_row_reduce<true>(pmax_o);
            if (m < M) {
                *reinterpret_cast<u32x2*>(out + static_cast<size_t>(m) * N + n0) = u32x2{pack_bf16x2(hv[0], hv[1]), pack_bf16x2(hv[2], hv[3])};
                if (prod.raw_out != nullptr)
                    *reinterpret_cast<u32x2*>(prod.raw_out + static_cast<size_t>(m) * N + n0) =
                        u32x2{o[0] | (static_cast<uint32_t>(o[1]) << 16), o[2] | (static_cast<uint32_t>(o[3]) << 16)};
                if (g == 0) prod.stats_out[static_cast<size_t>(m) * (N / 16) + n0 / 16] = float2{ssq_o, pmax_o};
            }
        } else if (m < M) {
            const EpilogueRegs eregs = finish_epilogue(ep, eraw[e]);
            uint16_t o[4];
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                if constexpr (sizeof(Act) == 2) o[v] = apply_epilogue<float>(ep.kind, eregs, v, sum[v] * kBf16WeightUndo);
                else o[v] = apply_epilogue<int>(ep.kind, eregs, v, sum[v] >> kI8WeightShift);
            }
            const u32x2 pk = {o[0] | (static_cast<uint32_t>(o[1]) << 16), o[2] | (static_cast<uint32_t>(o[3]) << 16)};
            *reinterpret_cast<u32x2*>(out + static_cast<size_t>(m) * N + n0) = pk;
        }
    }
}

}  // namespace terna
