// Small-M TernaSpMM kernel on the P2 layout for up to 16 activation rows and a K that one workgroup holds in flight:
// the straight-line form of decode_packed_kernel.h (same work split, same operand order, same arithmetic, the same
// results bit for bit), built around what bounds a launch of a few microseconds -- not bytes and not MFMA, but
//   (a) the one round trip to HBM, which cannot start before the wave has its addresses, and
//   (b) the instructions of its waves: a 64-lane instruction occupies its SIMD for four cycles and the four waves
//       that share a SIMD take turns, so every vector instruction of the prologue and the epilogue is paid 16 cycles.
//
//   * Every load of a wave is a raw buffer load: the address is a scalar offset (band, tile) plus one per-lane
//     offset computed once, rows the batch does not have are switched off by an out-of-range lane offset (the
//     hardware returns zeros and touches no memory) -- no 64-bit address arithmetic, no masked branches, and the
//     compiler's wait counters stay exact because nothing is loaded inside a branch.
//   * Loads return in the order they were issued.  The activations (a few KB, cache resident) are requested first and
//     turned into MFMA operands for ALL of the wave's tiles while the weights -- requested last, from HBM -- are still
//     on their way; once they arrive a band-tile costs one cross-lane permutation, the 2-bit expansion and the MFMA.
//   * TMAX tiles per wave, all in flight at once: no prefetch ring, no loop-carried wait.  Tiles past K re-read the
//     wave's first tile (a cache hit) and are skipped by a scalar branch.
//   * The cross-wave sum and the epilogue are spread over four waves per band (one accumulator per lane, 16 LDS reads
//     and one division each) instead of one wave doing four of everything; four neighbouring lanes then pack their
//     bf16 results into one 8-byte store.  The order of the additions is wave 0, 1, 2, ... as before.
#pragma once

#include "packed_common.h"
#include "norm_quant_kernel.h"

namespace terna {

// The weight-scale group of one output column (the rule of ws_group_decode4 / ws_group_prefill for a single column).
__device__ __forceinline__ int ws_group_of(int n, int N, int ws_num, int kind)
{
    if (ws_num == 1) return 0;
    if (kind == EP_I8_PREFILL) return ws_group_prefill(n, N, ws_num);
    if (ws_num == 3 && N == 3840) return n < 2560 ? 0 : (n < 3200 ? 1 : 2);
    return n / (N / ws_num);
}

template <typename Act, int WAVES, int TMAX, int NB = 1, bool GUARD = false>
__global__ __launch_bounds__(WAVES * 64) void terna_decode_flat_kernel(
    const Act* __restrict__ x, const uint32_t* __restrict__ packed, uint16_t* __restrict__ out,
    int M, int N, int K, Epilogue ep, RepackGuard guard)
{
    if constexpr (GUARD) {                       // the extra, checking workgroup is the first of the grid: see decode_packed_kernel.h
        if (blockIdx.x == 0) {
            if (threadIdx.x < 64) repack_guard_role(guard, threadIdx.x);
            return;
        }
    }
    using T = ActTraits<Act>;
    using Acc = typename T::Acc;
    using AccScalar = typename T::AccScalar;
    using XS = XSlab<Act>;
    constexpr bool BF16 = sizeof(Act) == 2;
    constexpr int TASKS = 4 * NB;                // finishing waves: four per band (one 16-lane group of accumulators each)
    static_assert(TASKS <= WAVES, "one finishing task per wave at most");

    __shared__ Acc red[WAVES][NB][64];
    __shared__ __align__(16) uint8_t xslab_all[WAVES][16 * XS::kPitch];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int band0 = (static_cast<int>(blockIdx.x) - (GUARD ? 1 : 0)) * NB;
    const int ktiles = K >> 6;
    const int i = lane & 15, g = lane >> 4;

    // this wave's tiles: wave, wave + WAVES, ...; a slot past K falls back to the wave's first tile (tile 0 for a
    // wave that has none) -- scalar selects only
    int jt[TMAX];
    bool tv[TMAX];
    const int jfirst = wave < ktiles ? wave : 0;
#pragma unroll
    for (int t = 0; t < TMAX; ++t) {
        const int j = wave + WAVES * t;
        tv[t] = j < ktiles;
        jt[t] = tv[t] ? j : jfirst;
    }

    // ---- (1) the activations: coalesced 16-byte pieces of the [16 rows][64 columns] slab of every tile
    const __amdgpu_buffer_rsrc_t rx = make_raw_buffer(x, static_cast<uint32_t>(M) * K * sizeof(Act));
    int xoff[XS::kLoads];
#pragma unroll
    for (int h = 0; h < XS::kLoads; ++h) {
        const int row = XS::row_of(lane, h);
        xoff[h] = row < M ? (row * K + XS::col_of(lane)) * static_cast<int>(sizeof(Act)) : kBufferOutOfRange;
    }
    u32x4 xr[TMAX][XS::kLoads];
#pragma unroll
    for (int t = 0; t < TMAX; ++t)
#pragma unroll
        for (int h = 0; h < XS::kLoads; ++h)
            xr[t][h] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rx, xoff[h], jt[t] * (64 * static_cast<int>(sizeof(Act))), 0));
    __builtin_amdgcn_sched_barrier(0);           // the weight loads stay behind the activation loads

    // ---- (2) the weights: lane L loads word L of a band-tile (consecutive lanes, consecutive words: one 256-byte line)
    const __amdgpu_buffer_rsrc_t rw = make_raw_buffer(packed, static_cast<uint32_t>(N >> 4) * static_cast<uint32_t>(ktiles) * 256u);
    uint32_t wword[NB][TMAX];
#pragma unroll
    for (int t = 0; t < TMAX; ++t)
#pragma unroll
        for (int b = 0; b < NB; ++b)
            wword[b][t] = __builtin_amdgcn_raw_buffer_load_b32(rw, lane * 4, ((band0 + b) * ktiles + jt[t]) * 256, 0);
    __builtin_amdgcn_sched_barrier(0);

    // ---- (3) what the finishing waves need at the very end: wave 4u + q finishes the accumulators of lanes 16q .. 16q+15
    // of band u, lane l the element (l & 3) of lane 16q + (l >> 2): batch row l >> 2, output column 4q + (l & 3)
    const int fin_band = band0 + (wave < TASKS ? wave >> 2 : 0);
    const int fin_m = lane >> 2;
    const int fin_n = fin_band * 16 + 4 * (wave & 3) + (lane & 3);
    uint32_t es = 0u, ew = 0u;
    if (wave < TASKS) {
        const int grp = ws_group_of(fin_n, N, ep.ws_num, ep.kind);
        if constexpr (BF16) {
            ew = __float_as_uint(ep.scale[grp]);
        } else {
            es = ep.s[fin_m < M ? fin_m : 0];
            ew = ep.ws[grp];
        }
    }

    // ---- (4) activations -> MFMA operand order through the wave's LDS slot, every tile, before any weight is needed
    uint8_t* slab = xslab_all[wave];
    u32x4 bx[TMAX][BF16 ? 2 : 1];
#pragma unroll
    for (int t = 0; t < TMAX; ++t) {
        if (tv[t]) {
#pragma unroll
            for (int h = 0; h < XS::kLoads; ++h) *reinterpret_cast<u32x4*>(slab + XS::write_off(lane, h)) = xr[t][h];
            if constexpr (BF16) {
                const uint8_t* src = slab + i * XS::kPitch + g * 32;
                bx[t][0] = *reinterpret_cast<const u32x4*>(src);          // columns 16g .. 16g+7
                bx[t][1] = *reinterpret_cast<const u32x4*>(src + 16);     // columns 16g+8 .. 16g+15
            } else {
                bx[t][0] = *reinterpret_cast<const u32x4*>(slab + i * XS::kPitch + g * 16);
            }
        }
    }
    __builtin_amdgcn_sched_barrier(0);           // nothing that needs a weight word moves up into the staging

    // ---- (5) the weights: operand order by one LDS-crossbar permutation, 2-bit expansion, MFMA
    const int operand_src = (i * 4 + g) * 4;
    Acc acc[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) acc[b] = Acc{0, 0, 0, 0};
#pragma unroll
    for (int t = 0; t < TMAX; ++t) {
        if (tv[t]) {
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const uint32_t w = static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(operand_src, static_cast<int>(wword[b][t])));
                if constexpr (BF16) {
                    const bf16x8 a0 = __builtin_bit_cast(bf16x8, expand_chunk_bf16(w << 4));
                    const bf16x8 a1 = __builtin_bit_cast(bf16x8, expand_chunk_bf16(w));
                    acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, __builtin_bit_cast(bf16x8, bx[t][0]), acc[b], 0, 0, 0);
                    acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, __builtin_bit_cast(bf16x8, bx[t][1]), acc[b], 0, 0, 0);
                } else {
                    acc[b] = __builtin_amdgcn_mfma_i32_16x16x64_i8(expand_word_i8(w), __builtin_bit_cast(i32x4, bx[t][0]), acc[b], 0, 0, 0);
                }
            }
        }
    }

    // ---- (6) cross-wave sum in wave order and the epilogue, one accumulator per lane of the finishing waves
#pragma unroll
    for (int b = 0; b < NB; ++b) red[wave][b][lane] = acc[b];
    if (wave < TASKS) asm volatile("" : "+v"(es), "+v"(ew));      // requested in (3): must not sink below the barrier
    __syncthreads();
    if (wave < TASKS) {
        const AccScalar* rp = reinterpret_cast<const AccScalar*>(&red[0][wave >> 2][0]) + 64 * (wave & 3) + lane;
        AccScalar sum = rp[0];
#pragma unroll
        for (int w = 1; w < WAVES; ++w) sum += rp[w * (NB * 256)];
        EpilogueRegs e;
        uint16_t o;
        if constexpr (BF16) {
            e.s = 1.0f;
            e.w[0] = __uint_as_float(ew);
            o = apply_epilogue<float>(ep.kind, e, 0, sum * kBf16WeightUndo);
        } else {
            e.s = __uint_as_float(es << 16);
            e.w[0] = __uint_as_float(ew << 16);
            o = apply_epilogue<int>(ep.kind, e, 0, sum >> kI8WeightShift);
        }
        // four neighbouring lanes hold four consecutive columns of one batch row: one 8-byte store by the first of them
        const uint32_t o32 = o;
        const uint32_t p2 = o32 | (dpp_permute_u32<kDppSwapPairs>(o32) << 16);
        const uint32_t p4 = dpp_permute_u32<kDppSwapHalfQuads>(p2);
        if ((lane & 3) == 0 && fin_m < M)
            *reinterpret_cast<u32x2*>(out + static_cast<size_t>(fin_m) * N + fin_n) = u32x2{p2, p4};
    }
}

}  // namespace terna
