// Small-M TernaSpMM kernel on the P2 layout, up to 16 activation rows, four band-tiles per load.
//
// What bounds a launch of three microseconds is not bytes and not MFMA: it is the one round trip to HBM, which starts when
// a wave's weight load has been ISSUED, plus what the wave still has to do once the data is there.  Two facts of the
// memory pipeline shape the kernel:
//   * the CU's address unit takes a wave's load instruction in about twelve cycles whatever its width, one after the other
//     for all sixteen waves: a design with one 256-byte load per band-tile and one activation load per tile (96 of them
//     for K = 2560) has its last request out a thousand cycles after the first;
//   * the vector cache returns data in the order of the requests, for all waves of the CU together: a cache-resident
//     activation requested behind somebody's weight load arrives with the weights, not before.
// So: few, wide loads, the weights first, and as little as possible between their arrival and the MFMA.
//   * weights: one 16-byte load per lane fetches FOUR consecutive band-tiles (1 KB) -- lane L = 16 t + i receives the four
//     words of weight row i of tile t, i.e. the row's 64 columns in groups of 16.  No cross-lane permutation is needed:
//     MFMA number c of the chunk takes component c of every lane as its A operand (row i, tile t, columns 16c .. 16c+15)
//     and the B operand is read to match (batch row m, tile t, the same 16 columns): the k index of the instruction runs
//     over (tile, column) instead of the 64 columns of one tile.  Integer sums do not depend on that order; the fp32 sums
//     of the bf16 family are added in an order of their own (within the family's tolerance).
//   * activations: the chunk's [MR rows][256 columns] slab, 16 lanes along a row (bf16: 32), MR / 4 (MR / 2) coalesced
//     16-byte loads; through the wave's own LDS slot (row pitch + 16 bytes: conflict free) into operand order.  No
//     workgroup barrier before the MFMAs.  Rows the batch does not have and columns past K get an out-of-range lane
//     offset: the hardware returns zeros and touches no memory.
//   * wave w takes chunks w, w + 16, ... (CT at most); a wave without a chunk goes straight to the barrier of the sum.
//   * cross-wave sum and epilogue: four waves, one accumulator per lane (decode_flat_kernel.h).
#pragma once

#include "decode_flat_kernel.h"

namespace terna {

constexpr int kChunkWaves = 16;

template <typename Act, int CT, int MR, bool GUARD = false>
__global__ __launch_bounds__(kChunkWaves * 64) void terna_decode_chunk_kernel(
    const Act* __restrict__ x, const uint32_t* __restrict__ packed, uint16_t* __restrict__ out,
    int M, int N, int K, Epilogue ep, RepackGuard guard)
{
    // GUARD: one extra workgroup checks the cached copy's fingerprint (decode_packed_kernel.h).  It is the FIRST of the grid:
    // its check is two dependent memory round trips, longer than a band's work, and starts ahead of the bands' dispatch.
    if constexpr (GUARD) {
        if (blockIdx.x == 0) {
            if (threadIdx.x < 64) repack_guard_role(guard, threadIdx.x);
            return;
        }
    }
    using T = ActTraits<Act>;
    using Acc = typename T::Acc;
    using AccScalar = typename T::AccScalar;
    constexpr bool BF16 = sizeof(Act) == 2;
    constexpr int SZ = static_cast<int>(sizeof(Act));
    constexpr int WAVES = kChunkWaves;
    constexpr int PIECES = BF16 ? 8 : 4;         // 16-byte B operands per chunk and lane (64 columns of one tile)
    constexpr int ROWLANES = 16 * SZ;            // lanes along a chunk row of 256 columns
    constexpr int ROWS_PER_LOAD = 64 / ROWLANES;
    constexpr int XL = MR / ROWS_PER_LOAD;       // activation loads per chunk
    constexpr int PITCH = 256 * SZ + 16;
    static_assert(MR == 4 || MR == 8 || MR == 16, "rows of the slab");

    __shared__ Acc red[WAVES][64];
    __shared__ __align__(16) uint8_t slab_all[WAVES][16 * PITCH];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int band = static_cast<int>(blockIdx.x) - (GUARD ? 1 : 0);
    const int ktiles = K >> 6;
    const int i = lane & 15, g = lane >> 4;

    // wave q < 4 finishes the accumulators of lanes 16q .. 16q+15, lane l the element (l & 3) of lane 16q + (l >> 2):
    // batch row l >> 2, output column 4q + (l & 3)
    const bool finisher = wave < 4;
    const int fin_m = lane >> 2;
    const int fin_n = band * 16 + 4 * (wave & 3) + (lane & 3);
    uint32_t es = 0u, ew = 0u;

    Acc acc = Acc{0, 0, 0, 0};
    // ---- (1) the weights, at once.  Tiles past K (the tail of a partial last chunk, a chunk slot this wave does not
    // have) come back as zeros; a wave without any chunk issues nothing
    const bool has_work = wave * 4 < ktiles;
    u32x4 wq[CT];
    if (has_work) {
        const __amdgpu_buffer_rsrc_t rw = make_raw_buffer(packed, static_cast<uint32_t>(N >> 4) * static_cast<uint32_t>(ktiles) * 256u);
#pragma unroll
        for (int t = 0; t < CT; ++t) {
            const int tile0 = (wave + WAVES * t) * 4;
            wq[t] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rw, tile0 + g < ktiles ? lane * 16 : kBufferOutOfRange,
                                                                                   (band * ktiles + tile0) * 256, 0));
        }
        __builtin_amdgcn_sched_barrier(0);       // nothing from below is scheduled ahead of the weight requests
    }
    // (A workgroup barrier here, so that every wave's weight requests precede anybody's activation requests, was measured:
    // slower -- the activations then arrive last and everything waits for them.)
    if (has_work) {
        // ---- (2) the activations of the wave's chunks
        const int rowbytes = K * SZ;
        const __amdgpu_buffer_rsrc_t rx = make_raw_buffer(x, static_cast<uint32_t>(M) * rowbytes);
        const int xrow = lane / ROWLANES, xcol = (lane % ROWLANES) * 16;       // this lane's row within a load, byte column within the chunk row
        u32x4 xr[CT][XL];
#pragma unroll
        for (int t = 0; t < CT; ++t) {
            const int col0 = (wave + WAVES * t) * (256 * SZ);                   // byte column of the chunk
#pragma unroll
            for (int h = 0; h < XL; ++h) {
                const int row = xrow + ROWS_PER_LOAD * h;
                const bool ok = row < M && col0 + xcol < rowbytes;
                xr[t][h] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rx, ok ? row * rowbytes + xcol : kBufferOutOfRange, col0, 0));
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        // ---- (3) what the finishing waves need at the very end
        if (finisher) {
            const int grp = ws_group_of(fin_n, N, ep.ws_num, ep.kind);
            if constexpr (BF16) {
                ew = __float_as_uint(ep.scale[grp]);
            } else {
                es = ep.s[fin_m < M ? fin_m : 0];
                ew = ep.ws[grp];
            }
        }
        // ---- (4) per chunk: activations through the wave's LDS slot into operand order, 2-bit expansion, MFMA
        uint8_t* slab = slab_all[wave];
        if constexpr (MR < 16) {                 // rows the slab never receives: zeros, once
            for (int o = MR * PITCH + lane * 16; o < 16 * PITCH; o += 64 * 16) *reinterpret_cast<u32x4*>(slab + o) = u32x4{0u, 0u, 0u, 0u};
        }
#pragma unroll
        for (int t = 0; t < CT; ++t) {
#pragma unroll
            for (int h = 0; h < XL; ++h) *reinterpret_cast<u32x4*>(slab + (xrow + ROWS_PER_LOAD * h) * PITCH + xcol) = xr[t][h];
            // lane (i, g): batch row i, tile g of the chunk -- its 64 columns, 16 bytes at a time
            const uint8_t* src = slab + i * PITCH + g * (64 * SZ);
            u32x4 bq[PIECES];
#pragma unroll
            for (int p = 0; p < PIECES; ++p) bq[p] = *reinterpret_cast<const u32x4*>(src + 16 * p);
            const uint32_t wc[4] = {wq[t].x, wq[t].y, wq[t].z, wq[t].w};
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                if constexpr (BF16) {
                    const bf16x8 a0 = __builtin_bit_cast(bf16x8, expand_chunk_bf16(wc[c] << 4));    // columns 16c .. 16c+7
                    const bf16x8 a1 = __builtin_bit_cast(bf16x8, expand_chunk_bf16(wc[c]));         // columns 16c+8 .. 16c+15
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, __builtin_bit_cast(bf16x8, bq[2 * c]), acc, 0, 0, 0);
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, __builtin_bit_cast(bf16x8, bq[2 * c + 1]), acc, 0, 0, 0);
                } else {
                    acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(expand_word_i8(wc[c]), __builtin_bit_cast(i32x4, bq[c]), acc, 0, 0, 0);
                }
            }
        }
    } else if (finisher) {                       // a finishing wave without a chunk (K < 256 * its number)
        const int grp = ws_group_of(fin_n, N, ep.ws_num, ep.kind);
        if constexpr (BF16) {
            ew = __float_as_uint(ep.scale[grp]);
        } else {
            es = ep.s[fin_m < M ? fin_m : 0];
            ew = ep.ws[grp];
        }
    }

    // ---- (5) cross-wave sum in wave order and the epilogue: one accumulator per lane of the finishing waves
    red[wave][lane] = acc;
    if (finisher) asm volatile("" : "+v"(es), "+v"(ew));          // requested above: must not sink below the barrier
    __syncthreads();
    if (finisher) {
        const AccScalar* rp = reinterpret_cast<const AccScalar*>(&red[0][0]) + 64 * wave + lane;
        AccScalar sum = rp[0];
#pragma unroll
        for (int w = 1; w < WAVES; ++w) sum += rp[w * 256];
        EpilogueRegs e;
        uint16_t o;
        if constexpr (BF16) {
            e.s = 1.0f;
            e.w[0] = __uint_as_float(ew);
            o = apply_epilogue<float>(EP_BF16, e, 0, sum * kBf16WeightUndo);
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

// The same for matrices of more than 256 bands (gate+up: 864): FOUR bands per workgroup, so that one round of workgroups
// covers the matrix.  A unit of work is (chunk, band pair): one activation slab, two weight loads, eight MFMAs into two
// accumulators; unit u = wave + 16 t (t < 2) is chunk u of pair 0 for u < chunks, chunk u - chunks of pair 1 behind it
// (chunks <= 16, so a wave has at most one unit of each pair and every SIMD gets the same number of units).  A wave
// leaves one accumulator per band in LDS (zeros for a pair it had no unit of); all 16 waves finish: wave 4b + q the
// accumulators of lanes 16q .. 16q+15 of band b.
// UNIT_BANDS = 4: a unit is a chunk with all four bands -- half as many activation loads and stagings, ten working waves
// instead of sixteen for K = 2560.  Measured on gate+up: the same at 8 rows (5.20 against 5.22 us), slower at 1 - 4 rows
// (5.06 against 4.83); not instantiated by the launcher.  (In the chained form, where the unit's activations are also
// normed and quantised, the whole-chunk unit is the faster one: chain_chunk_kernel.h.)
template <typename Act, int MR, bool GUARD = false, int UNIT_BANDS = 2>
__global__ __launch_bounds__(kChunkWaves * 64) void terna_decode_chunk4_kernel(
    const Act* __restrict__ x, const uint32_t* __restrict__ packed, uint16_t* __restrict__ out,
    int M, int N, int K, Epilogue ep, RepackGuard guard)
{
    if constexpr (GUARD) {                       // the checking workgroup comes first (see above)
        if (blockIdx.x == 0) {
            if (threadIdx.x < 64) repack_guard_role(guard, threadIdx.x);
            return;
        }
    }
    using T = ActTraits<Act>;
    using Acc = typename T::Acc;
    using AccScalar = typename T::AccScalar;
    constexpr bool BF16 = sizeof(Act) == 2;
    constexpr int SZ = static_cast<int>(sizeof(Act));
    constexpr int WAVES = kChunkWaves;
    constexpr int PIECES = BF16 ? 8 : 4;
    constexpr int ROWLANES = 16 * SZ;
    constexpr int ROWS_PER_LOAD = 64 / ROWLANES;
    constexpr int XL = MR / ROWS_PER_LOAD;
    constexpr int PITCH = 256 * SZ + 16;
    constexpr int SLAB_ROWS = MR < 16 ? MR + 1 : 16;             // one row of zeros for the batch rows the slab does not hold
    static_assert(MR == 4 || MR == 8 || MR == 16, "rows of the slab");

    __shared__ Acc red[WAVES][4][64];
    __shared__ __align__(16) uint8_t slab_all[WAVES][SLAB_ROWS * PITCH];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int band0 = (static_cast<int>(blockIdx.x) - (GUARD ? 1 : 0)) * 4;
    const int ktiles = K >> 6;
    const int chunks = (ktiles + 3) >> 2;
    const int i = lane & 15, g = lane >> 4;

    // this wave's units
    constexpr int UB = UNIT_BANDS;
    constexpr int UT = 4 / UB;                   // unit slots per wave: two (chunk, pair) units, or one whole chunk
    static_assert(UB == 2 || UB == 4, "a gate / up pair or all four bands");
    int upair[UT], uchunk[UT];
    bool uok[UT];
#pragma unroll
    for (int t = 0; t < UT; ++t) {
        const int u = wave + WAVES * t;
        if constexpr (UB == 2) {
            upair[t] = u >= chunks ? 1 : 0;
            uchunk[t] = u - upair[t] * chunks;
            uok[t] = u < 2 * chunks;
        } else {
            upair[t] = 0;
            uchunk[t] = u;
            uok[t] = u < chunks;
        }
    }

    // ---- (1) the weights of both units, at once (a unit the wave does not have: out of range, zeros)
    const __amdgpu_buffer_rsrc_t rw = make_raw_buffer(packed, static_cast<uint32_t>(N >> 4) * static_cast<uint32_t>(ktiles) * 256u);
    u32x4 wq[UT][UB];
#pragma unroll
    for (int t = 0; t < UT; ++t) {
        const int tile0 = uchunk[t] * 4;
        const int voff = uok[t] && tile0 + g < ktiles ? lane * 16 : kBufferOutOfRange;
#pragma unroll
        for (int b = 0; b < UB; ++b)
            wq[t][b] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rw, voff, ((band0 + UB * upair[t] + b) * ktiles + tile0) * 256, 0));
    }
    __builtin_amdgcn_sched_barrier(0);           // nothing from below is scheduled ahead of the weight requests
    // ---- (2) the activations of the units' chunks
    const int rowbytes = K * SZ;
    const __amdgpu_buffer_rsrc_t rx = make_raw_buffer(x, static_cast<uint32_t>(M) * rowbytes);
    const int xrow = lane / ROWLANES, xcol = (lane % ROWLANES) * 16;
    u32x4 xr[UT][XL];
#pragma unroll
    for (int t = 0; t < UT; ++t) {
        const int col0 = uchunk[t] * (256 * SZ);
#pragma unroll
        for (int h = 0; h < XL; ++h) {
            const int row = xrow + ROWS_PER_LOAD * h;
            const bool ok = uok[t] && row < M && col0 + xcol < rowbytes;
            xr[t][h] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rx, ok ? row * rowbytes + xcol : kBufferOutOfRange, col0, 0));
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    // ---- (3) what this wave needs to finish band wave / 4, lanes 16 (wave % 4) ..: batch row l >> 2, column 4 (wave % 4) + (l & 3)
    const int fin_m = lane >> 2;
    const int fin_n = (band0 + (wave >> 2)) * 16 + 4 * (wave & 3) + (lane & 3);
    uint32_t es = 0u, ew = 0u;
    {
        const int grp = ws_group_of(fin_n, N, ep.ws_num, ep.kind);
        if constexpr (BF16) {
            ew = __float_as_uint(ep.scale[grp]);
        } else {
            es = ep.s[fin_m < M ? fin_m : 0];
            ew = ep.ws[grp];
        }
    }
    // ---- (4) per unit: activations through the wave's LDS slot into operand order, 2-bit expansion, MFMA
    uint8_t* slab = slab_all[wave];
    if constexpr (MR < 16) {
        for (int o = MR * PITCH + lane * 16; o < SLAB_ROWS * PITCH; o += 64 * 16) *reinterpret_cast<u32x4*>(slab + o) = u32x4{0u, 0u, 0u, 0u};
    }
    Acc acc[UT][UB];
#pragma unroll
    for (int t = 0; t < UT; ++t) {
#pragma unroll
        for (int b = 0; b < UB; ++b) acc[t][b] = Acc{0, 0, 0, 0};
        if (uok[t]) {
#pragma unroll
            for (int h = 0; h < XL; ++h) *reinterpret_cast<u32x4*>(slab + (xrow + ROWS_PER_LOAD * h) * PITCH + xcol) = xr[t][h];
            const uint8_t* src = slab + (i < MR ? i : MR) * PITCH + g * (64 * SZ);
            u32x4 bq[PIECES];
#pragma unroll
            for (int p = 0; p < PIECES; ++p) bq[p] = *reinterpret_cast<const u32x4*>(src + 16 * p);
#pragma unroll
            for (int b = 0; b < UB; ++b) {
                const uint32_t wc[4] = {wq[t][b].x, wq[t][b].y, wq[t][b].z, wq[t][b].w};
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    if constexpr (BF16) {
                        const bf16x8 a0 = __builtin_bit_cast(bf16x8, expand_chunk_bf16(wc[c] << 4));
                        const bf16x8 a1 = __builtin_bit_cast(bf16x8, expand_chunk_bf16(wc[c]));
                        acc[t][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, __builtin_bit_cast(bf16x8, bq[2 * c]), acc[t][b], 0, 0, 0);
                        acc[t][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, __builtin_bit_cast(bf16x8, bq[2 * c + 1]), acc[t][b], 0, 0, 0);
                    } else {
                        acc[t][b] = __builtin_amdgcn_mfma_i32_16x16x64_i8(expand_word_i8(wc[c]), __builtin_bit_cast(i32x4, bq[c]), acc[t][b], 0, 0, 0);
                    }
                }
            }
        }
    }
    // ---- (5) one accumulator per band into LDS: unit 0 is of pair upair[0], unit 1 (if there is one) of pair 1
    if constexpr (UB == 2) {
        const bool first_is_pair0 = upair[0] == 0;                 // scalar
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            red[wave][b][lane] = first_is_pair0 ? acc[0][b] : Acc{0, 0, 0, 0};
            red[wave][2 + b][lane] = first_is_pair0 ? acc[UT - 1][b] : acc[0][b];
        }
    } else {
#pragma unroll
        for (int b = 0; b < 4; ++b) red[wave][b][lane] = acc[0][b];
    }
    asm volatile("" : "+v"(es), "+v"(ew));
    __syncthreads();
    {
        const AccScalar* rp = reinterpret_cast<const AccScalar*>(&red[0][wave >> 2][0]) + 16 * 4 * (wave & 3) + lane;
        AccScalar sum = rp[0];
#pragma unroll
        for (int w = 1; w < WAVES; ++w) sum += rp[w * (4 * 256)];
        EpilogueRegs e;
        uint16_t o;
        if constexpr (BF16) {
            e.s = 1.0f;
            e.w[0] = __uint_as_float(ew);
            o = apply_epilogue<float>(EP_BF16, e, 0, sum * kBf16WeightUndo);
        } else {
            e.s = __uint_as_float(es << 16);
            e.w[0] = __uint_as_float(ew << 16);
            o = apply_epilogue<int>(ep.kind, e, 0, sum >> kI8WeightShift);
        }
        const uint32_t o32 = o;
        const uint32_t p2 = o32 | (dpp_permute_u32<kDppSwapPairs>(o32) << 16);
        const uint32_t p4 = dpp_permute_u32<kDppSwapHalfQuads>(p2);
        if ((lane & 3) == 0 && fin_m < M)
            *reinterpret_cast<u32x2*>(out + static_cast<size_t>(fin_m) * N + fin_n) = u32x2{p2, p4};
    }
}

}  // namespace terna
