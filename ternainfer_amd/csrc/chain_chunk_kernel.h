// The chained small-M linear (decode_fused_kernel.h, FUSED_STATS: norm statistics from the producer of h) in the shape
// of decode_chunk_kernel.h: few, wide loads -- one 16-byte load per lane for four band-tiles of weights, 16-byte pieces
// of the bf16 activations and of the norm weights -- the weights requested first, and between their arrival and the MFMA
// only what needs them.  A launch of the per-tile form issued 200 narrow loads per workgroup (2-byte activation and
// norm-weight pieces per tile and lane at one row) and its last request left a thousand cycles after the first.
//
//   prologue   wave r < M does nothing but add up row r's partials (sum h^2, max |h * norm_w|) in a fixed order -- the
//              same in every workgroup, so all bands see identical int8 activations -- and leave rstd and the
//              quantisation scale in LDS (barrier 1, long before the weights are there).  The other 16 - M waves share the
//              chunks.  (A wave that did both had its weight requests held up behind the partials' round trip: register
//              copies and reuse make the compiler wait for loads in flight.)  Then per chunk of 256 columns, element-wise:
//                y = bf16((h * norm_w) * rstd),  q = clamp(rint(y * s))      (quant_value: the selected mode)
//              eight columns per lane, int8 into the wave's LDS slot, B operands out in operand order.
//              (Requesting partials, activations and norm weights from all waves first, a barrier, then the weights --
//              so that the prologue runs under the weights' round trip instead of behind it -- was measured: 3 % fewer
//              tokens per second; the later weight requests cost more than the overlap gains.)
//   matmul     as decode_chunk_kernel.h: MFMA number c of a chunk takes component c of the weight load.
//   epilogue   the accumulators go to LDS as a [batch row][column] matrix; wave q finishes batch rows 4q .. 4q+3, lane l
//              column l & 15 of row 4q + (l >> 4): one division per lane, and the sixteen columns of a row sit in sixteen
//              neighbouring lanes, so the partial statistics of the producing epilogues are data-parallel row reductions.
//                CEPI_STORE     out[m][n] = bf16((sum / s[m]) * ws[group(n)])
//                CEPI_RESIDUAL  h' = bf16(residual[m][n] + out[m][n]) stored instead, with (sum h'^2, max |h' * next_w|) per
//                               row and band (model.py:330, :334 + the statistics of the norm that follows)
//                CEPI_GATE      (terna_chain_gate_kernel) bands alternate gate / up rows: inner = bf16(bf16(relu(x1)^2) * x3)
//                               (model.py:279-280) stored, N / 2 columns, with its statistics under the ffn_sub_norm weights
#pragma once

#include "decode_chunk_kernel.h"
#include "decode_fused_kernel.h"

namespace terna {

enum ChainEpilogue { CEPI_STORE, CEPI_RESIDUAL, CEPI_GATE };

struct ChainIo {
    uint16_t* out;                   // bf16 [M][N] (CEPI_GATE: [M][N/2])
    const uint16_t* ws;              // bf16 [ws_num]
    int8_t* xq_out;                  // optional: the quantised activations [M][K] and their scales [M] (workgroup 0 writes)
    uint16_t* s_out;
    const uint16_t* residual;        // CEPI_RESIDUAL: bf16 [M][N]
    const uint16_t* next_w;          // producing epilogues: weights of the norm that follows
    float2* stats_out;               // [M][N/16] (CEPI_GATE: [M][N/32])
    uint16_t* raw_out;               // CEPI_RESIDUAL, optional: the linear's own output
    const uint16_t* s_in = nullptr;  // activations quantised already (XQ): their scales, bf16 [M]
};

constexpr int kChainSlabPitch = 256 + 16;
        // int8 slab row: 256 columns + 16 bytes (conflict-free operand reads)

// Row statistics from the producer's partials: wave r < M, all its lanes.  Leaves rstd / the multiplier / the bf16 scale
// of row r in LDS (lane 0) and publishes the scale when asked to.
__device__ __forceinline__ void chain_reduce_partials(const float2 (&part)[kStatsMaxPartials / 64], int row, int K, float eps, int quant_mode,
                                                      float* rstd_s, float* smul_s, float* sval_s, uint16_t* s_out, int lane)
{
    float sum = 0.0f, pmax = 0.0f;
#pragma unroll
    for (int t = 0; t < kStatsMaxPartials / 64; ++t) {      // entries past the count were out of range: zeros
        sum += part[t].x;
        pmax = fmaxf(pmax, part[t].y);
    }
    sum = wave_sum(sum);
    pmax = wave_max(pmax);
    if (lane == 0) {
        const float r = rsqrtf(sum / static_cast<float>(K) + eps);
        const float amax_y = fabsf(round_bf16(__fmul_rn(pmax, r)));      // = max |y| of the row, exactly
        uint16_t sb;
        const float s_mul = quant_scale(amax_y, quant_mode, &sb);
        rstd_s[row] = r;
        smul_s[row] = s_mul;
        sval_s[row] = bf16_bits_to_float(sb);
        if (s_out != nullptr) s_out[row] = sb;
    }
}

// NE (4 or 8) columns of one row: norm + quantisation, packed int8 (NE / 4 dwords).
template <int NE>
__device__ __forceinline__ void chain_quantise(const uint32_t (&hraw)[NE / 2], const uint32_t (&wraw)[NE / 2], float rstd, float s_mul, int quant_mode,
                                               uint32_t (&d)[NE / 4])
{
    float f[NE], w[NE];
#pragma unroll
    for (int j = 0; j < NE / 2; ++j) {
        f[2 * j] = __uint_as_float(hraw[j] << 16);
        f[2 * j + 1] = __uint_as_float(hraw[j] & 0xffff0000u);
        w[2 * j] = __uint_as_float(wraw[j] << 16);
        w[2 * j + 1] = __uint_as_float(wraw[j] & 0xffff0000u);
    }
#pragma unroll
    for (int j = 0; j < NE / 4; ++j) d[j] = 0u;
    const bool eager = quant_mode == QUANT_EAGER;            // uniform: one branch, not one per element
    if (eager) {
#pragma unroll
        for (int e = 0; e < NE; ++e) {
            const float y = round_bf16(__fmul_rn(__fmul_rn(f[e], w[e]), rstd));
            d[e >> 2] = __builtin_amdgcn_cvt_pk_u8_f32(quant_value(y, s_mul, QUANT_EAGER) + 128.0f, e & 3, d[e >> 2]);
        }
    } else {
#pragma unroll
        for (int e = 0; e < NE; ++e) {
            const float y = round_bf16(__fmul_rn(__fmul_rn(f[e], w[e]), rstd));
            d[e >> 2] = __builtin_amdgcn_cvt_pk_u8_f32(quant_value(y, s_mul, QUANT_ROUNDED) + 128.0f, e & 3, d[e >> 2]);
        }
    }
#pragma unroll
    for (int j = 0; j < NE / 4; ++j) d[j] ^= 0x80808080u;
}

// NBANDS = 1: one band per workgroup, a unit of work is a chunk; CEPI_STORE / CEPI_RESIDUAL.
// NBANDS = 4: gate+up with the bands of w1 and w3 interleaved (band 2j = rows 16j .. of w1, band 2j+1 the same rows of
//             w3), two gate / up pairs per workgroup so that one round of workgroups covers 864 bands; CEPI_GATE.  A unit of
//             work is (chunk, pair) -- unit u is chunk u of pair 0 for u < chunks, chunk u - chunks of pair 1 behind it --
//             or, UNIT_BANDS = 4, a chunk with all four bands: its activations are then normed and quantised once.
// The 16 - M working waves take the units round robin, CT each at most.
// MR = 1, 2, 4 or 8 >= M: rows of the wave's LDS slot.  One row: 64 lanes x 4 columns; more: 32 lanes x 8 columns, two rows
// per load.
// XQ: the activations are quantised already (`hin` is int8 [M][K], io.s_in their scales; a launch of
// terna_quant_stats_kernel or of the norm kernel made them): no reducing waves, no statistics, no barrier ahead of the
// matmul; all 16 waves share the units and a chunk's rows go from the load to the LDS slot as they are (16 bytes per lane,
// four rows per load).  The producing epilogues are the same.  MR = 16 exists in this form only.
template <int NBANDS, int CT, int MR, int EPI, int UNIT_BANDS = (NBANDS == 4 ? 2 : 1), bool XQ = false>
__global__ __launch_bounds__(kChunkWaves * 64) void terna_chain_chunk_kernel(
    const void* __restrict__ hin, const uint16_t* __restrict__ norm_w, const uint32_t* __restrict__ packed,
    const float2* __restrict__ stats_in, int M, int N, int K, int stats_count, float eps, int ws_num, int quant_mode, ChainIo io)
{
    static_assert((NBANDS == 1 && (EPI == CEPI_STORE || EPI == CEPI_RESIDUAL)) || (NBANDS == 4 && EPI == CEPI_GATE), "see above");
    static_assert(MR == 1 || MR == 2 || MR == 4 || MR == 8 || (XQ && MR == 16), "rows of the slab (sixteen: quantised rows only)");
    constexpr int WAVES = kChunkWaves;
    constexpr int NE = MR == 1 ? 4 : 8;          // columns per lane and load
    constexpr int LPR = 256 / NE;                // lanes along a chunk row
    constexpr int RPL = 64 / LPR;                // rows per load
    constexpr int XL = MR / RPL;                 // activation loads per chunk
    constexpr int FW = (MR + 3) / 4;             // finishing waves per band (pair)
    constexpr int UB = UNIT_BANDS;               // bands per unit of work
    static_assert(UB == NBANDS || (NBANDS == 4 && UB == 2), "a unit covers the workgroup's bands or one gate / up pair");
    constexpr int UPAIRS = NBANDS / UB;          // units per chunk
    constexpr int PT = kStatsMaxPartials / 64;
    constexpr int XLQ = (MR + 3) / 4;            // XQ: 16-byte loads per lane and chunk (four rows of 256 bytes each)

    __shared__ int red[WAVES][NBANDS][256];
    __shared__ __align__(16) uint8_t slab_all[WAVES][(MR + 1) * kChainSlabPitch];
    __shared__ float rstd_s[8], smul_s[8], sval_s[8];
    const uint16_t* h = static_cast<const uint16_t*>(hin);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int band0 = blockIdx.x * NBANDS;
    const int ktiles = K >> 6;
    const int chunks = (ktiles + 3) >> 2;
    const int i = lane & 15, g = lane >> 4;
    const bool writer = blockIdx.x == 0;

    // this wave's units of work
    const int reducers = XQ ? 0 : M;
    const bool reducer = wave < reducers;
    const int workers = WAVES - reducers;
    int upair[CT], uchunk[CT];
    bool uok[CT];
#pragma unroll
    for (int t = 0; t < CT; ++t) {
        const int u = wave - reducers + workers * t;
        if constexpr (UPAIRS == 2) {
            upair[t] = u >= chunks ? 1 : 0;
            uchunk[t] = u - upair[t] * chunks;
            uok[t] = !reducer && u < 2 * chunks;
        } else {
            upair[t] = 0;
            uchunk[t] = u;
            uok[t] = !reducer && u < chunks;
        }
    }
    const bool has_work = uok[0];

    // What a wave requests: a reducing wave its row's partials; a working wave the weights, then the activations and norm
    // weights of its chunks; a finishing wave the epilogue's operands on top.
    float2 part[PT];
    auto request_partials = [&]() {
        const __amdgpu_buffer_rsrc_t rs = make_raw_buffer(stats_in, static_cast<uint32_t>(M) * stats_count * 8u);
#pragma unroll
        for (int t = 0; t < PT; ++t) {
            const int idx = lane + 64 * t;
            const u32x2 v = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(rs, idx < stats_count ? (wave * stats_count + idx) * 8 : kBufferOutOfRange, 0, 0));
            part[t] = float2{__uint_as_float(v.x), __uint_as_float(v.y)};
        }
    };
    // Finishing: the accumulators of a band lie in LDS as a [batch row][column] matrix; task (p, q) = band (pair) p, batch
    // rows 4q .. 4q+3 goes to wave p FW + q: lane l has row 4q + (l >> 4), column l & 15.
    constexpr int FTASKS = (NBANDS == 4 ? 2 : 1) * FW;
    const bool finisher = wave < FTASKS;
    const int fin_p = wave / FW, fin_q = wave % FW;
    const int fin_m = 4 * fin_q + (lane >> 4);
    const int fin_col = lane & 15;
    const int out_cols = EPI == CEPI_GATE ? N / 2 : N;
    const int fin_n = (EPI == CEPI_GATE ? (static_cast<int>(blockIdx.x) * 2 + fin_p) : band0) * 16 + fin_col;   // output column
    uint32_t ew = 0u, ew3 = 0u, eres = 0u, enw = 0u, es = 0u;
    auto request_epilogue = [&]() {
        if constexpr (XQ) es = io.s_in[fin_m < M ? fin_m : 0];
        if constexpr (EPI == CEPI_GATE) {
            ew = io.ws[0];                       // gate rows (w1) and up rows (w3): one scale each
            ew3 = io.ws[1];
            enw = io.next_w[fin_n];
        } else {
            ew = io.ws[ws_num == 1 ? 0 : ws_group_decode(fin_n, N, ws_num)];
            if constexpr (EPI == CEPI_RESIDUAL) {
                eres = io.residual[static_cast<size_t>(fin_m < M ? fin_m : 0) * N + fin_n];
                enw = io.next_w[fin_n];
            }
        }
    };
    u32x4 wq[CT][UB];
    uint32_t xr[XQ ? 1 : CT][XL][NE / 2], nw[XQ ? 1 : CT][NE / 2];
    u32x4 xq8[XQ ? CT : 1][XLQ];
    const int xrow0 = XQ ? lane >> 4 : lane / LPR;               // row within a load, first of this lane's columns in the chunk
    const int xcol = XQ ? (lane & 15) * 16 : (lane % LPR) * NE;
    uint8_t* slab = slab_all[wave];
    if (has_work) {
        const __amdgpu_buffer_rsrc_t rw = make_raw_buffer(packed, static_cast<uint32_t>(N >> 4) * static_cast<uint32_t>(ktiles) * 256u);
#pragma unroll
        for (int t = 0; t < CT; ++t) {
            const int tile0 = uchunk[t] * 4;
            const int voff = uok[t] && tile0 + g < ktiles ? lane * 16 : kBufferOutOfRange;
#pragma unroll
            for (int b = 0; b < UB; ++b)
                wq[t][b] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rw, voff, ((band0 + UB * upair[t] + b) * ktiles + tile0) * 256, 0));
        }
        if constexpr (XQ) {
            const __amdgpu_buffer_rsrc_t rx = make_raw_buffer(hin, static_cast<uint32_t>(M) * K);
#pragma unroll
            for (int t = 0; t < CT; ++t) {
                const int col0 = uchunk[t] * 256;
                const bool col_ok = uok[t] && col0 + xcol < K;
#pragma unroll
                for (int q = 0; q < XLQ; ++q) {
                    const int row = xrow0 + 4 * q;
                    xq8[t][q] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rx, row < M && col_ok ? row * K + xcol : kBufferOutOfRange, col0, 0));
                }
            }
        } else {
        const __amdgpu_buffer_rsrc_t rx = make_raw_buffer(h, static_cast<uint32_t>(M) * K * 2u);
        const __amdgpu_buffer_rsrc_t rn = make_raw_buffer(norm_w, static_cast<uint32_t>(K) * 2u);
#pragma unroll
        for (int t = 0; t < CT; ++t) {
            const int col0 = uchunk[t] * 256;
            const bool col_ok = uok[t] && col0 + xcol < K;
#pragma unroll
            for (int q = 0; q < XL; ++q) {
                const int row = xrow0 + RPL * q;
                const int voff = row < M && col_ok ? (row * K + xcol) * 2 : kBufferOutOfRange;
                if constexpr (NE == 8) {
                    const u32x4 v = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rx, voff, col0 * 2, 0));
                    xr[t][q][0] = v.x; xr[t][q][1] = v.y; xr[t][q][2] = v.z; xr[t][q][3] = v.w;
                } else {
                    const u32x2 v = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(rx, voff, col0 * 2, 0));
                    xr[t][q][0] = v.x; xr[t][q][1] = v.y;
                }
            }
            const int woff = col_ok ? xcol * 2 : kBufferOutOfRange;
            if constexpr (NE == 8) {
                const u32x4 v = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rn, woff, col0 * 2, 0));
                nw[t][0] = v.x; nw[t][1] = v.y; nw[t][2] = v.z; nw[t][3] = v.w;
            } else {
                const u32x2 v = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(rn, woff, col0 * 2, 0));
                nw[t][0] = v.x; nw[t][1] = v.y;
            }
        }
        }
        if (finisher) request_epilogue();
        // the row of zeros behind the slab's MR rows
        for (int o = MR * kChainSlabPitch + lane * 16; o < (MR + 1) * kChainSlabPitch; o += 64 * 16) *reinterpret_cast<u32x4*>(slab + o) = u32x4{0u, 0u, 0u, 0u};
    } else {
        if (reducer) {
            request_partials();
            if (finisher) request_epilogue();
            chain_reduce_partials(part, wave, K, eps, quant_mode, rstd_s, smul_s, sval_s, writer ? io.s_out : nullptr, lane);
        } else if (finisher) {
            request_epilogue();
        }
    }
    if constexpr (!XQ) __syncthreads();          // barrier 1: the rows' statistics are in LDS

    // ---- per unit: norm + quantisation into the LDS slot, operands out, 2-bit expansion, MFMA
    constexpr int NACC = UPAIRS;                 // accumulator sets: one per pair that has units of its own
    i32x4 acc[NACC][UB];
#pragma unroll
    for (int p = 0; p < NACC; ++p)
#pragma unroll
        for (int b = 0; b < UB; ++b) acc[p][b] = i32x4{0, 0, 0, 0};
    if (has_work) {
#pragma unroll
        for (int t = 0; t < CT; ++t) {
            if (t > 0 && !uok[t]) continue;      // scalar
            const int col0 = uchunk[t] * 256;
            if constexpr (XQ) {
#pragma unroll
                for (int q = 0; q < XLQ; ++q) {
                    const int row = xrow0 + 4 * q;
                    if (row < MR) *reinterpret_cast<u32x4*>(slab + row * kChainSlabPitch + xcol) = xq8[t][q];
                }
            } else {
#pragma unroll
            for (int q = 0; q < XL; ++q) {
                const int row = xrow0 + RPL * q;
                const int rc = row < M ? row : 0;
                uint32_t d[NE / 4];
                chain_quantise<NE>(xr[t][q], nw[t], rstd_s[rc], smul_s[rc], quant_mode, d);
                const bool pub = writer && io.xq_out != nullptr && row < M && col0 + xcol < K && upair[t] == 0;
                if constexpr (NE == 8) {
                    *reinterpret_cast<u32x2*>(slab + row * kChainSlabPitch + xcol) = u32x2{d[0], d[1]};
                    if (pub) *reinterpret_cast<u32x2*>(io.xq_out + static_cast<size_t>(row) * K + col0 + xcol) = u32x2{d[0], d[1]};
                } else {
                    *reinterpret_cast<uint32_t*>(slab + row * kChainSlabPitch + xcol) = d[0];
                    if (pub) *reinterpret_cast<uint32_t*>(io.xq_out + static_cast<size_t>(row) * K + col0 + xcol) = d[0];
                }
            }
            }
            const uint8_t* src = slab + (i < MR ? i : MR) * kChainSlabPitch + g * 64;
            u32x4 bq[4];
#pragma unroll
            for (int p = 0; p < 4; ++p) bq[p] = *reinterpret_cast<const u32x4*>(src + 16 * p);
            auto multiply = [&](i32x4 (&dst)[UB]) {
#pragma unroll
                for (int b = 0; b < UB; ++b) {
                    const uint32_t wc[4] = {wq[t][b].x, wq[t][b].y, wq[t][b].z, wq[t][b].w};
#pragma unroll
                    for (int c = 0; c < 4; ++c)
                        dst[b] = __builtin_amdgcn_mfma_i32_16x16x64_i8(expand_word_i8(wc[c]), __builtin_bit_cast(i32x4, bq[c]), dst[b], 0, 0, 0);
                }
            };
            if constexpr (UPAIRS == 2) {
                if (upair[t] == 0) multiply(acc[0]);             // scalar
                else multiply(acc[1]);
            } else {
                multiply(acc[0]);
            }
        }
    }
    // ---- accumulators to LDS as [batch row][column] per band (lane (m, g) holds columns 4g .. 4g+3 of row m), barrier 2
#pragma unroll
    for (int p = 0; p < NACC; ++p)
#pragma unroll
        for (int b = 0; b < UB; ++b) *reinterpret_cast<i32x4*>(&red[wave][UB * p + b][i * 16 + 4 * g]) = acc[p][b];
    if (finisher) asm volatile("" : "+v"(ew), "+v"(ew3), "+v"(eres), "+v"(enw), "+v"(es));
    __syncthreads();
    if (finisher) {
        const bool row_ok = fin_m < M;
        EpilogueRegs e;
        e.s = XQ ? __uint_as_float(es << 16) : sval_s[row_ok ? fin_m : 0];
        if constexpr (EPI == CEPI_GATE) {
            const int* rp = &red[0][2 * fin_p][64 * fin_q + lane];
            int sum1 = rp[0], sum3 = rp[256];
#pragma unroll
            for (int w = 1; w < WAVES; ++w) {
                sum1 += rp[w * (NBANDS * 256)];
                sum3 += rp[w * (NBANDS * 256) + 256];
            }
            e.w[0] = __uint_as_float(ew << 16);
            const float x1 = bf16_bits_to_float(apply_epilogue<int>(EP_I8_DECODE, e, 0, sum1 >> kI8WeightShift));
            e.w[0] = __uint_as_float(ew3 << 16);
            const float x3 = bf16_bits_to_float(apply_epilogue<int>(EP_I8_DECODE, e, 0, sum3 >> kI8WeightShift));
            const float p = fmaxf(x1, 0.0f);
            const float hv = row_ok ? round_bf16(round_bf16(p * p) * x3) : 0.0f;
            float ssq = hv * hv;
            float pmax = fabsf(__fmul_rn(hv, __uint_as_float(enw << 16)));
            ssq = group_reduce<16, false>(ssq);
            pmax = group_reduce<16, true>(pmax);
            const uint32_t h32 = float_to_bf16_bits(hv);
            const uint32_t hp = h32 | (dpp_permute_u32<kDppSwapPairs>(h32) << 16);
            if (row_ok) {
                if ((lane & 1) == 0) *reinterpret_cast<uint32_t*>(io.out + static_cast<size_t>(fin_m) * out_cols + fin_n) = hp;
                if (fin_col == 0) io.stats_out[static_cast<size_t>(fin_m) * (out_cols / 16) + fin_n / 16] = float2{ssq, pmax};
            }
        } else {
            const int* rp = &red[0][0][64 * fin_q + lane];
            int sum = rp[0];
#pragma unroll
            for (int w = 1; w < WAVES; ++w) sum += rp[w * (NBANDS * 256)];
            e.w[0] = __uint_as_float(ew << 16);
            const uint16_t o = apply_epilogue<int>(EP_I8_DECODE, e, 0, sum >> kI8WeightShift);
            const uint32_t o32 = o;
            const uint32_t op = o32 | (dpp_permute_u32<kDppSwapPairs>(o32) << 16);
            if constexpr (EPI == CEPI_STORE) {
                if ((lane & 1) == 0 && row_ok) *reinterpret_cast<uint32_t*>(io.out + static_cast<size_t>(fin_m) * N + fin_n) = op;
            } else {
                const float hv = row_ok ? round_bf16(__uint_as_float(eres << 16) + bf16_bits_to_float(o)) : 0.0f;
                float ssq = hv * hv;
                float pmax = fabsf(__fmul_rn(hv, __uint_as_float(enw << 16)));
                ssq = group_reduce<16, false>(ssq);
                pmax = group_reduce<16, true>(pmax);
                const uint32_t h32 = float_to_bf16_bits(hv);
                const uint32_t hp = h32 | (dpp_permute_u32<kDppSwapPairs>(h32) << 16);
                if (row_ok) {
                    if ((lane & 1) == 0) {
                        *reinterpret_cast<uint32_t*>(io.out + static_cast<size_t>(fin_m) * N + fin_n) = hp;
                        if (io.raw_out != nullptr) *reinterpret_cast<uint32_t*>(io.raw_out + static_cast<size_t>(fin_m) * N + fin_n) = op;
                    }
                    if (fin_col == 0) io.stats_out[static_cast<size_t>(fin_m) * (N / 16) + fin_n / 16] = float2{ssq, pmax};
                }
            }
        }
    }
}

// The same linear with the norm's statistics taken INSIDE (no producer left them): the O projection behind the attention.
//   CPRO_NORM  x is bf16 [M][K]
//   CPRO_ATTN  one row: x is the fp32 buffer a deferred-merge attention launch left (attention_kernel.h) -- per head the
//              score maxima and sums of its ASP splits, then the splits' unnormalised results; a lane merges its four
//              columns with attention_merge's arithmetic, so the row has the bits the merge kernel would give
// One band per workgroup, every wave works (unit = chunk, wave w takes chunks w, w + 16, ...).  The prologue is a chain
// of its own here -- values, partial statistics per wave, barrier, totals, norm, quantisation -- so everything it reads
// (cache resident) is requested by ALL waves first, then a barrier, then the weights: the vector cache returns data in
// the order of the requests of the whole CU, and what is requested behind a weight load arrives with the weights.  The
// chain then runs under the weights' round trip.  Sums of squares: per lane in column order, the lanes of a row pairwise
// (group_reduce), the waves pairwise -- the same in every workgroup.
enum ChainPrologue { CPRO_NORM, CPRO_ATTN };

template <int PRO, int CT, int MR, int EPI, int ASP = 1, int AHD = 128>
__global__ __launch_bounds__(kChunkWaves * 64) void terna_chain_norm_kernel(
    const void* __restrict__ xin, const uint16_t* __restrict__ norm_w, const uint32_t* __restrict__ packed,
    int M, int N, int K, float eps, int ws_num, int quant_mode, ChainIo io)
{
    static_assert(EPI == CEPI_STORE || EPI == CEPI_RESIDUAL, "one band per workgroup");
    static_assert(MR == 1 || MR == 2 || MR == 4 || MR == 8, "rows of the slab");
    static_assert(PRO != CPRO_ATTN || MR == 1, "the attention merge feeds a single row");
    static_assert(AHD % 4 == 0 && 256 % AHD == 0 && ASP >= 1 && ASP <= kAttentionMaxSplits, "a lane's four columns lie inside one head");
    constexpr int WAVES = kChunkWaves;
    constexpr int NE = MR == 1 ? 4 : 8;
    constexpr int LPR = 256 / NE;
    constexpr int RPL = 64 / LPR;
    constexpr int XL = MR / RPL;
    constexpr int FW = (MR + 3) / 4;
    constexpr int PASSES = (MR + 3) / 4;         // four rows' totals per pass over the waves' partials

    __shared__ int red[WAVES][256];
    __shared__ __align__(16) uint8_t slab_all[WAVES][(MR + 1) * kChainSlabPitch];
    __shared__ float2 part_s[8][WAVES];          // per row and wave: (sum of squares, max |value * norm weight|)
    __shared__ float stat_w[WAVES][8][2];        // per wave, its own copy: rstd and the multiplier of every row

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int band = blockIdx.x;
    const int ktiles = K >> 6;
    const int chunks = (ktiles + 3) >> 2;
    const int i = lane & 15, g = lane >> 4;
    const bool writer = blockIdx.x == 0;
    int uchunk[CT];
    bool uok[CT];
#pragma unroll
    for (int t = 0; t < CT; ++t) {
        uchunk[t] = wave + WAVES * t;
        uok[t] = uchunk[t] < chunks;
    }
    const bool has_work = uok[0];
    const bool finisher = wave < FW;
    const int fin_m = 4 * wave + (lane >> 4);
    const int fin_n = band * 16 + (lane & 15);
    uint32_t ew = 0u, eres = 0u, enw = 0u;
    const int xrow0 = lane / LPR, xcol = (lane % LPR) * NE;
    uint8_t* slab = slab_all[wave];

    // ---- (1) everything the prologue reads, all waves; barrier; (2) the weights
    uint32_t xr[CT][XL][NE / 2], nw[CT][NE / 2];
    constexpr int SQ = PRO == CPRO_ATTN ? (ASP > 4 ? 4 : 2) : 1;                 // statistic quads of a head that matter
    f32x4 ast[PRO == CPRO_ATTN ? CT : 1][SQ], ao[PRO == CPRO_ATTN ? CT : 1][ASP];
    if (has_work) {
        const __amdgpu_buffer_rsrc_t rn = make_raw_buffer(norm_w, static_cast<uint32_t>(K) * 2u);
#pragma unroll
        for (int t = 0; t < CT; ++t) {
            const int col0 = uchunk[t] * 256;
            const bool col_ok = uok[t] && col0 + xcol < K;
            if constexpr (PRO == CPRO_ATTN) {
                const int heads = K / AHD;
                const __amdgpu_buffer_rsrc_t rp = make_raw_buffer(xin, static_cast<uint32_t>(heads) * (kAttentionStatFloats + ASP * AHD) * 4u);
                const int c = col0 + xcol;
                const int head = c / AHD, d = c % AHD;             // AHD is a power of two times ... a constant: shifts
#pragma unroll
                for (int q4 = 0; q4 < SQ; ++q4) {
                    const int quad = SQ == 2 ? 2 * q4 : q4;        // maxima 0-3 (4-7), sums 0-3 (4-7)
                    ast[t][q4] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rp, col_ok ? (head * kAttentionStatFloats + 4 * quad) * 4 : kBufferOutOfRange, 0, 0));
                }
#pragma unroll
                for (int jj = 0; jj < ASP; ++jj)
                    ao[t][jj] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(
                        rp, col_ok ? (heads * kAttentionStatFloats + (head * ASP + jj) * AHD + d) * 4 : kBufferOutOfRange, 0, 0));
            } else {
                const __amdgpu_buffer_rsrc_t rx = make_raw_buffer(xin, static_cast<uint32_t>(M) * K * 2u);
#pragma unroll
                for (int q = 0; q < XL; ++q) {
                    const int row = xrow0 + RPL * q;
                    const int voff = row < M && col_ok ? (row * K + xcol) * 2 : kBufferOutOfRange;
                    if constexpr (NE == 8) {
                        const u32x4 v = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rx, voff, col0 * 2, 0));
                        xr[t][q][0] = v.x; xr[t][q][1] = v.y; xr[t][q][2] = v.z; xr[t][q][3] = v.w;
                    } else {
                        const u32x2 v = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(rx, voff, col0 * 2, 0));
                        xr[t][q][0] = v.x; xr[t][q][1] = v.y;
                    }
                }
            }
            const int woff = col_ok ? xcol * 2 : kBufferOutOfRange;
            if constexpr (NE == 8) {
                const u32x4 v = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rn, woff, col0 * 2, 0));
                nw[t][0] = v.x; nw[t][1] = v.y; nw[t][2] = v.z; nw[t][3] = v.w;
            } else {
                const u32x2 v = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(rn, woff, col0 * 2, 0));
                nw[t][0] = v.x; nw[t][1] = v.y;
            }
        }
    }
    if (finisher) {
        ew = io.ws[ws_num == 1 ? 0 : ws_group_decode(fin_n, N, ws_num)];
        if constexpr (EPI == CEPI_RESIDUAL) {
            eres = io.residual[static_cast<size_t>(fin_m < M ? fin_m : 0) * N + fin_n];
            enw = io.next_w[fin_n];
        }
    }
    __builtin_amdgcn_s_barrier();                // every cache-resident request of the CU is out
    u32x4 wq[CT];
    if (has_work) {
        const __amdgpu_buffer_rsrc_t rw = make_raw_buffer(packed, static_cast<uint32_t>(N >> 4) * static_cast<uint32_t>(ktiles) * 256u);
#pragma unroll
        for (int t = 0; t < CT; ++t) {
            const int tile0 = uchunk[t] * 4;
            wq[t] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rw, uok[t] && tile0 + g < ktiles ? lane * 16 : kBufferOutOfRange,
                                                                                   (band * ktiles + tile0) * 256, 0));
        }
        for (int o = MR * kChainSlabPitch + lane * 16; o < (MR + 1) * kChainSlabPitch; o += 64 * 16) *reinterpret_cast<u32x4*>(slab + o) = u32x4{0u, 0u, 0u, 0u};
    }

    // ---- (3) the values (CPRO_ATTN: merged and rounded to bf16) and this wave's partial statistics per row
    float pss[XL], pmx[XL];
#pragma unroll
    for (int q = 0; q < XL; ++q) pss[q] = pmx[q] = 0.0f;
    if (has_work) {
#pragma unroll
        for (int t = 0; t < CT; ++t) {
            if constexpr (PRO == CPRO_ATTN) {
                float am[kAttentionMaxSplits], al[kAttentionMaxSplits];
#pragma unroll
                for (int jj = 0; jj < ASP; ++jj) {
                    am[jj] = ast[t][jj >> 2][jj & 3];
                    al[jj] = ast[t][(SQ / 2) + (jj >> 2)][jj & 3];
                }
                float m_all = -INFINITY;
#pragma unroll
                for (int jj = 0; jj < ASP; ++jj) m_all = fmaxf(m_all, am[jj]);
                float wj[ASP], den = 0.0f;
#pragma unroll
                for (int jj = 0; jj < ASP; ++jj) {
                    wj[jj] = __expf(am[jj] - m_all);
                    den = fmaf(wj[jj], al[jj], den);
                }
                float merged[4];
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    float num = 0.0f;
#pragma unroll
                    for (int jj = 0; jj < ASP; ++jj) num = fmaf(wj[jj], ao[t][jj][c], num);
                    merged[c] = uok[t] && uchunk[t] * 256 + xcol < K ? num / den : 0.0f;
                }
                xr[t][0][0] = pack_bf16x2(merged[0], merged[1]);
                xr[t][0][1] = pack_bf16x2(merged[2], merged[3]);
            }
#pragma unroll
            for (int q = 0; q < XL; ++q) {
#pragma unroll
                for (int j = 0; j < NE / 2; ++j) {
                    const float f0 = __uint_as_float(xr[t][q][j] << 16), f1 = __uint_as_float(xr[t][q][j] & 0xffff0000u);
                    const float w0 = __uint_as_float(nw[t][j] << 16), w1 = __uint_as_float(nw[t][j] & 0xffff0000u);
                    pss[q] = fmaf(f0, f0, pss[q]);
                    pss[q] = fmaf(f1, f1, pss[q]);
                    pmx[q] = fmaxf(pmx[q], fmaxf(fabsf(__fmul_rn(f0, w0)), fabsf(__fmul_rn(f1, w1))));
                }
            }
        }
    }
#pragma unroll
    for (int q = 0; q < XL; ++q) {
        const float a = group_reduce<LPR, false>(pss[q]);
        const float b = group_reduce<LPR, true>(pmx[q]);
        if ((lane % LPR) == 0) part_s[xrow0 + RPL * q][wave] = float2{a, b};
    }
    __syncthreads();                             // barrier 1: every wave's partials

    // ---- (4) totals per row -> rstd and the quantisation scale; every wave for itself (lane 16 r + w: row r, wave w)
    float sval_mine = 0.0f;                      // finishing waves: the bf16 scale of this lane's row fin_m
#pragma unroll
    for (int ps = 0; ps < PASSES; ++ps) {
        const int row = 4 * ps + (lane >> 4);
        const float2 v = part_s[row < MR ? row : 0][lane & 15];
        const float total = group_reduce<16, false>(v.x);
        const float pmax = group_reduce<16, true>(v.y);
        const float r = rsqrtf(total / static_cast<float>(K) + eps);
        const float amax_y = fabsf(round_bf16(__fmul_rn(pmax, r)));          // = max |y| of the row, exactly
        uint16_t sb;
        const float s_mul = quant_scale(amax_y, quant_mode, &sb);
        if ((lane & 15) == 0 && row < MR) {
            stat_w[wave][row][0] = r;
            stat_w[wave][row][1] = s_mul;
            if (writer && wave == 0 && io.s_out != nullptr && row < M) io.s_out[row] = sb;
        }
        if (ps == wave) sval_mine = bf16_bits_to_float(sb);                  // finishing wave q: rows 4q .. 4q+3 = pass q, same lanes
    }

    // ---- (5) norm + quantisation into the LDS slot, operands out; then the weights: 2-bit expansion, MFMA
    i32x4 acc = i32x4{0, 0, 0, 0};
    if (has_work) {
        u32x4 bq[CT][4];
#pragma unroll
        for (int t = 0; t < CT; ++t) {
            const int col0 = uchunk[t] * 256;
#pragma unroll
            for (int q = 0; q < XL; ++q) {
                const int row = xrow0 + RPL * q;
                uint32_t d[NE / 4];
                chain_quantise<NE>(xr[t][q], nw[t], stat_w[wave][row][0], stat_w[wave][row][1], quant_mode, d);
                const bool pub = writer && io.xq_out != nullptr && row < M && uok[t] && col0 + xcol < K;
                if constexpr (NE == 8) {
                    *reinterpret_cast<u32x2*>(slab + row * kChainSlabPitch + xcol) = u32x2{d[0], d[1]};
                    if (pub) *reinterpret_cast<u32x2*>(io.xq_out + static_cast<size_t>(row) * K + col0 + xcol) = u32x2{d[0], d[1]};
                } else {
                    *reinterpret_cast<uint32_t*>(slab + row * kChainSlabPitch + xcol) = d[0];
                    if (pub) *reinterpret_cast<uint32_t*>(io.xq_out + static_cast<size_t>(row) * K + col0 + xcol) = d[0];
                }
            }
            const uint8_t* src = slab + (i < MR ? i : MR) * kChainSlabPitch + g * 64;
#pragma unroll
            for (int p = 0; p < 4; ++p) bq[t][p] = *reinterpret_cast<const u32x4*>(src + 16 * p);
        }
        __builtin_amdgcn_sched_barrier(0);       // nothing that needs a weight word moves up
#pragma unroll
        for (int t = 0; t < CT; ++t) {
            if (t > 0 && !uok[t]) continue;      // scalar
            const uint32_t wc[4] = {wq[t].x, wq[t].y, wq[t].z, wq[t].w};
#pragma unroll
            for (int c = 0; c < 4; ++c)
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(expand_word_i8(wc[c]), __builtin_bit_cast(i32x4, bq[t][c]), acc, 0, 0, 0);
        }
    }

    // ---- (6) accumulators to LDS as [batch row][column], barrier 2, finishing (as terna_chain_chunk_kernel)
    *reinterpret_cast<i32x4*>(&red[wave][i * 16 + 4 * g]) = acc;
    if (finisher) asm volatile("" : "+v"(ew), "+v"(eres), "+v"(enw));
    __syncthreads();
    if (finisher) {
        const bool row_ok = fin_m < M;
        const int* rp = &red[0][64 * wave + lane];
        int sum = rp[0];
#pragma unroll
        for (int w = 1; w < WAVES; ++w) sum += rp[w * 256];
        EpilogueRegs e;
        e.s = sval_mine;
        e.w[0] = __uint_as_float(ew << 16);
        const uint16_t o = apply_epilogue<int>(EP_I8_DECODE, e, 0, sum >> kI8WeightShift);
        const uint32_t o32 = o;
        const uint32_t op = o32 | (dpp_permute_u32<kDppSwapPairs>(o32) << 16);
        if constexpr (EPI == CEPI_STORE) {
            if ((lane & 1) == 0 && row_ok) *reinterpret_cast<uint32_t*>(io.out + static_cast<size_t>(fin_m) * N + fin_n) = op;
        } else {
            const float hv = row_ok ? round_bf16(__uint_as_float(eres << 16) + bf16_bits_to_float(o)) : 0.0f;
            float ssq = hv * hv;
            float pmax = fabsf(__fmul_rn(hv, __uint_as_float(enw << 16)));
            ssq = group_reduce<16, false>(ssq);
            pmax = group_reduce<16, true>(pmax);
            const uint32_t h32 = float_to_bf16_bits(hv);
            const uint32_t hp = h32 | (dpp_permute_u32<kDppSwapPairs>(h32) << 16);
            if (row_ok) {
                if ((lane & 1) == 0) {
                    *reinterpret_cast<uint32_t*>(io.out + static_cast<size_t>(fin_m) * N + fin_n) = hp;
                    if (io.raw_out != nullptr) *reinterpret_cast<uint32_t*>(io.raw_out + static_cast<size_t>(fin_m) * N + fin_n) = op;
                }
                if ((lane & 15) == 0) io.stats_out[static_cast<size_t>(fin_m) * (N / 16) + band] = float2{ssq, pmax};
            }
        }
    }
}

}  // namespace terna
