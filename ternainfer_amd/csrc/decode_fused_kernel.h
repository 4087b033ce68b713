// Small-M TernaSpMM on the P2 layout with its prologue inside: [residual add] -> RMSNorm ->
// per-row int8 quantisation -> ternary matmul -> scale epilogue, one launch.
//
// In terna_decode_packed_kernel every workgroup (one 16-row band of W) already reads the whole
// activation row block: its waves take the band's 64-column tiles round robin.  So the row
// statistics the prologue needs (sum of squares, then max |y|) cost each workgroup two
// reductions over data it holds anyway, and the separate norm/quantise launch -- 4 us of a
// 9 us pair in a decode step -- disappears.  Every workgroup recomputes the same statistics from
// the same values in the same order, so all bands see identical int8 activations.
//
//   h  = x, or bf16(x + residual)            (workgroup 0 also writes h to sum_out: the new stream),
//        or bf16(bf16(relu(x1)^2) * x3)      (gated FFN: x = [x1 | x3], 2K columns per row),
//        or the single-token attention's output row merged from the partial results of its splits
//        (FUSED_ATTN, one row: `x` is then the fp32 buffer a deferred-merge attention launch left, see
//        attention_kernel.h; the merge arithmetic is attention_merge's, so the row has the bits the merge kernel gives)
//   y  = bf16(h * rsqrt(mean(h^2) + eps) * norm_w)
//   s  = bf16(127 / max(max|y|, 1e-5)),  q = clamp(rint(y * s), -128, 127)
//   out[m][n] = bf16((sum_k q[m][k] W[n][k] / s[m]) * ws[group(n)])      (decode epilogue)
//
// Phases of a wave (T = its tiles, at most TMAX):
//   A  request everything: T weight words, T activation pieces (x, residual), then the norm
//      weights of its columns; h -> registers (packed bf16), sum of squares per row
//   B  rows' sums: the lanes that share a row (data-parallel permutes), then the waves in LDS -- barrier 1
//   C  y -> registers, max |y| per row, same reduction                      -- barrier 2
//   D  per tile: quantise, int8 slab -> wave-private LDS -> operand order (a single row: gathered
//      with data-parallel permutes, no LDS), MFMA
//   E  cross-wave sum of the accumulators + epilogue (wave b finishes band b) -- barrier 3
//
// FUSED_STATS: the row statistics come from the PRODUCER of h instead.  The launch that wrote h also left, per row and
// per 16 (or more) columns, the partial sums of h^2 and the partial maxima of |h * norm_w| (both exact products of two
// bf16 values); here one wave per row adds / maximises the partials in a fixed order -- the same order in every
// workgroup, so all bands see identical int8 activations -- and the rest is element-wise:
//   y = bf16((h * norm_w) * rstd)        max|y| = bf16(max|h * norm_w| * rstd) exactly: both roundings are monotone
// One barrier instead of two, no second pass over the row, and the row need not stay in registers.
//
// Epilogues (EPI): FEPI_PLAIN stores bf16 out[m][n].  The other two make this launch the producer for the next one:
//   FEPI_RESIDUAL  h' = bf16(residual[m][n] + out[m][n]) is stored (the new residual stream, model.py:330, :334) with
//                  the statistics of h' under the NEXT norm's weights, one partial per row and 16-row band;
//   FEPI_GLU       the bands of W alternate between the gate and the up matrix (band 2j = rows 16j.. of w1, band
//                  2j+1 = the same rows of w3; a load-time permutation), so the workgroup holds matching x1 / x3 and
//                  stores inner = bf16(bf16(relu(x1)^2) * x3) (model.py:279-280) -- N/2 columns instead of N -- with
//                  its statistics under the ffn_sub_norm weights.
//
// NB = bands of W per workgroup.  The prologue is repeated by every workgroup, so a matrix with
// more bands than the chip has CUs (gate+up: 864) would repeat it once per *round* of workgroups
// on every CU; with NB bands per workgroup the grid fits one round, the prologue runs once per CU
// and its result feeds NB accumulators.
#pragma once

#include "decode_packed_kernel.h"
#include "norm_quant_kernel.h"
#include "attention_kernel.h"

namespace terna {

// MP consecutive columns of one activation row, as a lane holds them: bf16 storage in, floats out.
template <int MP> struct RowPiece;
template <> struct RowPiece<16> {
    u32x4 v[2];
    __device__ void load(const uint16_t* p) { v[0] = reinterpret_cast<const u32x4*>(p)[0]; v[1] = reinterpret_cast<const u32x4*>(p)[1]; }
    __device__ void store(uint16_t* p) const { reinterpret_cast<u32x4*>(p)[0] = v[0]; reinterpret_cast<u32x4*>(p)[1] = v[1]; }
    __device__ void zero() { v[0] = v[1] = u32x4{0u, 0u, 0u, 0u}; }
    __device__ void unpack(float f[16]) const { unpack_bf16x8(v[0], f); unpack_bf16x8(v[1], f + 8); }
    __device__ void pack(const float f[16]) { v[0] = pack_bf16x8(f); v[1] = pack_bf16x8(f + 8); }
};
template <> struct RowPiece<8> {
    u32x4 v;
    __device__ void load(const uint16_t* p) { v = *reinterpret_cast<const u32x4*>(p); }
    __device__ void store(uint16_t* p) const { *reinterpret_cast<u32x4*>(p) = v; }
    __device__ void zero() { v = u32x4{0u, 0u, 0u, 0u}; }
    __device__ void unpack(float f[8]) const { unpack_bf16x8(v, f); }
    __device__ void pack(const float f[8]) { v = pack_bf16x8(f); }
};
template <> struct RowPiece<4> {
    u32x2 v;
    __device__ void load(const uint16_t* p) { v = *reinterpret_cast<const u32x2*>(p); }
    __device__ void store(uint16_t* p) const { *reinterpret_cast<u32x2*>(p) = v; }
    __device__ void zero() { v = u32x2{0u, 0u}; }
    __device__ void unpack(float f[4]) const
    {
        f[0] = __uint_as_float(v.x << 16); f[1] = __uint_as_float(v.x & 0xffff0000u);
        f[2] = __uint_as_float(v.y << 16); f[3] = __uint_as_float(v.y & 0xffff0000u);
    }
    __device__ void pack(const float f[4]) { v = u32x2{pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3])}; }
};
template <> struct RowPiece<2> {
    uint32_t v;
    __device__ void load(const uint16_t* p) { v = *reinterpret_cast<const uint32_t*>(p); }
    __device__ void store(uint16_t* p) const { *reinterpret_cast<uint32_t*>(p) = v; }
    __device__ void zero() { v = 0u; }
    __device__ void unpack(float f[2]) const { f[0] = __uint_as_float(v << 16); f[1] = __uint_as_float(v & 0xffff0000u); }
    __device__ void pack(const float f[2]) { v = pack_bf16x2(f[0], f[1]); }
};
template <> struct RowPiece<1> {
    uint16_t v;
    __device__ void load(const uint16_t* p) { v = *p; }
    __device__ void store(uint16_t* p) const { *p = v; }
    __device__ void zero() { v = 0; }
    __device__ void unpack(float f[1]) const { f[0] = bf16_bits_to_float(v); }
    __device__ void pack(const float f[1]) { v = float_to_bf16_bits(f[0]); }
};

// MP = rows a wave's 64 lanes cover at once (M <= MP): 64/MP lanes walk along a row, MP columns
// each, so a lane handles MP elements per tile -- the prologue arithmetic, which every workgroup
// repeats, costs in proportion to the batch rows that exist, not to the 16 the MFMA tile has.
enum FusedMode { FUSED_PLAIN, FUSED_RESIDUAL, FUSED_GLU, FUSED_ATTN, FUSED_STATS };
enum FusedEpilogue { FEPI_PLAIN, FEPI_RESIDUAL, FEPI_GLU };

constexpr int kStatsMaxPartials = 448;           // partials per row a consumer adds up: 7 per lane of one wave

// What the newer prologue / epilogues need beyond the original argument list (passed by value, last).
struct FusedExtra {
    const float2* stats_in;          // FUSED_STATS: [M][stats_count] (sum of h^2, max |h * norm_w|)
    int stats_count;
    const uint16_t* epi_residual;    // FEPI_RESIDUAL: bf16 [M][N], the stream the output is added to
    const uint16_t* epi_next_w;      // FEPI_RESIDUAL / FEPI_GLU: weights of the norm that follows (bf16 [N] / [N/2])
    float2* stats_out;               // [M][N/16] / [M][N/32]
    uint16_t* raw_out;               // FEPI_RESIDUAL, optional: the linear's own output bf16 [M][N] as well
};

// ASP / AHD (FUSED_ATTN only): splits and head size of the attention whose partial results the row is merged from --
// compile-time, so that a head's statistics are two scalar loads and no address needs a division.
template <int WAVES, int TMAX, int MODE, int MP, int NB = 1, int ASP = 1, int AHD = 64, int EPI = FEPI_PLAIN>
__global__ __launch_bounds__(WAVES * 64) void terna_decode_fused_kernel(
    // what the first loads depend on comes first: the leading sixteen dwords of the arguments arrive in scalar registers
    const uint16_t* __restrict__ x, const uint16_t* __restrict__ residual, const uint16_t* __restrict__ norm_w,
    const uint32_t* __restrict__ packed, int M, int N, int K, float eps, uint16_t* __restrict__ sum_out,
    uint16_t* __restrict__ out, const uint16_t* __restrict__ ws, int ws_num, int8_t* __restrict__ xq_out,
    uint16_t* __restrict__ s_out, int quant_mode, FusedExtra ex)
{
    static_assert(MODE != FUSED_ATTN || MP == 1, "the attention merge feeds a single row");
    static_assert(MODE != FUSED_STATS || MP <= WAVES, "one reducing wave per row");
    static_assert(EPI != FEPI_GLU || NB % 2 == 0, "gate and up bands come in pairs");
    static_assert(AHD % 64 == 0 && ASP >= 1 && ASP <= kAttentionMaxSplits, "a 64-column tile lies inside one head");
    using XQ = XSlab<int8_t>;
    using Piece = RowPiece<MP>;
    constexpr int LPR = 64 / MP;                     // lanes per row
    static_assert(NB <= WAVES, "one finishing wave per band");
    __shared__ i32x4 red[WAVES][NB][64];
    __shared__ __align__(16) uint8_t slab_all[WAVES][16 * XQ::kPitch];
    __shared__ __align__(16) float stat[2][16][WAVES];
    __shared__ float s_row[16];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int band0 = blockIdx.x * NB;               // first of this workgroup's NB bands
    const int ktiles = K >> 6;
    const int i = lane & 15, g = lane >> 4;          // operand coordinates: weight row / batch row i, 16-column group g
    const int row = lane / LPR, cl = (lane % LPR) * MP;   // load coordinates: batch row, first of MP columns
    const bool row_ok = row < M;
    const bool writer = blockIdx.x == 0;             // the workgroup that publishes h, q and s
    constexpr bool RES = MODE == FUSED_RESIDUAL || MODE == FUSED_GLU;   // a second operand: the residual, or x3 of the gate
    const size_t pitch = MODE == FUSED_GLU ? 2 * static_cast<size_t>(K) : K;
    const uint16_t* second = MODE == FUSED_GLU ? x + K : residual;

    // ---- phase A: request everything
    // Straight-line code: every load is unconditional on a clamped address and what must be zero is
    // zeroed by a select afterwards.  Loads inside branches end up with a full wait at every join,
    // i.e. one memory round trip per tile.
    uint32_t wword[NB][TMAX];
    Piece xr[TMAX], rr[TMAX], nw[TMAX];
    constexpr int AT = MODE == FUSED_ATTN ? TMAX : 1;
    f32x4 ast[AT][4];                                // FUSED_ATTN: score maxima and sums of numerators of the tile's head
    float ao[AT][ASP];                               //             unnormalised result of every split, this lane's dimension
    bool use[TMAX];
#pragma unroll
    for (int t = 0; t < TMAX; ++t) {
        const int j = wave + WAVES * t;
        const bool valid = j < ktiles;
        const int jc = valid ? j : 0;
        use[t] = valid && row_ok;
#pragma unroll
        for (int b = 0; b < NB; ++b) wword[b][t] = packed[(static_cast<size_t>(band0 + b) * ktiles + jc) * 64 + lane];   // word L; operand order below
        const size_t off = static_cast<size_t>(row_ok ? row : 0) * pitch + jc * 64 + cl;
        if constexpr (MODE == FUSED_ATTN) {
            // column jc * 64 + lane of the one row = dimension d of head `head` (a tile lies inside one head);
            // the head's statistics are the same for the whole wave, its unnormalised results one float per lane and split
            const float* part = reinterpret_cast<const float*>(x);
            const int head = (jc * 64) / AHD;                           // wave-uniform
            const int d = jc * 64 - head * AHD + lane;
            const f32x4* stat = reinterpret_cast<const f32x4*>(part + static_cast<size_t>(head) * kAttentionStatFloats);
            const float* o_head = part + attention_stat_floats(static_cast<size_t>(K / AHD)) + static_cast<size_t>(head) * (ASP * AHD);
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) ast[t][q4] = stat[q4];      // maxima 0 .. 7, sums 0 .. 7
#pragma unroll
            for (int jj = 0; jj < ASP; ++jj) ao[t][jj] = o_head[jj * AHD + d];
        } else {
            xr[t].load(x + off);
        }
        if constexpr (RES) rr[t].load(second + off);
        nw[t].load(norm_w + jc * 64 + cl);
    }
    if constexpr (MODE == FUSED_ATTN) {
#pragma unroll
        for (int t = 0; t < TMAX; ++t) {             // attention_merge, on the values requested above
            float am[kAttentionMaxSplits], al[kAttentionMaxSplits];
#pragma unroll
            for (int jj = 0; jj < kAttentionMaxSplits; ++jj) {
                am[jj] = ast[t][jj >> 2][jj & 3];
                al[jj] = ast[t][2 + (jj >> 2)][jj & 3];
            }
            float m_all = -INFINITY;
#pragma unroll
            for (int jj = 0; jj < ASP; ++jj) m_all = fmaxf(m_all, am[jj]);
            float num = 0.0f, den = 0.0f;
#pragma unroll
            for (int jj = 0; jj < ASP; ++jj) {
                const float w = __expf(am[jj] - m_all);
                num = fmaf(w, ao[t][jj], num);
                den = fmaf(w, al[jj], den);
            }
            const float merged[1] = {num / den};
            xr[t].pack(merged);
        }
    }
#pragma unroll
    for (int t = 0; t < TMAX; ++t) {
        if (!use[t]) {
            xr[t].zero();
            if constexpr (RES) rr[t].zero();
        }
        if (wave + WAVES * t >= ktiles) {
#pragma unroll
            for (int b = 0; b < NB; ++b) wword[b][t] = 0u;
        }
    }
    // wave b finishes band b: its weight-group scales are requested now, converted at the very end
    const Epilogue ep{nullptr, ws, nullptr, ws_num, EP_I8_DECODE};
    constexpr int NFIN = EPI == FEPI_GLU ? NB / 2 : NB;            // finishing waves (a gate / up pair shares one)
    const bool finisher = wave < NFIN;
    const int my_band = band0 + (wave < NB ? wave : 0);
    EpilogueRaw eraw;
    if constexpr (EPI == FEPI_GLU) {
        eraw.s = 0u;
        eraw.w[0] = ws[0];                                         // gate rows (w1) and up rows (w3): one scale each
        eraw.w[1] = ws[1];
        eraw.w[2] = eraw.w[3] = 0u;
    } else {
        eraw = load_epilogue_raw_scales(ep, my_band * 16 + 4 * g, N);
    }
    // What the producing epilogues read besides the accumulators -- four stream values and four weights of the next
    // norm per lane -- is requested here as well, by the finishing waves (the others read one address: no traffic).
    u32x2 eres = {0u, 0u}, enw = {0u, 0u};
    const int out_cols = EPI == FEPI_GLU ? N / 2 : N;
    const int epi_col = EPI == FEPI_GLU ? (static_cast<int>(blockIdx.x) * NFIN + (finisher ? wave : 0)) * 16 + 4 * g : my_band * 16 + 4 * g;
    if constexpr (EPI != FEPI_PLAIN) {
        const size_t noff = finisher ? static_cast<size_t>(epi_col) : 0;
        enw = *reinterpret_cast<const u32x2*>(ex.epi_next_w + noff);
        if constexpr (EPI == FEPI_RESIDUAL) {
            const size_t roff = finisher ? static_cast<size_t>(i < M ? i : 0) * N + epi_col : 0;
            eres = *reinterpret_cast<const u32x2*>(ex.epi_residual + roff);
        }
    }
    // FUSED_STATS: wave r adds up the partials of row r (the other waves read one address: no traffic)
    constexpr int PT = MODE == FUSED_STATS ? kStatsMaxPartials / 64 : 1;
    float2 part[PT];
    if constexpr (MODE == FUSED_STATS) {
        const bool reducer = wave < M;
        const float2* sp = ex.stats_in + (reducer ? static_cast<size_t>(wave) * ex.stats_count : 0);
#pragma unroll
        for (int t = 0; t < PT; ++t) {
            const int idx = lane + 64 * t;
            part[t] = sp[reducer && idx < ex.stats_count ? idx : 0];
        }
    }
    // Requested here, used at the very end: without this the compiler moves the two loads next to their use, behind
    // the last barrier, and the launch ends with one more dependent trip to memory.
    if constexpr (EPI != FEPI_PLAIN) {
        pin_registers(enw);
        pin_registers(eres);
    }
    // this wave's LDS slot: rows the batch does not have stay zero (a single row needs no slot, see phase D)
    uint8_t* slab = slab_all[wave];
    if constexpr (MP != 1)
        for (int o = lane * 16; o < 16 * XQ::kPitch; o += 64 * 16) *reinterpret_cast<u32x4*>(slab + o) = u32x4{0u, 0u, 0u, 0u};

    float ssq = 0.0f;
#pragma unroll
    for (int t = 0; t < (MODE == FUSED_STATS ? 0 : TMAX); ++t) {
        const int j = wave + WAVES * t;
        float f[MP];
        xr[t].unpack(f);
        if constexpr (MODE == FUSED_RESIDUAL) {
            float r[MP];
            rr[t].unpack(r);
#pragma unroll
            for (int e = 0; e < MP; ++e) f[e] = round_bf16(f[e] + r[e]);
            xr[t].pack(f);
            if (writer && sum_out != nullptr && j < ktiles && row_ok)
                xr[t].store(sum_out + static_cast<size_t>(row) * K + j * 64 + cl);
        } else if constexpr (MODE == FUSED_GLU) {
            float r[MP];
            rr[t].unpack(r);
#pragma unroll
            for (int e = 0; e < MP; ++e) {
                const float p = fmaxf(f[e], 0.0f);
                f[e] = round_bf16(round_bf16(p * p) * r[e]);
            }
            xr[t].pack(f);
        }
#pragma unroll
        for (int e = 0; e < MP; ++e) ssq = fmaf(f[e], f[e], ssq);
    }

    // ---- phase B: sum of squares per row (LPR lanes share a row, then the waves)
    auto row_reduce = [&](float v, int which, bool is_max) {
        v = is_max ? group_reduce<LPR, true>(v) : group_reduce<LPR, false>(v);
        if ((lane % LPR) == 0) stat[which][row][wave] = v;
        __syncthreads();
        const f32x4* p = reinterpret_cast<const f32x4*>(stat[which][row]);
        float r = 0.0f;
#pragma unroll
        for (int q4 = 0; q4 < WAVES / 4; ++q4) {
            const f32x4 c = p[q4];
            if (is_max) r = fmaxf(fmaxf(r, fmaxf(c.x, c.y)), fmaxf(c.z, c.w));
            else r += (c.x + c.y) + (c.z + c.w);
        }
        return r;
    };
    float rstd, s;
    uint16_t s_bits = 0;
    if constexpr (MODE == FUSED_STATS) {
        // ---- phases B + C from the producer's partials: one wave per row, a fixed order, one barrier
        if (wave < M) {
            float sum = 0.0f, pmax = 0.0f;
#pragma unroll
            for (int t = 0; t < PT; ++t) {
                if (lane + 64 * t < ex.stats_count) {
                    sum += part[t].x;
                    pmax = fmaxf(pmax, part[t].y);
                }
            }
            sum = wave_sum(sum);
            pmax = wave_max(pmax);
            if (lane == 0) {
                const float r = rsqrtf(sum / static_cast<float>(K) + eps);
                const float amax_y = fabsf(round_bf16(__fmul_rn(pmax, r)));      // = max |y| of the row, exactly
                uint16_t sb;
                const float s_mul = quant_scale(amax_y, quant_mode, &sb);
                stat[0][wave][0] = r;
                stat[1][wave][0] = s_mul;
                s_row[wave] = bf16_bits_to_float(sb);
                if (writer && s_out != nullptr) s_out[wave] = sb;
            }
        }
        __syncthreads();
        rstd = stat[0][row_ok ? row : 0][0];
        s = stat[1][row_ok ? row : 0][0];
    } else {
    ssq = row_reduce(ssq, 0, false);
    rstd = rsqrtf(ssq / static_cast<float>(K) + eps);

    // ---- phase C: y in place of h, max |y| per row
    float amax = 0.0f;
#pragma unroll
    for (int t = 0; t < TMAX; ++t) {
        float w[MP], f[MP];
        nw[t].unpack(w);
        xr[t].unpack(f);
        const bool valid = wave + WAVES * t < ktiles;
#pragma unroll
        for (int e = 0; e < MP; ++e) {
            f[e] = round_bf16(__fmul_rn(__fmul_rn(f[e], w[e]), rstd));
            if (valid) amax = fmaxf(amax, fabsf(f[e]));
        }
        xr[t].pack(f);
    }
    amax = row_reduce(amax, 1, true);
    s = quant_scale(amax, quant_mode, &s_bits);      // what multiplies; the epilogue divides by the bf16 value
    if (wave == 0 && (lane % LPR) == 0) {
        s_row[row] = bf16_bits_to_float(s_bits);
        if (writer && s_out != nullptr && row_ok) s_out[row] = s_bits;
    }
    }

    // ---- phase D: quantise a tile, turn it into operand order through the wave's LDS slot, multiply
    i32x4 acc[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) acc[b] = i32x4{0, 0, 0, 0};
#pragma unroll
    for (int t = 0; t < TMAX; ++t) {
        const int j = wave + WAVES * t;
        if (j < ktiles) {
            float f[MP];
            xr[t].unpack(f);
            if constexpr (MODE == FUSED_STATS) {                  // the norm, element-wise: rstd came from the partials
                float w[MP];
                nw[t].unpack(w);
#pragma unroll
                for (int e = 0; e < MP; ++e) f[e] = round_bf16(__fmul_rn(__fmul_rn(f[e], w[e]), rstd));
            }
            // int8 bytes, packed four to a dword: clamp(rint(y * s)) + 128 is an integer in [0, 255] that one
            // conversion drops into its byte; the xor takes the 128 out again (two's complement)
            constexpr int ND = MP >= 4 ? MP / 4 : 1;
            constexpr uint32_t kBias = MP >= 4 ? 0x80808080u : (MP == 2 ? 0x8080u : 0x80u);
            uint32_t d[ND];
            const bool eager = quant_mode == QUANT_EAGER;                    // uniform: one branch per tile, not per element
#pragma unroll
            for (int e4 = 0; e4 < ND; ++e4) {
                uint32_t wd = 0u;
                if (eager) {
#pragma unroll
                    for (int e = 4 * e4; e < 4 * e4 + 4 && e < MP; ++e)
                        wd = __builtin_amdgcn_cvt_pk_u8_f32(quant_value(f[e], s, QUANT_EAGER) + 128.0f, e & 3, wd);
                } else {
#pragma unroll
                    for (int e = 4 * e4; e < 4 * e4 + 4 && e < MP; ++e)
                        wd = __builtin_amdgcn_cvt_pk_u8_f32(quant_value(f[e], s, QUANT_ROUNDED) + 128.0f, e & 3, wd);
                }
                d[e4] = wd ^ kBias;
            }
            uint8_t* dst = slab + row * XQ::kPitch + cl;
            int8_t* gdst = xq_out + static_cast<size_t>(row_ok ? row : 0) * K + j * 64 + cl;
            const bool publish = writer && xq_out != nullptr && row_ok;
            i32x4 bq;
            if constexpr (MP == 1) {
                // One row: lane c holds the byte of column c.  Four neighbouring bytes into the dword of lane 4d,
                // the four dwords of 16 columns into lane 16g -- the only lanes whose MFMA operand (batch row 0,
                // columns 16g .. 16g+15) is not zero.  No LDS.
                if (publish) *gdst = static_cast<int8_t>(d[0]);
                const uint32_t b1 = d[0];
                const uint32_t b2 = b1 | (dpp_permute_u32<kDppSwapPairs>(b1) << 8);          // even lanes: columns c, c+1
                const uint32_t b4 = b2 | (dpp_permute_u32<kDppSwapHalfQuads>(b2) << 16);     // lanes 4d: columns 4d .. 4d+3
                const uint32_t d1 = dpp_permute_u32<kDppRowShl4>(b4), d2 = dpp_permute_u32<kDppRowShl8>(b4),
                               d3 = dpp_permute_u32<kDppRowShl12>(b4);
                const bool first = i == 0;
                bq = i32x4{static_cast<int>(first ? b4 : 0u), static_cast<int>(first ? d1 : 0u),
                           static_cast<int>(first ? d2 : 0u), static_cast<int>(first ? d3 : 0u)};
            } else {
                if constexpr (MP == 2) {
                    *reinterpret_cast<uint16_t*>(dst) = static_cast<uint16_t>(d[0]);
                    if (publish) *reinterpret_cast<uint16_t*>(gdst) = static_cast<uint16_t>(d[0]);
                } else if constexpr (MP == 4) {
                    *reinterpret_cast<uint32_t*>(dst) = d[0];
                    if (publish) *reinterpret_cast<uint32_t*>(gdst) = d[0];
                } else if constexpr (MP == 8) {
                    *reinterpret_cast<u32x2*>(dst) = u32x2{d[0], d[1]};
                    if (publish) *reinterpret_cast<u32x2*>(gdst) = u32x2{d[0], d[1]};
                } else {
                    *reinterpret_cast<u32x4*>(dst) = u32x4{d[0], d[1], d[2], d[3]};
                    if (publish) *reinterpret_cast<u32x4*>(gdst) = u32x4{d[0], d[1], d[2], d[3]};
                }
                bq = __builtin_bit_cast(i32x4, *reinterpret_cast<const u32x4*>(slab + i * XQ::kPitch + g * 16));
            }
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                // lane L loaded word L of the band-tile (consecutive lanes, consecutive words: the memory pipeline takes
                // such a load in a quarter of the steps); the operand of lane L is word (L & 15) * 4 + (L >> 4)
                const uint32_t w = static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute((i * 4 + g) * 4, static_cast<int>(wword[b][t])));
                acc[b] = __builtin_amdgcn_mfma_i32_16x16x64_i8(expand_word_i8(w), bq, acc[b], 0, 0, 0);
            }
        }
    }

    // ---- phase E: cross-wave sum in wave order + the decode epilogue (lane: batch row i, output rows 4g .. 4g+3)
#pragma unroll
    for (int b = 0; b < NB; ++b) red[wave][b][lane] = acc[b];
    __syncthreads();
    if (finisher) {
        EpilogueRegs e = finish_epilogue(ep, eraw);
        e.s = s_row[i < M ? i : 0];
        if constexpr (EPI == FEPI_GLU) {
            // gate band 2 * wave and up band 2 * wave + 1: x1, x3 of the same sixteen features
            i32x4 sum1 = red[0][2 * wave][lane], sum3 = red[0][2 * wave + 1][lane];
#pragma unroll
            for (int w = 1; w < WAVES; ++w) {
                sum1 += red[w][2 * wave][lane];
                sum3 += red[w][2 * wave + 1][lane];
            }
            const float w1 = __uint_as_float(eraw.w[0] << 16), w3 = __uint_as_float(eraw.w[1] << 16);
            float nwv[4], hv[4];
            nwv[0] = __uint_as_float(enw.x << 16); nwv[1] = __uint_as_float(enw.x & 0xffff0000u);
            nwv[2] = __uint_as_float(enw.y << 16); nwv[3] = __uint_as_float(enw.y & 0xffff0000u);
            float ssq_o = 0.0f, pmax_o = 0.0f;
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                e.w[v] = w1;
                const float x1 = bf16_bits_to_float(apply_epilogue<int>(EP_I8_DECODE, e, v, sum1[v] >> kI8WeightShift));
                e.w[v] = w3;
                const float x3 = bf16_bits_to_float(apply_epilogue<int>(EP_I8_DECODE, e, v, sum3[v] >> kI8WeightShift));
                const float p = fmaxf(x1, 0.0f);
                hv[v] = i < M ? round_bf16(round_bf16(p * p) * x3) : 0.0f;
                ssq_o = fmaf(hv[v], hv[v], ssq_o);
                pmax_o = fmaxf(pmax_o, fabsf(__fmul_rn(hv[v], nwv[v])));
            }
            // the four lanes (g = 0 .. 3) of a batch row hold the band's sixteen features between them
            ssq_o = cross_row_reduce<false>(ssq_o);
            pmax_o = cross_row_reduce<true>(pmax_o);
            if (i < M) {
                *reinterpret_cast<u32x2*>(out + static_cast<size_t>(i) * out_cols + epi_col) =
                    u32x2{pack_bf16x2(hv[0], hv[1]), pack_bf16x2(hv[2], hv[3])};
                if (g == 0) ex.stats_out[static_cast<size_t>(i) * (out_cols / 16) + epi_col / 16] = float2{ssq_o, pmax_o};
            }
        } else {
            i32x4 sum = red[0][wave][lane];
#pragma unroll
            for (int w = 1; w < WAVES; ++w) sum += red[w][wave][lane];
            uint16_t o[4];
#pragma unroll
            for (int v = 0; v < 4; ++v) o[v] = apply_epilogue<int>(EP_I8_DECODE, e, v, sum[v] >> kI8WeightShift);
            const u32x2 pk = {o[0] | (static_cast<uint32_t>(o[1]) << 16), o[2] | (static_cast<uint32_t>(o[3]) << 16)};
            if constexpr (EPI == FEPI_PLAIN) {
                if (i < M) *reinterpret_cast<u32x2*>(out + static_cast<size_t>(i) * N + epi_col) = pk;
            } else {
                float rv[4], nwv[4], hv[4];
                rv[0] = __uint_as_float(eres.x << 16); rv[1] = __uint_as_float(eres.x & 0xffff0000u);
                rv[2] = __uint_as_float(eres.y << 16); rv[3] = __uint_as_float(eres.y & 0xffff0000u);
                nwv[0] = __uint_as_float(enw.x << 16); nwv[1] = __uint_as_float(enw.x & 0xffff0000u);
                nwv[2] = __uint_as_float(enw.y << 16); nwv[3] = __uint_as_float(enw.y & 0xffff0000u);
                float ssq_o = 0.0f, pmax_o = 0.0f;
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    hv[v] = i < M ? round_bf16(rv[v] + bf16_bits_to_float(o[v])) : 0.0f;
                    ssq_o = fmaf(hv[v], hv[v], ssq_o);
                    pmax_o = fmaxf(pmax_o, fabsf(__fmul_rn(hv[v], nwv[v])));
                }
                ssq_o = cross_row_reduce<false>(ssq_o);
                pmax_o = cross_row_reduce<true>(pmax_o);
                if (i < M) {
                    *reinterpret_cast<u32x2*>(out + static_cast<size_t>(i) * N + epi_col) =
                        u32x2{pack_bf16x2(hv[0], hv[1]), pack_bf16x2(hv[2], hv[3])};
                    if (ex.raw_out != nullptr) *reinterpret_cast<u32x2*>(ex.raw_out + static_cast<size_t>(i) * N + epi_col) = pk;
                    if (g == 0) ex.stats_out[static_cast<size_t>(i) * (N / 16) + epi_col / 16] = float2{ssq_o, pmax_o};
                }
            }
        }
    }
}

}  // namespace terna
