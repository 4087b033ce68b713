// C ABI of the chained small-M linears of a decode step: every launch is the consumer of the row statistics its
// producer left and the producer of the statistics its consumer needs (decode_fused_kernel.h: FUSED_STATS prologue,
// FEPI_RESIDUAL / FEPI_GLU epilogues).  Declarations: include/ternaspmm.h.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

#include "../../include/ternaspmm.h"
#include "host_util.h"
#include "decode_fused_kernel.h"
#include "chain_chunk_kernel.h"
#include "launchers.h"

using namespace terna;

namespace {

// Row statistics of a bf16 matrix h [M][K] under the weights of the norm that will read it: per row and per 512 columns
// (sum of h^2, max |h * norm_w|), in the form the FUSED_STATS prologue adds up -- for a row block that no producing
// epilogue wrote (the embedding rows in front of the first block).  One workgroup of 256 threads per row.
__global__ __launch_bounds__(256) void terna_row_stats_kernel(const uint16_t* __restrict__ h, const uint16_t* __restrict__ norm_w,
                                                               float2* __restrict__ stats_out, int K, int count)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const size_t row = blockIdx.x;
    for (int p = wave; p < count; p += 4) {
        const int c = p * 512 + lane * 8;
        float ssq = 0.0f, pmax = 0.0f;
        if (c < K) {                                    // K is a multiple of 8
            float f[8], w[8];
            unpack_bf16x8(*reinterpret_cast<const u32x4*>(h + row * K + c), f);
            unpack_bf16x8(*reinterpret_cast<const u32x4*>(norm_w + c), w);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                ssq = fmaf(f[e], f[e], ssq);
                pmax = fmaxf(pmax, fabsf(__fmul_rn(f[e], w[e])));
            }
        }
        ssq = wave_sum(ssq);
        pmax = wave_max(pmax);
        if (lane == 0) stats_out[row * count + p] = float2{ssq, pmax};
    }
}

// The inputs of a single-token step in one launch: x_out[b] = embedding[tokens[b]] with its partials under norm_w (as
// terna_row_stats_kernel leaves them), and the rows of the RoPE table at the sequences' positions, cos rows then sin rows
// (rope_out [2][B][half]; table [S][2][half]).  A token or position outside its table is clamped (device memory the host
// cannot check).  One workgroup of 256 threads per sequence.
__global__ __launch_bounds__(256) void terna_step_inputs_kernel(const long long* __restrict__ tokens, const long long* __restrict__ pos,
                                                                 int per_seq, const uint16_t* __restrict__ embedding, int V, int K,
                                                                 const float* __restrict__ rope_table, int S, int half,
                                                                 const uint16_t* __restrict__ norm_w, uint16_t* __restrict__ x_out,
                                                                 float2* __restrict__ stats_out, float* __restrict__ rope_out, int count)
{
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int b = blockIdx.x, B = gridDim.x;
    long long t = tokens[b], p = pos[per_seq ? b : 0];
    t = t < 0 ? 0 : (t >= V ? V - 1 : t);
    p = p < 0 ? 0 : (p >= S ? S - 1 : p);
    const uint16_t* row = embedding + static_cast<size_t>(t) * K;
    if (tid < 2 * half / 4) {                           // half is a multiple of 4: 16-byte pieces, cos row then sin row
        const int which = tid / (half / 4), piece = tid - which * (half / 4);
        const f32x4 v = *reinterpret_cast<const f32x4*>(rope_table + (static_cast<size_t>(p) * 2 + which) * half + 4 * piece);
        *reinterpret_cast<f32x4*>(rope_out + (static_cast<size_t>(which) * B + b) * half + 4 * piece) = v;
    }
    for (int part = wave; part < count; part += 4) {
        const int c = part * 512 + lane * 8;
        float ssq = 0.0f, pmax = 0.0f;
        if (c < K) {                                    // K is a multiple of 8
            const u32x4 hv = *reinterpret_cast<const u32x4*>(row + c);
            *reinterpret_cast<u32x4*>(x_out + static_cast<size_t>(b) * K + c) = hv;
            float f[8], w[8];
            unpack_bf16x8(hv, f);
            unpack_bf16x8(*reinterpret_cast<const u32x4*>(norm_w + c), w);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                ssq = fmaf(f[e], f[e], ssq);
                pmax = fmaxf(pmax, fabsf(__fmul_rn(f[e], w[e])));
            }
        }
        ssq = wave_sum(ssq);
        pmax = wave_max(pmax);
        if (lane == 0) stats_out[static_cast<size_t>(b) * count + part] = float2{ssq, pmax};
    }
}

// Band permutation of a P2 gate+up matrix ([w1; w3], N = 2F rows) for the FEPI_GLU epilogue: band 2j <- band j (rows
// 16j .. of w1), band 2j + 1 <- band F/16 + j (the same rows of w3).  One workgroup per destination band.
__global__ __launch_bounds__(256) void terna_interleave_gate_up_kernel(const uint32_t* __restrict__ src, uint32_t* __restrict__ dst,
                                                                        int N, int K)
{
    const int half_bands = N / 32;
    const int dst_band = blockIdx.x;
    const int src_band = (dst_band & 1) * half_bands + (dst_band >> 1);
    const size_t words = static_cast<size_t>(K >> 6) * 64;
    const u32x4* s4 = reinterpret_cast<const u32x4*>(src + src_band * words);
    u32x4* d4 = reinterpret_cast<u32x4*>(dst + dst_band * words);
    for (size_t q = threadIdx.x; q < words / 4; q += 256) d4[q] = s4[q];
}

// Norm + quantisation of h [M][K] as a launch of its own, from the producer's partials (no reduction over the row here):
// for row counts at which every consuming workgroup repeating the element-wise work costs more than this launch.
// Grid (M, ceil(K / 2048)); every wave adds up the partials of its row in the same fixed order as the FUSED_STATS
// prologue, so the (xq, s) written here are the ones that prologue would have formed.
__global__ __launch_bounds__(256) void terna_quant_stats_kernel(const uint16_t* __restrict__ h, const float2* __restrict__ stats, int count,
                                                                 const uint16_t* __restrict__ norm_w, int K, float eps,
                                                                 int8_t* __restrict__ xq_out, uint16_t* __restrict__ s_out, int quant_mode)
{
    const int lane = threadIdx.x & 63;
    const size_t row = blockIdx.x;
    const int c = (blockIdx.y * 256 + threadIdx.x) * 8;
    const bool in = c < K;                                       // K is a multiple of 8
    const u32x4 hv = *reinterpret_cast<const u32x4*>(h + row * K + (in ? c : 0));
    const u32x4 wv = *reinterpret_cast<const u32x4*>(norm_w + (in ? c : 0));
    constexpr int PT = kStatsMaxPartials / 64;
    float2 part[PT];
#pragma unroll
    for (int t = 0; t < PT; ++t) {
        const int idx = lane + 64 * t;
        part[t] = stats[row * count + (idx < count ? idx : 0)];
    }
    float sum = 0.0f, pmax = 0.0f;
#pragma unroll
    for (int t = 0; t < PT; ++t) {
        if (lane + 64 * t < count) {
            sum += part[t].x;
            pmax = fmaxf(pmax, part[t].y);
        }
    }
    sum = wave_sum(sum);
    pmax = wave_max(pmax);
    const float rstd = rsqrtf(sum / static_cast<float>(K) + eps);
    uint16_t sb;
    const float s = quant_scale(fabsf(round_bf16(__fmul_rn(pmax, rstd))), quant_mode, &sb);
    if (blockIdx.y == 0 && threadIdx.x == 0) s_out[row] = sb;
    if (!in) return;
    float f[8], w[8];
    unpack_bf16x8(hv, f);
    unpack_bf16x8(wv, w);
    uint32_t d[2] = {0u, 0u};
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const float y = round_bf16(__fmul_rn(__fmul_rn(f[e], w[e]), rstd));
        d[e >> 2] = __builtin_amdgcn_cvt_pk_u8_f32(quant_value(y, s, quant_mode) + 128.0f, e & 3, d[e >> 2]);
    }
    *reinterpret_cast<u32x2*>(xq_out + row * K + c) = u32x2{d[0] ^ 0x80808080u, d[1] ^ 0x80808080u};
}

// One launch of terna_decode_fused_kernel<WAVES, TMAX, MODE, MP, NB, ASP, AHD, EPI> with MP picked by M (1, 2, 4, 8).
struct ChainArgs {
    const uint16_t* x;
    const uint16_t* residual;
    const uint16_t* norm_w;
    const uint32_t* packed;
    int M, N, K;
    float eps;
    uint16_t* sum_out;
    uint16_t* out;
    const uint16_t* ws;
    int ws_num;
    int8_t* xq_out;
    uint16_t* s_out;
    int qmode;
    FusedExtra ex;
    dim3 grid;
    hipStream_t st;
};

template <int WAVES, int TMAX, int MODE, int MP, int NB, int ASP, int AHD, int EPI>
void launch_one(const ChainArgs& a)
{
    terna_decode_fused_kernel<WAVES, TMAX, MODE, MP, NB, ASP, AHD, EPI><<<a.grid, dim3(WAVES * 64), 0, a.st>>>(
        a.x, a.residual, a.norm_w, a.packed, a.M, a.N, a.K, a.eps, a.sum_out, a.out, a.ws, a.ws_num, a.xq_out, a.s_out, a.qmode,
        a.ex);
}

template <int WAVES, int TMAX, int MODE, int NB, int EPI>
void launch_by_rows(const ChainArgs& a)
{
    if (a.M == 1) launch_one<WAVES, TMAX, MODE, 1, NB, 1, 64, EPI>(a);
    else if (a.M == 2) launch_one<WAVES, TMAX, MODE, 2, NB, 1, 64, EPI>(a);
    else if (a.M <= 4) launch_one<WAVES, TMAX, MODE, 4, NB, 1, 64, EPI>(a);
    else launch_one<WAVES, TMAX, MODE, 8, NB, 1, 64, EPI>(a);
}

template <int EPI>
void launch_attn(const ChainArgs& a, int splits, int head_dim)
{
#define TERNA_CHAIN_ATTN(SP, HD) launch_one<8, 5, FUSED_ATTN, 1, 1, SP, HD, EPI>(a)
    if (head_dim == 128) {
        if (splits == 1) TERNA_CHAIN_ATTN(1, 128);
        else if (splits == 2) TERNA_CHAIN_ATTN(2, 128);
        else if (splits == 4) TERNA_CHAIN_ATTN(4, 128);
        else TERNA_CHAIN_ATTN(8, 128);
    } else {
        if (splits == 1) TERNA_CHAIN_ATTN(1, 64);
        else if (splits == 2) TERNA_CHAIN_ATTN(2, 64);
        else if (splits == 4) TERNA_CHAIN_ATTN(4, 64);
        else TERNA_CHAIN_ATTN(8, 64);
    }
#undef TERNA_CHAIN_ATTN
}

// The statistics-given prologue in the wide-load form (chain_chunk_kernel.h): M waves add up the partials, the other
// 16 - M share `units` units of work, up to three each.  Returns false where that does not cover the matrix.
template <int NBANDS, int EPI, int UNIT_BANDS = (NBANDS == 4 ? 2 : 1)>
bool launch_chunk_by_rows(const ChainArgs& a, int units)
{
    const ChainIo io{a.out, a.ws, a.xq_out, a.s_out, a.ex.epi_residual, a.ex.epi_next_w, a.ex.stats_out, a.ex.raw_out};
    const int workers = kChunkWaves - a.M;
    const int ct = (units + workers - 1) / workers;
    if (ct > 3) return false;
#define TERNA_CHAIN_CHUNK(CT, MR)                                                                                       \
    terna_chain_chunk_kernel<NBANDS, CT, MR, EPI, UNIT_BANDS><<<a.grid, dim3(kChunkWaves * 64), 0, a.st>>>(                \
        a.x, a.norm_w, a.packed, a.ex.stats_in, a.M, a.N, a.K, a.ex.stats_count, a.eps, a.ws_num, a.qmode, io)
#define TERNA_CHAIN_CHUNK_CT(MR)                                                                                        \
    do {                                                                                                                \
        if (ct == 1) TERNA_CHAIN_CHUNK(1, MR);                                                                          \
        else if (ct == 2) TERNA_CHAIN_CHUNK(2, MR);                                                                     \
        else TERNA_CHAIN_CHUNK(3, MR);                                                                                  \
    } while (0)
    if (a.M == 1) TERNA_CHAIN_CHUNK_CT(1);
    else if (a.M == 2) TERNA_CHAIN_CHUNK_CT(2);
    else if (a.M <= 4) TERNA_CHAIN_CHUNK_CT(4);
    else TERNA_CHAIN_CHUNK_CT(8);
#undef TERNA_CHAIN_CHUNK_CT
#undef TERNA_CHAIN_CHUNK
    return true;
}

// Activations quantised already (int8 rows + scales), producing epilogue, up to 16 rows: all 16 waves share the units.
template <int NBANDS, int EPI>
bool launch_chunk_quantised(const ChainArgs& a, const uint16_t* s_in, int units)
{
    ChainIo io{a.out, a.ws, nullptr, nullptr, a.ex.epi_residual, a.ex.epi_next_w, a.ex.stats_out, a.ex.raw_out};
    io.s_in = s_in;
    const int ct = (units + kChunkWaves - 1) / kChunkWaves;
    if (ct > 3 || a.M > 16) return false;
#define TERNA_CHAIN_XQ(CT, MR)                                                                                          \
    do {                                                                                                                \
        auto kernel = terna_chain_chunk_kernel<NBANDS, CT, MR, EPI, (NBANDS == 4 ? 2 : 1), true>;                         \
        kernel<<<a.grid, dim3(kChunkWaves * 64), 0, a.st>>>(a.x, nullptr, a.packed, nullptr, a.M, a.N, a.K, 0, 0.0f, a.ws_num, 0, io); \
    } while (0)
#define TERNA_CHAIN_XQ_CT(MR)                                                                                           \
    do {                                                                                                                \
        if (ct == 1) TERNA_CHAIN_XQ(1, MR);                                                                             \
        else if (ct == 2) TERNA_CHAIN_XQ(2, MR);                                                                        \
        else TERNA_CHAIN_XQ(3, MR);                                                                                     \
    } while (0)
    if (a.M <= 8) TERNA_CHAIN_XQ_CT(8);
    else TERNA_CHAIN_XQ_CT(16);
#undef TERNA_CHAIN_XQ_CT
#undef TERNA_CHAIN_XQ
    return true;
}

// The statistics-inside prologues in the wide-load form (terna_chain_norm_kernel): plain rows ...
template <int EPI>
bool launch_norm_chunk_by_rows(const ChainArgs& a, int chunks)
{
    const ChainIo io{a.out, a.ws, a.xq_out, a.s_out, a.ex.epi_residual, a.ex.epi_next_w, a.ex.stats_out, a.ex.raw_out};
    if (chunks > 2 * kChunkWaves) return false;
#define TERNA_CHAIN_NORM(CT, MR)                                                                                        \
    terna_chain_norm_kernel<CPRO_NORM, CT, MR, EPI><<<a.grid, dim3(kChunkWaves * 64), 0, a.st>>>(                         \
        a.x, a.norm_w, a.packed, a.M, a.N, a.K, a.eps, a.ws_num, a.qmode, io)
#define TERNA_CHAIN_NORM_CT(MR)                                                                                         \
    do {                                                                                                                \
        if (chunks <= kChunkWaves) TERNA_CHAIN_NORM(1, MR);                                                             \
        else TERNA_CHAIN_NORM(2, MR);                                                                                   \
    } while (0)
    if (a.M == 1) TERNA_CHAIN_NORM_CT(1);
    else if (a.M == 2) TERNA_CHAIN_NORM_CT(2);
    else if (a.M <= 4) TERNA_CHAIN_NORM_CT(4);
    else TERNA_CHAIN_NORM_CT(8);
#undef TERNA_CHAIN_NORM_CT
#undef TERNA_CHAIN_NORM
    return true;
}

// ... and the single row merged from a deferred attention's partial results (K <= 4096)
template <int EPI>
bool launch_attn_chunk(const ChainArgs& a, int splits, int head_dim, int chunks)
{
    const ChainIo io{a.out, a.ws, a.xq_out, a.s_out, a.ex.epi_residual, a.ex.epi_next_w, a.ex.stats_out, a.ex.raw_out};
    if (chunks > kChunkWaves || a.M != 1) return false;
#define TERNA_CHAIN_ATTN(SP, HD)                                                                                        \
    terna_chain_norm_kernel<CPRO_ATTN, 1, 1, EPI, SP, HD><<<a.grid, dim3(kChunkWaves * 64), 0, a.st>>>(                   \
        a.x, a.norm_w, a.packed, a.M, a.N, a.K, a.eps, a.ws_num, a.qmode, io)
    if (head_dim == 128) {
        if (splits == 1) TERNA_CHAIN_ATTN(1, 128);
        else if (splits == 2) TERNA_CHAIN_ATTN(2, 128);
        else if (splits == 4) TERNA_CHAIN_ATTN(4, 128);
        else TERNA_CHAIN_ATTN(8, 128);
    } else {
        if (splits == 1) TERNA_CHAIN_ATTN(1, 64);
        else if (splits == 2) TERNA_CHAIN_ATTN(2, 64);
        else if (splits == 4) TERNA_CHAIN_ATTN(4, 64);
        else TERNA_CHAIN_ATTN(8, 64);
    }
#undef TERNA_CHAIN_ATTN
    return true;
}

// TERNASPMM_CHAIN_CHUNK=0 keeps the per-tile kernels (tuning aid).
bool chain_chunk_enabled()
{
    static const bool on = [] {
        const char* v = tuning_env("TERNASPMM_CHAIN_CHUNK");
        return !(v && std::atoi(v) == 0);
    }();
    return on;
}

}  // namespace

namespace terna {

bool launch_norm_linear_chunk(const uint16_t* x, const uint16_t* norm_w, const uint32_t* packed, uint16_t* out, const uint16_t* ws,
                              int ws_num, int8_t* xq_out, uint16_t* s_out, int M, int N, int K, float eps, int quant_mode,
                              hipStream_t st)
{
    if (!chain_chunk_enabled() || M < 1 || M > 8 || static_cast<long long>(N) * K / 4 >= (1ll << 31)) return false;
    ChainArgs a{};
    a.x = x;
    a.norm_w = norm_w;
    a.packed = packed;
    a.M = M; a.N = N; a.K = K;
    a.eps = eps;
    a.out = out;
    a.ws = ws;
    a.ws_num = ws_num;
    a.xq_out = xq_out;
    a.s_out = s_out;
    a.qmode = quant_mode;
    a.ex = FusedExtra{};
    a.grid = dim3(N / 16);
    a.st = st;
    return launch_norm_chunk_by_rows<CEPI_STORE>(a, (K / 64 + 3) / 4);
}

}  // namespace terna

extern "C" {

int ternaspmm_row_stats_count(int K) { return K < 8 || (K & 7) ? -1 : (K + 511) / 512; }

int ternaspmm_row_stats(const terna_bf16* h, const terna_bf16* norm_weight, float* stats_out, int M, int K, terna_stream stream)
{
    const int count = ternaspmm_row_stats_count(K);
    if (M < 1 || count < 1 || count > kStatsMaxPartials) {
        std::fprintf(stderr, "ternaspmm_row_stats: unsupported arguments (M=%d K=%d)\n", M, K);
        return -1;
    }
    terna_row_stats_kernel<<<dim3(M), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(h, norm_weight, reinterpret_cast<float2*>(stats_out), K, count);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("ternaspmm_row_stats", e, __LINE__);
    return count;
}

int ternaspmm_step_inputs(const long long* tokens, const long long* pos, int per_sequence, const terna_bf16* embedding, int V, int K,
                          const float* rope_table, int S, int rope_half, const terna_bf16* norm_weight, terna_bf16* x_out,
                          float* stats_out, float* rope_out, int B, terna_stream stream)
{
    const int count = ternaspmm_row_stats_count(K);
    if (B < 1 || B > 65535 || V < 1 || S < 1 || count < 1 || count > kStatsMaxPartials || rope_half < 4 || (rope_half & 3) || rope_half > 512 ||
        tokens == nullptr || pos == nullptr || embedding == nullptr || rope_table == nullptr || norm_weight == nullptr || x_out == nullptr ||
        stats_out == nullptr || rope_out == nullptr ||
        ((reinterpret_cast<uintptr_t>(embedding) | reinterpret_cast<uintptr_t>(x_out) | reinterpret_cast<uintptr_t>(norm_weight) |
          reinterpret_cast<uintptr_t>(rope_table) | reinterpret_cast<uintptr_t>(rope_out)) & 15)) {
        std::fprintf(stderr, "ternaspmm_step_inputs: unsupported arguments (B=%d V=%d K=%d S=%d rope_half=%d)\n", B, V, K, S, rope_half);
        return -1;
    }
    terna_step_inputs_kernel<<<dim3(B), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
        tokens, pos, per_sequence != 0, embedding, V, K, rope_table, S, rope_half, norm_weight, x_out, reinterpret_cast<float2*>(stats_out),
        rope_out, count);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("ternaspmm_step_inputs", e, __LINE__);
    return count;
}

int ternaspmm_interleave_gate_up(const void* packed, void* packed_out, int N, int K, terna_stream stream)
{
    if (N < 64 || K < 64 || (N % 64) || (K % 64) || packed == packed_out) return -1;
    terna_interleave_gate_up_kernel<<<dim3(N / 16), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<const uint32_t*>(packed), static_cast<uint32_t*>(packed_out), N, K);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("ternaspmm_interleave_gate_up", e, __LINE__);
    return 0;
}

int ternaspmm_quant_from_stats(const terna_bf16* h, const float* stats, int stats_count, const terna_bf16* norm_weight, float eps,
                               int8_t* xq_out, terna_bf16* s_out, int M, int K, terna_stream stream)
{
    if (M < 1 || K < 8 || (K & 7) || stats_count < 1 || stats_count > kStatsMaxPartials || h == nullptr || stats == nullptr ||
        norm_weight == nullptr || xq_out == nullptr || s_out == nullptr) {
        std::fprintf(stderr, "ternaspmm_quant_from_stats: unsupported arguments (M=%d K=%d partials=%d)\n", M, K, stats_count);
        return -1;
    }
    terna_quant_stats_kernel<<<dim3(M, (K + 2047) / 2048), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
        h, reinterpret_cast<const float2*>(stats), stats_count, norm_weight, K, eps, xq_out, s_out, quant_mode());
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("ternaspmm_quant_from_stats", e, __LINE__);
    return 0;
}

int ternaspmm_fused_linear(const ternaspmm_fused_linear_desc* d, terna_stream stream)
{
    if (d == nullptr) return -1;
    const int M = d->M, N = d->N, K = d->K;
    const int pro = d->prologue, epi = d->epilogue;
    if (pro == TERNASPMM_PROLOGUE_QUANTISED) {
        // activations already quantised (ternaspmm_quant_from_stats, ternaspmm_rmsnorm_quant): the matmul of
        // bitlinear_TernaSpMM_packed with a producing epilogue
        const bool gate = epi == TERNASPMM_EPILOGUE_GATE;
        const int bands = N / 16, chunks = (K / 64 + 3) / 4;
        if (!shape_ok(M, N, K) || !groups_ok(d->ws_num) || !i8_depth_ok(K) || M > 16 || (epi != TERNASPMM_EPILOGUE_RESIDUAL && !gate) ||
            d->x == nullptr || d->s_in == nullptr || d->packed == nullptr || d->ws == nullptr || d->out == nullptr ||
            d->next_norm_weight == nullptr || d->stats_out == nullptr)
            return -1;
        if (gate ? (d->ws_num != 2 || bands % 4 != 0 || bands / 2 > kStatsMaxPartials) : (d->residual == nullptr || bands > kStatsMaxPartials))
            return -1;
        const hipStream_t st = static_cast<hipStream_t>(stream);
        ChainArgs a{};
        a.x = static_cast<const uint16_t*>(d->x);
        a.packed = static_cast<const uint32_t*>(d->packed);
        a.M = M; a.N = N; a.K = K;
        a.out = d->out;
        a.ws = d->ws;
        a.ws_num = d->ws_num;
        a.ex = FusedExtra{nullptr, 0, d->residual, d->next_norm_weight, reinterpret_cast<float2*>(d->stats_out), d->raw_out};
        a.st = st;
        const bool wide = chain_chunk_enabled() && static_cast<long long>(N) * K / 4 < (1ll << 31);
        bool done = false;
        if (gate) {
            // four bands (two gate / up pairs) per workgroup, a unit of work is a chunk of one pair
            a.grid = dim3(bands / 4);
            done = wide && launch_chunk_quantised<4, CEPI_GATE>(a, d->s_in, 2 * chunks);
            if (!done) return -1;
        } else {
            a.grid = dim3(bands);
            done = wide && launch_chunk_quantised<1, CEPI_RESIDUAL>(a, d->s_in, chunks);
            if (!done) {
                const Epilogue ep{d->s_in, d->ws, nullptr, d->ws_num, EP_I8_DECODE};
                launch_decode_packed_producer(static_cast<const int8_t*>(d->x), static_cast<const uint32_t*>(d->packed), d->out, ep, M, N, K,
                                              d->residual, d->next_norm_weight, d->stats_out, d->raw_out, st);
            }
        }
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess) die("ternaspmm_fused_linear", e, __LINE__);
        return gate ? bands / 2 : bands;
    }
    if (!shape_ok(M, N, K) || !groups_ok(d->ws_num) || M > 8) return -1;
    const int ktiles = K / 64, bands = N / 16;
    if (pro != TERNASPMM_PROLOGUE_NORM && pro != TERNASPMM_PROLOGUE_ATTENTION && pro != TERNASPMM_PROLOGUE_STATS) return -1;
    if (epi != TERNASPMM_EPILOGUE_STORE && epi != TERNASPMM_EPILOGUE_RESIDUAL && epi != TERNASPMM_EPILOGUE_GATE) return -1;
    if (d->x == nullptr || d->norm_weight == nullptr || d->packed == nullptr || d->ws == nullptr || d->out == nullptr) return -1;
    if ((d->xq_out != nullptr) != (d->s_out != nullptr)) return -1;
    if (pro == TERNASPMM_PROLOGUE_STATS && (d->stats_in == nullptr || d->stats_count < 1 || d->stats_count > kStatsMaxPartials)) return -1;
    if (epi != TERNASPMM_EPILOGUE_STORE && (d->next_norm_weight == nullptr || d->stats_out == nullptr)) return -1;
    if (epi == TERNASPMM_EPILOGUE_RESIDUAL && d->residual == nullptr) return -1;
    if (epi == TERNASPMM_EPILOGUE_GATE && (d->ws_num != 2 || bands % 4 != 0)) return -1;
    const int out_partials = epi == TERNASPMM_EPILOGUE_RESIDUAL ? bands : (epi == TERNASPMM_EPILOGUE_GATE ? bands / 2 : 0);
    if (out_partials > kStatsMaxPartials) return -1;

    ChainArgs a{};
    a.x = static_cast<const uint16_t*>(d->x);
    a.norm_w = d->norm_weight;
    a.packed = static_cast<const uint32_t*>(d->packed);
    a.M = M; a.N = N; a.K = K;
    a.eps = d->eps;
    a.out = d->out;
    a.ws = d->ws;
    a.ws_num = d->ws_num;
    a.xq_out = d->xq_out;
    a.s_out = d->s_out;
    a.qmode = quant_mode();
    a.ex = FusedExtra{reinterpret_cast<const float2*>(d->stats_in), d->stats_count, d->residual, d->next_norm_weight,
                      reinterpret_cast<float2*>(d->stats_out), d->raw_out};
    a.st = static_cast<hipStream_t>(stream);

    if (pro == TERNASPMM_PROLOGUE_ATTENTION) {
        // the O projection of a single-row step with the deferred attention merge inside (x = the partial results)
        const int hd = d->head_dim, sp = d->attention_splits;
        if (M != 1 || (hd != 64 && hd != 128) || K % hd != 0 || (sp != 1 && sp != 2 && sp != 4 && sp != 8) || ktiles > 8 * 5 ||
            bands > 65535 || epi == TERNASPMM_EPILOGUE_GATE)
            return -1;
        a.grid = dim3(bands);
        const bool wide = chain_chunk_enabled() && static_cast<long long>(N) * K / 4 < (1ll << 31);
        const int chunks = (ktiles + 3) / 4;
        if (epi == TERNASPMM_EPILOGUE_RESIDUAL) {
            if (!(wide && launch_attn_chunk<CEPI_RESIDUAL>(a, sp, hd, chunks))) launch_attn<FEPI_RESIDUAL>(a, sp, hd);
        } else {
            if (!(wide && launch_attn_chunk<CEPI_STORE>(a, sp, hd, chunks))) launch_attn<FEPI_PLAIN>(a, sp, hd);
        }
    } else if (epi == TERNASPMM_EPILOGUE_GATE) {
        // gate+up, bands interleaved: four bands (two gate / up pairs) per workgroup
        if (pro != TERNASPMM_PROLOGUE_STATS || ktiles > 8 * 5) return -1;
        a.grid = dim3(bands / 4);
        const bool wide = chain_chunk_enabled() && static_cast<long long>(N) * K / 4 < (1ll << 31);
        // a unit of work: a chunk with all four bands, so that its activations are normed and quantised once per workgroup
        // (units of a chunk and ONE gate / up pair, spread over more waves: 1159 against 1180 tokens/s at one row, 3740
        // against 3871 at four)
        const bool done = wide && launch_chunk_by_rows<4, CEPI_GATE, 4>(a, (ktiles + 3) / 4);
        if (!done) launch_by_rows<8, 5, FUSED_STATS, 4, FEPI_GLU>(a);
    } else if (pro == TERNASPMM_PROLOGUE_STATS) {
        const bool res = epi == TERNASPMM_EPILOGUE_RESIDUAL;
        a.grid = dim3(bands);
        const int chunks = (ktiles + 3) / 4;
        const bool wide = chain_chunk_enabled() && static_cast<long long>(N) * K / 4 < (1ll << 31);
        if (wide && (res ? launch_chunk_by_rows<1, CEPI_RESIDUAL>(a, chunks) : launch_chunk_by_rows<1, CEPI_STORE>(a, chunks))) {
            // launched
        } else if (ktiles <= 8 * 5) {
            if (res) launch_by_rows<8, 5, FUSED_STATS, 1, FEPI_RESIDUAL>(a);
            else launch_by_rows<8, 5, FUSED_STATS, 1, FEPI_PLAIN>(a);
        } else if (ktiles <= 16 * 7) {
            if (res) launch_by_rows<16, 7, FUSED_STATS, 1, FEPI_RESIDUAL>(a);
            else launch_by_rows<16, 7, FUSED_STATS, 1, FEPI_PLAIN>(a);
        } else {
            return -1;
        }
    } else {
        // the norm's statistics taken inside (two workgroup-wide reductions), producing epilogue
        if (epi != TERNASPMM_EPILOGUE_RESIDUAL || ktiles > 8 * 5) return -1;     // (with a plain store: bitlinear_TernaSpMM_packed_fused)
        a.grid = dim3(bands);
        const bool wide = chain_chunk_enabled() && static_cast<long long>(N) * K / 4 < (1ll << 31);
        if (!(wide && launch_norm_chunk_by_rows<CEPI_RESIDUAL>(a, (ktiles + 3) / 4))) launch_by_rows<8, 5, FUSED_PLAIN, 1, FEPI_RESIDUAL>(a);
    }
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("ternaspmm_fused_linear", e, __LINE__);
    return out_partials;
}

}  // extern "C"
