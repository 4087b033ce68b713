// C ABI of the fused prologue of a ternary linear: norm / gate / activation quantisation as kernels of their own
// (norm_quant_kernel.h) and inside the small-M linear (decode_fused_kernel.h).  Declarations: include/ternaspmm.h.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

#include "../../include/ternaspmm.h"
#include "host_util.h"
#include "norm_quant_kernel.h"
#include "decode_fused_kernel.h"
#include "launchers.h"

using namespace terna;

extern "C" {

void ternaspmm_rmsnorm_quant(const terna_bf16* x, const terna_bf16* residual, terna_bf16* sum_out,
                             const terna_bf16* weight, float eps, terna_bf16* y_out, int8_t* xq_out,
                             terna_bf16* s_out, int M, int K, terna_stream stream)
{
    if (M < 1 || K < 8 || (K & 7) || K > 8 * kNormThreads * kNormMaxVecs || (xq_out != nullptr) != (s_out != nullptr)) {
        std::fprintf(stderr, "ternaspmm_rmsnorm_quant: unsupported arguments (M=%d K=%d)\n", M, K);
        return;
    }
    // as many 8-element vectors per thread as the row needs (1, 2 or 4), the residual's loads only where there is one
    const int nv = (K / 8 + kNormThreads - 1) / kNormThreads;
    const dim3 grid(M), block(kNormThreads);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int qm = quant_mode();
#define TERNA_NORM(NV, SECOND) terna_norm_quant_kernel<false, NV, SECOND><<<grid, block, 0, st>>>(x, residual, weight, K, eps, sum_out, y_out, xq_out, s_out, qm)
    if (residual != nullptr) {
        if (nv <= 1) TERNA_NORM(1, true);
        else if (nv <= 2) TERNA_NORM(2, true);
        else TERNA_NORM(4, true);
    } else {
        if (nv <= 1) TERNA_NORM(1, false);
        else if (nv <= 2) TERNA_NORM(2, false);
        else TERNA_NORM(4, false);
    }
#undef TERNA_NORM
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("ternaspmm_rmsnorm_quant", e, __LINE__);
}

void ternaspmm_relu2_mul_rmsnorm_quant(const terna_bf16* x13, const terna_bf16* weight, float eps, terna_bf16* y_out,
                                       int8_t* xq_out, terna_bf16* s_out, int M, int F, terna_stream stream)
{
    if (M < 1 || F < 8 || (F & 7) || F > 8 * kNormThreads * kNormMaxVecs || (xq_out != nullptr) != (s_out != nullptr)) {
        std::fprintf(stderr, "ternaspmm_relu2_mul_rmsnorm_quant: unsupported arguments (M=%d F=%d)\n", M, F);
        return;
    }
    const int nv = (F / 8 + kNormThreads - 1) / kNormThreads;
    const dim3 grid(M), block(kNormThreads);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int qm = quant_mode();
#define TERNA_NORM(NV) terna_norm_quant_kernel<true, NV, true><<<grid, block, 0, st>>>(x13, nullptr, weight, F, eps, nullptr, y_out, xq_out, s_out, qm)
    if (nv <= 1) TERNA_NORM(1);
    else if (nv <= 2) TERNA_NORM(2);
    else TERNA_NORM(4);
#undef TERNA_NORM
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("ternaspmm_relu2_mul_rmsnorm_quant", e, __LINE__);
}

// One band per workgroup repeats the prologue in every workgroup: only where one round of workgroups covers the matrix.
static bool bands_fit_one_round(int N) { return N / 16 <= 256; }

// mode: FUSED_PLAIN / FUSED_RESIDUAL / FUSED_GLU.  Returns 1 when a launch was enqueued.
static int launch_decode_fused(int mode, const terna_bf16* x, const terna_bf16* residual, terna_bf16* sum_out,
                               const terna_bf16* norm_weight, float eps, const void* packed, terna_bf16* out,
                               const terna_bf16* ws, int ws_num, int8_t* xq_out, terna_bf16* s_out, int M, int N,
                               int K, hipStream_t st)
{
    if (!shape_ok(M, N, K) || !groups_ok(ws_num) || M > 16) return 0;
    // Rows longer than the per-tile kernels below take (48 band-tiles), no second operand, up to 8 rows: the wide-load
    // kernel of the chained step's NORM prologue.  For the shorter rows it measured level with the kernels here at
    // 1-4 rows and 2 % behind at 6-8 rows in a whole decode step, so they keep those.
    if (mode == FUSED_PLAIN && K / 64 > 16 * 3)
        return bands_fit_one_round(N) && launch_norm_linear_chunk(x, norm_weight, static_cast<const uint32_t*>(packed), out, ws, ws_num,
                                                                  xq_out, s_out, M, N, K, eps, quant_mode(), st)
                   ? 1
                   : 0;
    const int ktiles = K / 64;
    const int bands = N / 16;
    static const int forced_waves = [] {
        const char* v = tuning_env("TERNASPMM_FUSED_WAVES");
        return v ? std::atoi(v) : 0;
    }();
    // 8 waves of up to 5 band-tiles where K allows (measured: +2 % tokens/s over 16 waves of 3 once the weight loads
    // were lane-contiguous), 16 waves for longer K and for the gate variant; TERNASPMM_FUSED_WAVES=8|16 forces one
    const bool wide = forced_waves == 16 ? true : (forced_waves == 8 ? mode == FUSED_GLU : mode == FUSED_GLU || ktiles > 8 * 5);
    const uint32_t* p = static_cast<const uint32_t*>(packed);
    // More bands than CUs: four bands per workgroup, so that the grid is one round and the prologue runs once
    // per CU.  TERNASPMM_FUSED_BANDS=1 switches that off, TERNASPMM_FUSED_BANDS_WAVES=16 picks the 16-wave
    // variant of it (tuning aids).
    static const int forced_nb = [] {
        const char* v = tuning_env("TERNASPMM_FUSED_BANDS");
        return v ? std::atoi(v) : 0;
    }();
    static const int nb_waves = [] {
        const char* v = tuning_env("TERNASPMM_FUSED_BANDS_WAVES");
        return v && std::atoi(v) == 16 ? 16 : 8;
    }();
    const bool multi = forced_nb != 1 && bands > 256 && bands % 4 == 0 && mode != FUSED_GLU;
    const bool multi8 = multi && nb_waves == 8 && ktiles <= 8 * 5;
    const bool multi16 = multi && !multi8 && ktiles <= 16 * 3;
    const dim3 grid(multi16 || multi8 ? bands / 4 : bands);
    const int qmode = quant_mode();
#define TERNA_FUSED(WAVES, TMAX, MODE, MP, NB)                                                                     \
    terna_decode_fused_kernel<WAVES, TMAX, MODE, MP, NB><<<grid, dim3(WAVES * 64), 0, st>>>(                       \
        x, residual, norm_weight, p, M, N, K, eps, sum_out, out, ws, ws_num, xq_out, s_out, qmode, FusedExtra{})
#define TERNA_FUSED_M(WAVES, TMAX, MODE, NB)                                                                       \
    do {                                                                                                           \
        if (M == 1) TERNA_FUSED(WAVES, TMAX, MODE, 1, NB);                                                         \
        else if (M == 2) TERNA_FUSED(WAVES, TMAX, MODE, 2, NB);                                                    \
        else if (M <= 4) TERNA_FUSED(WAVES, TMAX, MODE, 4, NB);                                                    \
        else if (M <= 8) TERNA_FUSED(WAVES, TMAX, MODE, 8, NB);                                                    \
        else TERNA_FUSED(WAVES, TMAX, MODE, 16, NB);                                                               \
    } while (0)
    if (mode == FUSED_GLU) {
        // long K (the down projection): the variants for up to four rows, whose per-lane state is small
        if (M > 4 || !wide || ktiles > 16 * 7) return 0;
        if (M == 1) TERNA_FUSED(16, 7, FUSED_GLU, 1, 1);
        else if (M == 2) TERNA_FUSED(16, 7, FUSED_GLU, 2, 1);
        else TERNA_FUSED(16, 7, FUSED_GLU, 4, 1);
    } else if (multi16) {
        if (mode == FUSED_RESIDUAL) TERNA_FUSED_M(16, 3, FUSED_RESIDUAL, 4);
        else TERNA_FUSED_M(16, 3, FUSED_PLAIN, 4);
    } else if (multi8) {
        if (mode == FUSED_RESIDUAL) TERNA_FUSED_M(8, 5, FUSED_RESIDUAL, 4);
        else TERNA_FUSED_M(8, 5, FUSED_PLAIN, 4);
    } else if (wide) {
        if (ktiles > 16 * 3) return 0;
        if (mode == FUSED_RESIDUAL) TERNA_FUSED_M(16, 3, FUSED_RESIDUAL, 1);
        else TERNA_FUSED_M(16, 3, FUSED_PLAIN, 1);
    } else {
        if (ktiles > 8 * 5) return 0;
        if (mode == FUSED_RESIDUAL) TERNA_FUSED_M(8, 5, FUSED_RESIDUAL, 1);
        else TERNA_FUSED_M(8, 5, FUSED_PLAIN, 1);
    }
#undef TERNA_FUSED_M
#undef TERNA_FUSED
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("bitlinear_TernaSpMM_packed_fused", e, __LINE__);
    return 1;
}

int bitlinear_TernaSpMM_packed_fused(const terna_bf16* x, const terna_bf16* residual, terna_bf16* sum_out,
                                     const terna_bf16* norm_weight, float eps, const void* packed, terna_bf16* out,
                                     const terna_bf16* ws, int ws_num, int8_t* xq_out, terna_bf16* s_out, int M,
                                     int N, int K, terna_stream stream)
{
    return launch_decode_fused(residual ? FUSED_RESIDUAL : FUSED_PLAIN, x, residual, sum_out, norm_weight, eps, packed, out,
                               ws, ws_num, xq_out, s_out, M, N, K, static_cast<hipStream_t>(stream));
}

int bitlinear_TernaSpMM_packed_fused_attn(const float* partial, int splits, int head_dim, const terna_bf16* norm_weight, float eps,
                                          const void* packed, terna_bf16* out, const terna_bf16* ws, int ws_num,
                                          int8_t* xq_out, terna_bf16* s_out, int M, int N, int K, terna_stream stream)
{
    if (!shape_ok(M, N, K) || !groups_ok(ws_num)) return 0;
    const int ktiles = K / 64;
    if (M != 1 || (head_dim != 64 && head_dim != 128) || K % head_dim != 0 || (splits != 1 && splits != 2 && splits != 4 && splits != 8) ||
        partial == nullptr || N / 16 > 65535 || ktiles > 8 * 5)
        return 0;
    const dim3 grid(N / 16);
    const uint16_t* x = reinterpret_cast<const uint16_t*>(partial);
    const uint32_t* p = static_cast<const uint32_t*>(packed);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int qmode = quant_mode();
#define TERNA_FUSED_ATTN(SP, HD)                                                                                   \
    terna_decode_fused_kernel<8, 5, FUSED_ATTN, 1, 1, SP, HD><<<grid, dim3(8 * 64), 0, st>>>(                      \
        x, nullptr, norm_weight, p, M, N, K, eps, nullptr, out, ws, ws_num, xq_out, s_out, qmode, FusedExtra{})
#define TERNA_FUSED_ATTN_HD(HD)                                                                                    \
    do {                                                                                                           \
        if (splits == 1) TERNA_FUSED_ATTN(1, HD);                                                                  \
        else if (splits == 2) TERNA_FUSED_ATTN(2, HD);                                                             \
        else if (splits == 4) TERNA_FUSED_ATTN(4, HD);                                                             \
        else TERNA_FUSED_ATTN(8, HD);                                                                              \
    } while (0)
    if (head_dim == 128) TERNA_FUSED_ATTN_HD(128);
    else TERNA_FUSED_ATTN_HD(64);
#undef TERNA_FUSED_ATTN_HD
#undef TERNA_FUSED_ATTN
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("bitlinear_TernaSpMM_packed_fused_attn", e, __LINE__);
    return 1;
}

int bitlinear_TernaSpMM_packed_fused_glu(const terna_bf16* x13, const terna_bf16* norm_weight, float eps,
                                         const void* packed, terna_bf16* out, const terna_bf16* ws, int ws_num,
                                         int8_t* xq_out, terna_bf16* s_out, int M, int N, int F, terna_stream stream)
{
    return launch_decode_fused(FUSED_GLU, x13, nullptr, nullptr, norm_weight, eps, packed, out, ws, ws_num, xq_out, s_out,
                               M, N, F, static_cast<hipStream_t>(stream));
}

}  // extern "C"
