// C ABI of the tail of a decode step: bf16 LM head (lm_head_kernel.h) and greedy sampling (argmax_kernel.h).
// Declarations: include/ternaspmm.h.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

#include "../../include/ternaspmm.h"
#include "host_util.h"
#include "argmax_kernel.h"
#include "lm_head_kernel.h"

using namespace terna;

extern "C" {

void ternaspmm_argmax_bf16(const terna_bf16* x, long long* out, int B, int V, terna_stream stream)
{
    if (B < 1 || V < 1) {
        std::fprintf(stderr, "ternaspmm_argmax_bf16: unsupported arguments (B=%d V=%d)\n", B, V);
        return;
    }
    terna_argmax_bf16_kernel<<<dim3(B), dim3(kArgmaxThreads), 0, static_cast<hipStream_t>(stream)>>>(x, out, V);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("ternaspmm_argmax_bf16", e, __LINE__);
}

size_t ternaspmm_greedy_step_state_bytes(int B) { return B < 1 ? 0 : greedy_state_bytes(B); }

void ternaspmm_greedy_step_bf16(const terna_bf16* logits, long long* tok, long long* history, int history_len,
                                long long* counters, void* state, int B, int V, terna_stream stream)
{
    if (B < 1 || B > 65535 || V < 1 || !state || (reinterpret_cast<uintptr_t>(state) & 7) || (history && history_len < 1)) {
        std::fprintf(stderr, "ternaspmm_greedy_step_bf16: unsupported arguments (B=%d V=%d history_len=%d state=%p)\n", B, V,
                     history_len, state);
        return;
    }
    terna_greedy_step_kernel<<<dim3(kGreedyChunks, B), dim3(kGreedyThreads), 0, static_cast<hipStream_t>(stream)>>>(
        logits, tok, history, history_len, counters, static_cast<unsigned long long*>(state), B, V);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("ternaspmm_greedy_step_bf16", e, __LINE__);
}

void ternaspmm_lm_head_bf16(const terna_bf16* x, const terna_bf16* w, terna_bf16* logits, int M, int V, int K,
                            terna_stream stream)
{
    if (M < 1 || M > 16 || V < 1 || K < 32 || (K & 31) || K > 16384 || (reinterpret_cast<uintptr_t>(x) & 15) ||
        (reinterpret_cast<uintptr_t>(w) & 15)) {
        std::fprintf(stderr, "ternaspmm_lm_head_bf16: unsupported arguments (M=%d V=%d K=%d)\n", M, V, K);
        return;
    }
    // the unpadded layout where it buys a second workgroup per CU (TERNASPMM_LM_HEAD_SWIZZLE=0 keeps the padded one)
    static const bool swizzle_on = [] {
        const char* v = tuning_env("TERNASPMM_LM_HEAD_SWIZZLE");
        return !(v && std::atoi(v) == 0);
    }();
    const bool swizzled = swizzle_on && M > 4 && (K & 63) == 0 && lm_head_lds_bytes(M, K) > 80 * 1024 && lm_head_lds_bytes_swizzled(M, K) <= 80 * 1024;
    const size_t lds = swizzled ? lm_head_lds_bytes_swizzled(M, K) : lm_head_lds_bytes(M, K);
    if (lds > 160 * 1024) {
        std::fprintf(stderr, "ternaspmm_lm_head_bf16: M=%d rows of K=%d do not fit the 160 KB of LDS\n", M, K);
        return;
    }
    if (lds > 64 * 1024) allow_dynamic_lds(terna_lm_head_kernel, 160 * 1024, "hipFuncSetAttribute(lm head)", __LINE__);
    const int blocks = (V + 15) / 16;
    const int wgs_needed = (blocks + kLmWaves - 1) / kLmWaves;
    static const int forced = [] {
        const char* v = tuning_env("TERNASPMM_LM_HEAD_WGS");
        return v ? std::atoi(v) : 0;
    }();
    const int cap = forced > 0 ? forced : 512;               // two workgroups per CU measure fastest (256: 137 us, 512: 115 us, 1024: 119 us on 657 MB)
    const int grid = wgs_needed < cap ? wgs_needed : cap;
    static const int quad = [] {
        const char* v = tuning_env("TERNASPMM_LM_HEAD_QUAD");
        return v ? std::atoi(v) : 1;
    }();
    const int ksteps = K / 128;
    static const bool quad32 = [] {                     // TERNASPMM_LM_HEAD_QUAD32=0: 5 - 8 rows through the 16-row kernel
        const char* v = tuning_env("TERNASPMM_LM_HEAD_QUAD32");
        return !(v && std::atoi(v) == 0);
    }();
    if (quad && quad32 && M > 4 && M <= 8 && (K & 63) == 0) {
        const int qwgs = ((V + 7) / 8 + kLmWaves - 1) / kLmWaves;
        const dim3 qgrid(qwgs < cap ? qwgs : cap);
        if ((K / 64) % 10 == 0) {
            if (lds > 64 * 1024) allow_dynamic_lds(terna_lm_head_quad32_kernel<10>, 160 * 1024, "hipFuncSetAttribute(lm head)", __LINE__);
            terna_lm_head_quad32_kernel<10><<<qgrid, dim3(kLmWaves * 64), lds, static_cast<hipStream_t>(stream)>>>(x, w, logits, M, V, K);
        } else {
            if (lds > 64 * 1024) allow_dynamic_lds(terna_lm_head_quad32_kernel<8>, 160 * 1024, "hipFuncSetAttribute(lm head)", __LINE__);
            terna_lm_head_quad32_kernel<8><<<qgrid, dim3(kLmWaves * 64), lds, static_cast<hipStream_t>(stream)>>>(x, w, logits, M, V, K);
        }
    } else if (quad && M <= 4 && (K & 127) == 0) {
        const int qwgs = ((V + 3) / 4 + kLmWaves - 1) / kLmWaves;
        const dim3 qgrid(qwgs < cap ? qwgs : cap);
        if (ksteps % 10 == 0) {
            if (lds > 64 * 1024) allow_dynamic_lds(terna_lm_head_quad_kernel<10>, 160 * 1024, "hipFuncSetAttribute(lm head)", __LINE__);
            terna_lm_head_quad_kernel<10><<<qgrid, dim3(kLmWaves * 64), lds, static_cast<hipStream_t>(stream)>>>(x, w, logits, M, V, K);
        } else {
            if (lds > 64 * 1024) allow_dynamic_lds(terna_lm_head_quad_kernel<8>, 160 * 1024, "hipFuncSetAttribute(lm head)", __LINE__);
            terna_lm_head_quad_kernel<8><<<qgrid, dim3(kLmWaves * 64), lds, static_cast<hipStream_t>(stream)>>>(x, w, logits, M, V, K);
        }
    } else {
        terna_lm_head_kernel<<<dim3(grid), dim3(kLmWaves * 64), lds, static_cast<hipStream_t>(stream)>>>(x, w, logits, M, V, K, swizzled ? 1 : 0);
    }
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("ternaspmm_lm_head_bf16", e, __LINE__);
}

}  // extern "C"
