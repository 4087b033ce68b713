// C ABI of the multi-token attention of a prompt pass (prefill_attention_kernel.h).  Declaration: include/ternaspmm.h.
// A translation unit of its own because it is compiled with -mllvm -amdgpu-mfma-vgpr-form: the kernels rescale their
// running output between matrix instructions, and with the accumulators in the matrix core's own registers every
// round would copy them out and back (64 - 100 copies per 24 matrix instructions).
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

#include "../../include/ternaspmm.h"
#include "host_util.h"
#include "prefill_attention_kernel.h"

using namespace terna;

extern "C" {

void ternaspmm_prefill_attention(const terna_bf16* q, const terna_bf16* cache_k, const terna_bf16* cache_v,
                                 const long long* pos, int per_sequence, terna_bf16* out, int B, int T, int H, int KV, int D, int S,
                                 float scale, terna_stream stream)
{
    if (!attention_args_ok("ternaspmm_prefill_attention", B, H, KV, D, S) || T < 1 || B > 65535 || H > 65535) {
        if (T < 1 || B > 65535 || H > 65535) std::fprintf(stderr, "ternaspmm_prefill_attention: unsupported arguments (B=%d T=%d H=%d)\n", B, T, H);
        return;
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    // The query heads of a kv head in one workgroup (keys and values fetched once for all of them) when there are
    // 1, 2, 4 or 8 per kv head; else one wave per head.  TERNASPMM_PREFILL_ATTN_GROUP=0 forces the latter (tuning aid;
    // the results are the same bits).
    static const bool group_off = [] {
        const char* v = tuning_env("TERNASPMM_PREFILL_ATTN_GROUP");
        return v && std::atoi(v) == 0;
    }();
    const int G = H / KV;
    const int ps = per_sequence != 0;
    const dim3 ggrid((T + 15) / 16, KV, B);
#define TERNA_GROUP_ATTN(DD, GG) \
    terna_prefill_attention_group_kernel<DD, GG><<<ggrid, dim3(64 * GG), 0, st>>>(q, cache_k, cache_v, pos, out, T, H, KV, S, scale, ps)
    if (!group_off && D == 128 && G == 4) TERNA_GROUP_ATTN(128, 4);
    else if (!group_off && D == 128 && G == 8) TERNA_GROUP_ATTN(128, 8);
    else if (!group_off && D == 128 && G == 2) TERNA_GROUP_ATTN(128, 2);
    else if (!group_off && D == 128 && G == 1) TERNA_GROUP_ATTN(128, 1);
    else if (!group_off && D == 64 && G == 4) TERNA_GROUP_ATTN(64, 4);
    else if (!group_off && D == 64 && G == 8) TERNA_GROUP_ATTN(64, 8);
    else if (!group_off && D == 64 && G == 2) TERNA_GROUP_ATTN(64, 2);
    else if (!group_off && D == 64 && G == 1) TERNA_GROUP_ATTN(64, 1);
#undef TERNA_GROUP_ATTN
    else {
        const dim3 grid((T + 15) / 16, H, B);
        if (D == 128) terna_prefill_attention_kernel<128><<<grid, dim3(64), 0, st>>>(q, cache_k, cache_v, pos, out, T, H, KV, S, scale, ps);
        else terna_prefill_attention_kernel<64><<<grid, dim3(64), 0, st>>>(q, cache_k, cache_v, pos, out, T, H, KV, S, scale, ps);
    }
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("ternaspmm_prefill_attention", e, __LINE__);
}

}  // extern "C"
