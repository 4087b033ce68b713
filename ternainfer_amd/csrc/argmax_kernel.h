// Greedy sampling step of the decode loop: index of the largest logit of each row.
//
// The reference takes torch.argmax over the LM head's output (generate.py:283, 305); here it is one
// launch of one workgroup per row.  Ties go to the
// lowest index; NaN never wins a comparison (a row of NaNs returns 0).
#pragma once

#include "norm_quant_kernel.h"

namespace terna {

constexpr int kArgmaxThreads = 1024;
constexpr int kArgmaxBatch = 16;             // 16-byte loads in flight per thread: 256 KB per workgroup and round

__device__ __forceinline__ void argmax_merge(float& best, int& idx, float v, int i)
{
    if (v > best || (v == best && i < idx)) {
        best = v;
        idx = i;
    }
}

// x bf16 [B][V]; out int64 [B].
__global__ __launch_bounds__(kArgmaxThreads) void terna_argmax_bf16_kernel(const uint16_t* __restrict__ x,
                                                                           long long* __restrict__ out, int V)
{
    __shared__ float sv[kArgmaxThreads / 64];
    __shared__ int si[kArgmaxThreads / 64];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint16_t* row = x + static_cast<size_t>(blockIdx.x) * V;
    float best = -INFINITY;
    int idx = 0x7fffffff;
    // rows start 16-byte aligned when V is a multiple of 8; otherwise everything goes through the scalar tail
    const int nvec = (V & 7) == 0 ? V >> 3 : 0;
    for (int base = 0; base < nvec; base += kArgmaxThreads * kArgmaxBatch) {
        u32x4 raw[kArgmaxBatch];
#pragma unroll
        for (int u = 0; u < kArgmaxBatch; ++u) {
            const int v = base + u * kArgmaxThreads + tid;
            raw[u] = *reinterpret_cast<const u32x4*>(row + 8 * static_cast<size_t>(v < nvec ? v : nvec - 1));
        }
#pragma unroll
        for (int u = 0; u < kArgmaxBatch; ++u) {
            const int v = base + u * kArgmaxThreads + tid;
            if (v < nvec) {
                float f[8];
                unpack_bf16x8(raw[u], f);
#pragma unroll
                for (int e = 0; e < 8; ++e) {    // a thread's indices ascend: a strict compare keeps the first maximum
                    const bool better = f[e] > best;
                    best = better ? f[e] : best;
                    idx = better ? 8 * v + e : idx;
                }
            }
        }
    }
    for (int i = nvec * 8 + tid; i < V; i += kArgmaxThreads) argmax_merge(best, idx, bf16_bits_to_float(row[i]), i);
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        const float ov = __shfl_xor(best, off);
        const int oi = __shfl_xor(idx, off);
        argmax_merge(best, idx, ov, oi);
    }
    if (lane == 0) {
        sv[wave] = best;
        si[wave] = idx;
    }
    __syncthreads();
    if (wave == 0) {
        best = lane < kArgmaxThreads / 64 ? sv[lane] : -INFINITY;
        idx = lane < kArgmaxThreads / 64 ? si[lane] : 0x7fffffff;
#pragma unroll
        for (int off = 8; off >= 1; off >>= 1) {
            const float ov = __shfl_xor(best, off);
            const int oi = __shfl_xor(idx, off);
            argmax_merge(best, idx, ov, oi);
        }
        if (lane == 0) out[blockIdx.x] = idx == 0x7fffffff ? 0 : idx;
    }
}

}  // namespace terna
