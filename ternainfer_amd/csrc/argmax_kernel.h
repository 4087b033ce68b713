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

// ---- the whole bookkeeping of a greedy decode step in one launch -------------------------------
// kGreedyChunks workgroups share a row (one CU streams a 256 KB row in about 8 us; sixteen take
// 16 KB each), leave (value, index) of their chunk in `state`, and the last workgroup of the grid
// to arrive -- counted in the first word of `state`, zero before the first launch and zero again
// after every launch -- merges every row's chunks in index order (the result does not depend on
// which workgroup that is), writes the tokens, appends them to the history and advances the
// counters.  The partials and the count go through device-scope relaxed atomics, past the per-XCD
// L2, as in the split attention: stores complete at the barrier, the arrival is counted after it,
// and the merging workgroup reads after it has seen the full count.
constexpr int kGreedyChunks = 16;
constexpr int kGreedyThreads = 256;
constexpr int kGreedyBatch = 4;              // 16-byte loads in flight per thread

constexpr size_t greedy_state_bytes(int B) { return 8 * (1 + static_cast<size_t>(B) * kGreedyChunks); }

// x bf16 [B][V]; tok int64 [B]; history int64 [B][history_len] or null; counters int64 [2] or null;
// state: greedy_state_bytes(B), 8-byte aligned.  Grid (kGreedyChunks, B).
__global__ __launch_bounds__(kGreedyThreads) void terna_greedy_step_kernel(const uint16_t* __restrict__ x, long long* __restrict__ tok,
                                                                           long long* __restrict__ history, int history_len,
                                                                           long long* __restrict__ counters,
                                                                           unsigned long long* state, int B, int V)
{
    __shared__ float sv[kGreedyThreads / 64];
    __shared__ int si[kGreedyThreads / 64];
    __shared__ int last_flag;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int chunk = blockIdx.x, b = blockIdx.y;
    const uint16_t* row = x + static_cast<size_t>(b) * V;
    float best = -INFINITY;
    int idx = 0x7fffffff;
    const int nvec = (V & 7) == 0 ? V >> 3 : 0;              // as above: unaligned rows go through the scalar tail
    const int per = (nvec + kGreedyChunks - 1) / kGreedyChunks;
    const int v0 = chunk * per, v1 = v0 + per < nvec ? v0 + per : nvec;
    for (int base = v0; base < v1; base += kGreedyThreads * kGreedyBatch) {
        u32x4 raw[kGreedyBatch];
#pragma unroll
        for (int u = 0; u < kGreedyBatch; ++u) {
            const int v = base + u * kGreedyThreads + tid;
            raw[u] = *reinterpret_cast<const u32x4*>(row + 8 * static_cast<size_t>(v < v1 ? v : v1 - 1));
        }
#pragma unroll
        for (int u = 0; u < kGreedyBatch; ++u) {
            const int v = base + u * kGreedyThreads + tid;
            if (v < v1) {
                float f[8];
                unpack_bf16x8(raw[u], f);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const bool better = f[e] > best;
                    best = better ? f[e] : best;
                    idx = better ? 8 * v + e : idx;
                }
            }
        }
    }
    if (chunk == kGreedyChunks - 1)                          // the scalar tail holds the highest indices: last chunk
        for (int i = nvec * 8 + tid; i < V; i += kGreedyThreads) argmax_merge(best, idx, bf16_bits_to_float(row[i]), i);
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
    int* arrived = reinterpret_cast<int*>(state);
    unsigned long long* partial = state + 1;
    if (tid == 0) {
#pragma unroll
        for (int w = 1; w < kGreedyThreads / 64; ++w) argmax_merge(best, idx, sv[w], si[w]);
        const unsigned long long packed = (static_cast<unsigned long long>(__float_as_uint(best)) << 32) | static_cast<unsigned>(idx);
        __hip_atomic_store(partial + b * kGreedyChunks + chunk, packed, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        // the arrival below must not overtake this store (another memory channel): wait for its acknowledgement
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    __syncthreads();
    if (tid == 0)
        last_flag = __hip_atomic_fetch_add(arrived, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == B * kGreedyChunks - 1;
    __syncthreads();
    if (!last_flag) return;
    const long long step = counters ? counters[1] : 0;
    for (int r = tid; r < B; r += kGreedyThreads) {
        float m = -INFINITY;
        int mi = 0x7fffffff;
        for (int c = 0; c < kGreedyChunks; ++c) {
            const unsigned long long p = __hip_atomic_load(partial + r * kGreedyChunks + c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            argmax_merge(m, mi, __uint_as_float(static_cast<unsigned>(p >> 32)), static_cast<int>(p & 0xffffffffu));
        }
        const long long t = mi == 0x7fffffff ? 0 : mi;
        tok[r] = t;
        if (history && step < history_len) history[static_cast<size_t>(r) * history_len + step] = t;
    }
    __syncthreads();                                         // every thread has read the step number
    if (tid == 0) {
        if (counters) {
            counters[0] += 1;
            counters[1] = step + 1;
        }
        __hip_atomic_store(arrived, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);    // ready for the next launch
    }
}

}  // namespace terna
