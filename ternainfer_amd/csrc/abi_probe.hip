// Calibration probes: tiny kernels that measure what the machine gives, so that the figures a benchmark line is
// priced against (launch floor, streaming rate, cost of a device-wide synchronisation) come from the same run
// and the same library as the kernels themselves.  No counterpart in the reference.  Declarations: include/ternaspmm.h.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

#include "../../include/ternaspmm.h"
#include "host_util.h"
#include "terna_common.h"

using namespace terna;

namespace {

__global__ void terna_probe_empty_kernel() {}

// An empty body behind a launch of a given shape: what the dispatch of that many waves, the LDS allocation and the end
// of the kernel cost before any work.  One lane touches the LDS so that the allocation is not optimised away.
__global__ void terna_probe_empty_shape_kernel(int never)
{
    extern __shared__ uint32_t probe_lds[];
    if (never) probe_lds[threadIdx.x] = 1u;
}

constexpr int kProbeThreads = 256;
constexpr int kProbeUnroll = 16;             // 16-byte vectors in flight per thread
constexpr long long kProbeTile = static_cast<long long>(kProbeThreads) * kProbeUnroll;     // vectors per tile: 64 KB, contiguous

// Streaming read of `vecs` 16-byte vectors.  A workgroup takes contiguous 64 KB tiles (tile t, t + grid, ...): every
// load of a wave is one contiguous kilobyte and the sixteen loads a thread has in flight stay inside one tile -- the
// access pattern of the streaming kernels here (a lane walks along a weight row), and the one that reaches the rate
// those kernels reach; vectors a grid apart (8 MB strides, sixteen distant regions per workgroup at a time) measured
// 20 % lower.  Non-temporal loads: nothing is read twice.  The sum is written only if it takes a value it never takes.
__global__ __launch_bounds__(kProbeThreads) void terna_probe_read_kernel(const u32x4* __restrict__ src, long long vecs,
                                                                       u32x4* __restrict__ sink)
{
    u32x4 acc = {0u, 0u, 0u, 0u};
    const long long tiles = vecs / kProbeTile;
    for (long long t = blockIdx.x; t < tiles; t += gridDim.x) {
        const u32x4* p = src + t * kProbeTile + threadIdx.x;
        u32x4 v[kProbeUnroll];
#pragma unroll
        for (int u = 0; u < kProbeUnroll; ++u) v[u] = __builtin_nontemporal_load(p + u * kProbeThreads);
#pragma unroll
        for (int u = 0; u < kProbeUnroll; ++u) acc ^= v[u];
    }
    for (long long i = tiles * kProbeTile + static_cast<long long>(blockIdx.x) * kProbeThreads + threadIdx.x; i < vecs;
         i += static_cast<long long>(gridDim.x) * kProbeThreads)
        acc ^= src[i];
    if ((acc.x & acc.y & acc.z & acc.w) == 0xFFFFFFFFu && sink != nullptr) sink[0] = acc;   // practically never: keeps the loads alive
}

__global__ __launch_bounds__(kProbeThreads) void terna_probe_copy_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst,
                                                                       long long vecs)
{
    const long long tiles = vecs / kProbeTile;
    for (long long t = blockIdx.x; t < tiles; t += gridDim.x) {
        const u32x4* p = src + t * kProbeTile + threadIdx.x;
        u32x4* q = dst + t * kProbeTile + threadIdx.x;
        u32x4 v[kProbeUnroll];
#pragma unroll
        for (int u = 0; u < kProbeUnroll; ++u) v[u] = __builtin_nontemporal_load(p + u * kProbeThreads);
#pragma unroll
        for (int u = 0; u < kProbeUnroll; ++u) __builtin_nontemporal_store(v[u], q + u * kProbeThreads);
    }
    for (long long i = tiles * kProbeTile + static_cast<long long>(blockIdx.x) * kProbeThreads + threadIdx.x; i < vecs;
         i += static_cast<long long>(gridDim.x) * kProbeThreads)
        dst[i] = src[i];
}

// `rounds` device-wide synchronisations among the workgroups of the grid (all co-resident: the host caps the grid
// at one workgroup per CU): each workgroup publishes its flag = round with a device-scope store and wave 0 polls
// all flags with one 16-byte load per lane until every one has reached the round.  The wait is bounded: after
// kProbeMaxPolls polls a workgroup counts a time-out in state[kProbeMaxGroups] and leaves, and so will all others.
constexpr int kProbeMaxGroups = 256;
constexpr int kProbeMaxPolls = 1 << 16;
__global__ __launch_bounds__(kProbeThreads) void terna_probe_barrier_kernel(uint32_t* __restrict__ state, int rounds, uint32_t first)
{
    const int G = gridDim.x, wg = blockIdx.x, tid = threadIdx.x;
    __shared__ int gave_up;
    if (tid == 0) gave_up = 0;
    __syncthreads();
    const int fvecs = (G + 3) >> 2;
    for (int r = 0; r < rounds; ++r) {
        const uint32_t tag = first + static_cast<uint32_t>(r);
        uint32_t* flags = state + (r & 1) * kProbeMaxGroups;          // two sets: a fast workgroup never overwrites what a slow one still polls
        if (tid == 0) __hip_atomic_store(flags + wg, tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (tid < 64) {
            int polls = 0;
            for (;;) {
                bool ok = true;
                if (tid < fvecs) {
                    const unsigned long long* p = reinterpret_cast<const unsigned long long*>(flags) + 2 * tid;
                    const unsigned long long a = __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    const unsigned long long b = __hip_atomic_load(p + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    const uint32_t f[4] = {static_cast<uint32_t>(a), static_cast<uint32_t>(a >> 32), static_cast<uint32_t>(b),
                                           static_cast<uint32_t>(b >> 32)};
#pragma unroll
                    for (int e = 0; e < 4; ++e) ok = ok && (4 * tid + e >= G || static_cast<int>(f[e] - tag) >= 0);
                }
                if (__all(ok)) break;
                if (++polls > kProbeMaxPolls) {
                    if (tid == 0) gave_up = 1;
                    break;
                }
            }
        }
        __syncthreads();
        if (gave_up) {
            if (tid == 0) atomicAdd(state + 2 * kProbeMaxGroups, 1u);
            return;
        }
    }
}

int probe_grid(long long vecs)
{
    const long long want = (vecs + kProbeThreads - 1) / kProbeThreads;
    return static_cast<int>(want < 2048 ? (want < 1 ? 1 : want) : 2048);      // eight workgroups per CU at most
}

}  // namespace

extern "C" {

void ternaspmm_probe_empty(terna_stream stream)
{
    terna_probe_empty_kernel<<<1, 64, 0, static_cast<hipStream_t>(stream)>>>();
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("ternaspmm_probe_empty", e, __LINE__);
}

int ternaspmm_probe_empty_shape(int workgroups, int threads, int lds_bytes, terna_stream stream)
{
    if (workgroups < 1 || workgroups > (1 << 20) || threads < 64 || threads > 1024 || (threads & 63) || lds_bytes < 0 || lds_bytes > 64 * 1024)
        return -1;
    terna_probe_empty_shape_kernel<<<dim3(workgroups), dim3(threads), lds_bytes, static_cast<hipStream_t>(stream)>>>(0);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("ternaspmm_probe_empty_shape", e, __LINE__);
    return 0;
}

void ternaspmm_probe_read(const void* src, long long bytes, void* sink, terna_stream stream)
{
    if (src == nullptr || bytes < 16 || (reinterpret_cast<uintptr_t>(src) & 15)) {
        std::fprintf(stderr, "ternaspmm_probe_read: need a 16-byte aligned buffer of at least 16 bytes\n");
        return;
    }
    const long long vecs = bytes / 16;
    terna_probe_read_kernel<<<probe_grid(vecs), kProbeThreads, 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<const u32x4*>(src), vecs, static_cast<u32x4*>(sink));
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("ternaspmm_probe_read", e, __LINE__);
}

int ternaspmm_probe_read_grid(const void* src, long long bytes, void* sink, int workgroups, terna_stream stream)
{
    if (src == nullptr || bytes < 16 || (reinterpret_cast<uintptr_t>(src) & 15) || workgroups < 1 || workgroups > 4096) return -1;
    terna_probe_read_kernel<<<workgroups, kProbeThreads, 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<const u32x4*>(src), bytes / 16, static_cast<u32x4*>(sink));
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("ternaspmm_probe_read_grid", e, __LINE__);
    return 0;
}

void ternaspmm_probe_copy(const void* src, void* dst, long long bytes, terna_stream stream)
{
    if (src == nullptr || dst == nullptr || bytes < 16 || ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15)) {
        std::fprintf(stderr, "ternaspmm_probe_copy: need 16-byte aligned buffers of at least 16 bytes\n");
        return;
    }
    const long long vecs = bytes / 16;
    terna_probe_copy_kernel<<<probe_grid(vecs), kProbeThreads, 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<const u32x4*>(src), static_cast<u32x4*>(dst), vecs);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("ternaspmm_probe_copy", e, __LINE__);
}

size_t ternaspmm_probe_barrier_state_bytes(void) { return (2 * kProbeMaxGroups + 4) * sizeof(uint32_t); }

int ternaspmm_probe_barrier(void* state, int workgroups, int rounds, unsigned first_tag, terna_stream stream)
{
    if (state == nullptr || (reinterpret_cast<uintptr_t>(state) & 15) || workgroups < 1 || workgroups > kProbeMaxGroups ||
        rounds < 1 || rounds > (1 << 20)) {
        std::fprintf(stderr, "ternaspmm_probe_barrier: need 16-byte aligned state, 1 .. %d workgroups, 1 .. 2^20 rounds\n",
                     kProbeMaxGroups);
        return -1;
    }
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
        return -1;
    if (workgroups > cus) {       // every workgroup must be resident at once, or the ones that are would wait out their bound
        std::fprintf(stderr, "ternaspmm_probe_barrier: %d workgroups exceed the %d CUs of the device\n", workgroups, cus);
        return -1;
    }
    terna_probe_barrier_kernel<<<workgroups, kProbeThreads, 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<uint32_t*>(state), rounds, first_tag);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("ternaspmm_probe_barrier", e, __LINE__);
    return 0;
}

}  // extern "C"
