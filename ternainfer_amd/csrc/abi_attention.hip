// C ABI of the attention-side kernels of a decode step (attention_kernel.h): RoPE + cache write, single-token
// attention, both in one launch, the prefetching variant, and the variant that allocates nothing.  The multi-token
// attention of a prompt pass: abi_prefill_attention.hip.
// Declarations: include/ternaspmm.h.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <mutex>

#include "../../include/ternaspmm.h"
#include "host_util.h"
#include "attention_kernel.h"
#include "attention_grouped_kernel.h"

using namespace terna;

namespace {

// one word per thread; the grid covers the buffer exactly
__global__ void terna_fill_u32_kernel(uint32_t* p, uint32_t v) { p[blockIdx.x * blockDim.x + threadIdx.x] = v; }

// Waves per workgroup of the decode attention: with one workgroup per (sequence, head) and few of them
// on the chip, wider workgroups request more of the cache up front (64 slots of keys per wave).
// TERNASPMM_ATTN_WAVES=4|8 forces one (tuning aid).  Both entry points use the same rule, so their results
// stay bit-identical.
int attention_waves(int B, int H)
{
    static const int forced = [] {
        const char* v = tuning_env("TERNASPMM_ATTN_WAVES");
        const int w = v ? std::atoi(v) : 0;
        return (w == 4 || w == 8) ? w : 0;
    }();
    if (forced) return forced;
    return static_cast<long>(B) * H <= 512 ? 8 : 4;
}

// Workgroups of the attention grid that stand for (sequence, head) pairs: B * H, or -- when kv groups are kept on one
// XCD each (more than one head per group; TERNASPMM_ATTN_XCD_GROUPS=0 switches it off) -- whole rounds of 8 groups.
bool attention_groups_on(int H, int KV)
{
    static const int on = [] {
        const char* v = tuning_env("TERNASPMM_ATTN_XCD_GROUPS");
        return v ? std::atoi(v) : 1;
    }();
    return on && H > KV;
}
int attention_slots(int B, int H, int KV)
{
    if (!attention_groups_on(H, KV)) return B * H;
    return 8 * (H / KV) * ((B * KV + 7) / 8);
}

// Workspace of the split variant: one arrival counter per head (the caller zeroes them once), then
// kAttentionMaxSplits partial results of D + 2 floats per head.
size_t attention_counter_bytes(int B, int H) { return (static_cast<size_t>(B) * H * sizeof(int) + 255) & ~static_cast<size_t>(255); }

// Splits of the cache per head: as many as keep the grid within two workgroups per CU, at most 8; 1 without
// a workspace, and 1 for caches below 1024 slots, where the merge (three dependent trips to device memory,
// 4-5 us) costs more than streaming the prefix from one CU.  TERNASPMM_ATTN_SPLITS=1|2|4|8 forces one
// (tuning aid).
// Where the split variant keeps its arrival counters (one int per head, zero between launches) and its partial
// results: carved out of the caller's workspace, or the library's own static array (the entry point that
// allocates nothing).
struct AttentionScratch {
    int* arrived = nullptr;
    float* partial = nullptr;
};
AttentionScratch attention_scratch_of(void* workspace, int B, int H)
{
    if (workspace == nullptr) return {};
    return {static_cast<int*>(workspace),
            reinterpret_cast<float*>(static_cast<char*>(workspace) + attention_counter_bytes(B, H))};
}

int attention_splits(int B, int H, int S, const AttentionScratch& scratch)
{
    if (scratch.arrived == nullptr) return 1;
    static const int forced = [] {
        const char* v = tuning_env("TERNASPMM_ATTN_SPLITS");
        const int n = v ? std::atoi(v) : 0;
        return (n == 1 || n == 2 || n == 4 || n == 8) ? n : 0;
    }();
    if (forced) return forced;
    if (S < 1024) return 1;
    int sp = 1;
    while (sp < kAttentionMaxSplits && static_cast<long>(B) * H * sp * 2 <= 512) sp *= 2;
    return sp;
}

template <int D, bool ROPE, bool ADJ, int NW, bool SPLIT, int KT = 4>
void launch_attention_as(const uint16_t* q, uint16_t* ck, uint16_t* cv, const float* cos, const float* sin,
                         const long long* pos, int per_seq, uint16_t* out, int B, int H, int KV, int S, float scale, int splits,
                         const AttentionScratch& scratch, const AttentionPrefetch& pf_in, hipStream_t st, AttentionStats stats)
{
    if (stats.norm_w == nullptr || stats.out == nullptr) stats = AttentionStats{q, nullptr};   // (the kernel loads norm_w unconditionally)
    AttentionPrefetch pf = pf_in;
    if (splits > 1) pf.workgroups = 0;                       // the split grid is two-dimensional: no extra workgroups
    auto kernel = terna_decode_attention_kernel<D, ROPE, ADJ, NW, SPLIT, false, KT>;
    const size_t lds = decode_attention_lds_bytes(D, NW, S);
    if (lds > 64 * 1024) allow_dynamic_lds(kernel, 159 * 1024, "hipFuncSetAttribute(decode attention)", __LINE__);
    const int slots = attention_slots(B, H, KV);
    kernel<<<dim3(slots + pf.workgroups, splits), dim3(64 * NW), lds, st>>>(
        q, ck, cv, pos, H, KV, S, splits, slots, attention_groups_on(H, KV) ? B * KV : 0, per_seq, scale, cos, sin, out, scratch.partial,
        scratch.arrived, pf, stats);
}

// The split with the merge left to the next launch (DEFER): one-dimensional grid of (sequence, head, split) workgroups,
// padded to whole rounds of 8 (group, split) pairs when kv groups are kept on one XCD each, then the prefetching ones.
template <int D, bool ADJ>
void launch_attention_deferred(const uint16_t* qkv, uint16_t* ck, uint16_t* cv, const float* cos, const float* sin,
                               const long long* pos, int per_seq, float* partial, int splits, int B, int H, int KV, int S,
                               float scale, const AttentionPrefetch& pf_in, hipStream_t st)
{
    constexpr int NW = 4;                                     // a split is a short prefix: the narrow workgroup
    AttentionPrefetch pf = pf_in;
    auto kernel = terna_decode_attention_kernel<D, true, ADJ, NW, true, true>;
    const size_t lds = decode_attention_lds_bytes(D, NW, S);
    if (lds > 64 * 1024) allow_dynamic_lds(kernel, 160 * 1024, "hipFuncSetAttribute(decode attention, deferred merge)", __LINE__);
    const bool grouped = attention_groups_on(H, KV);
    const int slots = grouped ? 8 * (H / KV) * ((B * KV * splits + 7) / 8) : B * H * splits;
    kernel<<<dim3(slots + pf.workgroups), dim3(64 * NW), lds, st>>>(
        qkv, ck, cv, pos, H, KV, S, splits, slots, grouped ? B * KV : 0, per_seq, scale, cos, sin, nullptr, partial, nullptr, pf, AttentionStats{qkv, nullptr});
}

int prefetch_workgroups(const AttentionPrefetch& pf, int slots);

// The deferred-merge launch with one workgroup per (sequence, kv head, split) (attention_grouped_kernel.h).  Returns false
// where that form does not apply: one head per kv head, a group size other than 2 or 4, a score buffer beyond the LDS.
template <int D, bool ADJ>
bool launch_attention_grouped(const uint16_t* qkv, uint16_t* ck, uint16_t* cv, const float* cos, const float* sin, const long long* pos,
                              int per_seq, float* partial, int splits, int B, int H, int KV, int S, float scale,
                              const AttentionPrefetch& pf_in, hipStream_t st)
{
    static const int waves = [] {
        // 8 waves: measured ahead of 4 at 2 - 8 sequences with caches of 1528 slots (8 sequences: 1.351 against 1.410 ms
        // per decode step), level with them at 384 slots
        const char* v = tuning_env("TERNASPMM_ATTN_GROUPED_WAVES");
        return v && std::atoi(v) == 4 ? 4 : 8;
    }();
    if (KV < 1 || H % KV != 0) return false;
    const int gq = H / KV;
    if (gq != 2 && gq != 4) return false;
    const size_t lds = grouped_attention_lds_bytes(D, waves, gq, S);
    if (lds > 159 * 1024) return false;          // (160 KB per workgroup, the kernel's static LDS included)
    AttentionPrefetch pf = pf_in;
    const int slots = B * KV * splits;
    pf.workgroups = prefetch_workgroups(pf, slots);
#define TERNA_GROUPED(NWAVES, GQ)                                                                                          \
    do {                                                                                                                   \
        auto kernel = terna_decode_attention_grouped_kernel<D, ADJ, NWAVES, GQ>;                                            \
        if (lds > 64 * 1024) allow_dynamic_lds(kernel, 159 * 1024, "hipFuncSetAttribute(decode attention, kv groups)", __LINE__); \
        kernel<<<dim3(slots + pf.workgroups), dim3(64 * NWAVES), lds, st>>>(qkv, ck, cv, pos, KV, S, splits, slots, per_seq, scale, cos, sin, \
                                                                            partial, pf);                                  \
    } while (0)
    if (waves == 8) {
        if (gq == 4) TERNA_GROUPED(8, 4);
        else TERNA_GROUPED(8, 2);
    } else {
        if (gq == 4) TERNA_GROUPED(4, 4);
        else TERNA_GROUPED(4, 2);
    }
#undef TERNA_GROUPED
    return true;
}

template <bool ROPE, bool ADJ>
void launch_attention(const uint16_t* q, uint16_t* ck, uint16_t* cv, const float* cos, const float* sin,
                             const long long* pos, int per_seq, uint16_t* out, int B, int H, int KV, int D, int S, float scale,
                             const AttentionScratch& scratch, const AttentionPrefetch& pf, hipStream_t st,
                             AttentionStats stats = AttentionStats{nullptr, nullptr})
{
    const int splits = attention_splits(B, H, S, scratch);
    const int nw = splits > 1 ? 4 : attention_waves(B, H);       // a split is a short prefix: the narrow workgroup
#define TERNA_ATTN(DIM, NWAVES, SPLIT) \
    launch_attention_as<DIM, ROPE, ADJ, NWAVES, SPLIT>(q, ck, cv, cos, sin, pos, per_seq, out, B, H, KV, S, scale, splits, scratch, pf, st, stats)
    // the wide unsplit workgroup: as many key tiles in flight per wave as cover the cache (128 slots each), four at most
    static const bool all_tiles = [] {               // TERNASPMM_ATTN_KEY_TILES=4: always four (tuning aid)
        const char* v = tuning_env("TERNASPMM_ATTN_KEY_TILES");
        return v && std::atoi(v) == 4;
    }();
#define TERNA_ATTN_WIDE(DIM)                                                                                                         \
    do {                                                                                                                             \
        if (all_tiles) TERNA_ATTN(DIM, 8, false);                                                                                    \
        else if (S <= 256) launch_attention_as<DIM, ROPE, ADJ, 8, false, 2>(q, ck, cv, cos, sin, pos, per_seq, out, B, H, KV, S, scale, splits, scratch, pf, st, stats); \
        else if (S <= 384) launch_attention_as<DIM, ROPE, ADJ, 8, false, 3>(q, ck, cv, cos, sin, pos, per_seq, out, B, H, KV, S, scale, splits, scratch, pf, st, stats); \
        else TERNA_ATTN(DIM, 8, false);                                                                                              \
    } while (0)
    if (D == 128) {
        if (splits > 1) TERNA_ATTN(128, 4, true);
        else if (nw == 8) TERNA_ATTN_WIDE(128);
        else TERNA_ATTN(128, 4, false);
    } else {
        if (splits > 1) TERNA_ATTN(64, 4, true);
        else if (nw == 8) TERNA_ATTN_WIDE(64);
        else TERNA_ATTN(64, 4, false);
    }
#undef TERNA_ATTN_WIDE
#undef TERNA_ATTN
}

// The regions of a prefetching launch from the caller's host arrays; a region that breaks a rule is skipped.
AttentionPrefetch prefetch_regions(const void* const* pf_ptr, const long long* pf_bytes, const long long* pf_unit_bytes, int pf_count)
{
    AttentionPrefetch pf{};
    for (int r = 0; r < pf_count && pf.count < kAttentionPrefetchRegions; ++r) {
        const bool broadcast = pf_unit_bytes[r] == 0;        // every XCD fetches the whole (small) region
        if (pf_ptr[r] == nullptr || (reinterpret_cast<uintptr_t>(pf_ptr[r]) & 15) || pf_bytes[r] < 16 || pf_bytes[r] > (1ll << 30) ||
            (!broadcast && (pf_unit_bytes[r] < 16 || (pf_unit_bytes[r] & 15) || pf_unit_bytes[r] > (1ll << 30))) ||
            (broadcast && pf_bytes[r] > (1ll << 20)))
            continue;
        const int c = pf.count++;
        pf.base[c] = static_cast<const u32x4*>(pf_ptr[r]);
        pf.total_vecs[c] = pf_bytes[r] / 16;
        pf.unit_vecs[c] = broadcast ? 0 : static_cast<int>(pf_unit_bytes[r] / 16);
        pf.units[c] = broadcast ? 1 : (pf.total_vecs[c] + pf.unit_vecs[c] - 1) / pf.unit_vecs[c];
    }
    return pf;
}

// The attention takes `slots` workgroups; the rest of the chip prefetches (none when few CUs are left).
int prefetch_workgroups(const AttentionPrefetch& pf, int slots)
{
    static const int forced_wgs = [] {
        const char* v = tuning_env("TERNASPMM_ATTN_PREFETCH_WGS");
        return v ? std::atoi(v) / 8 * 8 : -1;
    }();
    // With fewer than 96 CUs left the few prefetching workgroups outlast the attention (measured, 2B shape, regions of
    // 10 MB: 9 - 11 sequences -- 64 and 32 workgroups -- ran 10 - 20 % slower per step than without prefetch).
    return pf.count > 0 && slots <= 160 ? (forced_wgs >= 0 ? forced_wgs : (256 - slots) / 8 * 8) : 0;
}

}  // namespace

// ---- the entry point that allocates nothing (ternaspmm_decode_attention_static) -------------------------------
// Its split-attention scratch lives in this file-scope device array instead of a caller workspace: kStaticHeads
// arrival counters first -- at a fixed place whatever the call's size, so that the zeros every launch leaves behind
// are the zeros the next one starts from -- then kAttentionMaxSplits partial results of up to 128 + 2 floats per head.
// Every GPU the library runs on holds its own copy of the array, at its own address, until the process ends.
constexpr int kStaticHeads = 256;                                       // B * H of one call
constexpr size_t kStaticCounterBytes = kStaticHeads * sizeof(int);     // 1 KiB, a multiple of 256
constexpr size_t kStaticScratchBytes =
    kStaticCounterBytes + static_cast<size_t>(kStaticHeads) * kAttentionMaxSplits * (128 + 2) * sizeof(float);   // ~1.02 MiB
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// Device address of `scratch` on the current device (in host code the array's name is only a handle for this lookup).
// Looked up once per device; the first sight also clears the counters with a fill kernel on the caller's stream.
static unsigned char* static_scratch(hipStream_t st, int line)
{
    static std::mutex mutex;
    static unsigned char* ptr_of[64] = {};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) die("hipGetDevice", e, line);
    if (dev < 0 || dev >= 64) {
        std::fprintf(stderr, "ternaspmm_decode_attention_static: device ordinal %d is outside 0 .. 63\n", dev);
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(mutex);
    if (ptr_of[dev] == nullptr) {
        // the first call on a device clears the counters with a launch on the caller's stream: recorded into a graph
        // it would run at replay time only, and calls made before the first replay would find the array as it was
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(st, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone) {
            (void)hipGetLastError();
            std::fprintf(stderr, "ternaspmm_decode_attention_static: the first call on a device must be made outside stream "
                                 "capture (it sets the library's scratch array up); nothing was recorded\n");
            return nullptr;
        }
        unsigned char* ptr = nullptr;
        e = hipGetSymbolAddress(reinterpret_cast<void**>(&ptr), HIP_SYMBOL(scratch));
        if (e != hipSuccess || ptr == nullptr) die("hipGetSymbolAddress(scratch)", e, line);
        static_assert(kStaticCounterBytes % (256 * sizeof(uint32_t)) == 0, "fill grid");
        terna_fill_u32_kernel<<<dim3(kStaticCounterBytes / (256 * sizeof(uint32_t))), dim3(256), 0, st>>>(
            reinterpret_cast<uint32_t*>(ptr), 0u);
        e = hipGetLastError();
        if (e != hipSuccess) die("scratch clear", e, line);
        ptr_of[dev] = ptr;
    }
    return ptr_of[dev];
}

extern "C" {

void ternaspmm_rope_kv_store(const terna_bf16* qkv, const float* cos, const float* sin, const long long* pos,
                             int per_sequence, terna_bf16* q_out, terna_bf16* cache_k, terna_bf16* cache_v, int B, int T, int H,
                             int KV, int D, int S, int adjacent, terna_stream stream)
{
    if (B < 1 || T < 1 || H < 1 || KV < 1 || D < 2 || (D & 1) || S < 1) {
        std::fprintf(stderr, "ternaspmm_rope_kv_store: unsupported arguments\n");
        return;
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (adjacent)
        terna_rope_kv_store_kernel<true><<<dim3(B * T), dim3(256), 0, st>>>(qkv, cos, sin, pos, q_out, cache_k, cache_v, T, H, KV, D, S, per_sequence != 0);
    else
        terna_rope_kv_store_kernel<false><<<dim3(B * T), dim3(256), 0, st>>>(qkv, cos, sin, pos, q_out, cache_k, cache_v, T, H, KV, D, S, per_sequence != 0);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("ternaspmm_rope_kv_store", e, __LINE__);
}

long long ternaspmm_attention_workspace_bytes(int B, int H, int D)
{
    if (B < 1 || H < 1 || D < 1) return -1;
    return static_cast<long long>(attention_counter_bytes(B, H)) +
           static_cast<long long>(B) * H * kAttentionMaxSplits * (D + 2) * sizeof(float);
}

void ternaspmm_decode_attention(const terna_bf16* q, const terna_bf16* cache_k, const terna_bf16* cache_v,
                                const long long* pos, int per_sequence, terna_bf16* out, int B, int H, int KV, int D, int S,
                                float scale, void* workspace, terna_stream stream)
{
    if (!attention_args_ok("ternaspmm_decode_attention", B, H, KV, D, S)) return;
    // the kernel writes the caches only in its ROPE variant
    launch_attention<false, false>(q, const_cast<uint16_t*>(cache_k), const_cast<uint16_t*>(cache_v), nullptr, nullptr, pos,
                                   per_sequence != 0, out, B, H, KV, D, S, scale, attention_scratch_of(workspace, B, H), AttentionPrefetch{},
                                   static_cast<hipStream_t>(stream));
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("ternaspmm_decode_attention", e, __LINE__);
}

int ternaspmm_decode_attention_static(const terna_bf16* q, const terna_bf16* cache_k, const terna_bf16* cache_v,
                                      const long long* pos, int per_sequence, terna_bf16* out, int B, int H, int KV, int D, int S,
                                      float scale, terna_stream stream)
{
    if (!attention_args_ok("ternaspmm_decode_attention_static", B, H, KV, D, S)) return -1;
    if (static_cast<long>(B) * H > kStaticHeads) {
        std::fprintf(stderr,
                     "ternaspmm_decode_attention_static: B * H = %ld heads exceed the %d the library's static scratch holds; "
                     "use ternaspmm_decode_attention with a workspace\n", static_cast<long>(B) * H, kStaticHeads);
        return -1;
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    unsigned char* base = static_scratch(st, __LINE__);
    if (base == nullptr) return -1;
    const AttentionScratch sc{reinterpret_cast<int*>(base), reinterpret_cast<float*>(base + kStaticCounterBytes)};
    launch_attention<false, false>(q, const_cast<uint16_t*>(cache_k), const_cast<uint16_t*>(cache_v), nullptr, nullptr, pos,
                                   per_sequence != 0, out, B, H, KV, D, S, scale, sc, AttentionPrefetch{}, st);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("ternaspmm_decode_attention_static", e, __LINE__);
    return 0;
}

void ternaspmm_rope_decode_attention(const terna_bf16* qkv, const float* cos, const float* sin, const long long* pos,
                                     int per_sequence, terna_bf16* cache_k, terna_bf16* cache_v, terna_bf16* out, int B, int H, int KV,
                                     int D, int S, float scale, int adjacent, void* workspace, terna_stream stream)
{
    if (!attention_args_ok("ternaspmm_rope_decode_attention", B, H, KV, D, S)) return;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const AttentionScratch scratch = attention_scratch_of(workspace, B, H);
    if (adjacent) launch_attention<true, true>(qkv, cache_k, cache_v, cos, sin, pos, per_sequence != 0, out, B, H, KV, D, S, scale, scratch, AttentionPrefetch{}, st);
    else launch_attention<true, false>(qkv, cache_k, cache_v, cos, sin, pos, per_sequence != 0, out, B, H, KV, D, S, scale, scratch, AttentionPrefetch{}, st);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("ternaspmm_rope_decode_attention", e, __LINE__);
}

int ternaspmm_rope_decode_attention_stats(const terna_bf16* qkv, const float* cos, const float* sin, const long long* pos, int per_sequence,
                                          terna_bf16* cache_k, terna_bf16* cache_v, terna_bf16* out, int B, int H, int KV, int D, int S,
                                          float scale, int adjacent, const terna_bf16* norm_weight, float* stats_out, terna_stream stream)
{
    if (!attention_args_ok("ternaspmm_rope_decode_attention_stats", B, H, KV, D, S)) return -1;
    if (norm_weight == nullptr || stats_out == nullptr || H > 448) return -1;      // (448: partials per row a consumer adds up)
    hipStream_t st = static_cast<hipStream_t>(stream);
    const AttentionStats stats{norm_weight, reinterpret_cast<float2*>(stats_out)};
    // no workspace: the unsplit launch, whose workgroups hold whole output rows of their heads
    if (adjacent) launch_attention<true, true>(qkv, cache_k, cache_v, cos, sin, pos, per_sequence != 0, out, B, H, KV, D, S, scale, AttentionScratch{}, AttentionPrefetch{}, st, stats);
    else launch_attention<true, false>(qkv, cache_k, cache_v, cos, sin, pos, per_sequence != 0, out, B, H, KV, D, S, scale, AttentionScratch{}, AttentionPrefetch{}, st, stats);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("ternaspmm_rope_decode_attention_stats", e, __LINE__);
    return H;
}

void ternaspmm_rope_decode_attention_prefetch(const terna_bf16* qkv, const float* cos, const float* sin, const long long* pos,
                                              int per_sequence, terna_bf16* cache_k, terna_bf16* cache_v, terna_bf16* out, int B, int H, int KV,
                                              int D, int S, float scale, int adjacent, void* workspace,
                                              const void* const* pf_ptr, const long long* pf_bytes, const long long* pf_unit_bytes,
                                              int pf_count, terna_stream stream)
{
    if (!attention_args_ok("ternaspmm_rope_decode_attention_prefetch", B, H, KV, D, S)) return;
    AttentionPrefetch pf = prefetch_regions(pf_ptr, pf_bytes, pf_unit_bytes, pf_count);
    const int slots = attention_slots(B, H, KV);
    pf.workgroups = prefetch_workgroups(pf, slots);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const AttentionScratch scratch = attention_scratch_of(workspace, B, H);
    if (adjacent) launch_attention<true, true>(qkv, cache_k, cache_v, cos, sin, pos, per_sequence != 0, out, B, H, KV, D, S, scale, scratch, pf, st);
    else launch_attention<true, false>(qkv, cache_k, cache_v, cos, sin, pos, per_sequence != 0, out, B, H, KV, D, S, scale, scratch, pf, st);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("ternaspmm_rope_decode_attention_prefetch", e, __LINE__);
}

long long ternaspmm_attention_partial_bytes(int B, int H, int D)
{
    if (B < 1 || H < 1 || D < 1) return -1;
    return static_cast<long long>(sizeof(float)) *
           (static_cast<long long>(attention_stat_floats(static_cast<size_t>(B) * H)) + static_cast<long long>(B) * H * kAttentionMaxSplits * D);
}

int ternaspmm_attention_partial_splits(int B, int H, int S)
{
    if (B < 1 || H < 1 || S < 1) return -1;
    // The launch is bound by what ONE CU streams, so a split should not get more than about 512 slots -- but the consumer
    // of the partial results reads splits x the bytes of a merged row (measured on the 2B shapes, one sequence: four splits
    // cost the O projection 0.9 us, eight 1.7 us): four splits up to 1024 slots, eight beyond, fewer when the
    // (sequence, head, split) workgroups would not fit the chip or a split would get less than two tiles.
    // Long caches of several sequences (more heads than the chip has CUs): an unsplit workgroup walks up to S slots alone
    // while a split costs a merge pass, so split there as well, up to about four workgroups per CU (measured, 8 sequences
    // of the 2B shape at slot 1500 of 2048: unsplit 25.5 us, four splits 18.2 us + 2.2 us for the merge launch).
    const int want = S > 1024 ? kAttentionMaxSplits : 4;
    const long fill = S > 1024 ? 1024 : 256;
    int sp = 1;
    while (sp < want && static_cast<long>(B) * H * sp * 2 <= fill && 32 * sp * 2 <= S) sp *= 2;
    return sp;
}

int ternaspmm_attention_partial_splits_kv(int B, int H, int KV, int S)
{
    if (B < 1 || H < 1 || KV < 1 || H % KV != 0 || S < 1) return -1;
    const int gq = H / KV;
    // several sequences whose kv groups share a workgroup (2 or 4 heads per kv head): the grid is B * KV * splits
    // workgroups, and a cache of more than 512 slots already pays for the split (the unsplit launch requests 512 slots of
    // keys up front and walks the rest in dependent round trips; measured, 8 sequences of the 2B shape, 728 slots:
    // 1.316 ms per step unsplit, 1.235 with four splits; 428 slots: 1.204 against 1.219)
    if (B >= 2 && (gq == 2 || gq == 4) && S > 512 && S <= 1024) {
        int sp = 1;
        while (sp < 4 && static_cast<long>(B) * KV * sp * 2 <= 256) sp *= 2;
        return sp;
    }
    return ternaspmm_attention_partial_splits(B, H, S);
}

void ternaspmm_rope_decode_attention_partial(const terna_bf16* qkv, const float* cos, const float* sin, const long long* pos,
                                             int per_sequence, terna_bf16* cache_k, terna_bf16* cache_v, float* partial, int splits,
                                             int B, int H, int KV, int D, int S, float scale, int adjacent,
                                             const void* const* pf_ptr, const long long* pf_bytes, const long long* pf_unit_bytes,
                                             int pf_count, terna_stream stream)
{
    if (!attention_args_ok("ternaspmm_rope_decode_attention_partial", B, H, KV, D, S)) return;
    if (splits < 1 || splits > kAttentionMaxSplits || (splits & (splits - 1)) || partial == nullptr ||
        static_cast<long>(B) * H * splits > 65536) {
        std::fprintf(stderr, "ternaspmm_rope_decode_attention_partial: unsupported splits=%d (1, 2, 4 or 8) or no partial buffer\n", splits);
        return;
    }
    AttentionPrefetch pf = prefetch_regions(pf_ptr, pf_bytes, pf_unit_bytes, pf_count);
    hipStream_t st = static_cast<hipStream_t>(stream);
    // several sequences: the heads of a kv group share a workgroup (TERNASPMM_ATTN_GROUPED=0|1 forces either form)
    static const int forced_grouped = [] {
        const char* v = tuning_env("TERNASPMM_ATTN_GROUPED");
        return v ? std::atoi(v) : -1;
    }();
    if (forced_grouped >= 0 ? forced_grouped != 0 : B >= 2) {
        bool done;
        if (D == 128) done = adjacent ? launch_attention_grouped<128, true>(qkv, cache_k, cache_v, cos, sin, pos, per_sequence != 0, partial, splits, B, H, KV, S, scale, pf, st)
                                      : launch_attention_grouped<128, false>(qkv, cache_k, cache_v, cos, sin, pos, per_sequence != 0, partial, splits, B, H, KV, S, scale, pf, st);
        else done = adjacent ? launch_attention_grouped<64, true>(qkv, cache_k, cache_v, cos, sin, pos, per_sequence != 0, partial, splits, B, H, KV, S, scale, pf, st)
                             : launch_attention_grouped<64, false>(qkv, cache_k, cache_v, cos, sin, pos, per_sequence != 0, partial, splits, B, H, KV, S, scale, pf, st);
        if (done) {
            const hipError_t e = hipGetLastError();
            if (e != hipSuccess) die("ternaspmm_rope_decode_attention_partial", e, __LINE__);
            return;
        }
    }
    const bool grouped = attention_groups_on(H, KV);
    const int slots = grouped ? 8 * (H / KV) * ((B * KV * splits + 7) / 8) : B * H * splits;
    pf.workgroups = prefetch_workgroups(pf, slots);
#define TERNA_DEFER(DIM, ADJ) \
    launch_attention_deferred<DIM, ADJ>(qkv, cache_k, cache_v, cos, sin, pos, per_sequence != 0, partial, splits, B, H, KV, S, scale, pf, st)
    if (D == 128) {
        if (adjacent) TERNA_DEFER(128, true);
        else TERNA_DEFER(128, false);
    } else {
        if (adjacent) TERNA_DEFER(64, true);
        else TERNA_DEFER(64, false);
    }
#undef TERNA_DEFER
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("ternaspmm_rope_decode_attention_partial", e, __LINE__);
}

void ternaspmm_attention_merge(const float* partial, int splits, terna_bf16* out, int B, int H, int D, terna_stream stream)
{
    if (B < 1 || H < 1 || (D != 64 && D != 128) || splits < 1 || splits > kAttentionMaxSplits) {
        std::fprintf(stderr, "ternaspmm_attention_merge: unsupported arguments (H=%d D=%d splits=%d)\n", H, D, splits);
        return;
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (D == 128) terna_attention_merge_kernel<128><<<dim3(B * H), dim3(128), 0, st>>>(partial, out, B * H, splits);
    else terna_attention_merge_kernel<64><<<dim3(B * H), dim3(64), 0, st>>>(partial, out, B * H, splits);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("ternaspmm_attention_merge", e, __LINE__);
}

int ternaspmm_attention_merge_rmsnorm_quant(const float* partial, int splits, const terna_bf16* norm_weight, float eps, terna_bf16* o_out,
                                            int8_t* xq_out, terna_bf16* s_out, int B, int H, int D, terna_stream stream)
{
    const long long K = static_cast<long long>(H) * D;
    if (B < 1 || H < 1 || (D != 64 && D != 128) || (splits != 1 && splits != 2 && splits != 4 && splits != 8) || K > 2048 * 2 ||
        partial == nullptr || norm_weight == nullptr || xq_out == nullptr || s_out == nullptr)
        return -1;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int qmode = quant_mode();
#define TERNA_MERGE_NQ(DIM, SP)                                                                                           \
    do {                                                                                                                  \
        if (K <= 2048)                                                                                                    \
            terna_attention_merge_norm_quant_kernel<DIM, SP, 1><<<dim3(B), dim3(kNormThreads), 0, st>>>(                   \
                partial, norm_weight, H, B * H, eps, o_out, nullptr, xq_out, s_out, qmode);                               \
        else                                                                                                              \
            terna_attention_merge_norm_quant_kernel<DIM, SP, 2><<<dim3(B), dim3(kNormThreads), 0, st>>>(                   \
                partial, norm_weight, H, B * H, eps, o_out, nullptr, xq_out, s_out, qmode);                               \
    } while (0)
#define TERNA_MERGE_NQ_D(DIM)                                                                                             \
    do {                                                                                                                  \
        if (splits == 1) TERNA_MERGE_NQ(DIM, 1);                                                                          \
        else if (splits == 2) TERNA_MERGE_NQ(DIM, 2);                                                                     \
        else if (splits == 4) TERNA_MERGE_NQ(DIM, 4);                                                                     \
        else TERNA_MERGE_NQ(DIM, 8);                                                                                      \
    } while (0)
    if (D == 128) TERNA_MERGE_NQ_D(128);
    else TERNA_MERGE_NQ_D(64);
#undef TERNA_MERGE_NQ_D
#undef TERNA_MERGE_NQ
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("ternaspmm_attention_merge_rmsnorm_quant", e, __LINE__);
    return 0;
}

}  // extern "C"
