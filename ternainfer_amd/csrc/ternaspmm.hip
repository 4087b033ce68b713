// libternaspmm.so: the extern "C" boundary of the TernaSpMM path on MI355X (gfx950) -- the reference's eight
// symbols, the bf16-activation family, the load-time repack and the host encoder.  Declarations and the reference
// interface each symbol stands for: include/ternaspmm.h.  The kernels are instantiated in launch_*.hip; the glue
// kernels of a decode step have their entry points in abi_fused.hip, abi_attention.hip and abi_head.hip.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <mutex>
#include <unordered_map>

#include "../../include/ternaspmm.h"
#include "format_host.h"
#include "host_util.h"
#include "launchers.h"
#include "repack_cache.h"

using namespace terna;

namespace terna {
namespace {
std::atomic<int> g_quant_mode{-1};     // -1: not decided yet (environment)
}
int quant_mode()
{
    int m = g_quant_mode.load(std::memory_order_relaxed);
    if (m < 0) {
        const char* v = std::getenv("TERNASPMM_QUANT_MODE");
        m = v != nullptr ? std::atoi(v) : 0;
        if (m < QUANT_ROUNDED || m > QUANT_EAGER) m = QUANT_ROUNDED;
        g_quant_mode.store(m, std::memory_order_relaxed);
    }
    return m;
}
}  // namespace terna

namespace {

enum Route { ROUTE_AUTO, ROUTE_DECODE, ROUTE_PREFILL };

// Which P2 kernel runs a call of M rows when the caller leaves the choice to the library: the small-M dot-product
// kernel or the MFMA-tiled one.  (The epilogue arithmetic of the int8 family follows the reference's M <= 64 rule
// whatever kernel computes the sums.)
// By measurement on the four BitNet-2B matrices at M = 16 .. 256 (us per launch, P2 layout, small-M kernel / MFMA-tiled
// kernel with split-K scratch): the small-M kernel's time grows with every 16 rows, the MFMA-tiled one is flat but
// pays a fill / drain of 10 us or more.
//   gate+up (864 bands)  bf16 M=32  8.7 / 17.4   M=48 23.1 / 18.1      int8 M=32  6.5 / 10.7   M=48 12.4 / 11.6
//   QKV (240 bands)      bf16 M=64  7.9 / 11.8   M=96 13.2 / 12.7      int8 M=128 8.5 / 10.9   M=192 11.1 / 10.9
//   O (160 bands)        bf16 M=64  7.6 / 11.4   M=96 12.5 / 12.1      int8 M=192 8.3 / 10.6   M=256 10.6 / 10.8
//   down (K = 6912)      bf16 M=64 14.2 / 14.4   M=96 24.6 / 15.5      int8 M=64  9.2 / 12.2   M=96 14.2 / 12.8
// Without scratch the MFMA-tiled kernel cannot split K and walks all of it in every workgroup (QKV bf16 16-17 us flat,
// down 38-44 us), which moves the cut up.
bool packed_small_kernel(int M, int N, int K, bool int8, bool has_scratch)
{
    if (N / 16 > 512) return M <= 32;
    if (!has_scratch) return M <= (K > 4096 ? 256 : 128);
    if (int8 && K <= 4096) return M <= (N / 16 <= 160 ? 192 : 128);
    return M <= 64;
}

// Scratch for split-K is worth counting on when it holds two planes of partial sums or more.
bool scratch_for_split(const void* scratch, size_t bytes, int M, int N)
{
    return scratch != nullptr && (reinterpret_cast<uintptr_t>(scratch) & 15) == 0 && bytes >= static_cast<size_t>(8) * M * N;
}

// What a call on reference-format pointers does, decided on the host before anything is enqueued (also what
// ternaspmm_plan_reference_call reports).  The caller's workspace is used within the bytes the reference itself would
// write there and never beyond (reference_workspace_bytes): with a cached P2 copy all of them may hold split-K planes;
// without one a large-M call puts its per-call P2 transcode (N*K/4 bytes) first and the planes behind it.
enum CallKernel {
    CALL_REF_SMALL = 0,        // small-M kernel on the reference format
    CALL_REF_FUSED_LARGE = 1,  // MFMA-tiled kernel that decodes the reference format on the fly (no workspace)
    CALL_TRANSCODE_LARGE = 2,  // transcode into the workspace, then the MFMA-tiled P2 kernel
    CALL_P2_SMALL = 3,         // small-M kernel on the cached P2 copy
    CALL_P2_LARGE = 4,         // MFMA-tiled kernel on the cached P2 copy
};
struct CallPlan {
    CallKernel kernel;
    size_t p2_bytes;           // bytes of the workspace that receive transcoded weights (CALL_TRANSCODE_LARGE)
    size_t scratch_offset;     // where split-K planes may start
    size_t scratch_bytes;      // ... and how many bytes they may take
};
CallPlan plan_call(bool int8, Route route, int M, int N, int K, int split_k, const void* workspace, bool cached)
{
    const bool ref_prefill_path = route == ROUTE_PREFILL || (route == ROUTE_AUTO && M > 64);
    const bool aligned = workspace != nullptr && (reinterpret_cast<uintptr_t>(workspace) & 15) == 0;
    const size_t avail = aligned ? reference_workspace_bytes(ref_prefill_path, M, N, K, split_k) : 0;
    CallPlan plan{CALL_REF_SMALL, 0, 0, 0};
    if (cached) {
        bool small;
        if (int8) small = packed_small_kernel(M, N, K, true, scratch_for_split(workspace, avail, M, N));   // integer sums: any kernel, same bits
        else small = route == ROUTE_DECODE || (route == ROUTE_AUTO && packed_small_kernel(M, N, K, false, scratch_for_split(workspace, avail, M, N)));
        plan.kernel = small ? CALL_P2_SMALL : CALL_P2_LARGE;
        if (!small) plan.scratch_bytes = avail;
        return plan;
    }
    const bool small = int8 ? M <= 64 : (route == ROUTE_DECODE || (route == ROUTE_AUTO && M <= 64));
    if (small) return plan;
    const size_t p2_bytes = (static_cast<size_t>(N) * K / 4 + 255) & ~static_cast<size_t>(255);
    if (aligned && avail >= p2_bytes) {
        plan.kernel = CALL_TRANSCODE_LARGE;
        plan.p2_bytes = static_cast<size_t>(N) * K / 4;
        plan.scratch_offset = p2_bytes;
        plan.scratch_bytes = avail - p2_bytes;
    } else {
        plan.kernel = CALL_REF_FUSED_LARGE;
    }
    return plan;
}

// ---- repack cache behind the reference-format entry points (on unless TERNASPMM_REPACK_CACHE=0).
// An unmodified call site keeps passing the four format tensors; the first call that sees a weight (identified by
// device, pointers and shape) allocates N*K/4 bytes, repacks into them, records a fingerprint of the source tensors
// and waits; every later call runs the P2 kernels.  A first sight during stream capture (where nothing may be
// allocated) is served by the reference-format kernels instead.  The bookkeeping -- least recently used copies go
// when a byte limit is reached, copies a captured graph may hold are never released behind its back -- is
// repack_cache.h.
// The pointers alone are not trusted: every launch on a cached copy recomputes the fingerprint from the tensors the
// caller passes (an extra workgroup of the small-M launch, a one-wave launch next to a large-M one) and, when it differs
// from the recorded one -- weights freed or rewritten, other data at the same addresses -- reports the copy's id in
// host-visible memory.  A launch cannot be taken back: the ONE launch that found the mismatch has used the old copy.
// The next call into the library drops that copy, says so, and goes on (the weight gets a fresh copy at its next
// sight); with TERNASPMM_REPACK_CACHE_STRICT=1 it ends the process instead, as every error of this library does
// (kernels/TernaSpMM.cu:15-22).  ternaspmm_repack_cache_clear() after freeing or reloading weights avoids the window.
struct RepackLaunch {
    const uint32_t* packed;           // N*K/4 bytes of P2, then (256-byte aligned) the recorded fingerprint
    RepackGuard guard;                // what the launches on this copy check (passed to them by value)
};
constexpr uint32_t kStaleSlots = 1023;     // host-visible words 1 .. 1023: id of a stale copy at [1 + id % 1023]; word 0: any
void release_device(void* p) { (void)hipFree(p); }     // waits for the launches that still read it
std::mutex g_repack_mutex;
RepackCachePolicy<RepackLaunch> g_repack_cache(release_device, ~static_cast<size_t>(0));
bool g_repack_limit_set = false;      // the default limit (an eighth of the device's memory) is fixed at the first copy
uint32_t* g_repack_stale = nullptr;   // pinned host memory, mapped into every device
int g_repack_on = -1;                 // -1: not decided yet (environment), 0 / 1
int g_repack_strict = -1;
uint64_t g_repack_warned = 0;

bool repack_cache_on()
{
    if (g_repack_on < 0) {
        const char* v = std::getenv("TERNASPMM_REPACK_CACHE");
        g_repack_on = (v == nullptr || std::atoi(v) != 0) ? 1 : 0;
    }
    return g_repack_on == 1;
}

// Copies the device-side checks have reported stale since the last look: dropped here (not during stream capture:
// releasing memory waits for the device).
void repack_cache_collect_stale(int line)
{
    volatile uint32_t* flags = g_repack_stale;
    if (flags == nullptr || flags[0] == 0) return;
    flags[0] = 0;                                        // before the scan: a report that arrives meanwhile raises it again
    for (uint32_t slot = 1; slot <= kStaleSlots; ++slot) {
        const uint32_t id = flags[slot];
        if (id == 0) continue;
        flags[slot] = 0;
        if (!g_repack_cache.retire(id)) continue;
        if (g_repack_strict < 0) {
            const char* v = std::getenv("TERNASPMM_REPACK_CACHE_STRICT");
            g_repack_strict = (v != nullptr && std::atoi(v) != 0) ? 1 : 0;
        }
        if (g_repack_strict == 1 || g_repack_warned++ < 8) {
            std::printf("TernaSpMM %s (line %d): a cached repacked weight no longer matched the tensors it was made from -- "
                        "weights were freed or rewritten without ternaspmm_repack_cache_clear().  The copy was dropped; the one "
                        "launch that found the mismatch had already used it and its output is invalid.\n",
                        g_repack_strict == 1 ? "Error" : "Warning", line);
            std::fflush(stdout);
        }
        if (g_repack_strict == 1) std::exit(EXIT_FAILURE);
    }
}

// The cached P2 copy of a weight (made on first sight) and the guard its launches carry; false: no copy, the
// reference-format kernels serve the call.
bool cached_packed(const Weights& w, int N, int K, hipStream_t st, RepackLaunch* launch, int line)
{
    std::lock_guard<std::mutex> lock(g_repack_mutex);
    if (!repack_cache_on()) return false;
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &capturing) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    const bool capture = capturing != hipStreamCaptureStatusNone;
    if (!capture) repack_cache_collect_stale(line);
    RepackKey key{0, w.bitmap, w.sign_words, w.tile_off, N, K};
    if (hipGetDevice(&key.device) != hipSuccess) return false;
    if (auto* slot = g_repack_cache.find(key)) {
        if (capture) slot->pinned = true;                 // the graph being captured will hold this copy's address
        *launch = slot->payload;                          // (a copy: the launch takes the guard by value)
        return true;
    }
    if (capture) return false;
    if (g_repack_stale == nullptr) {
        void* flag = nullptr;
        if (hipHostMalloc(&flag, (kStaleSlots + 1) * sizeof(uint32_t), hipHostMallocMapped | hipHostMallocPortable) != hipSuccess) {
            (void)hipGetLastError();
            return false;
        }
        g_repack_stale = static_cast<uint32_t*>(flag);
        for (uint32_t i = 0; i <= kStaleSlots; ++i) g_repack_stale[i] = 0;
    }
    if (!g_repack_limit_set) {
        g_repack_limit_set = true;
        size_t limit = 0;
        if (const char* v = std::getenv("TERNASPMM_REPACK_CACHE_LIMIT_MB")) {
            limit = static_cast<size_t>(std::strtoull(v, nullptr, 10)) << 20;
        } else {
            size_t free_b = 0, total_b = 0;
            if (hipMemGetInfo(&free_b, &total_b) == hipSuccess) limit = total_b / 8;
            else (void)hipGetLastError();
        }
        if (limit > 0) g_repack_cache.set_limit(limit);
    }
    const size_t p2_bytes = (static_cast<size_t>(N) * K / 4 + 255) & ~static_cast<size_t>(255);
    if (!g_repack_cache.make_room(p2_bytes + 256)) return false;
    void* buf = nullptr;
    if (hipMalloc(&buf, p2_bytes + 256) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    unsigned long long* expect = reinterpret_cast<unsigned long long*>(static_cast<char*>(buf) + p2_bytes);
    RepackGuard g{w.bitmap, w.tile_off, w.sign_words, expect, g_repack_stale, N / 64 * (K / 64), 0, g_repack_cache.next_id()};
    // the length of the sign stream decides where the check samples it
    hipError_t e = hipMemcpyAsync(&g.total_bits, w.tile_off + g.tiles, sizeof(int), hipMemcpyDeviceToHost, st);
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    if (e != hipSuccess) die("repack cache", e, __LINE__);
    launch_repack(w, static_cast<uint32_t*>(buf), N, K, st);
    launch_repack_fingerprint(g, expect, st);
    e = hipStreamSynchronize(st);                        // later calls may come on other streams
    if (e != hipSuccess) die("repack cache", e, __LINE__);
    *launch = RepackLaunch{static_cast<const uint32_t*>(buf), g};
    g_repack_cache.insert(key, buf, p2_bytes + 256, *launch);
    return true;
}

template <typename Act>
void run_planned(const CallPlan& plan, const Act* x, const Weights& w, const RepackLaunch& cached, uint16_t* out,
                 const Epilogue& ep, int M, int N, int K, void* workspace, hipStream_t st)
{
    char* scratch = plan.scratch_bytes ? static_cast<char*>(workspace) + plan.scratch_offset : nullptr;
    switch (plan.kernel) {
    case CALL_P2_SMALL:
        launch_decode_packed<Act>(x, cached.packed, out, ep, M, N, K, st, &cached.guard);
        break;
    case CALL_P2_LARGE:
        if (!launch_prefill_packed<Act>(x, cached.packed, out, ep, M, N, K, scratch, plan.scratch_bytes, st, &cached.guard))
            launch_repack_guard(&cached.guard, st);
        break;
    case CALL_REF_SMALL:
        launch_decode<Act>(x, w, out, ep, M, N, K, st);
        break;
    case CALL_TRANSCODE_LARGE:
        launch_repack(w, static_cast<uint32_t*>(workspace), N, K, st);
        launch_prefill_packed<Act>(x, static_cast<const uint32_t*>(workspace), out, ep, M, N, K, scratch, plan.scratch_bytes, st);
        break;
    case CALL_REF_FUSED_LARGE:
        launch_prefill<Act>(x, w, out, ep, M, N, K, st);
        break;
    }
}

void run_i8(Route route, int8_t* x, uint64_t* bitmap, int* tile_off, uint16_t* median_off, uint32_t* sign_words,
            uint16_t* out, uint16_t* s, uint16_t* ws, int ws_num, int M, int N, int K, int split_k, void* workspace,
            hipStream_t st, int line)
{
    if (!shape_ok(M, N, K) || !groups_ok(ws_num) || !i8_depth_ok(K)) return;
    // The reference picks its path, and with it the epilogue arithmetic, by M <= 64
    // (kernels/TernaSpMM.cu:34); the forced entry points pin one of the two.
    const bool decode_rule = route == ROUTE_DECODE || (route == ROUTE_AUTO && M <= 64);
    const Epilogue ep{s, ws, nullptr, ws_num, decode_rule ? EP_I8_DECODE : EP_I8_PREFILL};
    const Weights w{bitmap, tile_off, median_off, sign_words};
    RepackLaunch cached{};
    const bool have = cached_packed(w, N, K, st, &cached, line);
    run_planned<int8_t>(plan_call(true, route, M, N, K, split_k, workspace, have), x, w, cached, out, ep, M, N, K, workspace, st);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("bitlinear_TernaSpMM", e, line);
}

void run_bf16(Route route, const uint16_t* x, const uint64_t* bitmap, const int* tile_off,
              const uint16_t* median_off, const uint32_t* sign_words, uint16_t* out, const float* scale,
              int ws_num, int M, int N, int K, int split_k, void* workspace, hipStream_t st, int line)
{
    if (!shape_ok(M, N, K) || !groups_ok(ws_num)) return;
    const Epilogue ep{nullptr, nullptr, scale, ws_num, EP_BF16};
    const Weights w{bitmap, tile_off, median_off, sign_words};
    RepackLaunch cached{};
    const bool have = cached_packed(w, N, K, st, &cached, line);
    run_planned<uint16_t>(plan_call(false, route, M, N, K, split_k, workspace, have), x, w, cached, out, ep, M, N, K, workspace, st);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("bitlinear_TernaSpMM_bf16", e, line);
}

__global__ void sleep_kernel(long long ticks)
{
    // wall_clock64 counts at a fixed 100 MHz; every lane leaves once the span has passed.
    const long long start = wall_clock64();
    while (wall_clock64() - start < ticks) __builtin_amdgcn_s_sleep(8);
}

}  // namespace

extern "C" {

void checkLastCudaError(int line)
{
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("checkLastCudaError", e, line);
}

void bitlinear_TernaSpMM(int8_t* x, uint64_t* bitmap, int* tile_off, uint16_t* median_off, uint32_t* sign_words,
                         terna_bf16* out, terna_bf16* s, terna_bf16* ws, int ws_num, int M, int N, int K,
                         int SPLIT_K, int32_t* workspace, terna_stream stream)
{
    run_i8(ROUTE_AUTO, x, bitmap, tile_off, median_off, sign_words, out, s, ws, ws_num, M, N, K, SPLIT_K, workspace,
           static_cast<hipStream_t>(stream), __LINE__);
}

void bitlinear_TernaSpMM_decode(int8_t* x, uint64_t* bitmap, int* tile_off, uint16_t* median_off,
                                uint32_t* sign_words, terna_bf16* out, terna_bf16* s, terna_bf16* ws, int ws_num,
                                int M, int N, int K, int SPLIT_K, int32_t* workspace, terna_stream stream)
{
    run_i8(ROUTE_DECODE, x, bitmap, tile_off, median_off, sign_words, out, s, ws, ws_num, M, N, K, SPLIT_K, workspace,
           static_cast<hipStream_t>(stream), __LINE__);
}

void bitlinear_TernaSpMM_prefill(int8_t* x, uint64_t* bitmap, int* tile_off, uint16_t* median_off,
                                 uint32_t* sign_words, terna_bf16* out, terna_bf16* s, terna_bf16* ws, int ws_num,
                                 int M, int N, int K, int SPLIT_K, int32_t* workspace, terna_stream stream)
{
    run_i8(ROUTE_PREFILL, x, bitmap, tile_off, median_off, sign_words, out, s, ws, ws_num, M, N, K, SPLIT_K, workspace,
           static_cast<hipStream_t>(stream), __LINE__);
}

void bitlinear_TernaSpMM_benchmark(int mode, int warmup_iters, int bench_iters, int8_t* x, uint64_t* bitmap,
                                   int* tile_off, uint16_t* median_off, uint32_t* sign_words, terna_bf16* out,
                                   terna_bf16* s, terna_bf16* ws, int ws_num, int M, int N, int K, int SPLIT_K,
                                   int32_t* workspace, terna_stream stream)
{
    // mode 0 = auto, 1 = prefill, 2 = decode (kernels/TernaSpMM.cu:165-173)
    const Route route = mode == 1 ? ROUTE_PREFILL : (mode == 2 ? ROUTE_DECODE : ROUTE_AUTO);
    hipStream_t st = static_cast<hipStream_t>(stream);
    for (int it = 0; it < warmup_iters; ++it)
        run_i8(route, x, bitmap, tile_off, median_off, sign_words, out, s, ws, ws_num, M, N, K, SPLIT_K, workspace, st, __LINE__);
    hipError_t e = hipStreamSynchronize(st);
    if (e != hipSuccess) die("benchmark warm-up", e, __LINE__);

    hipEvent_t start, stop;
    if ((e = hipEventCreate(&start)) != hipSuccess) die("hipEventCreate", e, __LINE__);
    if ((e = hipEventCreate(&stop)) != hipSuccess) die("hipEventCreate", e, __LINE__);
    (void)hipEventRecord(start, st);
    for (int it = 0; it < bench_iters; ++it)
        run_i8(route, x, bitmap, tile_off, median_off, sign_words, out, s, ws, ws_num, M, N, K, SPLIT_K, workspace, st, __LINE__);
    (void)hipEventRecord(stop, st);
    if ((e = hipEventSynchronize(stop)) != hipSuccess) die("benchmark loop", e, __LINE__);
    float total_ms = 0.0f;
    (void)hipEventElapsedTime(&total_ms, start, stop);
    const float avg_us = bench_iters > 0 ? total_ms * 1000.0f / bench_iters : 0.0f;
    std::printf("Shape(M=%d, N=%d, K=%d): %.2f us (avg over %d iters, warmup=%d)\n", M, N, K, avg_us, bench_iters,
                warmup_iters);
    std::fflush(stdout);
    (void)hipEventDestroy(start);
    (void)hipEventDestroy(stop);
}

void reorder_WT_h(terna_bf16* W, terna_bf16* W_reordered, int N, int K) { reorder_bf16(W, W_reordered, N, K); }

int convert_reorderd(terna_bf16* A_h, int N, int K, int tile_N, int warp_subtile_N, int subtile_N, int tile_K,
                     int warp_subtile_K, int subtile_K, uint64_t** bitmap, int** tile_off, uint16_t** median_off,
                     uint32_t** sign_words, int* max_nnz_count)
{
    if (tile_N != 64 || warp_subtile_N != 16 || subtile_N != 8 || tile_K != 64 || warp_subtile_K != 64 ||
        subtile_K != 8)
        return -1;
    int64_t n_bitmap, n_off, n_med, cap_words;
    if (encode_sizes(N, K, &n_bitmap, &n_off, &n_med, &cap_words) != 0) return -1;
    *sign_words = static_cast<uint32_t*>(std::malloc(static_cast<size_t>(cap_words) * 4 + 4));
    *tile_off = static_cast<int*>(std::malloc(static_cast<size_t>(n_off) * sizeof(int)));
    // three trailing entries of slack: the reference's consumer reads that far past the end
    *median_off = static_cast<uint16_t*>(std::calloc(static_cast<size_t>(n_med) + 4, sizeof(uint16_t)));
    *bitmap = nullptr;
    // pinned, as the reference allocates it (kernels/TernaSpMM.cu:317); callers release it with hipHostFree
    if (hipHostMalloc(reinterpret_cast<void**>(bitmap), static_cast<size_t>(n_bitmap) * 8, hipHostMallocDefault) !=
        hipSuccess) {
        (void)hipGetLastError();
        *bitmap = nullptr;
    }
    if (!*sign_words || !*tile_off || !*median_off || !*bitmap) return -1;
    int max_nnz = 0;
    const int64_t words = encode_reordered_bf16(A_h, N, K, *bitmap, *tile_off, *median_off, *sign_words, &max_nnz);
    if (words < 0) return -1;
    if (max_nnz_count) *max_nnz_count = max_nnz;
    uint32_t* shrunk = static_cast<uint32_t*>(std::realloc(*sign_words, static_cast<size_t>(words) * 4 + 4));
    if (shrunk) *sign_words = shrunk;
    return (N / 64) * (K / 64);
}

void gpu_sleep(double us, terna_stream stream)
{
    const long long ticks = us > 0 ? static_cast<long long>(us * 100.0) : 0;
    sleep_kernel<<<1, 64, 0, static_cast<hipStream_t>(stream)>>>(ticks);
}

void bitlinear_TernaSpMM_bf16(const terna_bf16* x, const uint64_t* bitmap, const int* tile_off,
                              const uint16_t* median_off, const uint32_t* sign_words, terna_bf16* out,
                              const float* scale, int ws_num, int M, int N, int K, int SPLIT_K,
                              void* workspace, terna_stream stream)
{
    run_bf16(ROUTE_AUTO, x, bitmap, tile_off, median_off, sign_words, out, scale, ws_num, M, N, K, SPLIT_K, workspace,
             static_cast<hipStream_t>(stream), __LINE__);
}

void bitlinear_TernaSpMM_bf16_decode(const terna_bf16* x, const uint64_t* bitmap, const int* tile_off,
                                     const uint16_t* median_off, const uint32_t* sign_words, terna_bf16* out,
                                     const float* scale, int ws_num, int M, int N, int K, int SPLIT_K,
                                     void* workspace, terna_stream stream)
{
    run_bf16(ROUTE_DECODE, x, bitmap, tile_off, median_off, sign_words, out, scale, ws_num, M, N, K, SPLIT_K, workspace,
             static_cast<hipStream_t>(stream), __LINE__);
}

void bitlinear_TernaSpMM_bf16_prefill(const terna_bf16* x, const uint64_t* bitmap, const int* tile_off,
                                      const uint16_t* median_off, const uint32_t* sign_words, terna_bf16* out,
                                      const float* scale, int ws_num, int M, int N, int K, int SPLIT_K,
                                      void* workspace, terna_stream stream)
{
    run_bf16(ROUTE_PREFILL, x, bitmap, tile_off, median_off, sign_words, out, scale, ws_num, M, N, K, SPLIT_K, workspace,
             static_cast<hipStream_t>(stream), __LINE__);
}

int ternaspmm_encode_sizes(int N, int K, int64_t* bitmap_len, int64_t* tile_off_len, int64_t* median_len,
                           int64_t* sign_words_capacity)
{
    return encode_sizes(N, K, bitmap_len, tile_off_len, median_len, sign_words_capacity);
}

int64_t ternaspmm_encode_i8(const int8_t* W, int N, int K, uint64_t* bitmap, int* tile_off, uint16_t* median_off,
                            uint32_t* sign_words)
{
    return encode_i8(W, N, K, bitmap, tile_off, median_off, sign_words);
}

void ternaspmm_decompress_bf16(const uint64_t* bitmap, const int* tile_off, const uint16_t* median_off,
                               const uint32_t* sign_words, terna_bf16* W_dense, int N, int K, terna_stream stream)
{
    if (!shape_ok(1, N, K)) return;
    launch_decompress(Weights{bitmap, tile_off, median_off, sign_words}, W_dense, N, K, static_cast<hipStream_t>(stream));
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("ternaspmm_decompress_bf16", e, __LINE__);
}

int64_t ternaspmm_packed_bytes(int N, int K)
{
    if (N < 64 || K < 64 || (N % 64) || (K % 64)) return -1;
    return static_cast<int64_t>(N) * K / 4;
}

void ternaspmm_repack(const uint64_t* bitmap, const int* tile_off, const uint16_t* median_off,
                      const uint32_t* sign_words, void* packed, int N, int K, terna_stream stream)
{
    if (!shape_ok(1, N, K)) return;
    launch_repack(Weights{bitmap, tile_off, median_off, sign_words}, static_cast<uint32_t*>(packed), N, K,
                  static_cast<hipStream_t>(stream));
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("ternaspmm_repack", e, __LINE__);
}

void bitlinear_TernaSpMM_bf16_packed_ws(const terna_bf16* x, const void* packed, terna_bf16* out, const float* scale,
                                        int ws_num, int M, int N, int K, int route, void* workspace,
                                        long long workspace_bytes, terna_stream stream)
{
    if (!shape_ok(M, N, K) || !groups_ok(ws_num)) return;
    const Epilogue ep{nullptr, nullptr, scale, ws_num, EP_BF16};
    const uint32_t* p = static_cast<const uint32_t*>(packed);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool small = route == 2 || (route != 1 && packed_small_kernel(M, N, K, false, workspace != nullptr && workspace_bytes > 0));
    if (small) launch_decode_packed<uint16_t>(x, p, out, ep, M, N, K, st);
    else launch_prefill_packed<uint16_t>(x, p, out, ep, M, N, K, workspace, workspace_bytes > 0 ? static_cast<size_t>(workspace_bytes) : 0, st);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("bitlinear_TernaSpMM_bf16_packed", e, __LINE__);
}

void bitlinear_TernaSpMM_bf16_packed(const terna_bf16* x, const void* packed, terna_bf16* out, const float* scale,
                                     int ws_num, int M, int N, int K, int route, terna_stream stream)
{
    bitlinear_TernaSpMM_bf16_packed_ws(x, packed, out, scale, ws_num, M, N, K, route, nullptr, 0, stream);
}

void bitlinear_TernaSpMM_packed_ws(const int8_t* x, const void* packed, terna_bf16* out, const terna_bf16* s,
                                   const terna_bf16* ws, int ws_num, int M, int N, int K, int route, void* workspace,
                                   long long workspace_bytes, terna_stream stream)
{
    if (!shape_ok(M, N, K) || !groups_ok(ws_num) || !i8_depth_ok(K)) return;
    const int rule = route & 3, kernel = route & 12;
    const bool decode_rule = rule == 2 || (rule != 1 && M <= 64);
    const Epilogue ep{s, ws, nullptr, ws_num, decode_rule ? EP_I8_DECODE : EP_I8_PREFILL};
    const uint32_t* p = static_cast<const uint32_t*>(packed);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool small = kernel == 4 || (kernel != 8 && packed_small_kernel(M, N, K, true, workspace != nullptr && workspace_bytes > 0));
    if (small) launch_decode_packed<int8_t>(x, p, out, ep, M, N, K, st);
    else launch_prefill_packed<int8_t>(x, p, out, ep, M, N, K, workspace, workspace_bytes > 0 ? static_cast<size_t>(workspace_bytes) : 0, st);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("bitlinear_TernaSpMM_packed", e, __LINE__);
}

void bitlinear_TernaSpMM_packed(const int8_t* x, const void* packed, terna_bf16* out, const terna_bf16* s,
                                const terna_bf16* ws, int ws_num, int M, int N, int K, int route, terna_stream stream)
{
    bitlinear_TernaSpMM_packed_ws(x, packed, out, s, ws, ws_num, M, N, K, route, nullptr, 0, stream);
}

void ternaspmm_repack_cache_clear(void)
{
    std::lock_guard<std::mutex> lock(g_repack_mutex);
    g_repack_cache.clear();                               // hipFree waits for the launches that still read a copy
    if (g_repack_stale != nullptr)
        for (uint32_t i = 0; i <= kStaleSlots; ++i) g_repack_stale[i] = 0;
}

int ternaspmm_repack_cache_enable(int on)
{
    std::lock_guard<std::mutex> lock(g_repack_mutex);
    const int was = repack_cache_on() ? 1 : 0;
    g_repack_on = on ? 1 : 0;
    return was;
}

long long ternaspmm_repack_cache_limit(long long bytes)
{
    std::lock_guard<std::mutex> lock(g_repack_mutex);
    const size_t was = g_repack_cache.limit();
    if (bytes >= 0) {
        g_repack_cache.set_limit(static_cast<size_t>(bytes));
        g_repack_limit_set = true;
    }
    return was > static_cast<size_t>(INT64_MAX) ? -1 : static_cast<long long>(was);
}

void ternaspmm_repack_cache_stats(long long out[6])
{
    std::lock_guard<std::mutex> lock(g_repack_mutex);
    out[0] = static_cast<long long>(g_repack_cache.entries());
    out[1] = static_cast<long long>(g_repack_cache.used());
    out[2] = static_cast<long long>(g_repack_cache.retired());
    out[3] = static_cast<long long>(g_repack_cache.evicted());
    out[4] = static_cast<long long>(g_repack_cache.parked_bytes());
    out[5] = g_repack_cache.limit() > static_cast<size_t>(INT64_MAX) ? -1 : static_cast<long long>(g_repack_cache.limit());
}

int ternaspmm_plan_reference_call(int int8_activations, int route, int M, int N, int K, int SPLIT_K, const void* workspace,
                                  int cached, long long* workspace_bytes_used)
{
    if (M < 1 || N < 64 || K < 64 || (N % 64) || (K % 64) || route < 0 || route > 2) return -1;
    const Route r = route == 1 ? ROUTE_PREFILL : (route == 2 ? ROUTE_DECODE : ROUTE_AUTO);
    const CallPlan plan = plan_call(int8_activations != 0, r, M, N, K, SPLIT_K, workspace, cached != 0);
    size_t used = plan.p2_bytes;
    if (plan.kernel == CALL_P2_LARGE || plan.kernel == CALL_TRANSCODE_LARGE) {
        const void* scratch = plan.scratch_bytes ? static_cast<const char*>(workspace) + plan.scratch_offset : nullptr;
        const void* x_aligned = reinterpret_cast<const void*>(uintptr_t{256});          // any 16-byte aligned address: the common case
        const PrefillPlan pp = int8_activations ? plan_prefill_packed<int8_t>(x_aligned, M, N, K, scratch, plan.scratch_bytes)
                                                : plan_prefill_packed<uint16_t>(x_aligned, M, N, K, scratch, plan.scratch_bytes);
        if (pp.scratch_used) used = plan.scratch_offset + pp.scratch_used;
    }
    if (workspace_bytes_used) *workspace_bytes_used = static_cast<long long>(used);
    return static_cast<int>(plan.kernel);
}

int ternaspmm_quant_mode(int mode)
{
    const int was = quant_mode();
    if (mode >= QUANT_ROUNDED && mode <= QUANT_EAGER) g_quant_mode.store(mode, std::memory_order_relaxed);
    return was;
}

const char* ternaspmm_version(void) { return "ternaspmm-gfx950 0.1"; }

}  // extern "C"
