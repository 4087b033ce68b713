// libternaspmm.so: the extern "C" boundary of the TernaSpMM path on MI355X (gfx950).
// Declarations and the reference interface each symbol stands for: include/ternaspmm.h.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <mutex>
#include <unordered_map>

#include "../../include/ternaspmm.h"
#include "decode_kernel.h"
#include "decompress_kernel.h"
#include "prefill_kernel.h"
#include "decode_packed_kernel.h"
#include "prefill_packed_kernel.h"
#include "norm_quant_kernel.h"
#include "decode_fused_kernel.h"
#include "attention_kernel.h"
#include "argmax_kernel.h"
#include "lm_head_kernel.h"
#include "format_host.h"

using namespace terna;

namespace {

[[noreturn]] void die(const char* what, hipError_t e, int line)
{
    std::printf("Last Cuda Error Detected at line: %d, Error: %s (%s).\n", line, hipGetErrorString(e), what);
    std::fflush(stdout);
    std::exit(EXIT_FAILURE);
}

bool shape_ok(int M, int N, int K)
{
    if (M < 1 || N < 64 || K < 64 || (N % 64) || (K % 64)) {
        std::printf("TernaSpMM Error: unsupported shape M=%d N=%d K=%d (need M >= 1, N %% 64 == 0, K %% 64 == 0)\n",
                    M, N, K);
        std::fflush(stdout);
        return false;
    }
    return true;
}

// weight_scale has four slots (convert/convert_TernaInfer.py:176-194): one to four scale groups per matrix
bool groups_ok(int ws_num)
{
    if (ws_num < 1 || ws_num > 4) {
        std::printf("TernaSpMM Error: unsupported ws_num=%d (need 1 .. 4)\n", ws_num);
        std::fflush(stdout);
        return false;
    }
    return true;
}

struct Weights {
    const uint64_t* bitmap;
    const int* tile_off;
    const uint16_t* median_off;
    const uint32_t* sign_words;
};

// Dynamic-LDS opt-in of one kernel, once per (kernel, device) of the process: the attribute is per device.
void allow_dynamic_lds_ptr(const void* kernel, int bytes, const char* what, int line)
{
    static std::mutex mutex;
    static std::unordered_map<const void*, uint64_t> done;       // kernel -> bit per device ordinal
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = -1;
    std::lock_guard<std::mutex> lock(mutex);
    uint64_t& mask = done[kernel];
    if (dev >= 0 && ((mask >> dev) & 1u)) return;
    const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e != hipSuccess) die(what, e, line);
    if (dev >= 0) mask |= uint64_t{1} << dev;
}
template <typename Kernel>
void allow_dynamic_lds(Kernel kernel, int bytes, const char* what, int line)
{
    allow_dynamic_lds_ptr(reinterpret_cast<const void*>(kernel), bytes, what, line);
}

// Small-M kernel: one workgroup per 16-row band; up to 64 batch rows per workgroup.
template <typename Act, int WAVES, int MB, int DEPTH>
void launch_decode_as(const Act* x, const Weights& w, uint16_t* out, const Epilogue& ep, int M, int N, int K,
                      hipStream_t st)
{
    const dim3 grid(N / 16, (M + 16 * MB - 1) / (16 * MB));
    terna_decode_kernel<Act, WAVES, MB, DEPTH><<<grid, dim3(WAVES * 64), 0, st>>>(
        x, w.bitmap, w.tile_off, w.median_off, w.sign_words, out, ep, M, N, K);
}

// Shape of the small-M launch.  With one workgroup per 16-row band, a matrix with few bands
// (N/16 <= 256: at most one workgroup per CU) is bound by each wave's serial share of K, so it
// gets 16 waves and a deeper prefetch ring; a matrix with many bands is bound by how many
// workgroups fit on the chip at once, so it gets 8 waves and the leaner ring (<= 64 VGPRs).
// TERNASPMM_DECODE_WAVES=4|8|16 forces one variant (tuning aid).
int decode_waves_override()
{
    static const int waves = [] {
        const char* v = std::getenv("TERNASPMM_DECODE_WAVES");
        const int w = v ? std::atoi(v) : 0;
        return (w == 4 || w == 8 || w == 16) ? w : 0;
    }();
    return waves;
}

template <typename Act>
void launch_decode(const Act* x, const Weights& w, uint16_t* out, const Epilogue& ep, int M, int N, int K,
                   hipStream_t st)
{
    const int forced = decode_waves_override();
    const bool wide = forced ? forced == 16 : (N / 16 <= 256);
    if (M <= 16) {
        const bool narrow = forced ? forced == 4 : (N / 16 > 512);      // as on the P2 layout: fewer, longer-lived waves
        if (narrow) launch_decode_as<Act, 4, 1, 2>(x, w, out, ep, M, N, K, st);
        else if (wide) launch_decode_as<Act, 16, 1, 2>(x, w, out, ep, M, N, K, st);
        else launch_decode_as<Act, 8, 1, 1>(x, w, out, ep, M, N, K, st);
    } else if (M <= 32) {
        if (wide) launch_decode_as<Act, 16, 2, 1>(x, w, out, ep, M, N, K, st);
        else launch_decode_as<Act, 8, 2, 1>(x, w, out, ep, M, N, K, st);
    } else {
        launch_decode_as<Act, 8, 4, 1>(x, w, out, ep, M, N, K, st);
    }
}

// Large-M kernel: 256 output features x 64*MT batch rows per workgroup, MFMA-tiled.
template <typename Act, int MT>
void launch_prefill_as(const Act* x, const Weights& w, uint16_t* out, const Epilogue& ep, int M, int N, int K,
                       hipStream_t st)
{
    using S = PrefillSmem<MT>;
    auto kernel = terna_prefill_kernel<Act, MT>;
    allow_dynamic_lds(kernel, S::kBytes, "hipFuncSetAttribute(prefill)", __LINE__);
    const dim3 grid((N + kPrefillBN - 1) / kPrefillBN, (M + S::BM - 1) / S::BM);
    kernel<<<grid, dim3(256), S::kBytes, st>>>(x, w.bitmap, w.tile_off, w.median_off, w.sign_words, out, ep, M, N, K);
}

template <typename Act>
void launch_prefill(const Act* x, const Weights& w, uint16_t* out, const Epilogue& ep, int M, int N, int K,
                    hipStream_t st)
{
    if (K > 128 * 64) {                     // the MFMA kernel keeps per-step offsets for at most 128 steps
        launch_decode(x, w, out, ep, M, N, K, st);
        return;
    }
    // Largest batch tile that still gives every CU a workgroup; small problems take the smallest.
    const int n_tiles = (N + kPrefillBN - 1) / kPrefillBN;
    if (n_tiles * ((M + 255) / 256) >= 256) launch_prefill_as<Act, 4>(x, w, out, ep, M, N, K, st);
    else if (n_tiles * ((M + 127) / 128) >= 256) launch_prefill_as<Act, 2>(x, w, out, ep, M, N, K, st);
    else launch_prefill_as<Act, 1>(x, w, out, ep, M, N, K, st);
}

// ---- P2 layout (load-time repack): see packed_common.h -------------------------------------------
void launch_repack(const Weights& w, uint32_t* packed, int N, int K, hipStream_t st)
{
    terna_repack_kernel<4><<<dim3(N / 16), dim3(256), 0, st>>>(w.bitmap, w.tile_off, w.median_off, w.sign_words,
                                                              packed, N, K);
}

template <typename Act, int WAVES, int MB, int DEPTH, int NB = 1>
void launch_decode_packed_as(const Act* x, const uint32_t* packed, uint16_t* out, const Epilogue& ep, int M, int N,
                             int K, hipStream_t st)
{
    const dim3 grid(N / 16 / NB, (M + 16 * MB - 1) / (16 * MB));
    terna_decode_packed_kernel<Act, WAVES, MB, DEPTH, NB><<<grid, dim3(WAVES * 64), 0, st>>>(x, packed, out, ep, M, N, K);
}

template <typename Act>
void launch_decode_packed(const Act* x, const uint32_t* packed, uint16_t* out, const Epilogue& ep, int M, int N, int K,
                          hipStream_t st)
{
    const int forced = decode_waves_override();
    const bool wide = forced ? forced == 16 : (N / 16 <= 256);
    if (M <= 16) {
        // more than 512 bands (gate+up): per-wave set-up is as expensive as a few band-tiles, so fewer waves
        // with more band-tiles each win (measured 7.4 against 8.2 us)
        const bool narrow = forced ? forced == 4 : (N / 16 > 512);
        // ... and every workgroup stages the same activations: two bands per workgroup share one staging (N is a
        // multiple of 64, so the band count is even).  Measured on gate+up, cold: 6.4 us against 7.3 us; four
        // bands 6.7 us.  TERNASPMM_DECODE_BANDS=1 switches that off (tuning aid).
        static const bool multi_off = [] {
            const char* v = std::getenv("TERNASPMM_DECODE_BANDS");
            return v && std::atoi(v) == 1;
        }();
        if (narrow && !forced && !multi_off) launch_decode_packed_as<Act, 8, 1, 2, 2>(x, packed, out, ep, M, N, K, st);
        else if (narrow) launch_decode_packed_as<Act, 4, 1, 3>(x, packed, out, ep, M, N, K, st);
        else if (wide) launch_decode_packed_as<Act, 16, 1, 3>(x, packed, out, ep, M, N, K, st);
        else launch_decode_packed_as<Act, 8, 1, 2>(x, packed, out, ep, M, N, K, st);
    } else if (M <= 32) {
        if (wide) launch_decode_packed_as<Act, 16, 2, 2>(x, packed, out, ep, M, N, K, st);
        else launch_decode_packed_as<Act, 8, 2, 2>(x, packed, out, ep, M, N, K, st);
    } else {
        launch_decode_packed_as<Act, 8, 4, 1>(x, packed, out, ep, M, N, K, st);
    }
}

template <typename Act, int MB, int NA = 2>
void launch_prefill_packed_as(const Act* x, const uint32_t* packed, uint16_t* out, const Epilogue& ep, int M, int N,
                              int K, hipStream_t st)
{
    using S = PackedPrefillSmem<MB>;
    auto kernel = terna_prefill_packed_kernel<Act, MB, NA>;
    allow_dynamic_lds(kernel, S::kBytes, "hipFuncSetAttribute(prefill packed)", __LINE__);
    constexpr int BN = 128 * NA;
    const dim3 grid((N + BN - 1) / BN, (M + S::BM - 1) / S::BM);
    kernel<<<grid, dim3(256), S::kBytes, st>>>(x, packed, out, ep, M, N, K);
}

template <typename Act, int MB, int NA>
void launch_prefill_packed_dma_as(const Act* x, const uint32_t* packed, uint16_t* out, const Epilogue& ep, int M,
                                  int N, int K, hipStream_t st)
{
    using S = PackedPrefillDmaSmem<MB>;
    auto kernel = terna_prefill_packed_dma_kernel<Act, MB, NA>;
    allow_dynamic_lds(kernel, S::kBytes, "hipFuncSetAttribute(prefill packed dma)", __LINE__);
    constexpr int BN = 128 * NA;
    const dim3 grid((N + BN - 1) / BN, (M + S::BM - 1) / S::BM);
    static const int xcd_forced = [] {
        const char* v = std::getenv("TERNASPMM_PREFILL_XCD_MAP");
        return v ? std::atoi(v) : -1;
    }();
    // XCD-aware tile order (see the kernel): pays once the activations no longer fit one XCD's 4 MiB L2 --
    // below that the default order, which fetches every weight tile on one XCD only, moves less data.
    // TERNASPMM_PREFILL_XCD_MAP=0|1 forces it off / on (tuning aid).
    const bool big_x = static_cast<size_t>(M) * K * sizeof(Act) > (4u << 20);
    const int xcd_map = (grid.y % 8 == 0) && (xcd_forced < 0 ? big_x : xcd_forced != 0);
    kernel<<<grid, dim3(256), S::kBytes, st>>>(x, packed, out, ep, M, N, K, xcd_map);
}

// The direct-to-LDS kernel addresses both operands as a 64-bit base plus a 32-bit byte offset and
// loads 16-byte pieces of the activation rows.
inline bool prefill_dma_ok(const void* x, size_t act_bytes, int M, int N, int K)
{
    static const bool off = [] {
        const char* v = std::getenv("TERNASPMM_PREFILL_DMA");
        return v && std::atoi(v) == 0;
    }();
    return !off && (reinterpret_cast<uintptr_t>(x) & 15) == 0 && static_cast<uint64_t>(M) * K * act_bytes < (1ull << 32) &&
           static_cast<uint64_t>(N) * K / 4 < (1ull << 32);
}

template <typename Act>
void launch_prefill_packed(const Act* x, const uint32_t* packed, uint16_t* out, const Epilogue& ep, int M, int N, int K,
                           hipStream_t st)
{
    // Batch rows per workgroup (64 / 128 / 256).  Measured on MI355X the 64-row tile wins at every
    // BitNet-2B shape: it runs four waves per SIMD, and occupancy hides more latency than the taller
    // tiles save in weight expansion.  TERNASPMM_PREFILL_BM=64|128|256 forces one (tuning aid).
    static const int forced = [] {
        const char* v = std::getenv("TERNASPMM_PREFILL_BM");
        const int bm = v ? std::atoi(v) : 0;
        return (bm == 64 || bm == 96 || bm == 128 || bm == 256) ? bm : 0;
    }();
    static const int forced_bn = [] {
        const char* v = std::getenv("TERNASPMM_PREFILL_BN");
        const int bn = v ? std::atoi(v) : 0;
        return (bn == 128 || bn == 256) ? bn : 0;
    }();
    const int bm = forced ? forced : 64;
    // 256-feature tiles expand every weight once per 64 batch rows with two MFMAs per operand read;
    // when they would leave most of the 1024 workgroup slots of the chip empty, 128-feature tiles
    // double the workgroup count instead.  TERNASPMM_PREFILL_BN=128|256 forces one (tuning aid).
    const long wg256 = static_cast<long>((N + 255) / 256) * ((M + 63) / 64);
    const int bn = forced_bn ? forced_bn : (wg256 <= 640 ? 128 : 256);
    if (prefill_dma_ok(x, sizeof(Act), M, N, K) && (bm == 64 || bm == 128)) {
        if (bm == 64 && bn == 128) launch_prefill_packed_dma_as<Act, 2, 1>(x, packed, out, ep, M, N, K, st);
        else if (bm == 128 && forced_bn == 128) launch_prefill_packed_dma_as<Act, 4, 1>(x, packed, out, ep, M, N, K, st);
        else if (bm == 128) launch_prefill_packed_dma_as<Act, 4, 2>(x, packed, out, ep, M, N, K, st);
        else launch_prefill_packed_dma_as<Act, 2, 2>(x, packed, out, ep, M, N, K, st);
        return;
    }
    if (bm == 64 && bn == 128) launch_prefill_packed_as<Act, 2, 1>(x, packed, out, ep, M, N, K, st);
    else if (bm == 256) launch_prefill_packed_as<Act, 8>(x, packed, out, ep, M, N, K, st);
    else if (bm == 96) launch_prefill_packed_as<Act, 3>(x, packed, out, ep, M, N, K, st);
    else if (bm == 128) launch_prefill_packed_as<Act, 4>(x, packed, out, ep, M, N, K, st);
    else launch_prefill_packed_as<Act, 2>(x, packed, out, ep, M, N, K, st);
}

// Large-M call on reference-format pointers: with a 16-byte aligned workspace of N*K/4 bytes the
// weights are first transcoded to P2 there (one cheap pass) and the P2 kernel does the GEMM;
// without one the fused reference-format kernel runs.
template <typename Act>
void launch_large_m(const Act* x, const Weights& w, uint16_t* out, const Epilogue& ep, int M, int N, int K,
                    void* workspace, hipStream_t st)
{
    if (workspace && (reinterpret_cast<uintptr_t>(workspace) & 15) == 0) {
        uint32_t* packed = static_cast<uint32_t*>(workspace);
        launch_repack(w, packed, N, K, st);
        launch_prefill_packed(x, packed, out, ep, M, N, K, st);
    } else {
        launch_prefill(x, w, out, ep, M, N, K, st);
    }
}

enum Route { ROUTE_AUTO, ROUTE_DECODE, ROUTE_PREFILL };

// ---- opt-in repack cache behind the reference-format entry points (TERNASPMM_REPACK_CACHE=1).
// An unmodified call site keeps passing the four format tensors; the first call that sees a weight
// (identified by device, pointers and shape) allocates N*K/4 bytes, repacks into them and waits for
// the repack; every later call runs the P2 kernels.  The cache trusts the pointers: a caller that
// frees or rewrites weights must call ternaspmm_repack_cache_clear().  A first sight during stream
// capture (where nothing may be allocated) is served by the reference-format kernels instead.
struct RepackKey {
    int device;
    const void* bitmap;
    const void* signs;
    const void* offsets;
    int n, k;
    bool operator==(const RepackKey& o) const
    {
        return device == o.device && bitmap == o.bitmap && signs == o.signs && offsets == o.offsets && n == o.n && k == o.k;
    }
};
struct RepackKeyHash {
    size_t operator()(const RepackKey& key) const
    {
        size_t h = std::hash<const void*>()(key.bitmap);
        h = h * 1000003u ^ std::hash<const void*>()(key.signs);
        h = h * 1000003u ^ std::hash<const void*>()(key.offsets);
        return h * 1000003u ^ (static_cast<size_t>(key.n) << 20) ^ static_cast<size_t>(key.k) ^ (static_cast<size_t>(key.device) << 40);
    }
};
std::mutex g_repack_mutex;
std::unordered_map<RepackKey, void*, RepackKeyHash> g_repack_cache;

const uint32_t* cached_packed(const Weights& w, int N, int K, hipStream_t st)
{
    static const bool on = [] {
        const char* v = std::getenv("TERNASPMM_REPACK_CACHE");
        return v && std::atoi(v) != 0;
    }();
    if (!on) return nullptr;
    RepackKey key{0, w.bitmap, w.sign_words, w.tile_off, N, K};
    if (hipGetDevice(&key.device) != hipSuccess) return nullptr;
    std::lock_guard<std::mutex> lock(g_repack_mutex);
    const auto it = g_repack_cache.find(key);
    if (it != g_repack_cache.end()) return static_cast<const uint32_t*>(it->second);
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone) {
        (void)hipGetLastError();
        return nullptr;
    }
    void* buf = nullptr;
    if (hipMalloc(&buf, static_cast<size_t>(N) * K / 4) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    launch_repack(w, static_cast<uint32_t*>(buf), N, K, st);
    const hipError_t e = hipStreamSynchronize(st);       // later calls may come on other streams
    if (e != hipSuccess) die("repack cache", e, __LINE__);
    g_repack_cache.emplace(key, buf);
    return static_cast<const uint32_t*>(buf);
}

void run_i8(Route route, int8_t* x, uint64_t* bitmap, int* tile_off, uint16_t* median_off, uint32_t* sign_words,
            uint16_t* out, uint16_t* s, uint16_t* ws, int ws_num, int M, int N, int K, void* workspace,
            hipStream_t st, int line)
{
    if (!shape_ok(M, N, K) || !groups_ok(ws_num)) return;
    // The reference picks its path, and with it the epilogue arithmetic, by M <= 64
    // (kernels/TernaSpMM.cu:34); the forced entry points pin one of the two.
    const bool decode_rule = route == ROUTE_DECODE || (route == ROUTE_AUTO && M <= 64);
    const Epilogue ep{s, ws, nullptr, ws_num, decode_rule ? EP_I8_DECODE : EP_I8_PREFILL};
    const Weights w{bitmap, tile_off, median_off, sign_words};
    if (const uint32_t* p2 = cached_packed(w, N, K, st)) {
        if (M <= 64) launch_decode_packed<int8_t>(x, p2, out, ep, M, N, K, st);
        else launch_prefill_packed<int8_t>(x, p2, out, ep, M, N, K, st);
    } else if (M <= 64) launch_decode<int8_t>(x, w, out, ep, M, N, K, st);
    else launch_large_m<int8_t>(x, w, out, ep, M, N, K, workspace, st);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("bitlinear_TernaSpMM", e, line);
}

void run_bf16(Route route, const uint16_t* x, const uint64_t* bitmap, const int* tile_off,
              const uint16_t* median_off, const uint32_t* sign_words, uint16_t* out, const float* scale,
              int ws_num, int M, int N, int K, void* workspace, hipStream_t st, int line)
{
    if (!shape_ok(M, N, K) || !groups_ok(ws_num)) return;
    const Epilogue ep{nullptr, nullptr, scale, ws_num, EP_BF16};
    const Weights w{bitmap, tile_off, median_off, sign_words};
    const bool small = route == ROUTE_DECODE || (route == ROUTE_AUTO && M <= 64);
    if (const uint32_t* p2 = cached_packed(w, N, K, st)) {
        if (small) launch_decode_packed<uint16_t>(x, p2, out, ep, M, N, K, st);
        else launch_prefill_packed<uint16_t>(x, p2, out, ep, M, N, K, st);
    } else if (small) launch_decode<uint16_t>(x, w, out, ep, M, N, K, st);
    else launch_large_m<uint16_t>(x, w, out, ep, M, N, K, workspace, st);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("bitlinear_TernaSpMM_bf16", e, line);
}

__global__ void sleep_kernel(long long ticks)
{
    // wall_clock64 counts at a fixed 100 MHz; every lane leaves once the span has passed.
    const long long start = wall_clock64();
    while (wall_clock64() - start < ticks) __builtin_amdgcn_s_sleep(8);
}

// Waves per workgroup of the decode attention: with one workgroup per (sequence, head) and few of them
// on the chip, wider workgroups request more of the cache up front (64 slots of keys per wave).
// TERNASPMM_ATTN_WAVES=4|8 forces one (tuning aid).  Both entry points use the same rule, so their results
// stay bit-identical.
int attention_waves(int B, int H)
{
    static const int forced = [] {
        const char* v = std::getenv("TERNASPMM_ATTN_WAVES");
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
        const char* v = std::getenv("TERNASPMM_ATTN_XCD_GROUPS");
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
int attention_splits(int B, int H, int S, const void* workspace)
{
    if (workspace == nullptr) return 1;
    static const int forced = [] {
        const char* v = std::getenv("TERNASPMM_ATTN_SPLITS");
        const int n = v ? std::atoi(v) : 0;
        return (n == 1 || n == 2 || n == 4 || n == 8) ? n : 0;
    }();
    if (forced) return forced;
    if (S < 1024) return 1;
    int sp = 1;
    while (sp < kAttentionMaxSplits && static_cast<long>(B) * H * sp * 2 <= 512) sp *= 2;
    return sp;
}

template <int D, bool ROPE, bool ADJ, int NW, bool SPLIT>
void launch_attention_as(const uint16_t* q, uint16_t* ck, uint16_t* cv, const float* cos, const float* sin,
                         const long long* pos, uint16_t* out, int B, int H, int KV, int S, float scale, int splits,
                         void* workspace, const AttentionPrefetch& pf_in, hipStream_t st)
{
    AttentionPrefetch pf = pf_in;
    if (splits > 1) pf.workgroups = 0;                       // the split grid is two-dimensional: no extra workgroups
    auto kernel = terna_decode_attention_kernel<D, ROPE, ADJ, NW, SPLIT>;
    const size_t lds = decode_attention_lds_bytes(D, NW, S);
    if (lds > 64 * 1024) allow_dynamic_lds(kernel, 160 * 1024, "hipFuncSetAttribute(decode attention)", __LINE__);
    int* arrived = static_cast<int*>(workspace);
    float* partial = workspace ? reinterpret_cast<float*>(static_cast<char*>(workspace) + attention_counter_bytes(B, H)) : nullptr;
    const int slots = attention_slots(B, H, KV);
    kernel<<<dim3(slots + pf.workgroups, splits), dim3(64 * NW), lds, st>>>(q, ck, cv, cos, sin, pos, out, H, KV, S, scale,
                                                                           partial, arrived, splits, pf, slots,
                                                                           attention_groups_on(H, KV) ? B * KV : 0);
}

template <bool ROPE, bool ADJ>
void launch_attention(const uint16_t* q, uint16_t* ck, uint16_t* cv, const float* cos, const float* sin,
                             const long long* pos, uint16_t* out, int B, int H, int KV, int D, int S, float scale,
                             void* workspace, const AttentionPrefetch& pf, hipStream_t st)
{
    const int splits = attention_splits(B, H, S, workspace);
    const int nw = splits > 1 ? 4 : attention_waves(B, H);       // a split is a short prefix: the narrow workgroup
#define TERNA_ATTN(DIM, NWAVES, SPLIT) \
    launch_attention_as<DIM, ROPE, ADJ, NWAVES, SPLIT>(q, ck, cv, cos, sin, pos, out, B, H, KV, S, scale, splits, workspace, pf, st)
    if (D == 128) {
        if (splits > 1) TERNA_ATTN(128, 4, true);
        else if (nw == 8) TERNA_ATTN(128, 8, false);
        else TERNA_ATTN(128, 4, false);
    } else {
        if (splits > 1) TERNA_ATTN(64, 4, true);
        else if (nw == 8) TERNA_ATTN(64, 8, false);
        else TERNA_ATTN(64, 4, false);
    }
#undef TERNA_ATTN
}

bool attention_args_ok(const char* who, int B, int H, int KV, int D, int S)
{
    if (B < 1 || H < 1 || KV < 1 || H % KV != 0 || (D != 64 && D != 128) || S < 1 || S > 8192) {
        std::fprintf(stderr, "%s: unsupported arguments (H=%d KV=%d D=%d S=%d)\n", who, H, KV, D, S);
        return false;
    }
    return true;
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
                         int /*SPLIT_K*/, int32_t* workspace, terna_stream stream)
{
    run_i8(ROUTE_AUTO, x, bitmap, tile_off, median_off, sign_words, out, s, ws, ws_num, M, N, K, workspace,
           static_cast<hipStream_t>(stream), __LINE__);
}

void bitlinear_TernaSpMM_decode(int8_t* x, uint64_t* bitmap, int* tile_off, uint16_t* median_off,
                                uint32_t* sign_words, terna_bf16* out, terna_bf16* s, terna_bf16* ws, int ws_num,
                                int M, int N, int K, int /*SPLIT_K*/, int32_t* workspace, terna_stream stream)
{
    run_i8(ROUTE_DECODE, x, bitmap, tile_off, median_off, sign_words, out, s, ws, ws_num, M, N, K, workspace,
           static_cast<hipStream_t>(stream), __LINE__);
}

void bitlinear_TernaSpMM_prefill(int8_t* x, uint64_t* bitmap, int* tile_off, uint16_t* median_off,
                                 uint32_t* sign_words, terna_bf16* out, terna_bf16* s, terna_bf16* ws, int ws_num,
                                 int M, int N, int K, int /*SPLIT_K*/, int32_t* workspace, terna_stream stream)
{
    run_i8(ROUTE_PREFILL, x, bitmap, tile_off, median_off, sign_words, out, s, ws, ws_num, M, N, K, workspace,
           static_cast<hipStream_t>(stream), __LINE__);
}

void bitlinear_TernaSpMM_benchmark(int mode, int warmup_iters, int bench_iters, int8_t* x, uint64_t* bitmap,
                                   int* tile_off, uint16_t* median_off, uint32_t* sign_words, terna_bf16* out,
                                   terna_bf16* s, terna_bf16* ws, int ws_num, int M, int N, int K, int SPLIT_K,
                                   int32_t* workspace, terna_stream stream)
{
    // mode 0 = auto, 1 = prefill, 2 = decode (kernels/TernaSpMM.cu:165-173)
    const Route route = mode == 1 ? ROUTE_PREFILL : (mode == 2 ? ROUTE_DECODE : ROUTE_AUTO);
    (void)SPLIT_K;
    hipStream_t st = static_cast<hipStream_t>(stream);
    for (int it = 0; it < warmup_iters; ++it)
        run_i8(route, x, bitmap, tile_off, median_off, sign_words, out, s, ws, ws_num, M, N, K, workspace, st, __LINE__);
    hipError_t e = hipStreamSynchronize(st);
    if (e != hipSuccess) die("benchmark warm-up", e, __LINE__);

    hipEvent_t start, stop;
    if ((e = hipEventCreate(&start)) != hipSuccess) die("hipEventCreate", e, __LINE__);
    if ((e = hipEventCreate(&stop)) != hipSuccess) die("hipEventCreate", e, __LINE__);
    (void)hipEventRecord(start, st);
    for (int it = 0; it < bench_iters; ++it)
        run_i8(route, x, bitmap, tile_off, median_off, sign_words, out, s, ws, ws_num, M, N, K, workspace, st, __LINE__);
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
                              const float* scale, int ws_num, int M, int N, int K, int /*SPLIT_K*/,
                              void* workspace, terna_stream stream)
{
    run_bf16(ROUTE_AUTO, x, bitmap, tile_off, median_off, sign_words, out, scale, ws_num, M, N, K, workspace,
             static_cast<hipStream_t>(stream), __LINE__);
}

void bitlinear_TernaSpMM_bf16_decode(const terna_bf16* x, const uint64_t* bitmap, const int* tile_off,
                                     const uint16_t* median_off, const uint32_t* sign_words, terna_bf16* out,
                                     const float* scale, int ws_num, int M, int N, int K, int /*SPLIT_K*/,
                                     void* workspace, terna_stream stream)
{
    run_bf16(ROUTE_DECODE, x, bitmap, tile_off, median_off, sign_words, out, scale, ws_num, M, N, K, workspace,
             static_cast<hipStream_t>(stream), __LINE__);
}

void bitlinear_TernaSpMM_bf16_prefill(const terna_bf16* x, const uint64_t* bitmap, const int* tile_off,
                                      const uint16_t* median_off, const uint32_t* sign_words, terna_bf16* out,
                                      const float* scale, int ws_num, int M, int N, int K, int /*SPLIT_K*/,
                                      void* workspace, terna_stream stream)
{
    run_bf16(ROUTE_PREFILL, x, bitmap, tile_off, median_off, sign_words, out, scale, ws_num, M, N, K, workspace,
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
    terna_decompress_kernel<4><<<dim3(N / 16), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
        bitmap, tile_off, median_off, sign_words, W_dense, N, K);
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

void bitlinear_TernaSpMM_bf16_packed(const terna_bf16* x, const void* packed, terna_bf16* out, const float* scale,
                                     int ws_num, int M, int N, int K, int route, terna_stream stream)
{
    if (!shape_ok(M, N, K) || !groups_ok(ws_num)) return;
    const Epilogue ep{nullptr, nullptr, scale, ws_num, EP_BF16};
    const uint32_t* p = static_cast<const uint32_t*>(packed);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool small = route == 2 || (route != 1 && M <= 64);
    if (small) launch_decode_packed<uint16_t>(x, p, out, ep, M, N, K, st);
    else launch_prefill_packed<uint16_t>(x, p, out, ep, M, N, K, st);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("bitlinear_TernaSpMM_bf16_packed", e, __LINE__);
}

void bitlinear_TernaSpMM_packed(const int8_t* x, const void* packed, terna_bf16* out, const terna_bf16* s,
                                const terna_bf16* ws, int ws_num, int M, int N, int K, int route, terna_stream stream)
{
    if (!shape_ok(M, N, K) || !groups_ok(ws_num)) return;
    const bool decode_rule = route == 2 || (route != 1 && M <= 64);
    const Epilogue ep{s, ws, nullptr, ws_num, decode_rule ? EP_I8_DECODE : EP_I8_PREFILL};
    const uint32_t* p = static_cast<const uint32_t*>(packed);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (M <= 64) launch_decode_packed<int8_t>(x, p, out, ep, M, N, K, st);
    else launch_prefill_packed<int8_t>(x, p, out, ep, M, N, K, st);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("bitlinear_TernaSpMM_packed", e, __LINE__);
}

void ternaspmm_rmsnorm_quant(const terna_bf16* x, const terna_bf16* residual, terna_bf16* sum_out,
                             const terna_bf16* weight, float eps, terna_bf16* y_out, int8_t* xq_out,
                             terna_bf16* s_out, int M, int K, terna_stream stream)
{
    if (M < 1 || K < 8 || (K & 7) || K > 8 * kNormThreads * kNormMaxVecs || (xq_out != nullptr) != (s_out != nullptr)) {
        std::fprintf(stderr, "ternaspmm_rmsnorm_quant: unsupported arguments (M=%d K=%d)\n", M, K);
        return;
    }
    terna_norm_quant_kernel<false><<<dim3(M), dim3(kNormThreads), 0, static_cast<hipStream_t>(stream)>>>(
        x, residual, sum_out, weight, eps, y_out, xq_out, s_out, K);
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
    terna_norm_quant_kernel<true><<<dim3(M), dim3(kNormThreads), 0, static_cast<hipStream_t>(stream)>>>(
        x13, nullptr, nullptr, weight, eps, y_out, xq_out, s_out, F);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("ternaspmm_relu2_mul_rmsnorm_quant", e, __LINE__);
}

// mode: FUSED_PLAIN / FUSED_RESIDUAL / FUSED_GLU.  Returns 1 when a launch was enqueued.
static int launch_decode_fused(int mode, const terna_bf16* x, const terna_bf16* residual, terna_bf16* sum_out,
                               const terna_bf16* norm_weight, float eps, const void* packed, terna_bf16* out,
                               const terna_bf16* ws, int ws_num, int8_t* xq_out, terna_bf16* s_out, int M, int N,
                               int K, hipStream_t st)
{
    if (!shape_ok(M, N, K) || !groups_ok(ws_num) || M > 16) return 0;
    const int ktiles = K / 64;
    const int bands = N / 16;
    static const int forced_waves = [] {
        const char* v = std::getenv("TERNASPMM_FUSED_WAVES");
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
        const char* v = std::getenv("TERNASPMM_FUSED_BANDS");
        return v ? std::atoi(v) : 0;
    }();
    static const int nb_waves = [] {
        const char* v = std::getenv("TERNASPMM_FUSED_BANDS_WAVES");
        return v && std::atoi(v) == 16 ? 16 : 8;
    }();
    const bool multi = forced_nb != 1 && bands > 256 && bands % 4 == 0 && mode != FUSED_GLU;
    const bool multi8 = multi && nb_waves == 8 && ktiles <= 8 * 5;
    const bool multi16 = multi && !multi8 && ktiles <= 16 * 3;
    const dim3 grid(multi16 || multi8 ? bands / 4 : bands);
#define TERNA_FUSED(WAVES, TMAX, MODE, MP, NB)                                                                     \
    terna_decode_fused_kernel<WAVES, TMAX, MODE, MP, NB><<<grid, dim3(WAVES * 64), 0, st>>>(                       \
        x, residual, sum_out, norm_weight, eps, p, out, ws, ws_num, xq_out, s_out, M, N, K)
#define TERNA_FUSED_M(WAVES, TMAX, MODE, NB)                                                                       \
    do {                                                                                                           \
        if (M == 1) TERNA_FUSED(WAVES, TMAX, MODE, 1, NB);                                                         \
        else if (M <= 8) TERNA_FUSED(WAVES, TMAX, MODE, 8, NB);                                                    \
        else TERNA_FUSED(WAVES, TMAX, MODE, 16, NB);                                                               \
    } while (0)
    if (mode == FUSED_GLU) {
        // long K (the down projection): only the single-row variant, whose per-lane state is tiny
        if (M != 1 || !wide || ktiles > 16 * 7) return 0;
        TERNA_FUSED(16, 7, FUSED_GLU, 1, 1);
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

int bitlinear_TernaSpMM_packed_fused_glu(const terna_bf16* x13, const terna_bf16* norm_weight, float eps,
                                         const void* packed, terna_bf16* out, const terna_bf16* ws, int ws_num,
                                         int8_t* xq_out, terna_bf16* s_out, int M, int N, int F, terna_stream stream)
{
    return launch_decode_fused(FUSED_GLU, x13, nullptr, nullptr, norm_weight, eps, packed, out, ws, ws_num, xq_out, s_out,
                               M, N, F, static_cast<hipStream_t>(stream));
}

void ternaspmm_rope_kv_store(const terna_bf16* qkv, const float* cos, const float* sin, const long long* pos,
                             terna_bf16* q_out, terna_bf16* cache_k, terna_bf16* cache_v, int B, int T, int H,
                             int KV, int D, int S, int adjacent, terna_stream stream)
{
    if (B < 1 || T < 1 || H < 1 || KV < 1 || D < 2 || (D & 1) || S < 1) {
        std::fprintf(stderr, "ternaspmm_rope_kv_store: unsupported arguments\n");
        return;
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (adjacent)
        terna_rope_kv_store_kernel<true><<<dim3(B * T), dim3(256), 0, st>>>(qkv, cos, sin, pos, q_out, cache_k, cache_v, T, H, KV, D, S);
    else
        terna_rope_kv_store_kernel<false><<<dim3(B * T), dim3(256), 0, st>>>(qkv, cos, sin, pos, q_out, cache_k, cache_v, T, H, KV, D, S);
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
                                const long long* pos, terna_bf16* out, int B, int H, int KV, int D, int S,
                                float scale, void* workspace, terna_stream stream)
{
    if (!attention_args_ok("ternaspmm_decode_attention", B, H, KV, D, S)) return;
    // the kernel writes the caches only in its ROPE variant
    launch_attention<false, false>(q, const_cast<uint16_t*>(cache_k), const_cast<uint16_t*>(cache_v), nullptr, nullptr, pos,
                                   out, B, H, KV, D, S, scale, workspace, AttentionPrefetch{}, static_cast<hipStream_t>(stream));
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("ternaspmm_decode_attention", e, __LINE__);
}

void ternaspmm_rope_decode_attention(const terna_bf16* qkv, const float* cos, const float* sin, const long long* pos,
                                     terna_bf16* cache_k, terna_bf16* cache_v, terna_bf16* out, int B, int H, int KV,
                                     int D, int S, float scale, int adjacent, void* workspace, terna_stream stream)
{
    if (!attention_args_ok("ternaspmm_rope_decode_attention", B, H, KV, D, S)) return;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (adjacent) launch_attention<true, true>(qkv, cache_k, cache_v, cos, sin, pos, out, B, H, KV, D, S, scale, workspace, AttentionPrefetch{}, st);
    else launch_attention<true, false>(qkv, cache_k, cache_v, cos, sin, pos, out, B, H, KV, D, S, scale, workspace, AttentionPrefetch{}, st);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("ternaspmm_rope_decode_attention", e, __LINE__);
}

void ternaspmm_rope_decode_attention_prefetch(const terna_bf16* qkv, const float* cos, const float* sin, const long long* pos,
                                              terna_bf16* cache_k, terna_bf16* cache_v, terna_bf16* out, int B, int H, int KV,
                                              int D, int S, float scale, int adjacent, void* workspace,
                                              const void* const* pf_ptr, const long long* pf_bytes, const long long* pf_unit_bytes,
                                              int pf_count, terna_stream stream)
{
    if (!attention_args_ok("ternaspmm_rope_decode_attention_prefetch", B, H, KV, D, S)) return;
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
    // the heads take B*H CUs; the rest of the chip prefetches
    static const int forced_wgs = [] {
        const char* v = std::getenv("TERNASPMM_ATTN_PREFETCH_WGS");
        return v ? std::atoi(v) / 8 * 8 : -1;
    }();
    const int slots = attention_slots(B, H, KV);
    pf.workgroups = pf.count > 0 && slots < 232 ? (forced_wgs >= 0 ? forced_wgs : (256 - slots) / 8 * 8) : 0;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (adjacent) launch_attention<true, true>(qkv, cache_k, cache_v, cos, sin, pos, out, B, H, KV, D, S, scale, workspace, pf, st);
    else launch_attention<true, false>(qkv, cache_k, cache_v, cos, sin, pos, out, B, H, KV, D, S, scale, workspace, pf, st);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("ternaspmm_rope_decode_attention_prefetch", e, __LINE__);
}

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
    const size_t lds = lm_head_lds_bytes(M, K);
    if (lds > 160 * 1024) {
        std::fprintf(stderr, "ternaspmm_lm_head_bf16: M=%d rows of K=%d do not fit the 160 KB of LDS\n", M, K);
        return;
    }
    if (lds > 64 * 1024) allow_dynamic_lds(terna_lm_head_kernel, 160 * 1024, "hipFuncSetAttribute(lm head)", __LINE__);
    const int blocks = (V + 15) / 16;
    const int wgs_needed = (blocks + kLmWaves - 1) / kLmWaves;
    static const int forced = [] {
        const char* v = std::getenv("TERNASPMM_LM_HEAD_WGS");
        return v ? std::atoi(v) : 0;
    }();
    const int cap = forced > 0 ? forced : 512;               // two workgroups per CU measure fastest (256: 137 us, 512: 115 us, 1024: 119 us on 657 MB)
    const int grid = wgs_needed < cap ? wgs_needed : cap;
    static const int quad = [] {
        const char* v = std::getenv("TERNASPMM_LM_HEAD_QUAD");
        return v ? std::atoi(v) : 1;
    }();
    const int ksteps = K / 128;
    if (quad && M <= 4 && (K & 127) == 0) {
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
        terna_lm_head_kernel<<<dim3(grid), dim3(kLmWaves * 64), lds, static_cast<hipStream_t>(stream)>>>(x, w, logits, M, V, K);
    }
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) die("ternaspmm_lm_head_bf16", e, __LINE__);
}

void ternaspmm_repack_cache_clear(void)
{
    std::lock_guard<std::mutex> lock(g_repack_mutex);
    for (auto& kv : g_repack_cache) (void)hipFree(kv.second);
    g_repack_cache.clear();
}

const char* ternaspmm_version(void) { return "ternaspmm-gfx950 0.1"; }

}  // extern "C"
