// Launchers of the small-M kernel on the P2 layout and of the load-time repack (decode_packed_kernel.h,
// packed_common.h).
#include "launchers.h"
#include "host_util.h"
#include "decode_packed_kernel.h"
#include "decode_flat_kernel.h"
#include "decode_chunk_kernel.h"

namespace terna {

// ---- P2 layout (load-time repack): see packed_common.h -------------------------------------------
void launch_repack(const Weights& w, uint32_t* packed, int N, int K, hipStream_t st)
{
    terna_repack_kernel<4><<<dim3(N / 16), dim3(256), 0, st>>>(w.bitmap, w.tile_off, w.median_off, w.sign_words,
                                                              packed, N, K);
}

template <typename Act, int WAVES, int MB, int DEPTH, int NB = 1>
void launch_decode_packed_as(const Act* x, const uint32_t* packed, uint16_t* out, const Epilogue& ep, int M, int N,
                             int K, const RepackGuard* guard, hipStream_t st)
{
    const dim3 grid(N / 16 / NB + (guard != nullptr ? 1 : 0), (M + 16 * MB - 1) / (16 * MB));
    if (guard != nullptr)
        terna_decode_packed_kernel<Act, WAVES, MB, DEPTH, NB, true><<<grid, dim3(WAVES * 64), 0, st>>>(x, packed, out, M, N, K, ep, *guard, PackedProducer{});
    else
        terna_decode_packed_kernel<Act, WAVES, MB, DEPTH, NB, false><<<grid, dim3(WAVES * 64), 0, st>>>(x, packed, out, M, N, K, ep, RepackGuard{}, PackedProducer{});
}

template <typename Act, int WAVES, int TMAX, int NB>
void launch_decode_flat_as(const Act* x, const uint32_t* packed, uint16_t* out, const Epilogue& ep, int M, int N, int K,
                           const RepackGuard* guard, hipStream_t st)
{
    const dim3 grid(N / 16 / NB + (guard != nullptr ? 1 : 0));
    if (guard != nullptr)
        terna_decode_flat_kernel<Act, WAVES, TMAX, NB, true><<<grid, dim3(WAVES * 64), 0, st>>>(x, packed, out, M, N, K, ep, *guard);
    else
        terna_decode_flat_kernel<Act, WAVES, TMAX, NB, false><<<grid, dim3(WAVES * 64), 0, st>>>(x, packed, out, M, N, K, ep, RepackGuard{});
}

// Up to 16 rows and a K whose tiles one workgroup holds in flight: the straight-line kernel (decode_flat_kernel.h).
// Returns false where it does not apply.  TERNASPMM_DECODE_FLAT=0 switches it off (tuning aid).
template <typename Act>
static bool try_decode_flat(const Act* x, const uint32_t* packed, uint16_t* out, const Epilogue& ep, int M, int N, int K,
                            hipStream_t st, const RepackGuard* guard)
{
    static const bool off = [] {
        const char* v = tuning_env("TERNASPMM_DECODE_FLAT");
        return v && std::atoi(v) == 0;
    }();
    const int ktiles = K / 64, bands = N / 16;
    if (off || M > 16 || static_cast<long long>(N) * K / 4 >= (1ll << 31)) return false;      // byte offsets are 32-bit
    if (bands > 512 && bands % 2 == 0 && ktiles <= 8 * 5) launch_decode_flat_as<Act, 8, 5, 2>(x, packed, out, ep, M, N, K, guard, st);
    else if (bands > 256 && ktiles <= 8 * 5) launch_decode_flat_as<Act, 8, 5, 1>(x, packed, out, ep, M, N, K, guard, st);
    else if (bands > 256) return false;
    else if (ktiles <= 16 * 3) launch_decode_flat_as<Act, 16, 3, 1>(x, packed, out, ep, M, N, K, guard, st);
    else if (ktiles <= 16 * 7) launch_decode_flat_as<Act, 16, 7, 1>(x, packed, out, ep, M, N, K, guard, st);
    else return false;
    return true;
}

template <typename Act, int CT, int MR>
void launch_decode_chunk_as(const Act* x, const uint32_t* packed, uint16_t* out, const Epilogue& ep, int M, int N, int K,
                            const RepackGuard* guard, hipStream_t st)
{
    const dim3 grid(N / 16 + (guard != nullptr ? 1 : 0));
    if (guard != nullptr)
        terna_decode_chunk_kernel<Act, CT, MR, true><<<grid, dim3(kChunkWaves * 64), 0, st>>>(x, packed, out, M, N, K, ep, *guard);
    else
        terna_decode_chunk_kernel<Act, CT, MR, false><<<grid, dim3(kChunkWaves * 64), 0, st>>>(x, packed, out, M, N, K, ep, RepackGuard{});
}

template <typename Act, int MR>
void launch_decode_chunk4_as(const Act* x, const uint32_t* packed, uint16_t* out, const Epilogue& ep, int M, int N, int K,
                             const RepackGuard* guard, hipStream_t st)
{
    const dim3 grid(N / 64 + (guard != nullptr ? 1 : 0));
    if (guard != nullptr)
        terna_decode_chunk4_kernel<Act, MR, true><<<grid, dim3(kChunkWaves * 64), 0, st>>>(x, packed, out, M, N, K, ep, *guard);
    else
        terna_decode_chunk4_kernel<Act, MR, false><<<grid, dim3(kChunkWaves * 64), 0, st>>>(x, packed, out, M, N, K, ep, RepackGuard{});
}

// Up to 16 rows, up to 32 chunks of four tiles (K <= 8192): the kernel with four band-tiles per load (decode_chunk_kernel.h).
// Returns false where it does not apply.  TERNASPMM_DECODE_CHUNK=0 switches it off, =2 gives every band a workgroup of
// its own whatever the band count, =3 leaves matrices of more than 256 bands to the other kernels (tuning aids).
template <typename Act>
static bool try_decode_chunk(const Act* x, const uint32_t* packed, uint16_t* out, const Epilogue& ep, int M, int N, int K,
                             hipStream_t st, const RepackGuard* guard)
{
    static const int mode = [] {
        const char* v = tuning_env("TERNASPMM_DECODE_CHUNK");
        return v ? std::atoi(v) : 1;
    }();
    const int ktiles = K / 64, bands = N / 16, chunks = (ktiles + 3) / 4;
    if (mode == 0 || M > 16 || chunks > 2 * kChunkWaves) return false;
    if (static_cast<long long>(N) * K / 4 >= (1ll << 31)) return false;      // byte offsets are 32-bit
    if (bands > 256 && mode != 2) {
        // four bands per workgroup: one round of workgroups up to 1024 bands (the bf16 slabs of 16 rows do not fit LDS)
        if (mode == 3 || bands % 4 != 0 || chunks > kChunkWaves || (sizeof(Act) == 2 && M > 8)) return false;
        if (M <= 4) launch_decode_chunk4_as<Act, 4>(x, packed, out, ep, M, N, K, guard, st);
        else if (M <= 8) launch_decode_chunk4_as<Act, 8>(x, packed, out, ep, M, N, K, guard, st);
        else if constexpr (sizeof(Act) == 1) launch_decode_chunk4_as<Act, 16>(x, packed, out, ep, M, N, K, guard, st);
        return true;
    }
#define TERNA_CHUNK(CT)                                                                                   \
    do {                                                                                                  \
        if (M <= 4) launch_decode_chunk_as<Act, CT, 4>(x, packed, out, ep, M, N, K, guard, st);            \
        else if (M <= 8) launch_decode_chunk_as<Act, CT, 8>(x, packed, out, ep, M, N, K, guard, st);       \
        else launch_decode_chunk_as<Act, CT, 16>(x, packed, out, ep, M, N, K, guard, st);                  \
    } while (0)
    if (chunks <= kChunkWaves) TERNA_CHUNK(1);
    else TERNA_CHUNK(2);
#undef TERNA_CHUNK
    return true;
}

template <typename Act>
void launch_decode_packed(const Act* x, const uint32_t* packed, uint16_t* out, const Epilogue& ep, int M, int N, int K,
                          hipStream_t st, const RepackGuard* guard)
{
    const int forced = decode_waves_override();
    if (!forced && try_decode_chunk(x, packed, out, ep, M, N, K, st, guard)) return;
    if (!forced && try_decode_flat(x, packed, out, ep, M, N, K, st, guard)) return;
    const bool wide = forced ? forced == 16 : (N / 16 <= 256);
    if (M <= 16) {
        // more than 512 bands (gate+up): per-wave set-up is as expensive as a few band-tiles, so fewer waves
        // with more band-tiles each win (measured 7.4 against 8.2 us)
        const bool narrow = forced ? forced == 4 : (N / 16 > 512);
        // ... and every workgroup stages the same activations: two bands per workgroup share one staging (N is a
        // multiple of 64, so the band count is even).  Measured on gate+up, cold: 6.4 us against 7.3 us; four
        // bands 6.7 us.  TERNASPMM_DECODE_BANDS=1 switches that off (tuning aid).
        static const bool multi_off = [] {
            const char* v = tuning_env("TERNASPMM_DECODE_BANDS");
            return v && std::atoi(v) == 1;
        }();
        if (narrow && !forced && !multi_off) launch_decode_packed_as<Act, 8, 1, 2, 2>(x, packed, out, ep, M, N, K, guard, st);
        else if (narrow) launch_decode_packed_as<Act, 4, 1, 3>(x, packed, out, ep, M, N, K, guard, st);
        else if (wide) launch_decode_packed_as<Act, 16, 1, 3>(x, packed, out, ep, M, N, K, guard, st);
        else launch_decode_packed_as<Act, 8, 1, 2>(x, packed, out, ep, M, N, K, guard, st);
    } else if (M <= 32) {
        // more than 512 bands: two bands per workgroup share the staging of the 32 activation rows, as above
        if (!forced && N / 16 > 512) launch_decode_packed_as<Act, 4, 2, 2, 2>(x, packed, out, ep, M, N, K, guard, st);
        else if (wide) launch_decode_packed_as<Act, 16, 2, 2>(x, packed, out, ep, M, N, K, guard, st);
        else launch_decode_packed_as<Act, 8, 2, 2>(x, packed, out, ep, M, N, K, guard, st);
    } else {
        launch_decode_packed_as<Act, 8, 4, 1>(x, packed, out, ep, M, N, K, guard, st);
    }
}

// The small-M int8 launch as a producer (residual add + the next norm's partial statistics in the epilogue): M <= 16.
void launch_decode_packed_producer(const int8_t* x, const uint32_t* packed, uint16_t* out, const Epilogue& ep, int M, int N, int K,
                                   const uint16_t* residual, const uint16_t* next_w, float* stats_out, uint16_t* raw_out, hipStream_t st)
{
    const PackedProducer prod{residual, next_w, reinterpret_cast<float2*>(stats_out), raw_out};
    const dim3 grid(N / 16, 1);
    if (N / 16 <= 256)
        terna_decode_packed_kernel<int8_t, 16, 1, 3, 1, false, true><<<grid, dim3(16 * 64), 0, st>>>(x, packed, out, M, N, K, ep, RepackGuard{}, prod);
    else
        terna_decode_packed_kernel<int8_t, 8, 1, 2, 1, false, true><<<grid, dim3(8 * 64), 0, st>>>(x, packed, out, M, N, K, ep, RepackGuard{}, prod);
}

// one wave each: record the fingerprint of a weight's reference-format tensors / check it as a launch of its own
__global__ __launch_bounds__(64) void terna_repack_fingerprint_kernel(RepackGuard g, unsigned long long* out)
{
    const unsigned long long now = repack_fingerprint(g, threadIdx.x);
    if (threadIdx.x == 0) *out = now;
}
__global__ __launch_bounds__(64) void terna_repack_guard_kernel(RepackGuard g) { repack_guard_role(g, threadIdx.x); }

void launch_repack_fingerprint(const RepackGuard& guard, unsigned long long* out, hipStream_t st)
{
    terna_repack_fingerprint_kernel<<<1, 64, 0, st>>>(guard, out);
}

void launch_repack_guard(const RepackGuard* guard, hipStream_t st) { terna_repack_guard_kernel<<<1, 64, 0, st>>>(*guard); }

template void launch_decode_packed<int8_t>(const int8_t*, const uint32_t*, uint16_t*, const Epilogue&, int, int, int, hipStream_t,
                                           const RepackGuard*);
template void launch_decode_packed<uint16_t>(const uint16_t*, const uint32_t*, uint16_t*, const Epilogue&, int, int, int, hipStream_t,
                                             const RepackGuard*);

}  // namespace terna
