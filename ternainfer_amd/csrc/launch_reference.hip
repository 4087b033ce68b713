// Launchers of the kernels that read the reference format directly (decode_kernel.h, prefill_kernel.h,
// decompress_kernel.h).
#include "launchers.h"
#include "host_util.h"
#include "decode_kernel.h"
#include "decompress_kernel.h"
#include "prefill_kernel.h"

namespace terna {

// Small-M kernel: one workgroup per 16-row band; up to 64 batch rows per workgroup.
template <typename Act, int WAVES, int MB, int DEPTH>
void launch_decode_as(const Act* x, const Weights& w, uint16_t* out, const Epilogue& ep, int M, int N, int K,
                      hipStream_t st)
{
    const dim3 grid(N / 16, (M + 16 * MB - 1) / (16 * MB));
    terna_decode_kernel<Act, WAVES, MB, DEPTH><<<grid, dim3(WAVES * 64), 0, st>>>(
        x, w.bitmap, w.tile_off, w.median_off, w.sign_words, out, M, N, K, ep);
}

// Shape of the small-M launch.  With one workgroup per 16-row band, a matrix with few bands
// (N/16 <= 256: at most one workgroup per CU) is bound by each wave's serial share of K, so it
// gets 16 waves and a deeper prefetch ring; a matrix with many bands is bound by how many
// workgroups fit on the chip at once, so it gets 8 waves and the leaner ring (<= 64 VGPRs).
// TERNASPMM_DECODE_WAVES=4|8|16 forces one variant (tuning aid).
int decode_waves_override()
{
    static const int waves = [] {
        const char* v = tuning_env("TERNASPMM_DECODE_WAVES");
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

void launch_decompress(const Weights& w, uint16_t* dense, int N, int K, hipStream_t st)
{
    terna_decompress_kernel<4><<<dim3(N / 16), dim3(256), 0, st>>>(w.bitmap, w.tile_off, w.median_off, w.sign_words, dense, N, K);
}

template void launch_decode<int8_t>(const int8_t*, const Weights&, uint16_t*, const Epilogue&, int, int, int, hipStream_t);
template void launch_decode<uint16_t>(const uint16_t*, const Weights&, uint16_t*, const Epilogue&, int, int, int, hipStream_t);
template void launch_prefill<int8_t>(const int8_t*, const Weights&, uint16_t*, const Epilogue&, int, int, int, hipStream_t);
template void launch_prefill<uint16_t>(const uint16_t*, const Weights&, uint16_t*, const Epilogue&, int, int, int, hipStream_t);

}  // namespace terna
