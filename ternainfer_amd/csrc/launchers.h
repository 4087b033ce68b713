// Host-side launchers of the TernaSpMM kernels.  Each kernel family is instantiated in a translation unit
// of its own (launch_*.hip), so that the library builds in parallel; the C ABI (ternaspmm.hip) only sees
// these declarations.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "terna_common.h"

namespace terna {

// The four tensors of the reference format.
struct Weights {
    const uint64_t* bitmap;
    const int* tile_off;
    const uint16_t* median_off;
    const uint32_t* sign_words;
};


// ---- reference format (launch_reference.hip) -------------------------------------------------------
// Small-M kernel on the reference format; Act = int8_t | uint16_t (bf16 storage).
template <typename Act>
void launch_decode(const Act* x, const Weights& w, uint16_t* out, const Epilogue& ep, int M, int N, int K, hipStream_t st);
// MFMA-tiled kernel that decodes the reference format on the fly (no workspace needed).
template <typename Act>
void launch_prefill(const Act* x, const Weights& w, uint16_t* out, const Epilogue& ep, int M, int N, int K, hipStream_t st);
// Reference format -> dense bf16 [N][K].
void launch_decompress(const Weights& w, uint16_t* dense, int N, int K, hipStream_t st);

// ---- P2 layout (launch_decode_packed.hip, launch_prefill_packed_*.hip) ---------------------------------
void launch_repack(const Weights& w, uint32_t* packed, int N, int K, hipStream_t st);
// `guard` (may be NULL): the launch also checks that `packed` still belongs to the caller's reference-format tensors.
template <typename Act>
void launch_decode_packed(const Act* x, const uint32_t* packed, uint16_t* out, const Epilogue& ep, int M, int N, int K,
                          hipStream_t st, const RepackGuard* guard = nullptr);
// The small-M int8 launch with the producing epilogue (M <= 16): out = bf16(residual + output), stats_out [M][N/16][2] under
// next_w; raw_out (optional) the output itself.
void launch_decode_packed_producer(const int8_t* x, const uint32_t* packed, uint16_t* out, const Epilogue& ep, int M, int N, int K,
                                   const uint16_t* residual, const uint16_t* next_w, float* stats_out, uint16_t* raw_out, hipStream_t st);
// Fingerprint of the reference-format tensors named by `guard` into *out / the check of it as a launch of its own.
void launch_repack_fingerprint(const RepackGuard& guard, unsigned long long* out, hipStream_t st);
void launch_repack_guard(const RepackGuard* guard, hipStream_t st);
// `scratch` (may be NULL; 16-byte aligned, scratch_bytes long): room for split-K partial sums when the shape has few
// output tiles for the chip; the call then enqueues two launches.  `guard` (may be NULL): the check of a cached copy;
// returns true when the launch carried it, false when the caller has to enqueue it (launch_repack_guard).
template <typename Act>
bool launch_prefill_packed(const Act* x, const uint32_t* packed, uint16_t* out, const Epilogue& ep, int M, int N, int K,
                           void* scratch, size_t scratch_bytes, hipStream_t st, const RepackGuard* guard = nullptr);
// What launch_prefill_packed does with a call (host arithmetic only, nothing is enqueued): the output tile, the
// grid, the split-K count and how many bytes of `scratch` the partial planes take (0 without a split; never more than
// scratch_bytes).
struct PrefillPlan {
    int bm, bn;                 // batch rows x output features per workgroup
    unsigned grid_x, grid_y;
    int steps;                  // K steps of one workgroup without a split
    int splits;
    bool direct_lds;            // activations loaded straight into LDS (16-byte aligned x, operands below 4 GiB)
    size_t scratch_used;        // splits * M * N * 4 when splits > 1
};
template <typename Act>
PrefillPlan plan_prefill_packed(const void* x, int M, int N, int K, const void* scratch, size_t scratch_bytes);

extern template void launch_decode<int8_t>(const int8_t*, const Weights&, uint16_t*, const Epilogue&, int, int, int, hipStream_t);
extern template void launch_decode<uint16_t>(const uint16_t*, const Weights&, uint16_t*, const Epilogue&, int, int, int, hipStream_t);
extern template void launch_prefill<int8_t>(const int8_t*, const Weights&, uint16_t*, const Epilogue&, int, int, int, hipStream_t);
extern template void launch_prefill<uint16_t>(const uint16_t*, const Weights&, uint16_t*, const Epilogue&, int, int, int, hipStream_t);
extern template void launch_decode_packed<int8_t>(const int8_t*, const uint32_t*, uint16_t*, const Epilogue&, int, int, int, hipStream_t,
                                                  const RepackGuard*);
extern template void launch_decode_packed<uint16_t>(const uint16_t*, const uint32_t*, uint16_t*, const Epilogue&, int, int, int, hipStream_t,
                                                    const RepackGuard*);
extern template bool launch_prefill_packed<int8_t>(const int8_t*, const uint32_t*, uint16_t*, const Epilogue&, int, int, int, void*, size_t,
                                                   hipStream_t, const RepackGuard*);
extern template bool launch_prefill_packed<uint16_t>(const uint16_t*, const uint32_t*, uint16_t*, const Epilogue&, int, int, int, void*, size_t,
                                                     hipStream_t, const RepackGuard*);

extern template PrefillPlan plan_prefill_packed<int8_t>(const void*, int, int, int, const void*, size_t);
extern template PrefillPlan plan_prefill_packed<uint16_t>(const void*, int, int, int, const void*, size_t);

// norm -> quantisation -> int8 linear on a P2 weight, statistics taken inside, plain store, up to 8 rows, in the
// wide-load form (chain_chunk_kernel.h; defined in abi_chain.hip).  False where the shape is not covered: nothing enqueued.
bool launch_norm_linear_chunk(const uint16_t* x, const uint16_t* norm_w, const uint32_t* packed, uint16_t* out, const uint16_t* ws,
                              int ws_num, int8_t* xq_out, uint16_t* s_out, int M, int N, int K, float eps, int quant_mode,
                              hipStream_t st);

// Tuning override shared by the two small-M launchers: TERNASPMM_DECODE_WAVES=4|8|16 forces one variant.
int decode_waves_override();

}  // namespace terna
