// Launchers of the MFMA-tiled kernels on the P2 layout (prefill_packed_kernel.h).  Compiled once per activation
// type (-DTERNA_PREFILL_ACT=int8_t | uint16_t): the two sets of instantiations build in parallel.
#include "launchers.h"
#include "host_util.h"
#include "prefill_packed_kernel.h"

#ifndef TERNA_PREFILL_ACT
#error "define TERNA_PREFILL_ACT (int8_t or uint16_t)"
#endif

namespace terna {
namespace {

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

}  // namespace

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

template void launch_prefill_packed<TERNA_PREFILL_ACT>(const TERNA_PREFILL_ACT*, const uint32_t*, uint16_t*, const Epilogue&, int, int, int,
                                                       hipStream_t);

}  // namespace terna
