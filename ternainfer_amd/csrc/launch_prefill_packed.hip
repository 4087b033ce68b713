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

// Split-K: with few output tiles for the chip (small M x N) every workgroup walks all of K alone and most CUs idle.
// Given scratch memory the K steps are spread over `splits` workgroups per tile, each leaves a plane of raw partial sums
// ([splits][M][N] fp32 / int32) and a second launch adds the planes in split order and applies the epilogue (the int8
// family stays bit-exact: integer sums; the bf16 family sums in another order, within its tolerance).
// Rule, from timings of the four BitNet-2B matrices at M = 128 .. 512 with 1 .. 8 splits (a step is 64 columns of bf16
// or 128 of int8 activations): a split must keep 13 steps or more; up to 96 tiles three splits (six up to 48 tiles);
// up to 192 tiles three splits if K gives 48 steps or more, else none (the second launch and the partial planes then
// cost more than the shorter chains save); above that none.  Measured: down projection at M = 256 / 512, bf16
// 44.5 -> 22.5 us / 44.8 -> 29.3 us, int8 25.1 -> 17.5 / 25.9 -> 21.8; O projection at M = 256, bf16 18.6 -> 14.8.
// TERNASPMM_PREFILL_SPLITS=1..8 forces a count (tuning aid).
int prefill_splits(long tiles, int steps, int M, int N, size_t scratch_bytes)
{
    static const int forced = [] {
        const char* v = tuning_env("TERNASPMM_PREFILL_SPLITS");
        const int n = v ? std::atoi(v) : 0;
        return n >= 1 && n <= 8 ? n : 0;
    }();
    const long fit = static_cast<long>(scratch_bytes / (static_cast<size_t>(M) * N * 4));
    long sp = 1;
    if (forced) sp = forced;
    else if (tiles <= 48) sp = 6;
    else if (tiles <= 96) sp = 3;
    else if (tiles <= 192 && steps >= 48) sp = 3;
    if (!forced && sp > steps / 13) sp = steps / 13;
    if (sp > steps) sp = steps;
    if (sp > fit) sp = fit;
    return sp < 1 ? 1 : static_cast<int>(sp);
}

template <typename Act, int MB, int NA>
void launch_prefill_packed_dma_as(const Act* x, const uint32_t* packed, uint16_t* out, const Epilogue& ep, int M,
                                  int N, int K, const PrefillPlan& plan, void* scratch, hipStream_t st, const RepackGuard* guard)
{
    using S = PackedPrefillDmaSmem<MB>;
    auto kernel = terna_prefill_packed_dma_kernel<Act, MB, NA>;
    allow_dynamic_lds(kernel, S::kBytes, "hipFuncSetAttribute(prefill packed dma)", __LINE__);
    const int splits = plan.splits;
    // The check of a cached copy rides in the launch: as one more row of workgroups in y, or -- with split-K planes, whose
    // workgroup -> XCD pattern an extra row per plane would shift -- as the first workgroup of the reduce launch.
    const bool guard_row = guard != nullptr && splits == 1;
    const dim3 grid(plan.grid_x, plan.grid_y + (guard_row ? 1 : 0), plan.splits);
    static const int xcd_forced = [] {
        const char* v = tuning_env("TERNASPMM_PREFILL_XCD_MAP");
        return v ? std::atoi(v) : -1;
    }();
    // XCD-aware tile order (see the kernel): pays once the activations no longer fit one XCD's 4 MiB L2 --
    // below that the default order, which fetches every weight tile on one XCD only, moves less data.
    // TERNASPMM_PREFILL_XCD_MAP=0|1 forces it off / on (tuning aid).
    const bool big_x = static_cast<size_t>(M) * K * sizeof(Act) > (4u << 20);
    const int xcd_map = (plan.grid_y % 8 == 0) && (xcd_forced < 0 ? big_x : xcd_forced != 0);
    kernel<<<grid, dim3(256), S::kBytes, st>>>(x, packed, out, ep, M, N, K, xcd_map, splits, splits > 1 ? scratch : nullptr,
                                               guard_row ? 1 : 0, guard_row ? *guard : RepackGuard{});
    if (splits > 1) {
        using AccT = typename std::conditional<sizeof(Act) == 1, int, float>::type;
        const long quads = static_cast<long>(M) * (N >> 2);
        const bool guard_first = guard != nullptr;
        terna_splitk_reduce_kernel<AccT><<<dim3(static_cast<unsigned>((quads + 255) / 256) + (guard_first ? 1 : 0)), dim3(256), 0, st>>>(
            static_cast<const AccT*>(scratch), out, ep, M, N, splits, guard_first ? 1 : 0, guard_first ? *guard : RepackGuard{});
    }
}

// The direct-to-LDS kernel addresses both operands as a 64-bit base plus a 32-bit byte offset and
// loads 16-byte pieces of the activation rows.
inline bool prefill_dma_ok(const void* x, size_t act_bytes, int M, int N, int K)
{
    static const bool off = [] {
        const char* v = tuning_env("TERNASPMM_PREFILL_DMA");
        return v && std::atoi(v) == 0;
    }();
    return !off && (reinterpret_cast<uintptr_t>(x) & 15) == 0 && static_cast<uint64_t>(M) * K * act_bytes < (1ull << 32) &&
           static_cast<uint64_t>(N) * K / 4 < (1ull << 32);
}

}  // namespace

template <typename Act>
PrefillPlan plan_prefill_packed(const void* x, int M, int N, int K, const void* scratch, size_t scratch_bytes)
{
    // Batch rows per workgroup (64 / 128 / 256).  Measured on MI355X the 64-row tile wins at every
    // BitNet-2B shape: it runs four waves per SIMD, and occupancy hides more latency than the taller
    // tiles save in weight expansion.  TERNASPMM_PREFILL_BM=64|128|256 forces one (tuning aid).
    static const int forced = [] {
        const char* v = tuning_env("TERNASPMM_PREFILL_BM");
        const int bm = v ? std::atoi(v) : 0;
        return (bm == 64 || bm == 96 || bm == 128 || bm == 256) ? bm : 0;
    }();
    static const int forced_bn = [] {
        const char* v = tuning_env("TERNASPMM_PREFILL_BN");
        const int bn = v ? std::atoi(v) : 0;
        return (bn == 128 || bn == 256) ? bn : 0;
    }();
    PrefillPlan plan{};
    plan.bm = forced ? forced : 64;
    // 256-feature tiles expand every weight once per 64 batch rows with two MFMAs per operand read;
    // when they would leave most of the 1024 workgroup slots of the chip empty, 128-feature tiles
    // double the workgroup count instead.  TERNASPMM_PREFILL_BN=128|256 forces one (tuning aid).
    const long wg256 = static_cast<long>((N + 255) / 256) * ((M + 63) / 64);
    plan.bn = forced_bn ? forced_bn : (wg256 <= 640 ? 128 : 256);
    plan.direct_lds = prefill_dma_ok(x, sizeof(Act), M, N, K) && (plan.bm == 64 || plan.bm == 128);
    if (plan.direct_lds) {
        if (plan.bm == 128 && forced_bn != 128) plan.bn = 256;
    } else if (!(plan.bm == 64 && plan.bn == 128)) {
        plan.bn = 256;                       // the register-staged kernel has 256-feature tiles except at 64 x 128
    }
    plan.grid_x = static_cast<unsigned>((N + plan.bn - 1) / plan.bn);
    plan.grid_y = static_cast<unsigned>((M + plan.bm - 1) / plan.bm);
    plan.steps = sizeof(Act) == 1 ? ((K >> 6) + 1) >> 1 : K >> 6;
    plan.splits = 1;
    const bool scratch_ok = plan.direct_lds && scratch != nullptr && (reinterpret_cast<uintptr_t>(scratch) & 15) == 0 && (N & 3) == 0;
    if (scratch_ok) plan.splits = prefill_splits(static_cast<long>(plan.grid_x) * plan.grid_y, plan.steps, M, N, scratch_bytes);
    plan.scratch_used = plan.splits > 1 ? static_cast<size_t>(plan.splits) * M * N * 4 : 0;
    return plan;
}

template <typename Act>
bool launch_prefill_packed(const Act* x, const uint32_t* packed, uint16_t* out, const Epilogue& ep, int M, int N, int K,
                           void* scratch, size_t scratch_bytes, hipStream_t st, const RepackGuard* guard)
{
    PrefillPlan plan = plan_prefill_packed<Act>(x, M, N, K, scratch, scratch_bytes);
    if (plan.direct_lds && !(plan.bm == 64 && plan.bn == 128) && !epilogue_scales_per_tile(ep, N)) {
        // weight-scale groups that change inside a 32-feature tile: only the 128 x 64 instantiation carries the per-column
        // epilogue (unsplit: it then uses no more scratch than the plan reported)
        plan.bm = 64;
        plan.bn = 128;
        plan.grid_x = static_cast<unsigned>((N + 127) / 128);
        plan.grid_y = static_cast<unsigned>((M + 63) / 64);
        plan.splits = 1;
        plan.scratch_used = 0;
    }
    if (plan.direct_lds) {
        if (plan.grid_y >= 65535u) guard = nullptr;         // (no room for the checking row: the caller launches the check itself)
        if (plan.bm == 64 && plan.bn == 128) launch_prefill_packed_dma_as<Act, 2, 1>(x, packed, out, ep, M, N, K, plan, scratch, st, guard);
        else if (plan.bm == 128 && plan.bn == 128) launch_prefill_packed_dma_as<Act, 4, 1>(x, packed, out, ep, M, N, K, plan, scratch, st, guard);
        else if (plan.bm == 128) launch_prefill_packed_dma_as<Act, 4, 2>(x, packed, out, ep, M, N, K, plan, scratch, st, guard);
        else launch_prefill_packed_dma_as<Act, 2, 2>(x, packed, out, ep, M, N, K, plan, scratch, st, guard);
        return guard != nullptr;
    }
    if (plan.bm == 64 && plan.bn == 128) launch_prefill_packed_as<Act, 2, 1>(x, packed, out, ep, M, N, K, st);
    else if (plan.bm == 256) launch_prefill_packed_as<Act, 8>(x, packed, out, ep, M, N, K, st);
    else if (plan.bm == 96) launch_prefill_packed_as<Act, 3>(x, packed, out, ep, M, N, K, st);
    else if (plan.bm == 128) launch_prefill_packed_as<Act, 4>(x, packed, out, ep, M, N, K, st);
    else launch_prefill_packed_as<Act, 2>(x, packed, out, ep, M, N, K, st);
    return false;
}

template bool launch_prefill_packed<TERNA_PREFILL_ACT>(const TERNA_PREFILL_ACT*, const uint32_t*, uint16_t*, const Epilogue&, int, int, int,
                                                       void*, size_t, hipStream_t, const RepackGuard*);
template PrefillPlan plan_prefill_packed<TERNA_PREFILL_ACT>(const void*, int, int, int, const void*, size_t);

}  // namespace terna
