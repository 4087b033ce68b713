// The two attention-side kernels of a decode step around the fused qkv linear:
//
//   terna_rope_kv_store_kernel   rotary embedding of q and k, q re-laid out per head, k and v
//                                written into the KV cache at the new tokens' slots
//   terna_decode_attention_kernel  one new token per sequence attending over its cache prefix
//
// They stand where the reference calls xformers' rope_padded (model.py:218-229) and
// fmha.memory_efficient_attention_forward (model.py:231-233); both are absent third-party
// operators, restated here from their definitions (RoPE with given cos/sin tables, pairing either
// adjacent dimensions -- rope_padded's default, which the reference's checkpoints are laid out for
// -- or the two halves of a head; softmax(q K^T / sqrt(D)) V over the valid cache slots).
// fp32 inside, bf16 storage.
#pragma once

#include "norm_quant_kernel.h"

namespace terna {

// qkv   bf16 [B*T][(H + 2*KV) * D]   row b*T + t: q heads, then k heads, then v heads
// cosv, sinv  fp32 [T][D/2]          angle of (token t, pair j)        } per_seq != 0: one row per (sequence, token),
// pos   int64 [T]                    cache slot of token t             } [B][T][D/2] and [B][T] -- sequences of a batch
//                                                                        with different prefix lengths
// q_out bf16 [B][H][T][D]
// cache_k, cache_v  bf16 [B][KV][S][D]
// Pair j of a head is (a, b) = (x[2j], x[2j + 1]) when ADJACENT, else (x[j], x[j + D/2]):
//   a' = a cos - b sin,   b' = b cos + a sin.
template <bool ADJACENT>
__global__ __launch_bounds__(256) void terna_rope_kv_store_kernel(
    const uint16_t* __restrict__ qkv, const float* __restrict__ cosv, const float* __restrict__ sinv,
    const long long* __restrict__ pos, uint16_t* __restrict__ q_out, uint16_t* __restrict__ cache_k,
    uint16_t* __restrict__ cache_v, int T, int H, int KV, int D, int S, int per_seq)
{
    const int row = blockIdx.x;                  // b*T + t
    const int b = row / T, t = row - b * T;
    const int tr = per_seq ? row : t;            // row of the position / angle tables
    const int half = D >> 1;
    const int slots = H + 2 * KV;
    const uint16_t* src = qkv + static_cast<size_t>(row) * slots * D;
    const long long slot = pos[tr];
    const bool slot_ok = slot >= 0 && slot < S;  // a position outside the cache writes no k / v row (q is still rotated)
    if ((half & 7) == 0) {
        // 8 pairs per thread: 16-byte loads and stores, for the 2B model one pass of 240 threads
        const int per = half >> 3;
        for (int i = threadIdx.x; i < slots * per; i += blockDim.x) {
            const int hs = i / per, j = (i - hs * per) * 8;          // pairs j .. j+7
            // the two 8-element chunks that hold those pairs
            const int off1 = ADJACENT ? 2 * j : j, off2 = ADJACENT ? 2 * j + 8 : j + half;
            float x1[8], x2[8], o1[8], o2[8];
            unpack_bf16x8(*reinterpret_cast<const u32x4*>(src + hs * D + off1), x1);
            unpack_bf16x8(*reinterpret_cast<const u32x4*>(src + hs * D + off2), x2);
            if (hs < H + KV) {
                const f32x4* cp = reinterpret_cast<const f32x4*>(cosv + tr * half + j);
                const f32x4* sp = reinterpret_cast<const f32x4*>(sinv + tr * half + j);
                const f32x4 c0 = cp[0], c1 = cp[1], s0 = sp[0], s1 = sp[1];
                if constexpr (ADJACENT) {
#pragma unroll
                    for (int m = 0; m < 4; ++m) {
#pragma clang fp contract(off)                   // every product and sum rounded once: a defined result
                        o1[2 * m] = x1[2 * m] * c0[m] - x1[2 * m + 1] * s0[m];
                        o1[2 * m + 1] = x1[2 * m + 1] * c0[m] + x1[2 * m] * s0[m];
                        o2[2 * m] = x2[2 * m] * c1[m] - x2[2 * m + 1] * s1[m];
                        o2[2 * m + 1] = x2[2 * m + 1] * c1[m] + x2[2 * m] * s1[m];
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
#pragma clang fp contract(off)
                        const float c = e < 4 ? c0[e & 3] : c1[e & 3], sn = e < 4 ? s0[e & 3] : s1[e & 3];
                        o1[e] = x1[e] * c - x2[e] * sn;
                        o2[e] = x2[e] * c + x1[e] * sn;
                    }
                }
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) { o1[e] = x1[e]; o2[e] = x2[e]; }
            }
            uint16_t* dst;
            if (hs < H) dst = q_out + ((static_cast<size_t>(b) * H + hs) * T + t) * D;
            else if (hs < H + KV) dst = cache_k + ((static_cast<size_t>(b) * KV + (hs - H)) * S + slot) * D;
            else dst = cache_v + ((static_cast<size_t>(b) * KV + (hs - H - KV)) * S + slot) * D;
            if (hs >= H && !slot_ok) continue;
            *reinterpret_cast<u32x4*>(dst + off1) = pack_bf16x8(o1);
            *reinterpret_cast<u32x4*>(dst + off2) = pack_bf16x8(o2);
        }
        return;
    }
    for (int i = threadIdx.x; i < slots * half; i += blockDim.x) {
        const int hs = i / half, j = i - hs * half;
        const int ia = ADJACENT ? 2 * j : j, ib = ADJACENT ? 2 * j + 1 : j + half;
        const float x1 = bf16_bits_to_float(src[hs * D + ia]);
        const float x2 = bf16_bits_to_float(src[hs * D + ib]);
        uint16_t* dst;
        float o1 = x1, o2 = x2;
        if (hs < H + KV) {
#pragma clang fp contract(off)
            const float c = cosv[tr * half + j], s = sinv[tr * half + j];
            o1 = x1 * c - x2 * s;
            o2 = x2 * c + x1 * s;
        }
        if (hs < H) dst = q_out + ((static_cast<size_t>(b) * H + hs) * T + t) * D;
        else if (hs < H + KV) dst = cache_k + ((static_cast<size_t>(b) * KV + (hs - H)) * S + slot) * D;
        else dst = cache_v + ((static_cast<size_t>(b) * KV + (hs - H - KV)) * S + slot) * D;
        if (hs >= H && !slot_ok) continue;
        dst[ia] = float_to_bf16_bits(o1);
        dst[ib] = float_to_bf16_bits(o2);
    }
}

// One workgroup of NW waves per (sequence, head).  q bf16 [B][H][D]; keys / values of kv head
// h / (H/KV) at slots 0 .. pos[0] (per_seq != 0: sequence b has its own prefix, slots 0 .. pos[b], and with ROPE its
// own angle row, cosv / sinv [B][D/2]); out bf16 [B][H*D].  Dynamic LDS: decode_attention_lds_bytes().
// What the waves request up front covers 64 * NW slots of keys (four 16-slot tiles per wave) and
// 4096 * NW / D slots of values, so with few workgroups on the chip (one per head) more waves mean
// fewer dependent memory round trips.
//   pass 1  q K^T on the matrix cores, 16 slots per MFMA tile, four tiles per wave requested up front
//   pass 2  softmax over the scores in LDS
//   pass 3  thread (slice, chunk): slots slice, slice+S', ... x 8 dimensions of V, eight rows in
//           flight per thread; the slices are summed through LDS
//
// ROPE = true folds terna_rope_kv_store_kernel (one token per sequence) into the same launch: `q` is
// then the fused qkv row of the new token (bf16 [B][(H + 2*KV)*D]); every workgroup rotates its own
// q head and the new key row of its kv head in registers (same arithmetic, bit for bit), uses them
// -- and the new value row -- in place of cache slot pos[0], and the first workgroup of each kv
// group writes the new key / value rows into the cache for the steps to come.  ADJACENT selects
// the pairing of the rotation, as in terna_rope_kv_store_kernel.
//
// Split over the cache (SP = gridDim.y > 1): one CU streams a cache prefix at a few tens of GB/s, so
// with few heads on the chip the launch is bound by that.  Workgroup (b, h, sp) then takes the
// 16-slot tiles sp, sp + SP, ... and leaves its unnormalised result, its score maximum and its
// sum of numerators in `partial` ([B*H][SP][D + 2] floats); the last of a head's SP workgroups
// to arrive (counted in `arrived`, one int per head, zero before the first launch and zero again
// after every launch) merges the SP partials in split order -- the result does not depend on
// which workgroup arrives last -- and writes the output row.
constexpr int kAttentionMaxSplits = 8;
//
// DEFER = true: the split without the hand-off.  The grid is one-dimensional (so that the prefetching workgroups fit
// behind it): workgroup -> (sequence, head, split), the splits of a kv group's heads spread over the XCDs like the
// groups themselves.  Every workgroup leaves its partial result with plain stores and ends; whoever consumes the
// attention output in the NEXT launch merges the splits (attention_merge below: the arithmetic of the in-launch
// merge, so the same bits) -- the launch boundary is the synchronisation, which takes the 5 - 6 us of the
// arrival counter and the merging workgroup's dependent reads out of the step.  Layout of `partial` then:
//   floats [B*H][2][kAttentionMaxSplits]   score maximum / sum of numerators of every split (attention_stat_floats)
//   floats [B*H][SP][D]                    unnormalised results
constexpr int kAttentionStatFloats = 2 * kAttentionMaxSplits;          // per head
__device__ __host__ inline size_t attention_stat_floats(size_t heads) { return heads * kAttentionStatFloats; }

// Output dimension d of head bh from its SP partial results, in split order.
__device__ __forceinline__ float attention_merge(const float* __restrict__ stat, const float* __restrict__ o_head, int SP, int D, int d)
{
    float m_all = -INFINITY;
    for (int j = 0; j < SP; ++j) m_all = fmaxf(m_all, stat[j]);
    float num = 0.0f, den = 0.0f;
    for (int j = 0; j < SP; ++j) {
        const float w = __expf(stat[j] - m_all);                       // an empty split: exp(-inf) = 0
        num = fmaf(w, o_head[j * D + d], num);
        den = fmaf(w, stat[kAttentionMaxSplits + j], den);
    }
    return num / den;
}

// out bf16 [B*H][D] from the partial results of a DEFER launch: one workgroup of D threads per head.
template <int D>
__global__ __launch_bounds__(D) void terna_attention_merge_kernel(const float* __restrict__ partial, uint16_t* __restrict__ out,
                                                                  int heads, int SP)
{
    const int bh = blockIdx.x;
    const float* stat = partial + static_cast<size_t>(bh) * kAttentionStatFloats;
    const float* o_head = partial + attention_stat_floats(heads) + static_cast<size_t>(bh) * SP * D;
    out[static_cast<size_t>(bh) * D + threadIdx.x] = float_to_bf16_bits(attention_merge(stat, o_head, SP, D, threadIdx.x));
}
// terna_attention_merge_kernel and the norm kernel behind it (norm_quant_kernel.h) as one launch: one workgroup per
// sequence forms its merged row -- H * D columns, rounded to bf16: the bits the merge kernel stores -- in registers and
// runs the norm kernel's passes on it.  Everything a thread reads (its heads' statistics, SP partial results of eight
// columns per vector, the norm weights) is requested before the first use.  o_out (optional): the merged row.
template <int D, int SP, int NV>
__global__ __launch_bounds__(kNormThreads) void terna_attention_merge_norm_quant_kernel(
    const float* __restrict__ partial, const uint16_t* __restrict__ weight, int H, int heads_total, float eps,
    uint16_t* __restrict__ o_out, uint16_t* __restrict__ y_out, int8_t* __restrict__ xq_out, uint16_t* __restrict__ s_out, int quant_mode)
{
    static_assert(D % 8 == 0 && SP >= 1 && SP <= kAttentionMaxSplits && kAttentionMaxSplits == 8, "a vector lies inside one head");
    const int tid = threadIdx.x;
    const size_t row = blockIdx.x;
    const int K = H * D, nvec = K >> 3;
    u32x4 raw_w[NV];
    f32x4 st[NV][4], po[NV][SP][2];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int v = tid + i * kNormThreads;
        const int vc = v < nvec ? v : nvec - 1;
        const int head = (8 * vc) / D, d = (8 * vc) % D;
        const size_t bh = row * H + head;
        raw_w[i] = *reinterpret_cast<const u32x4*>(weight + 8 * vc);
        const f32x4* sp = reinterpret_cast<const f32x4*>(partial + bh * kAttentionStatFloats);
#pragma unroll
        for (int q = 0; q < 4; ++q) st[i][q] = sp[q];
        const float* op = partial + attention_stat_floats(static_cast<size_t>(heads_total)) + bh * SP * D + d;
#pragma unroll
        for (int j = 0; j < SP; ++j) {
            po[i][j][0] = *reinterpret_cast<const f32x4*>(op + j * D);
            po[i][j][1] = *reinterpret_cast<const f32x4*>(op + j * D + 4);
        }
    }
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        pin_registers(raw_w[i]);
#pragma unroll
        for (int q = 0; q < 4; ++q) pin_registers(st[i][q]);
#pragma unroll
        for (int j = 0; j < SP; ++j) {
            pin_registers(po[i][j][0]);
            pin_registers(po[i][j][1]);
        }
    }
    float h[NV][8];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int v = tid + i * kNormThreads;
        if (v < nvec) {
            // attention_merge's arithmetic on the values in registers
            float mx[SP], dn[SP];
#pragma unroll
            for (int j = 0; j < SP; ++j) {
                mx[j] = st[i][j >> 2][j & 3];
                dn[j] = st[i][2 + (j >> 2)][j & 3];
            }
            float m_all = -INFINITY;
#pragma unroll
            for (int j = 0; j < SP; ++j) m_all = fmaxf(m_all, mx[j]);
            float wj[SP], den = 0.0f;
#pragma unroll
            for (int j = 0; j < SP; ++j) {
                wj[j] = __expf(mx[j] - m_all);
                den = fmaf(wj[j], dn[j], den);
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                float num = 0.0f;
#pragma unroll
                for (int j = 0; j < SP; ++j) num = fmaf(wj[j], po[i][j][e >> 2][e & 3], num);
                h[i][e] = round_bf16(num / den);
            }
            if (o_out != nullptr) *reinterpret_cast<u32x4*>(o_out + row * K + 8 * v) = pack_bf16x8(h[i]);
        }
    }
    norm_quant_passes<NV>(h, raw_w, K, eps, row, y_out, xq_out, s_out, quant_mode);
}

// Extra workgroups of the attention launch (blockIdx.x >= heads) that pull up to kAttentionPrefetchRegions regions of
// device memory through the caches while the heads' workgroups -- one CU each -- do the attention:
// the weights of the launches that follow.  Unit u of a region goes to a workgroup on XCD (u mod 8),
// where the consuming workgroup u runs if its dispatch is spread round robin from XCD 0 as well.
constexpr int kAttentionPrefetchRegions = 6;
struct AttentionPrefetch {
    const u32x4* base[kAttentionPrefetchRegions];
    long long units[kAttentionPrefetchRegions];
    long long total_vecs[kAttentionPrefetchRegions];
    int unit_vecs[kAttentionPrefetchRegions];     // 0: a small region that every XCD fetches whole
    int count;            // regions
    int workgroups;       // extra workgroups, a multiple of 8 (0: none)
};

// A prefetching workgroup's XCD owns the units u = xcd, xcd + 8, ... of every region (all of a
// region without units).  These shares, laid end to end, are cut into equal ranges for the XCD's
// prefetching workgroups, and a thread requests up to kPrefetchBatch of its range's 16-byte
// vectors before it waits for any: a workgroup's part is one memory round trip, whatever the
// sizes of the units (unit by unit, with a wait after each, the largest part took six).
constexpr int kPrefetchBatch = 16;

__device__ __forceinline__ void attention_prefetch_role(const AttentionPrefetch& pf, int heads, int nthreads)
{
    const int p = blockIdx.x - heads;
    const uint32_t xcd = blockIdx.x & 7;
    const uint32_t per_xcd = pf.workgroups >> 3;
    // rank of this workgroup among those of its XCD
    const uint32_t rank = (p - ((xcd - (heads & 7) + 8) & 7)) >> 3;
    uint32_t share[kAttentionPrefetchRegions], uv[kAttentionPrefetchRegions], tot[kAttentionPrefetchRegions];
    float inv[kAttentionPrefetchRegions];
    uint32_t all = 0;
#pragma unroll
    for (int r = 0; r < kAttentionPrefetchRegions; ++r) {
        const bool on = r < pf.count;
        uv[r] = on ? static_cast<uint32_t>(pf.unit_vecs[r]) : 0u;
        tot[r] = on ? static_cast<uint32_t>(pf.total_vecs[r]) : 0u;
        const uint32_t units = on ? static_cast<uint32_t>(pf.units[r]) : 0u;
        const uint32_t mine = units > xcd ? (units - xcd + 7) >> 3 : 0u;
        share[r] = uv[r] == 0 ? tot[r] : mine * uv[r];
        inv[r] = uv[r] ? 1.0f / static_cast<float>(uv[r]) : 0.0f;
        all += share[r];
    }
    const uint32_t lo = static_cast<uint32_t>(static_cast<unsigned long long>(all) * rank / per_xcd);
    const uint32_t hi = static_cast<uint32_t>(static_cast<unsigned long long>(all) * (rank + 1) / per_xcd);
    uint32_t seen = 0;
    for (uint32_t g0 = lo; g0 < hi; g0 += kPrefetchBatch * nthreads) {
        u32x4 q[kPrefetchBatch];
#pragma unroll
        for (int j = 0; j < kPrefetchBatch; ++j) {
            const uint32_t g = g0 + j * nthreads + threadIdx.x;
            // region of g and the offset in this XCD's share of it
            uint32_t off = g, r_uv = uv[0], r_tot = tot[0];
            float r_inv = inv[0];
            const u32x4* r_base = pf.base[0];
            bool found = off < share[0];
#pragma unroll
            for (int r = 1; r < kAttentionPrefetchRegions; ++r) {
                off -= found ? 0u : share[r - 1];
                const bool here = !found && off < share[r];
                r_uv = here ? uv[r] : r_uv;
                r_tot = here ? tot[r] : r_tot;
                r_inv = here ? inv[r] : r_inv;
                r_base = here ? pf.base[r] : r_base;
                found = found || here;
            }
            // vector `off` of the share -> unit xcd + 8 (off / uv), vector off % uv of it (shares stay below 2^24 vectors:
            // the float quotient is off by one at most)
            uint32_t unit = static_cast<uint32_t>(static_cast<float>(off) * r_inv);
            unit -= unit * r_uv > off ? 1u : 0u;
            unit += (unit + 1) * r_uv <= off ? 1u : 0u;
            const uint32_t v = r_uv ? (xcd + 8 * unit) * r_uv + (off - unit * r_uv) : off;
            const bool ok = g < hi && found && v < r_tot;
            q[j] = r_base[ok ? v : 0];           // past the range: the region's first vector again, no branch around the load
        }
#pragma unroll
        for (int j = 0; j < kPrefetchBatch; ++j) seen |= q[j].x & q[j].y & q[j].z & q[j].w;
    }
    if (seen == 0xffffffffu && pf.count > kAttentionPrefetchRegions) *const_cast<u32x4*>(pf.base[0]) = u32x4{seen, 0u, 0u, 0u};   // never true: keeps the loads
}

// The unsplit launch as a producer: per (sequence, head) the partial statistics of the norm that reads the attention
// output -- (sum of o^2, max |o * norm_w|) over the head's D columns of the stored bf16 row, the form
// terna_quant_stats_kernel adds up (H partials per row).  norm_w is loaded unconditionally and must always point at H * D
// readable elements (the launcher passes q when no statistics are wanted); out = nullptr: none written.
struct AttentionStats {
    const uint16_t* norm_w;
    float2* out;                  // [B][H]
};

constexpr size_t decode_attention_lds_bytes(int D, int NW, int S)
{
    return (static_cast<size_t>(S) + (64 * NW / (D / 8)) * D + 64 * NW) * sizeof(float);
}

template <int D, bool ROPE, bool ADJACENT = false, int NW = 4, bool SPLIT = false, bool DEFER = false, int KT = 4>
__global__ __launch_bounds__(64 * NW) void terna_decode_attention_kernel(
    // what the first loads depend on comes first: the leading sixteen dwords of the arguments arrive in scalar registers
    const uint16_t* __restrict__ q, uint16_t* __restrict__ cache_k, uint16_t* __restrict__ cache_v,
    const long long* __restrict__ pos, int H, int KV, int S, int splits, int heads, int groups, int per_seq, float scale,
    const float* __restrict__ cosv_all, const float* __restrict__ sinv_all, uint16_t* __restrict__ out,
    float* partial, int* arrived, AttentionPrefetch pf, AttentionStats stats)
{
    static_assert(D == 64 || D == 128, "head dimension");
    constexpr int CH = D / 8;                    // 8-dimension chunks of a row
    constexpr int NT = 64 * NW;
    constexpr int SLICES = NT / CH;
    constexpr int GROUPS = NT / D;               // threads per output dimension in the final sum
    extern __shared__ __align__(16) float lds[];
    float* part = lds;                           // [SLICES][D]
    float* part2 = lds + SLICES * D;             // [GROUPS][D]
    float* score = part2 + GROUPS * D;           // [S]
    __shared__ float red[2 * NW];
    __shared__ int last_flag;
    if (static_cast<int>(blockIdx.x) >= heads) {             // prefetch-only workgroups
        attention_prefetch_role(pf, heads, 64 * NW);
        return;
    }

    static_assert(!DEFER || SPLIT, "the deferred merge is a variant of the split kernel");
    // SP = splits of the cache (= gridDim.y, or folded into blockIdx.x when DEFER), sp = this workgroup's split;
    // constants in the unsplit kernel
    const int SP = SPLIT ? splits : 1;
    int sp = SPLIT && !DEFER ? blockIdx.y : 0;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    // Workgroup -> (sequence, head).  Workgroups go to the 8 XCDs round robin, and the H / KV heads of a kv group read
    // the same keys and values: with groups > 0 (= B * KV) the heads of group G all sit on XCD G mod 8, so that the
    // group's cache prefix crosses the fabric once and its other heads hit in that L2 (the grid is padded to whole
    // rounds of 8 groups; workgroups without a group leave).  groups = 0: heads in launch order.
    // DEFER: the same with (group, split) pairs in place of groups -- the heads of a group read the same tiles of a split.
    int b, h;
    if (groups > 0) {
        const int per = H / KV, q = blockIdx.x >> 3;
        int G = 8 * (q / per) + (blockIdx.x & 7);
        if (G >= (DEFER ? groups * SP : groups)) return;
        if constexpr (DEFER) {
            sp = G % SP;
            G /= SP;
        }
        b = G / KV;
        h = (G - b * KV) * per + q % per;
    } else {
        int u = blockIdx.x;
        if constexpr (DEFER) {
            sp = u % SP;
            u /= SP;
        }
        b = u / H;
        h = u - b * H;
    }
    // local slot l of this split (16 * local tile + row) -> cache slot
    auto cache_slot = [&](int l) { return (((l >> 4) * SP + sp) << 4) + (l & 15); };
    const int bh = b * H + h;
    const int kvh = h / (H / KV);
    const int pb = per_seq ? b : 0;              // row of the position / angle tables
    // (the position is requested here and first looked at after every other request of the launch has been issued: none
    // of their addresses depends on it, and waiting for it first put one memory round trip in front of all the others)
    const long long p0 = pos[pb];
    const float* cosv = cosv_all + pb * (D / 2);
    const float* sinv = sinv_all + pb * (D / 2);
    const uint16_t* kbase = cache_k + (static_cast<size_t>(b) * KV + kvh) * S * D;
    const uint16_t* vbase = cache_v + (static_cast<size_t>(b) * KV + kvh) * S * D;

    // Everything the first round of each pass needs is requested before anything is used: KT key
    // tiles per wave, the first VU value rows of this thread's slice, q.  Slots >= n hold stale or
    // unwritten cache lines; they are read (the cache is S slots long) and masked out below.
    //
    // ---- pass 1: scores on the matrix cores.  A tile is 16 cache slots; one v_mfma_f32_16x16x32_bf16
    // takes 16 / R of them, R = D / 32: a key row is R rows of the A operand, 32 dimensions each.
    // Lane L (row i = L & 15, k-block L >> 4) loads the 16-byte piece (i % R) + R (L >> 4) of slot
    // i / R, so four consecutive lanes fetch 64 consecutive bytes: the memory pipeline of a CU
    // handles a load four lanes at a time and takes one step per 64-byte segment these touch, and a
    // load whose consecutive lanes sit in different key rows (the plain operand layout: row L & 15)
    // streams at a quarter of the rate (25 against 80 bytes per clock from L2, measured).  The B
    // operand holds q's matching pieces in column i % R (zero elsewhere), so out[i][i % R] is the
    // partial score of row i and a slot's score is the sum over its R rows: the accumulator puts
    // them in R neighbouring lanes (columns 0 .. R-1), one quad permutation or two add them up.
    constexpr int NJ = D / 32;                   // MFMAs (32 dimensions each) per tile
    // KT key tiles in flight per wave (slots 0 .. 64 NW KT - 1 of the split; tiles beyond go through the loop below, one
    // dependent round trip each).  The launcher picks KT so that the requests just cover the cache: every request costs the
    // CU's address unit a slot whatever it returns, and a test in the kernel -- even a wave-uniform one on a kernel argument
    // -- made the waits around the requests conservative (8 sequences, caches of 384 slots: four tiles 6951 tokens/s,
    // three 7001, four with the fourth behind such a test 6919).
    constexpr int VU = 8;                        // value rows in flight per thread
    const int r16 = lane & 15, kblk = lane >> 4;
    const int chunk = tid % CH, slice = tid / CH;
    constexpr int R = D / 32;                    // operand rows per key row
    constexpr int SPM = 16 / R;                  // slots per MFMA
    const int rr = r16 % R, sl = r16 / R;
    const int piece = rr + R * kblk;             // this lane's 16 bytes (8 dimensions) of a key row, and of q
    u32x4 kr[KT][NJ], vr[VU], qb;
    // Cache rows come through raw buffer loads over the kv head's S rows: a slot past the cache costs an instruction slot
    // but neither a memory access nor a returned kilobyte (a clamped address did both).
    const __amdgpu_buffer_rsrc_t rk = make_raw_buffer(kbase, static_cast<uint32_t>(S) * D * 2u);
    const __amdgpu_buffer_rsrc_t rv = make_raw_buffer(vbase, static_cast<uint32_t>(S) * D * 2u);
    auto load_keys = [&](int ltile, u32x4 (&dst)[NJ]) {
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const int sk = 16 * (ltile * SP + sp) + SPM * j + sl;
            dst[j] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rk, (sk * D + 8 * piece) * 2, 0, 0));
        }
    };
    // Order of the requests: the new token's own row pieces and angles first (ROPE) -- loads return in order, so
    // the rotation can run while the cache rows are still on their way -- then the keys, then the values.
    u32x4 knew, vnew;                            // ROPE: the new token's key piece of this lane, value chunk of this thread
    u32x4 q_own, k_own, q_par, k_par;            // raw pieces of the new token's q / k rows (q_par, k_par: rotate-half partners)
    f32x4 cs[2], sn[2];
    const u32x4 zero4 = {0u, 0u, 0u, 0u};
    const int c = piece;                         // chunk c = dimensions 8c .. 8c+7
    const int cp = (c + CH / 2) % CH, ca = c % (CH / 2);      // rotate-half: the partner chunk, the angle chunk
    if constexpr (!ROPE) {
        qb = *reinterpret_cast<const u32x4*>(q + (static_cast<size_t>(b) * H + h) * D + 8 * piece);
    } else {
        const uint16_t* row = q + static_cast<size_t>(b) * (H + 2 * KV) * D;
        q_own = *reinterpret_cast<const u32x4*>(row + h * D + 8 * c);
        k_own = *reinterpret_cast<const u32x4*>(row + (H + kvh) * D + 8 * c);
        vnew = *reinterpret_cast<const u32x4*>(row + (H + KV + kvh) * D + 8 * chunk);
        if constexpr (ADJACENT) {                // a chunk holds the pairs 4c .. 4c+3 whole
            cs[0] = *reinterpret_cast<const f32x4*>(cosv + 4 * c);
            sn[0] = *reinterpret_cast<const f32x4*>(sinv + 4 * c);
        } else {                                 // the chunk and its rotation partner c +- CH/2
            q_par = *reinterpret_cast<const u32x4*>(row + h * D + 8 * cp);
            k_par = *reinterpret_cast<const u32x4*>(row + (H + kvh) * D + 8 * cp);
            cs[0] = *reinterpret_cast<const f32x4*>(cosv + 8 * ca);
            cs[1] = *reinterpret_cast<const f32x4*>(cosv + 8 * ca + 4);
            sn[0] = *reinterpret_cast<const f32x4*>(sinv + 8 * ca);
            sn[1] = *reinterpret_cast<const f32x4*>(sinv + 8 * ca + 4);
        }
    }
    uint32_t nw_raw = 0u;                        // this thread's norm weight (unsplit launch: the statistics of the output row)
    if constexpr (!SPLIT && !DEFER) nw_raw = stats.norm_w[h * D + (tid & (D - 1))];
    __builtin_amdgcn_sched_barrier(0);           // the requests above stay above the ones below
#pragma unroll
    for (int t = 0; t < KT; ++t) load_keys(wave + NW * t, kr[t]);
#pragma unroll
    for (int u = 0; u < VU; ++u) {
        const int sv = cache_slot(slice + u * SLICES);
        vr[u] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rv, (sv * D + chunk * 8) * 2, 0, 0));
    }
    __builtin_amdgcn_sched_barrier(0);           // everything is requested; only now the position is looked at
    // Prefix length: slots 0 .. pos.  It comes from device memory the host cannot check, so it is clamped to the
    // cache -- the LDS score buffer and every cache address are sized by S -- and a position outside [0, S) writes no
    // cache row below (the attention then runs over the clamped prefix; its result is not meaningful, but in bounds).
    const bool pos_ok = p0 >= 0 && p0 < S;
    const int n = p0 < 0 ? 1 : (p0 >= S ? S : static_cast<int>(p0) + 1);
    if constexpr (ROPE) {
        if constexpr (ADJACENT) {
            auto rotate = [&](const u32x4& own) {
                float a[8], o[8];
                unpack_bf16x8(own, a);
#pragma unroll
                for (int m = 0; m < 4; ++m) {
#pragma clang fp contract(off)                   // as terna_rope_kv_store_kernel: every product and sum rounded once
                    o[2 * m] = a[2 * m] * cs[0][m] - a[2 * m + 1] * sn[0][m];
                    o[2 * m + 1] = a[2 * m + 1] * cs[0][m] + a[2 * m] * sn[0][m];
                }
                return pack_bf16x8(o);
            };
            qb = rotate(q_own);
            knew = rotate(k_own);
        } else {
            const bool first_half = c < CH / 2;
            auto rotate = [&](const u32x4& own, const u32x4& par) {
                float a[8], p[8], o[8];
                unpack_bf16x8(own, a);
                unpack_bf16x8(par, p);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
#pragma clang fp contract(off)
                    const float cc = cs[e >> 2][e & 3], sv = sn[e >> 2][e & 3];
                    const float lo = a[e] * cc - p[e] * sv;    // own chunk in the first half:  x1 c - x2 s
                    const float hi = a[e] * cc + p[e] * sv;    // own chunk in the second half: x2 c + x1 s
                    o[e] = first_half ? lo : hi;
                }
                return pack_bf16x8(o);
            };
            qb = rotate(q_own, q_par);
            knew = rotate(k_own, k_par);
        }
        if (h % (H / KV) == 0 && sp == 0 && pos_ok) {      // this kv group's writer: slot pos of both caches
            const size_t slot_off = ((static_cast<size_t>(b) * KV + kvh) * S + (n - 1)) * D;
            if (wave == 0 && r16 < R) *reinterpret_cast<u32x4*>(cache_k + slot_off + 8 * c) = knew;   // r16 < R: every chunk once
            if (tid < CH) *reinterpret_cast<u32x4*>(cache_v + slot_off + 8 * chunk) = vnew;
        }
    }
    if (r16 >= R) qb = zero4;                    // B operand: q's pieces in columns 0 .. R-1 only

    float mx = -INFINITY;
    auto score_tile = [&](int ltile, const u32x4 (&kin)[NJ]) {       // ltile: local tile of this split
        const int tile = ltile * SP + sp;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            u32x4 k = kin[j];
            if constexpr (ROPE) {                // the new token's slot: its key row is in registers, not in the cache yet
                if (16 * tile + SPM * j + sl == n - 1) k = knew;
            }
            const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
            const f32x4 acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, k), __builtin_bit_cast(bf16x8, qb), zero, 0, 0, 0);
            // lane (column c = r16, rows 4 kblk + v): row i's partial score is out[i][i % R]
            if constexpr (R == 4) {              // rows 4 kblk + v of slot kblk: column v, lanes 16 kblk + 0 .. 3
                float x = r16 == 0 ? acc[0] : r16 == 1 ? acc[1] : r16 == 2 ? acc[2] : acc[3];
                x += dpp_permute<kDppSwapPairs>(x);
                x += dpp_permute<kDppSwapHalfQuads>(x);
                const int ls = SPM * j + kblk;   // slot within the tile
                if (r16 == 0 && 16 * tile + ls < n) {
                    const float d = x * scale;
                    score[16 * ltile + ls] = d;
                    mx = fmaxf(mx, d);
                }
            } else {                             // R == 2: rows 4 kblk + v of slots 2 kblk + (v >> 1): column v & 1
                float x0 = r16 == 0 ? acc[0] : acc[1];
                float x1 = r16 == 0 ? acc[2] : acc[3];
                x0 += dpp_permute<kDppSwapPairs>(x0);
                x1 += dpp_permute<kDppSwapPairs>(x1);
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const int ls = SPM * j + 2 * kblk + e;
                    if (r16 == 0 && 16 * tile + ls < n) {
                        const float d = (e ? x1 : x0) * scale;
                        score[16 * ltile + ls] = d;
                        mx = fmaxf(mx, d);
                    }
                }
            }
        }
    };
    const int tiles = (n + 15) >> 4;                                  // tiles with a valid slot, all splits
    const int ltiles = tiles > sp ? (tiles - sp + SP - 1) / SP : 0;  // ... of this split
    const int nl = 16 * ltiles;                                       // local slots (the last tile may be partly valid)
#pragma unroll
    for (int t = 0; t < KT; ++t)
        if (wave + NW * t < ltiles) score_tile(wave + NW * t, kr[t]);
    for (int tile = wave + NW * KT; tile < ltiles; tile += NW) {      // beyond the tiles requested up front: plain loop
        u32x4 k[NJ];
        load_keys(tile, k);
        score_tile(tile, k);
    }
    mx = wave_max(mx);
    if (lane == 0) red[wave] = mx;
    __syncthreads();
    mx = red[0];
#pragma unroll
    for (int w = 1; w < NW; ++w) mx = fmaxf(mx, red[w]);

    // ---- pass 2: softmax numerators and their sum (each thread revisits the slots it scored)
    float sum = 0.0f;
    for (int l = tid; l < nl; l += NT) {
        const float p = cache_slot(l) < n ? __expf(score[l] - mx) : 0.0f;
        score[l] = p;
        sum += p;
    }
    sum = wave_sum(sum);
    if (lane == 0) red[NW + wave] = sum;
    __syncthreads();
    sum = red[NW];
#pragma unroll
    for (int w = 1; w < NW; ++w) sum += red[NW + w];

    // ---- pass 3: weighted sum of the value rows, VU rows per round (the first round is already here)
    float acc[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    for (int l0 = slice; l0 < nl; l0 += VU * SLICES) {
        if (l0 != slice) {                       // all VU rows of the round requested before any is used
#pragma unroll
            for (int u = 0; u < VU; ++u) {
                const int l = l0 + u * SLICES;
                const int s = cache_slot(l);
                const bool ok = l < nl && s < n; // past the end: re-read slot 0, it gets weight 0 below
                vr[u] = *reinterpret_cast<const u32x4*>(vbase + static_cast<size_t>(ok ? s : 0) * D + chunk * 8);
            }
        }
#pragma unroll
        for (int u = 0; u < VU; ++u) {
            const int l = l0 + u * SLICES;
            const int s = cache_slot(l);
            const bool ok = l < nl && s < n;
            const float p = ok ? score[ok ? l : 0] : 0.0f;
            u32x4 row = vr[u];
            if constexpr (ROPE) row = (s == n - 1) ? vnew : row;
            row = ok ? row : u32x4{0u, 0u, 0u, 0u};          // never multiply stale cache contents (could be NaN)
            float vf[8];
            unpack_bf16x8(row, vf);
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[e] = fmaf(p, vf[e], acc[e]);
        }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) part[slice * D + chunk * 8 + e] = acc[e];
    __syncthreads();
    {                                            // GROUPS threads per dimension, SLICES / GROUPS slices each
        const int d = tid % D, grp = tid / D;
        float o = 0.0f;
#pragma unroll
        for (int sl = 0; sl < SLICES / GROUPS; ++sl) o += part[(grp * (SLICES / GROUPS) + sl) * D + d];
        part2[grp * D + d] = o;
    }
    __syncthreads();
    float o = 0.0f;
    if (tid < D) {
#pragma unroll
        for (int grp = 0; grp < GROUPS; ++grp) o += part2[grp * D + tid];
    }
    uint16_t* orow = out + (static_cast<size_t>(b) * H + h) * D;
    if ((!SPLIT || SP == 1) && !DEFER) {        // (DEFER has no output row: `out` is NULL there, also with one split)
        float v = 0.0f;
        if (tid < D) {
            const uint16_t ob = float_to_bf16_bits(o / sum);
            orow[tid] = ob;
            v = bf16_bits_to_float(ob);
        }
        if constexpr (!SPLIT) {
            if (stats.out != nullptr) {          // uniform: the row's statistics under the next norm, D columns = D / 64 waves
                float ssq = v * v;
                float pm = tid < D ? fabsf(__fmul_rn(v, __uint_as_float(nw_raw << 16))) : 0.0f;
                ssq = wave_sum(ssq);
                pm = wave_max(pm);
                if (lane == 0 && wave < D / 64) {
                    red[wave] = ssq;
                    red[NW + wave] = pm;
                }
                __syncthreads();
                if (tid == 0) {
                    float2 r{red[0], red[NW]};
                    if constexpr (D == 128) r = float2{red[0] + red[1], fmaxf(red[NW], red[NW + 1])};
                    stats.out[bh] = r;
                }
            }
        }
        return;
    }

    // ---- split: publish (o, mx, sum), count the arrival; the last workgroup of the head merges.
    // The partials and the counter are written and read with device-scope relaxed atomics: those go
    // past the per-XCD L2 to the memory all XCDs share, so no cache write-back or invalidate (what a
    // device-scope fence would cost every workgroup) is needed.  Order, made explicit: every storing
    // wave waits until the memory system has acknowledged its own partial stores (vmcnt(0): the
    // workgroup barrier alone orders instructions, not their completion, and the counter lives in
    // another memory channel than the partials), then the barrier, then ONE thread counts the arrival;
    // the merging workgroup issues its loads only after it has seen the full count.
    if constexpr (DEFER) {
        const int heads_total = groups > 0 ? groups * (H / KV) : heads / SP;           // B * H
        float* stat = partial + static_cast<size_t>(bh) * kAttentionStatFloats;
        float* o_out = partial + attention_stat_floats(static_cast<size_t>(heads_total)) + (static_cast<size_t>(bh) * SP + sp) * D;
        if (tid < D) o_out[tid] = o;
        if (tid == 0) {
            stat[sp] = mx;
            stat[kAttentionMaxSplits + sp] = sum;
        }
        return;
    }
    float* mine = partial + (static_cast<size_t>(bh) * SP + sp) * (D + 2);
    auto publish = [](float* p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); };
    auto fetch = [](const float* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); };
    if (tid < D) publish(mine + tid, o);
    if (tid == 0) {
        publish(mine + D, mx);
        publish(mine + D + 1, sum);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");     // this wave's partial stores have reached device memory
    __syncthreads();                             // ... and so have those of every other wave of the workgroup
    if (tid == 0)
        last_flag = __hip_atomic_fetch_add(arrived + bh, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == SP - 1;
    __syncthreads();
    if (!last_flag) return;
    if (tid < D) {
        const float* head = partial + static_cast<size_t>(bh) * SP * (D + 2);
        float m_all = -INFINITY;
        for (int j = 0; j < SP; ++j) m_all = fmaxf(m_all, fetch(head + j * (D + 2) + D));
        float num = 0.0f, den = 0.0f;
        for (int j = 0; j < SP; ++j) {
            const float w = __expf(fetch(head + j * (D + 2) + D) - m_all);      // an empty split: exp(-inf) = 0
            num = fmaf(w, fetch(head + j * (D + 2) + tid), num);
            den = fmaf(w, fetch(head + j * (D + 2) + D + 1), den);
        }
        orow[tid] = float_to_bf16_bits(num / den);
    }
    // every split has arrived: ready for the next launch
    if (tid == 0) __hip_atomic_store(arrived + bh, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace terna
