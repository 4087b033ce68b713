// Decode attention with the deferred merge (attention_kernel.h, DEFER) for several sequences, one workgroup per
// (sequence, KV HEAD, split) instead of one per (sequence, head, split): the GQ = H / KV heads of a kv group read the same
// keys and values, and in the per-head form each of them pulls every cache line from L2 again -- at eight sequences of
// the 2B shape that is four times the requests and four times the bytes into the CUs.  Here a cache line is requested
// once on the whole chip:
//
//   pass 1  the score MFMA of attention_kernel.h has the head's q pieces in columns 0 .. R-1 of its B operand (R = D / 32
//           operand rows per key row) and zeros elsewhere; head g of the group now takes columns R g .. R g + R - 1, so
//           the same instructions on the same key registers give the scores of all GQ heads (GQ R <= 16); the R partial
//           scores of a slot sit in R neighbouring lanes of the head's columns and a quad (pair) permutation adds them
//   pass 2  softmax numerators per head
//   pass 3  a thread's value rows, loaded once, are weighted with the GQ heads' numerators
//
// Every head's arithmetic is the per-head kernel's in the same order (an MFMA column does not depend on the other
// columns), so the partial results are the same bits.  RoPE and the cache write of the new token are folded in as there
// (split 0 writes the kv head's new rows).
#pragma once

#include "attention_kernel.h"

namespace terna {

constexpr size_t grouped_attention_lds_bytes(int D, int NW, int GQ, int S)
{
    return static_cast<size_t>(GQ) * ((64 * NW / (D / 8)) * D + 64 * NW + ((S + 15) & ~15)) * sizeof(float);
}

template <int D, bool ADJACENT, int NW, int GQ>
__global__ __launch_bounds__(64 * NW) void terna_decode_attention_grouped_kernel(
    const uint16_t* __restrict__ q, uint16_t* __restrict__ cache_k, uint16_t* __restrict__ cache_v,
    const long long* __restrict__ pos, int KV, int S, int splits, int slots, int per_seq, float scale,
    const float* __restrict__ cosv_all, const float* __restrict__ sinv_all, float* __restrict__ partial, AttentionPrefetch pf)
{
    static_assert(D == 64 || D == 128, "head dimension");
    constexpr int CH = D / 8;                    // 8-dimension chunks of a row
    constexpr int NT = 64 * NW;
    constexpr int SLICES = NT / CH;
    constexpr int GROUPS = NT / D;               // threads per output dimension in the final sum
    constexpr int R = D / 32;                    // operand rows per key row
    constexpr int SPM = 16 / R;                  // slots per MFMA
    constexpr int NJ = D / 32;                   // MFMAs (32 dimensions each) per tile
    constexpr int KT = 4;                        // key tiles in flight per wave
    constexpr int VU = 8;                        // value rows in flight per thread
    static_assert(GQ >= 2 && GQ * R <= 16, "the heads' columns fit one MFMA");
    extern __shared__ __align__(16) float lds[];
    float* part = lds;                           // [GQ][SLICES][D]
    float* part2 = part + GQ * SLICES * D;       // [GQ][GROUPS][D]
    float* score = part2 + GQ * GROUPS * D;      // [GQ][SS]
    const int SS = (S + 15) & ~15;               // a head's scores: whole tiles
    __shared__ float red[2][NW][GQ];
    if (static_cast<int>(blockIdx.x) >= slots) {             // prefetch-only workgroups
        attention_prefetch_role(pf, slots, NT);
        return;
    }
    const int SP = splits;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int sp = blockIdx.x % SP;
    const int grp_id = blockIdx.x / SP;          // (sequence, kv head)
    const int b = grp_id / KV, kvh = grp_id - b * KV;
    const int H = KV * GQ;
    auto cache_slot = [&](int l) { return (((l >> 4) * SP + sp) << 4) + (l & 15); };
    const int pb = per_seq ? b : 0;
    const long long p0 = pos[pb];
    const float* cosv = cosv_all + pb * (D / 2);
    const float* sinv = sinv_all + pb * (D / 2);
    const uint16_t* kbase = cache_k + (static_cast<size_t>(b) * KV + kvh) * S * D;
    const uint16_t* vbase = cache_v + (static_cast<size_t>(b) * KV + kvh) * S * D;

    const int r16 = lane & 15, kblk = lane >> 4;
    const int chunk = tid % CH, slice = tid / CH;
    const int rr = r16 % R, sl = r16 / R;        // operand row of a key row and the slot of the MFMA (A side);
    const int gq = sl < GQ ? sl : GQ - 1;        // on the B side sl is the head of this lane's column
    const bool col_on = sl < GQ;
    const int piece = rr + R * kblk;             // this lane's 16 bytes (8 dimensions) of a key row, and of its head's q
    u32x4 kr[KT][NJ], vr[VU], qb;
    auto load_keys = [&](int ltile, u32x4 (&dst)[NJ]) {
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const int sk = 16 * (ltile * SP + sp) + SPM * j + sl;
            dst[j] = *reinterpret_cast<const u32x4*>(kbase + static_cast<size_t>(sk < S ? sk : 0) * D + 8 * piece);
        }
    };
    // requests in the per-head kernel's order: the new token's pieces and angles, the keys, the values
    u32x4 knew, vnew, q_own, k_own, q_par, k_par;
    f32x4 cs[2], sn[2];
    const u32x4 zero4 = {0u, 0u, 0u, 0u};
    const int c = piece;
    const int cp = (c + CH / 2) % CH, ca = c % (CH / 2);
    {
        const uint16_t* row = q + static_cast<size_t>(b) * (H + 2 * KV) * D;
        const int hq = kvh * GQ + gq;
        q_own = *reinterpret_cast<const u32x4*>(row + hq * D + 8 * c);
        k_own = *reinterpret_cast<const u32x4*>(row + (H + kvh) * D + 8 * c);
        vnew = *reinterpret_cast<const u32x4*>(row + (H + KV + kvh) * D + 8 * chunk);
        if constexpr (ADJACENT) {
            cs[0] = *reinterpret_cast<const f32x4*>(cosv + 4 * c);
            sn[0] = *reinterpret_cast<const f32x4*>(sinv + 4 * c);
        } else {
            q_par = *reinterpret_cast<const u32x4*>(row + hq * D + 8 * cp);
            k_par = *reinterpret_cast<const u32x4*>(row + (H + kvh) * D + 8 * cp);
            cs[0] = *reinterpret_cast<const f32x4*>(cosv + 8 * ca);
            cs[1] = *reinterpret_cast<const f32x4*>(cosv + 8 * ca + 4);
            sn[0] = *reinterpret_cast<const f32x4*>(sinv + 8 * ca);
            sn[1] = *reinterpret_cast<const f32x4*>(sinv + 8 * ca + 4);
        }
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int t = 0; t < KT; ++t) load_keys(wave + NW * t, kr[t]);
#pragma unroll
    for (int u = 0; u < VU; ++u) {
        const int sv = cache_slot(slice + u * SLICES);
        vr[u] = *reinterpret_cast<const u32x4*>(vbase + static_cast<size_t>(sv < S ? sv : 0) * D + chunk * 8);
    }
    __builtin_amdgcn_sched_barrier(0);
    const bool pos_ok = p0 >= 0 && p0 < S;
    const int n = p0 < 0 ? 1 : (p0 >= S ? S : static_cast<int>(p0) + 1);
    if constexpr (ADJACENT) {
        auto rotate = [&](const u32x4& own) {
            float a[8], o[8];
            unpack_bf16x8(own, a);
#pragma unroll
            for (int m = 0; m < 4; ++m) {
#pragma clang fp contract(off)
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
                const float lo = a[e] * cc - p[e] * sv;
                const float hi = a[e] * cc + p[e] * sv;
                o[e] = first_half ? lo : hi;
            }
            return pack_bf16x8(o);
        };
        qb = rotate(q_own, q_par);
        knew = rotate(k_own, k_par);
    }
    if (sp == 0 && pos_ok) {                     // the kv head's new rows: slot pos of both caches
        const size_t slot_off = ((static_cast<size_t>(b) * KV + kvh) * S + (n - 1)) * D;
        if (wave == 0 && r16 < R) *reinterpret_cast<u32x4*>(cache_k + slot_off + 8 * c) = knew;
        if (tid < CH) *reinterpret_cast<u32x4*>(cache_v + slot_off + 8 * chunk) = vnew;
    }
    if (!col_on) qb = zero4;                     // B operand: the heads' pieces in columns 0 .. GQ R - 1 only

    // ---- pass 1: this lane keeps the running maximum of ITS head (columns R sl ..)
    float mx = -INFINITY;
    auto score_tile = [&](int ltile, const u32x4 (&kin)[NJ]) {
        const int tile = ltile * SP + sp;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            u32x4 k = kin[j];
            if (16 * tile + SPM * j + sl == n - 1) k = knew;     // the new token's slot: its key row is in registers
            const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
            const f32x4 acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, k), __builtin_bit_cast(bf16x8, qb), zero, 0, 0, 0);
            if constexpr (R == 4) {              // rows 4 kblk + v of slot kblk: the partial of column R g + v is in row v
                float x = rr == 0 ? acc[0] : rr == 1 ? acc[1] : rr == 2 ? acc[2] : acc[3];
                x += dpp_permute<kDppSwapPairs>(x);
                x += dpp_permute<kDppSwapHalfQuads>(x);
                const int ls = SPM * j + kblk;
                if (rr == 0 && col_on && 16 * tile + ls < n) {
                    const float d = x * scale;
                    score[gq * SS + 16 * ltile + ls] = d;
                    mx = fmaxf(mx, d);
                }
            } else {                             // R == 2: rows 4 kblk + v of slots 2 kblk + (v >> 1): column 2 g + (v & 1)
                float x0 = rr == 0 ? acc[0] : acc[1];
                float x1 = rr == 0 ? acc[2] : acc[3];
                x0 += dpp_permute<kDppSwapPairs>(x0);
                x1 += dpp_permute<kDppSwapPairs>(x1);
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const int ls = SPM * j + 2 * kblk + e;
                    if (rr == 0 && col_on && 16 * tile + ls < n) {
                        const float d = (e ? x1 : x0) * scale;
                        score[gq * SS + 16 * ltile + ls] = d;
                        mx = fmaxf(mx, d);
                    }
                }
            }
        }
    };
    const int tiles = (n + 15) >> 4;
    const int ltiles = tiles > sp ? (tiles - sp + SP - 1) / SP : 0;
    const int nl = 16 * ltiles;
#pragma unroll
    for (int t = 0; t < KT; ++t)
        if (wave + NW * t < ltiles) score_tile(wave + NW * t, kr[t]);
    for (int tile = wave + NW * KT; tile < ltiles; tile += NW) {
        u32x4 k[NJ];
        load_keys(tile, k);
        score_tile(tile, k);
    }
    mx = cross_row_reduce<true>(mx);             // over the four k-blocks: lanes with the same column
    if (kblk == 0 && rr == 0 && col_on) red[0][wave][gq] = mx;
    __syncthreads();
    float mxh[GQ], sum[GQ];
#pragma unroll
    for (int g = 0; g < GQ; ++g) {
        mxh[g] = red[0][0][g];
#pragma unroll
        for (int w = 1; w < NW; ++w) mxh[g] = fmaxf(mxh[g], red[0][w][g]);
        sum[g] = 0.0f;
    }

    // ---- pass 2: softmax numerators and their sums
    for (int l = tid; l < nl; l += NT) {
        const bool ok = cache_slot(l) < n;
#pragma unroll
        for (int g = 0; g < GQ; ++g) {
            const float p = ok ? __expf(score[g * SS + l] - mxh[g]) : 0.0f;
            score[g * SS + l] = p;
            sum[g] += p;
        }
    }
#pragma unroll
    for (int g = 0; g < GQ; ++g) {
        sum[g] = wave_sum(sum[g]);
        if (lane == 0) red[1][wave][g] = sum[g];
    }
    __syncthreads();
#pragma unroll
    for (int g = 0; g < GQ; ++g) {
        sum[g] = red[1][0][g];
#pragma unroll
        for (int w = 1; w < NW; ++w) sum[g] += red[1][w][g];
    }

    // ---- pass 3: weighted sums of the value rows, every row loaded once for the GQ heads
    float acc[GQ][8];
#pragma unroll
    for (int g = 0; g < GQ; ++g)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[g][e] = 0.0f;
    for (int l0 = slice; l0 < nl; l0 += VU * SLICES) {
        if (l0 != slice) {
#pragma unroll
            for (int u = 0; u < VU; ++u) {
                const int l = l0 + u * SLICES;
                const int s = cache_slot(l);
                const bool ok = l < nl && s < n;
                vr[u] = *reinterpret_cast<const u32x4*>(vbase + static_cast<size_t>(ok ? s : 0) * D + chunk * 8);
            }
        }
#pragma unroll
        for (int u = 0; u < VU; ++u) {
            const int l = l0 + u * SLICES;
            const int s = cache_slot(l);
            const bool ok = l < nl && s < n;
            u32x4 row = vr[u];
            row = (s == n - 1) ? vnew : row;
            row = ok ? row : u32x4{0u, 0u, 0u, 0u};
            float vf[8];
            unpack_bf16x8(row, vf);
#pragma unroll
            for (int g = 0; g < GQ; ++g) {
                const float p = ok ? score[g * SS + (ok ? l : 0)] : 0.0f;
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[g][e] = fmaf(p, vf[e], acc[g][e]);
            }
        }
    }
#pragma unroll
    for (int g = 0; g < GQ; ++g)
#pragma unroll
        for (int e = 0; e < 8; ++e) part[(g * SLICES + slice) * D + chunk * 8 + e] = acc[g][e];
    __syncthreads();
    {
        const int d = tid % D, grp = tid / D;
#pragma unroll
        for (int g = 0; g < GQ; ++g) {
            float o = 0.0f;
#pragma unroll
            for (int s2 = 0; s2 < SLICES / GROUPS; ++s2) o += part[(g * SLICES + grp * (SLICES / GROUPS) + s2) * D + d];
            part2[(g * GROUPS + grp) * D + d] = o;
        }
    }
    __syncthreads();
    const size_t heads_total = static_cast<size_t>(slots / SP) * GQ;      // B * H
    for (int idx = tid; idx < GQ * D; idx += NT) {
        const int g = idx / D, d = idx - g * D;
        float o = 0.0f;
#pragma unroll
        for (int grp = 0; grp < GROUPS; ++grp) o += part2[(g * GROUPS + grp) * D + d];
        const size_t bh = static_cast<size_t>(b) * H + kvh * GQ + g;
        partial[attention_stat_floats(heads_total) + (bh * SP + sp) * D + d] = o;
    }
    if (tid < GQ) {
        float* stat = partial + (static_cast<size_t>(b) * H + kvh * GQ + tid) * kAttentionStatFloats;
        float m = red[0][0][tid], s = red[1][0][tid];
#pragma unroll
        for (int w = 1; w < NW; ++w) {
            m = fmaxf(m, red[0][w][tid]);
            s += red[1][w][tid];
        }
        stat[sp] = m;
        stat[kAttentionMaxSplits + sp] = s;
    }
}

}  // namespace terna
