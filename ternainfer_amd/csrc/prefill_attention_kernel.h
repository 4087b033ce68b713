// Multi-token attention over the padded KV cache: the prompt pass of a block (model.py:231-233, where the
// reference calls fmha.memory_efficient_attention_forward on the cache after rope_padded has written the new rows).
//
//   q      bf16 [B][H][T][D]          rotated queries of the T new tokens (ternaspmm_rope_kv_store's q_out)
//   cache  bf16 [B][KV][S][D]         keys / values; the new tokens' rows are already in their slots
//   pos    int64 [T]                  cache slot of new token t; it sees the slots 0 .. pos[t]
//                                     (per_seq != 0: [B][T], sequence b's token t sees 0 .. pos[b][t])
//   out    bf16 [B*T][H*D]            row b*T + t: softmax(scale * q K^T) V, head h in columns h*D ..
//
// One wave per (sequence, head, block of 16 queries), flash-attention style over blocks of 32 cache slots, both
// products on the matrix cores (v_mfma_f32_16x16x32_bf16) in the TRANSPOSED form, so that a score tile comes out of
// the first product in exactly the register layout the second one wants as its B operand:
//   S^T = K Q^T :  A = 16 keys x 32 dims (16 bytes of a key row per lane, straight from the cache),
//                  B = Q^T, held in registers for the whole kernel; lane L ends up with keys 4 (L >> 4) + v,
//                  v = 0 .. 3, of query L & 15 -- all of a lane's scores belong to ONE query, so the running
//                  maximum, the rescale factor and the running sum are per-lane scalars, completed over the
//                  four lanes of a query with two cross-lane exchanges;
//   O^T = V^T P^T: B = P^T: the eight probabilities a lane holds after two score tiles (bf16), as they are;
//                  the k index of this product is a POSITION, position 8g + e of lane group g = L >> 4 standing for
//                  key 4g + e (e < 4) or 16 + 4g + e - 4 of the block -- any one-to-one assignment of keys to
//                  positions works as long as A uses the same one;
//                  A = V^T: row d, those eight keys -- gathered as eight 2-byte reads from the value block staged
//                  in LDS (row pitch 2 D + 8 bytes: the four lane groups fall into disjoint banks).
// fp32 running maximum / sum / output, exp via v_exp_f32, probabilities as a sum of two bf16 terms in the second product.
#pragma once

#include "norm_quant_kernel.h"

namespace terna {

constexpr int kPrefillAttnKeys = 32;          // cache slots per block

template <int D>
__global__ __launch_bounds__(64) void terna_prefill_attention_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ cache_k, const uint16_t* __restrict__ cache_v,
    const long long* __restrict__ pos, uint16_t* __restrict__ out, int T, int H, int KV, int S, float scale, int per_seq)
{
    static_assert(D == 64 || D == 128, "head size");
    constexpr int DS = D / 32;                // 32-dimension slices of a row (first product)
    constexpr int DT = D / 16;                // 16-dimension tiles of the output (second product)
    constexpr int PITCH = 2 * D + 8;          // bytes between value rows in LDS
    __shared__ __align__(16) uint8_t vblk[kPrefillAttnKeys * PITCH];

    const int lane = threadIdx.x;
    const int qi = lane & 15, g = lane >> 4;
    const int t0 = blockIdx.x * 16, h = blockIdx.y, b = blockIdx.z;
    const int kvh = h / (H / KV);
    const int t = t0 + qi < T ? t0 + qi : T - 1;                     // rows past T repeat the last one and are not stored
    // prefix length of this lane's query, clamped to the cache (pos comes from device memory)
    long long p64 = pos[(per_seq ? b * T : 0) + t];
    p64 = p64 < 0 ? 0 : (p64 >= S ? S - 1 : p64);
    const int my_last = static_cast<int>(p64);                        // last visible slot
    int n_keys = my_last + 1;
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) n_keys = max(n_keys, __shfl_xor(n_keys, off));
    n_keys = __builtin_amdgcn_readfirstlane(n_keys);                  // largest prefix of the block's queries

    const uint16_t* qrow = q + ((static_cast<size_t>(b) * H + h) * T + t) * D;
    bf16x8 bq[DS];
#pragma unroll
    for (int ds = 0; ds < DS; ++ds) bq[ds] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(qrow + 32 * ds + 8 * g));
    const uint16_t* kbase = cache_k + (static_cast<size_t>(b) * KV + kvh) * S * D;
    const uint16_t* vbase = cache_v + (static_cast<size_t>(b) * KV + kvh) * S * D;

    f32x4 o[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[dt] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    float m_run = -1e30f, l_run = 0.0f;

    for (int k0 = 0; k0 < n_keys; k0 += kPrefillAttnKeys) {
        // ---- requests of the block: key pieces for the two score tiles, value rows for LDS
        u32x4 kr[2][DS];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            int key = k0 + 16 * j + qi;
            key = key < S ? key : S - 1;
#pragma unroll
            for (int ds = 0; ds < DS; ++ds) kr[j][ds] = *reinterpret_cast<const u32x4*>(kbase + static_cast<size_t>(key) * D + 32 * ds + 8 * g);
        }
        constexpr int VPR = D / 8;            // 16-byte vectors per value row
        constexpr int VL = kPrefillAttnKeys * VPR / 64;
        u32x4 vr[VL];
#pragma unroll
        for (int u = 0; u < VL; ++u) {
            const int idx = lane + 64 * u;
            const int key = k0 + idx / VPR;
            // slots past the block's largest prefix were never written (they may hold anything, NaN included, and
            // 0 * NaN would poison the product): read an in-range row instead and zero it
            const u32x4 row = *reinterpret_cast<const u32x4*>(vbase + static_cast<size_t>(key < n_keys ? key : 0) * D + (idx % VPR) * 8);
            vr[u] = key < n_keys ? row : u32x4{0u, 0u, 0u, 0u};
        }
        // ---- scores, transposed: lane = (query qi, keys 4g + v of tile j)
        f32x4 s[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            s[j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int ds = 0; ds < DS; ++ds)
                s[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, kr[j][ds]), bq[ds], s[j], 0, 0, 0);
        }
        float blk_max = -1e30f;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int key = k0 + 16 * j + 4 * g + v;
                s[j][v] = key <= my_last ? s[j][v] * scale : -1e30f;
                blk_max = fmaxf(blk_max, s[j][v]);
            }
        blk_max = fmaxf(blk_max, __shfl_xor(blk_max, 16));
        blk_max = fmaxf(blk_max, __shfl_xor(blk_max, 32));
        const float m_new = fmaxf(m_run, blk_max);
        const float alpha = __expf(m_run - m_new);
        float p[8], psum = 0.0f;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int key = k0 + 16 * j + 4 * g + v;
                const float e = key <= my_last ? __expf(s[j][v] - m_new) : 0.0f;
                p[4 * j + v] = e;
                psum += e;
            }
        psum += __shfl_xor(psum, 16);
        psum += __shfl_xor(psum, 32);
        l_run = l_run * alpha + psum;
        m_run = m_new;
        // probabilities as two bf16 terms (value = hi + lo to 16 bits): a single bf16 rounding of P is a relative error of
        // 2^-9 per term, which shows when large value channels nearly cancel; the second product runs once per term
        const u32x4 p_hi = pack_bf16x8(p);
        float hi_f[8], p_lo_f[8];
        unpack_bf16x8(p_hi, hi_f);
#pragma unroll
        for (int e = 0; e < 8; ++e) p_lo_f[e] = p[e] - hi_f[e];
        const bf16x8 bp = __builtin_bit_cast(bf16x8, p_hi), bp_lo = __builtin_bit_cast(bf16x8, pack_bf16x8(p_lo_f));
        // ---- value block through LDS (the previous block's reads are done: one wave, program order + the barrier)
        __syncthreads();
#pragma unroll
        for (int u = 0; u < VL; ++u) {
            const int idx = lane + 64 * u;
            *reinterpret_cast<u32x2*>(vblk + (idx / VPR) * PITCH + (idx % VPR) * 16) = u32x2{vr[u].x, vr[u].y};
            *reinterpret_cast<u32x2*>(vblk + (idx / VPR) * PITCH + (idx % VPR) * 16 + 8) = u32x2{vr[u].z, vr[u].w};
        }
        __syncthreads();
        // ---- O^T += V^T P^T: position 8g + e <-> key 4g + e (e < 4), 16 + 4g + e - 4 (e >= 4)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            const uint8_t* col = vblk + (16 * dt + qi) * 2;
            uint32_t w[4];
#pragma unroll
            for (int e2 = 0; e2 < 4; ++e2) {
                const int ka = (e2 < 2 ? 4 * g + 2 * e2 : 16 + 4 * g + 2 * (e2 - 2));
                const uint32_t lo = *reinterpret_cast<const uint16_t*>(col + ka * PITCH);
                const uint32_t hi = *reinterpret_cast<const uint16_t*>(col + (ka + 1) * PITCH);
                w[e2] = lo | (hi << 16);
            }
#pragma unroll
            for (int v = 0; v < 4; ++v) o[dt][v] *= alpha;
            const bf16x8 va = __builtin_bit_cast(bf16x8, u32x4{w[0], w[1], w[2], w[3]});
            o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va, bp, o[dt], 0, 0, 0);
            o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va, bp_lo, o[dt], 0, 0, 0);
        }
    }

    if (t0 + qi < T) {
        const float inv = 1.0f / l_run;
        uint16_t* orow = out + (static_cast<size_t>(b) * T + t) * (static_cast<size_t>(H) * D) + static_cast<size_t>(h) * D;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            const u32x2 pk = {pack_bf16x2(o[dt][0] * inv, o[dt][1] * inv), pack_bf16x2(o[dt][2] * inv, o[dt][3] * inv)};
            *reinterpret_cast<u32x2*>(orow + 16 * dt + 4 * g) = pk;
        }
    }
}

}  // namespace terna
