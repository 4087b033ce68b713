// The two attention-side kernels of a decode step around the fused qkv linear:
//
//   terna_rope_kv_store_kernel   rotary embedding of q and k, q re-laid out per head, k and v
//                                written into the KV cache at the new tokens' slots
//   terna_decode_attention_kernel  one new token per sequence attending over its cache prefix
//
// They stand where the reference calls xformers' rope_padded (model.py:218-229) and
// fmha.memory_efficient_attention_forward (model.py:231-233); both are absent third-party
// operators, restated here from their definitions (rotate-half RoPE with given cos/sin tables;
// softmax(q K^T / sqrt(D)) V over the valid cache slots).  fp32 inside, bf16 storage.
#pragma once

#include "norm_quant_kernel.h"

namespace terna {

// qkv   bf16 [B*T][(H + 2*KV) * D]   row b*T + t: q heads, then k heads, then v heads
// cosv, sinv  fp32 [T][D/2]          angle of (token t, pair j)
// pos   int64 [T]                    cache slot of token t (same for every sequence)
// q_out bf16 [B][H][T][D]
// cache_k, cache_v  bf16 [B][KV][S][D]
// Pair j of a head is (x[j], x[j + D/2]):  x[j]' = x[j] cos - x[j + D/2] sin,
//                                          x[j + D/2]' = x[j + D/2] cos + x[j] sin.
__global__ __launch_bounds__(256) void terna_rope_kv_store_kernel(
    const uint16_t* __restrict__ qkv, const float* __restrict__ cosv, const float* __restrict__ sinv,
    const long long* __restrict__ pos, uint16_t* __restrict__ q_out, uint16_t* __restrict__ cache_k,
    uint16_t* __restrict__ cache_v, int T, int H, int KV, int D, int S)
{
    const int row = blockIdx.x;                  // b*T + t
    const int b = row / T, t = row - b * T;
    const int half = D >> 1;
    const int slots = H + 2 * KV;
    const uint16_t* src = qkv + static_cast<size_t>(row) * slots * D;
    const long long slot = pos[t];
    for (int i = threadIdx.x; i < slots * half; i += blockDim.x) {
        const int hs = i / half, j = i - hs * half;
        const float x1 = bf16_bits_to_float(src[hs * D + j]);
        const float x2 = bf16_bits_to_float(src[hs * D + j + half]);
        uint16_t* dst;
        float o1 = x1, o2 = x2;
        if (hs < H + KV) {
#pragma clang fp contract(off)                   // every product and sum rounded once: a defined result
            const float c = cosv[t * half + j], s = sinv[t * half + j];
            o1 = x1 * c - x2 * s;
            o2 = x2 * c + x1 * s;
        }
        if (hs < H) dst = q_out + ((static_cast<size_t>(b) * H + hs) * T + t) * D;
        else if (hs < H + KV) dst = cache_k + ((static_cast<size_t>(b) * KV + (hs - H)) * S + slot) * D;
        else dst = cache_v + ((static_cast<size_t>(b) * KV + (hs - H - KV)) * S + slot) * D;
        dst[j] = float_to_bf16_bits(o1);
        dst[j + half] = float_to_bf16_bits(o2);
    }
}

// One workgroup per (sequence, head).  q bf16 [B][H][D]; keys / values of kv head h / (H/KV) at
// slots 0 .. pos[0]; out bf16 [B][H*D].  Dynamic LDS: (S + 16*D) floats.
//   pass 1  16 groups of 16 lanes, group g takes slots g, g+16, ...; a lane holds D/16 dimensions
//           of q and of the key row (one 16-byte load for D = 128), the group sums by shuffles
//   pass 2  softmax over the scores in LDS
//   pass 3  thread (slice, chunk): slots slice, slice+16, ... x 8 dimensions of V; the 16 slices
//           are summed through LDS
template <int D>
__global__ __launch_bounds__(256) void terna_decode_attention_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ cache_k, const uint16_t* __restrict__ cache_v,
    const long long* __restrict__ pos, uint16_t* __restrict__ out, int H, int KV, int S, float scale)
{
    static_assert(D == 64 || D == 128, "head dimension");
    constexpr int PER = D / 16;                  // q / k dimensions per lane in pass 1
    constexpr int CH = D / 8;                    // 8-dimension chunks of a V row
    extern __shared__ float lds[];
    float* score = lds;                          // [S]
    float* part = lds + S;                       // [256 / CH][D]
    __shared__ float red[8];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int b = blockIdx.x / H, h = blockIdx.x - b * H;
    const int kvh = h / (H / KV);
    const int n = static_cast<int>(pos[0]) + 1;
    const uint16_t* kbase = cache_k + (static_cast<size_t>(b) * KV + kvh) * S * D;
    const uint16_t* vbase = cache_v + (static_cast<size_t>(b) * KV + kvh) * S * D;

    // ---- pass 1: scores
    const int grp = tid >> 4, sub = tid & 15;
    float qf[PER];
    {
        const uint16_t* qp = q + (static_cast<size_t>(b) * H + h) * D + sub * PER;
#pragma unroll
        for (int j = 0; j < PER; ++j) qf[j] = bf16_bits_to_float(qp[j]) * scale;
    }
    float mx = -INFINITY;
    for (int s = grp; s < n; s += 16) {
        const uint16_t* kp = kbase + static_cast<size_t>(s) * D + sub * PER;
        float kf[PER];
        if constexpr (PER == 8) {
            unpack_bf16x8(*reinterpret_cast<const u32x4*>(kp), kf);
        } else {
            const u32x2 v = *reinterpret_cast<const u32x2*>(kp);
            kf[0] = __uint_as_float(v.x << 16); kf[1] = __uint_as_float(v.x & 0xffff0000u);
            kf[2] = __uint_as_float(v.y << 16); kf[3] = __uint_as_float(v.y & 0xffff0000u);
        }
        float d = 0.0f;
#pragma unroll
        for (int j = 0; j < PER; ++j) d = fmaf(qf[j], kf[j], d);
#pragma unroll
        for (int off = 8; off >= 1; off >>= 1) d += __shfl_xor(d, off);
        if (sub == 0) score[s] = d;
        mx = fmaxf(mx, d);
    }
    mx = wave_max(mx);
    if (lane == 0) red[wave] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));

    // ---- pass 2: softmax numerators and their sum
    float sum = 0.0f;
    for (int s = tid; s < n; s += 256) {
        const float p = __expf(score[s] - mx);
        score[s] = p;
        sum += p;
    }
    sum = wave_sum(sum);
    if (lane == 0) red[4 + wave] = sum;
    __syncthreads();
    sum = (red[4] + red[5]) + (red[6] + red[7]);

    // ---- pass 3: weighted sum of the value rows
    const int chunk = tid % CH, slice = tid / CH;
    constexpr int SLICES = 256 / CH;
    float acc[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    for (int s = slice; s < n; s += SLICES) {
        float vf[8];
        unpack_bf16x8(*reinterpret_cast<const u32x4*>(vbase + static_cast<size_t>(s) * D + chunk * 8), vf);
        const float p = score[s];
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[j] = fmaf(p, vf[j], acc[j]);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) part[slice * D + chunk * 8 + j] = acc[j];
    __syncthreads();
    if (tid < D) {
        float o = 0.0f;
#pragma unroll
        for (int sl = 0; sl < SLICES; ++sl) o += part[sl * D + tid];
        out[(static_cast<size_t>(b) * H + h) * D + tid] = float_to_bf16_bits(o / sum);
    }
}

}  // namespace terna
