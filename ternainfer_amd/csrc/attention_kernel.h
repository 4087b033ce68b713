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
    if ((half & 7) == 0) {
        // 8 pairs per thread: 16-byte loads and stores, for the 2B model one pass of 240 threads
        const int per = half >> 3;
        for (int i = threadIdx.x; i < slots * per; i += blockDim.x) {
            const int hs = i / per, j = (i - hs * per) * 8;
            float x1[8], x2[8], o1[8], o2[8];
            unpack_bf16x8(*reinterpret_cast<const u32x4*>(src + hs * D + j), x1);
            unpack_bf16x8(*reinterpret_cast<const u32x4*>(src + hs * D + j + half), x2);
            if (hs < H + KV) {
                const f32x4* cp = reinterpret_cast<const f32x4*>(cosv + t * half + j);
                const f32x4* sp = reinterpret_cast<const f32x4*>(sinv + t * half + j);
                const f32x4 c0 = cp[0], c1 = cp[1], s0 = sp[0], s1 = sp[1];
#pragma unroll
                for (int e = 0; e < 8; ++e) {
#pragma clang fp contract(off)                   // every product and sum rounded once: a defined result
                    const float c = e < 4 ? c0[e & 3] : c1[e & 3], sn = e < 4 ? s0[e & 3] : s1[e & 3];
                    o1[e] = x1[e] * c - x2[e] * sn;
                    o2[e] = x2[e] * c + x1[e] * sn;
                }
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) { o1[e] = x1[e]; o2[e] = x2[e]; }
            }
            uint16_t* dst;
            if (hs < H) dst = q_out + ((static_cast<size_t>(b) * H + hs) * T + t) * D;
            else if (hs < H + KV) dst = cache_k + ((static_cast<size_t>(b) * KV + (hs - H)) * S + slot) * D;
            else dst = cache_v + ((static_cast<size_t>(b) * KV + (hs - H - KV)) * S + slot) * D;
            *reinterpret_cast<u32x4*>(dst + j) = pack_bf16x8(o1);
            *reinterpret_cast<u32x4*>(dst + j + half) = pack_bf16x8(o2);
        }
        return;
    }
    for (int i = threadIdx.x; i < slots * half; i += blockDim.x) {
        const int hs = i / half, j = i - hs * half;
        const float x1 = bf16_bits_to_float(src[hs * D + j]);
        const float x2 = bf16_bits_to_float(src[hs * D + j + half]);
        uint16_t* dst;
        float o1 = x1, o2 = x2;
        if (hs < H + KV) {
#pragma clang fp contract(off)
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
// slots 0 .. pos[0]; out bf16 [B][H*D].  Dynamic LDS: (S + D + 16*D) floats.
//   pass 1  one thread per cache slot: the whole key row is fetched with D/8 independent 16-byte
//           loads (all in flight together) and multiplied with q, which every lane reads from
//           LDS at the same address (a broadcast)
//   pass 2  softmax over the scores in LDS
//   pass 3  thread (slice, chunk): slots slice, slice+S', ... x 8 dimensions of V, four rows in
//           flight per thread; the slices are summed through LDS
template <int D>
__global__ __launch_bounds__(256) void terna_decode_attention_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ cache_k, const uint16_t* __restrict__ cache_v,
    const long long* __restrict__ pos, uint16_t* __restrict__ out, int H, int KV, int S, float scale)
{
    static_assert(D == 64 || D == 128, "head dimension");
    constexpr int CH = D / 8;                    // 8-dimension chunks of a row
    constexpr int SLICES = 256 / CH;
    extern __shared__ __align__(16) float lds[];
    float* qs = lds;                             // [D]  q * scale
    float* part = lds + D;                       // [SLICES][D]
    float* score = lds + D + SLICES * D;         // [S]
    __shared__ float red[8];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int b = blockIdx.x / H, h = blockIdx.x - b * H;
    const int kvh = h / (H / KV);
    const int n = static_cast<int>(pos[0]) + 1;
    const uint16_t* kbase = cache_k + (static_cast<size_t>(b) * KV + kvh) * S * D;
    const uint16_t* vbase = cache_v + (static_cast<size_t>(b) * KV + kvh) * S * D;

    if (tid < D) qs[tid] = bf16_bits_to_float(q[(static_cast<size_t>(b) * H + h) * D + tid]) * scale;
    __syncthreads();

    // ---- pass 1: scores
    float mx = -INFINITY;
    for (int s = tid; s < n; s += 256) {
        const u32x4* kp = reinterpret_cast<const u32x4*>(kbase + static_cast<size_t>(s) * D);
        u32x4 kr[CH];
#pragma unroll
        for (int c = 0; c < CH; ++c) kr[c] = kp[c];
        float d = 0.0f;
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            float kf[8];
            unpack_bf16x8(kr[c], kf);
            const f32x4 q0 = *reinterpret_cast<const f32x4*>(qs + 8 * c), q1 = *reinterpret_cast<const f32x4*>(qs + 8 * c + 4);
#pragma unroll
            for (int e = 0; e < 4; ++e) d = fmaf(q0[e], kf[e], d);
#pragma unroll
            for (int e = 0; e < 4; ++e) d = fmaf(q1[e], kf[4 + e], d);
        }
        score[s] = d;
        mx = fmaxf(mx, d);
    }
    mx = wave_max(mx);
    if (lane == 0) red[wave] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));

    // ---- pass 2: softmax numerators and their sum (each thread revisits the slots it scored)
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
    float acc[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    for (int s0 = slice; s0 < n; s0 += 4 * SLICES) {
        u32x4 vr[4];
        float p[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int s = s0 + u * SLICES;
            const int sc = s < n ? s : s0;       // past the end: re-read a valid row with weight 0
            vr[u] = *reinterpret_cast<const u32x4*>(vbase + static_cast<size_t>(sc) * D + chunk * 8);
            p[u] = s < n ? score[s] : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            float vf[8];
            unpack_bf16x8(vr[u], vf);
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[e] = fmaf(p[u], vf[e], acc[e]);
        }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) part[slice * D + chunk * 8 + e] = acc[e];
    __syncthreads();
    if (tid < D) {
        float o = 0.0f;
#pragma unroll
        for (int sl = 0; sl < SLICES; ++sl) o += part[sl * D + tid];
        out[(static_cast<size_t>(b) * H + h) * D + tid] = float_to_bf16_bits(o / sum);
    }
}

}  // namespace terna
