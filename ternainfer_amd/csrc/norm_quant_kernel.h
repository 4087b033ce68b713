// Fused prologue of a ternary linear: [residual add | relu(x1)^2 * x3] -> RMSNorm -> per-row
// absmax int8 quantisation, one workgroup per activation row.
//
// This is the glue the reference runs as separate PyTorch / xformers / Inductor kernels between two
// bitlinear calls (model.py:120-123 quant_input; model.py:236 attn_sub_norm; :280 ffn_sub_norm over
// squared_relu(x1) * x3; :330, :334 the residual adds and the two block norms).  Per row:
//
//   h  = x                                   (plain)
//      = bf16(x + residual)                  (residual add; h is also written back as the new stream)
//      = bf16(bf16(relu(x1)^2) * x3)         (gated FFN; x1 = row[0:F], x3 = row[F:2F])
//   y  = bf16(h * rsqrt(mean(h^2) + eps) * weight)          fp32 inside, one rounding at the end
//   s  = bf16(127 / max(max|y|, 1e-5));  q = clamp(rint(y * s), -128, 127)   (fp32 inside; `quant_mode` selects
//        which of the reference's ways of evaluating these two lines is reproduced: QuantMode in terna_common.h)
//
// The row stays in registers between the three passes; HBM sees each input element once and each
// output element once.  Rows are independent, so the grid is M workgroups of 256 threads.
#pragma once

#include "terna_common.h"

namespace terna {

constexpr int kNormThreads = 256;
constexpr int kNormMaxVecs = 4;                       // 8-element vectors per thread: K <= 8192

// Reductions over groups of LANES consecutive lanes (LANES = 2 .. 64, a power of two) with the data
// parallel primitives of the VALU instead of LDS-crossbar shuffles: a ds_bpermute round trip costs
// on the order of a hundred cycles and a 64-lane butterfly needs six of them in sequence; the
// quad / half-row / row permutations below are ordinary VALU operands.  Every lane of the wave must
// be active.  The result is the same in every lane of a group; the order of the additions is
// fixed (pairs, quads, eights, sixteens, then rows 0+1 and 2+3, then the halves).
template <int CTRL>
__device__ __forceinline__ float dpp_permute(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_permute_u32(uint32_t v)
{
    return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), CTRL, 0xf, 0xf, true));
}
constexpr int kDppRowShl4 = 0x104;        // lane i <- lane i + 4 within 16 lanes (0 past the row)
constexpr int kDppRowShl8 = 0x108;
constexpr int kDppRowShl12 = 0x10C;
constexpr int kDppSwapPairs = 0xB1;       // quad_perm [1, 0, 3, 2]: lane ^ 1
constexpr int kDppSwapHalfQuads = 0x4E;   // quad_perm [2, 3, 0, 1]: lane ^ 2
constexpr int kDppHalfRowMirror = 0x141;  // lane i <-> 7 - i within 8 lanes
constexpr int kDppRowMirror = 0x140;      // lane i <-> 15 - i within 16 lanes

template <int LANES, bool IS_MAX>
__device__ __forceinline__ float group_reduce(float v)
{
    static_assert(LANES >= 1 && LANES <= 64 && (LANES & (LANES - 1)) == 0, "group size");
    auto op = [](float a, float b) { return IS_MAX ? fmaxf(a, b) : a + b; };
    if constexpr (LANES >= 2) v = op(v, dpp_permute<kDppSwapPairs>(v));
    if constexpr (LANES >= 4) v = op(v, dpp_permute<kDppSwapHalfQuads>(v));
    if constexpr (LANES >= 8) v = op(v, dpp_permute<kDppHalfRowMirror>(v));     // quads are uniform by now
    if constexpr (LANES >= 16) v = op(v, dpp_permute<kDppRowMirror>(v));        // ... and so are the halves of a row
    if constexpr (LANES == 32) {
        // rows 0|1 and 2|3: lane ^ 16 through the row's uniform value of the neighbouring row
        const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
        const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 16));
        const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32));
        const float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 48));
        v = (threadIdx.x & 32) ? op(r2, r3) : op(r0, r1);
    }
    if constexpr (LANES == 64) {
        const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
        const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 16));
        const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32));
        const float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 48));
        v = op(op(r0, r1), op(r2, r3));
    }
    return v;
}

__device__ __forceinline__ float wave_sum(float v) { return group_reduce<64, false>(v); }
__device__ __forceinline__ float wave_max(float v) { return group_reduce<64, true>(v); }

__device__ __forceinline__ void unpack_bf16x8(const u32x4& v, float f[8])
{
    const uint32_t d[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        f[2 * j] = __uint_as_float(d[j] << 16);
        f[2 * j + 1] = __uint_as_float(d[j] & 0xffff0000u);
    }
}
__device__ __forceinline__ u32x4 pack_bf16x8(const float f[8])
{
    uint32_t d[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) d[j] = pack_bf16x2(f[2 * j], f[2 * j + 1]);
    return u32x4{d[0], d[1], d[2], d[3]};
}
__device__ __forceinline__ float round_bf16(float v) { return bf16_bits_to_float(float_to_bf16_bits(v)); }

// The passes behind the formation of a row, for every kernel that holds one in registers (h[i][j] = element
// 8 (tid + kNormThreads i) + j, vectors past K / 8 unused; raw_w the norm weights of the same elements): sum of squares
// -- per thread in element order, the lanes of a wave by group_reduce, the four waves pairwise -- then the norm, the row
// maximum, the scale and the int8 values.  y_out / xq_out + s_out: optional outputs.
template <int NV>
__device__ __forceinline__ void norm_quant_passes(float (&h)[NV][8], const u32x4 (&raw_w)[NV], int K, float eps, size_t row,
                                                  uint16_t* __restrict__ y_out, int8_t* __restrict__ xq_out,
                                                  uint16_t* __restrict__ s_out, int quant_mode)
{
    __shared__ float red[2][kNormThreads / 64];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int nvec = K >> 3;
    float ssq = 0.0f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        if (tid + i * kNormThreads < nvec) {
#pragma unroll
            for (int j = 0; j < 8; ++j) ssq = fmaf(h[i][j], h[i][j], ssq);
        }
    }
    ssq = wave_sum(ssq);
    if (lane == 0) red[0][wave] = ssq;
    __syncthreads();
    const float total = (red[0][0] + red[0][1]) + (red[0][2] + red[0][3]);
    const float rstd = rsqrtf(total / static_cast<float>(K) + eps);

    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int v = tid + i * kNormThreads;
        if (v < nvec) {
            float w[8];
            unpack_bf16x8(raw_w[i], w);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                h[i][j] = round_bf16(h[i][j] * rstd * w[j]);
                amax = fmaxf(amax, fabsf(h[i][j]));
            }
            if (y_out != nullptr) *reinterpret_cast<u32x4*>(y_out + row * K + 8 * v) = pack_bf16x8(h[i]);
        }
    }
    if (xq_out == nullptr) return;

    amax = wave_max(amax);
    if (lane == 0) red[1][wave] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(red[1][0], red[1][1]), fmaxf(red[1][2], red[1][3]));
    uint16_t s_bits;
    const float s = quant_scale(amax, quant_mode, &s_bits);
    if (tid == 0) s_out[row] = s_bits;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int v = tid + i * kNormThreads;
        if (v < nvec) {
            uint32_t q[2] = {0u, 0u};
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float r = quant_value(h[i][j], s, quant_mode);
                q[j >> 2] |= (static_cast<uint32_t>(static_cast<int>(r)) & 0xffu) << (8 * (j & 3));
            }
            *reinterpret_cast<u32x2*>(xq_out + row * K + 8 * v) = u32x2{q[0], q[1]};
        }
    }
}

// GLU = false: x [M][K], optional residual [M][K] and sum_out [M][K].
// GLU = true : x [M][2K] holding x1 | x3; residual / sum_out unused.
// NV = 8-element vectors per thread (K <= 2048 NV); SECOND = there is a second operand (the residual, or x3).
template <bool GLU, int NV = kNormMaxVecs, bool SECOND = true>
__global__ __launch_bounds__(kNormThreads) void terna_norm_quant_kernel(
    const uint16_t* __restrict__ x, const uint16_t* __restrict__ residual, const uint16_t* __restrict__ weight, int K,
    float eps, uint16_t* __restrict__ sum_out, uint16_t* __restrict__ y_out, int8_t* __restrict__ xq_out,
    uint16_t* __restrict__ s_out, int quant_mode)
{
    static_assert(!GLU || SECOND, "the gate has two operands");
    const int tid = threadIdx.x;
    const size_t row = blockIdx.x;
    const int nvec = K >> 3;
    const uint16_t* xr = x + row * static_cast<size_t>(GLU ? 2 * K : K);

    // Every global load of the row -- input, second operand, norm weight -- is issued before the
    // first use: with one row per workgroup the kernel's time is its chain of memory round trips, and the address
    // unit takes a wave's load in a dozen cycles whatever it fetches: no more loads than the row needs.
    // The loads are unconditional on clamped addresses (a load inside a branch is waited for at
    // the join, which would serialise them).
    u32x4 raw_x[NV], raw_b[NV], raw_w[NV];
    const uint16_t* br = GLU ? xr + K : (SECOND ? residual + row * K : xr);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int v = tid + i * kNormThreads;
        const int vc = v < nvec ? v : nvec - 1;
        raw_x[i] = *reinterpret_cast<const u32x4*>(xr + 8 * vc);
        if constexpr (SECOND) raw_b[i] = *reinterpret_cast<const u32x4*>(br + 8 * vc);
        raw_w[i] = *reinterpret_cast<const u32x4*>(weight + 8 * vc);
    }
    // pin the loads here: otherwise they are sunk into the branches below, next to their uses
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        pin_registers(raw_x[i]);
        if constexpr (SECOND) pin_registers(raw_b[i]);
        pin_registers(raw_w[i]);
    }

    float h[NV][8];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int v = tid + i * kNormThreads;
        if (v < nvec) {
            unpack_bf16x8(raw_x[i], h[i]);
            if constexpr (GLU) {
                float g[8];
                unpack_bf16x8(raw_b[i], g);
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float r = fmaxf(h[i][j], 0.0f);
                    h[i][j] = round_bf16(round_bf16(r * r) * g[j]);
                }
            } else if constexpr (SECOND) {
                float r[8];
                unpack_bf16x8(raw_b[i], r);
#pragma unroll
                for (int j = 0; j < 8; ++j) h[i][j] = round_bf16(h[i][j] + r[j]);
                if (sum_out != nullptr) *reinterpret_cast<u32x4*>(sum_out + row * K + 8 * v) = pack_bf16x8(h[i]);
            }
        }
    }
    norm_quant_passes<NV>(h, raw_w, K, eps, row, y_out, xq_out, s_out, quant_mode);
}

}  // namespace terna
