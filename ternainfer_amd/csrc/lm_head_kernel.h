// bf16 LM head of a decode step: logits[m][v] = sum_k x[m][k] * W[v][k] for M <= 16 rows of
// activations against the (tied) embedding matrix W [V][K] -- 657 MB for the 2B model, more than
// all ternary weights of a token together, read once per step: an HBM-bound GEMV
// (the reference: F.linear on the bf16 output matrix, model.py:367, 449-455).
//
// One wave owns 16 consecutive vocabulary rows at a time: v_mfma_f32_16x16x32_bf16 takes them as the
// A operand straight from memory (lane: row L & 15, 8 consecutive k of chunk L >> 4 -- the 16 bytes
// the lane loads) and the activations as B from LDS (staged once per workgroup; lanes of the batch
// rows >= M read row 0 and feed zeros).
// kLmUnroll loads of a lane are in flight before the first is used; a workgroup walks over row
// blocks blockIdx.x, blockIdx.x + gridDim.x, ... so that the activations are staged once.
#pragma once

#include "norm_quant_kernel.h"

namespace terna {

constexpr int kLmWaves = 4;
constexpr int kLmUnroll = 16;                    // k-steps of 32 in flight per lane (16 bytes each)

constexpr size_t lm_head_lds_bytes(int M, int K) { return static_cast<size_t>(M) * (K * 2 + 16); }
// Rows without padding, the 16-byte piece c of row r at position c ^ (r & 7) instead (the same spread over the banks; K a
// multiple of 64 so that a piece's partner is in the row): 16 rows of K = 2560 are then 80 KB, and two workgroups fit a CU.
constexpr size_t lm_head_lds_bytes_swizzled(int M, int K) { return static_cast<size_t>(M) * K * 2; }

__global__ __launch_bounds__(kLmWaves * 64) void terna_lm_head_kernel(const uint16_t* __restrict__ x,
                                                                      const uint16_t* __restrict__ w,
                                                                      uint16_t* __restrict__ logits, int M, int V, int K, int swizzled)
{
    extern __shared__ __align__(16) uint8_t xs[];            // [M][K * 2 + 16]: padded pitch, or [M][K * 2] swizzled
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int pitch = swizzled ? K * 2 : K * 2 + 16;
    const int row_vecs = K >> 3;                             // 16-byte pieces per row
    for (int p = tid; p < M * row_vecs; p += kLmWaves * 64) {
        const int r = p / row_vecs, c = p - r * row_vecs;
        *reinterpret_cast<u32x4*>(xs + r * pitch + 16 * (swizzled ? c ^ (r & 7) : c)) =
            *reinterpret_cast<const u32x4*>(x + static_cast<size_t>(r) * K + 8 * c);
    }
    __syncthreads();

    const int i = lane & 15, kg = lane >> 4;
    const int steps = K >> 5;
    const bool live = i < M;
    // B operand: batch row i, chunk kg of each step = piece 4 s + kg of the row; swizzled: (4 s + kg) ^ (i & 7), i.e. chunk
    // kg ^ (i & 3) of step s ^ ((i >> 2) & 1)
    const int row_b = live ? i : 0;
    const uint8_t* xrow = xs + row_b * pitch + 16 * (swizzled ? kg ^ (row_b & 3) : kg);
    const int step_flip = swizzled ? (row_b >> 2) & 1 : 0;
    const int blocks = (V + 15) >> 4;
    const bool wide_store = (V & 3) == 0 && (reinterpret_cast<uintptr_t>(logits) & 7) == 0;   // 8-byte stores of four logits
    for (int blk = blockIdx.x * kLmWaves + wave; blk < blocks; blk += gridDim.x * kLmWaves) {
        const int row = blk * 16 + i;
        const uint16_t* wrow = w + static_cast<size_t>(row < V ? row : V - 1) * K + 8 * kg;
        f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
        for (int s0 = 0; s0 < steps; s0 += kLmUnroll) {
            u32x4 a[kLmUnroll];
#pragma unroll
            for (int u = 0; u < kLmUnroll; ++u) {
                const int s = s0 + u < steps ? s0 + u : steps - 1;           // past the end: re-read, weight zero below
                a[u] = *reinterpret_cast<const u32x4*>(wrow + 32 * s);
            }
#pragma unroll
            for (int u = 0; u < kLmUnroll; ++u) {
                const int s = s0 + u;
                u32x4 b = *reinterpret_cast<const u32x4*>(xrow + 64 * ((s < steps ? s : steps - 1) ^ step_flip));
                if (s >= steps || !live) b = u32x4{0u, 0u, 0u, 0u};
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a[u]), __builtin_bit_cast(bf16x8, b), acc, 0, 0, 0);
            }
        }
        // lane: batch row i (the B column), vocabulary rows blk * 16 + 4 * kg .. + 3
        const int v0 = blk * 16 + 4 * kg;
        if (i < M && v0 < V) {
            uint16_t* dst = logits + static_cast<size_t>(i) * V + v0;
            if (wide_store) {                                // V % 4 == 0 and v0 % 4 == 0: v0 + 3 < V
                *reinterpret_cast<u32x2*>(dst) = u32x2{pack_bf16x2(acc[0], acc[1]), pack_bf16x2(acc[2], acc[3])};
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (v0 + e < V) dst[e] = float_to_bf16_bits(acc[e]);
            }
        }
    }
}

// Up to four rows of activations: a vocabulary row becomes four rows of the A operand (row i of A:
// vocabulary row i / 4, the 16-byte pieces (i % 4) + 4 (L >> 4) of a 128-column step), so that four
// consecutive lanes load 64 consecutive bytes -- a CU's memory pipeline takes one step per 64-byte
// segment that consecutive lanes touch, 16 per load here against 64 with one vocabulary row per
// operand row (above).  Column 4 m + r of B holds batch row m's matching pieces, out[i][4 m + i % 4]
// is a partial logit, and the four partials of a vocabulary row meet in the four lanes of a quad.
// UNROLL loads of a lane are in flight; it should divide K / 128.
template <int UNROLL>
__global__ __launch_bounds__(kLmWaves * 64) void terna_lm_head_quad_kernel(const uint16_t* __restrict__ x,
                                                                           const uint16_t* __restrict__ w,
                                                                           uint16_t* __restrict__ logits, int M, int V, int K)
{
    extern __shared__ __align__(16) uint8_t xs[];            // [M][K * 2 + 16]: padded pitch
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int pitch = K * 2 + 16;
    const int row_vecs = K >> 3;
    for (int p = tid; p < M * row_vecs; p += kLmWaves * 64) {
        const int r = p / row_vecs, c = p - r * row_vecs;
        *reinterpret_cast<u32x4*>(xs + r * pitch + 16 * c) = *reinterpret_cast<const u32x4*>(x + static_cast<size_t>(r) * K + 8 * c);
    }
    __syncthreads();

    const int i = lane & 15, kg = lane >> 4;
    const int piece = (i & 3) + 4 * kg;                      // 16 bytes of a 256-byte step of a row
    const int steps = K >> 7;
    const int m = i >> 2;                                    // B column i: batch row i / 4, pieces (i % 4) + 4 kg
    const bool live = m < M;
    const uint8_t* xrow = xs + (live ? m : 0) * pitch + 16 * piece;
    const int blocks = (V + 3) >> 2;
    for (int blk = blockIdx.x * kLmWaves + wave; blk < blocks; blk += gridDim.x * kLmWaves) {
        const int row = blk * 4 + (i >> 2);
        const uint16_t* wrow = w + static_cast<size_t>(row < V ? row : V - 1) * K + 8 * piece;
        f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
        for (int s0 = 0; s0 < steps; s0 += UNROLL) {
            u32x4 a[UNROLL];
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                const int s = s0 + u < steps ? s0 + u : steps - 1;
                a[u] = *reinterpret_cast<const u32x4*>(wrow + 128 * s);
            }
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                const int s = s0 + u;
                u32x4 b = *reinterpret_cast<const u32x4*>(xrow + 256 * (s < steps ? s : steps - 1));
                if (s >= steps || !live) b = u32x4{0u, 0u, 0u, 0u};
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a[u]), __builtin_bit_cast(bf16x8, b), acc, 0, 0, 0);
            }
        }
        // lane (column i, rows 4 kg + v): operand row 4 kg + v is vocabulary row blk * 4 + kg, pieces v (mod 4):
        // its partial for batch row m is in column 4 m + v
        float part = (i & 3) == 0 ? acc[0] : (i & 3) == 1 ? acc[1] : (i & 3) == 2 ? acc[2] : acc[3];
        part += dpp_permute<kDppSwapPairs>(part);
        part += dpp_permute<kDppSwapHalfQuads>(part);
        const int v = blk * 4 + kg;
        if ((i & 3) == 0 && live && v < V) logits[static_cast<size_t>(m) * V + v] = float_to_bf16_bits(part);
    }
}

// Five to eight rows of activations: the same trick on the 32 x 32 x 16 MFMA, whose 32 columns hold eight batch rows of four
// partials each.  Row i of A: vocabulary row i / 4 (eight per operand), the 16-byte pieces (i % 4) + 4 (L >> 5) of a
// 128-byte step; column 4 m + r of B: batch row m's pieces r + 4 (L >> 5); out[i][4 m + i % 4] is a partial logit, and the
// four partials of (vocabulary row, batch row) meet in the four lanes of a quad.  Four consecutive lanes load 64 consecutive
// bytes, as above.  UNROLL loads of a lane are in flight; it should divide K / 64.
template <int UNROLL>
__global__ __launch_bounds__(kLmWaves * 64) void terna_lm_head_quad32_kernel(const uint16_t* __restrict__ x,
                                                                             const uint16_t* __restrict__ w,
                                                                             uint16_t* __restrict__ logits, int M, int V, int K)
{
    extern __shared__ __align__(16) uint8_t xs[];            // [M][K * 2 + 16]: padded pitch
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int pitch = K * 2 + 16;
    const int row_vecs = K >> 3;
    for (int p = tid; p < M * row_vecs; p += kLmWaves * 64) {
        const int r = p / row_vecs, c = p - r * row_vecs;
        *reinterpret_cast<u32x4*>(xs + r * pitch + 16 * c) = *reinterpret_cast<const u32x4*>(x + static_cast<size_t>(r) * K + 8 * c);
    }
    __syncthreads();

    const int i = lane & 31, hb = lane >> 5;
    const int piece = (i & 3) + 4 * hb;                      // 16 bytes of a 128-byte step of a row (A and B alike)
    const int steps = K >> 6;
    const int m = i >> 2;                                    // B column i: batch row i / 4
    const bool live = m < M;
    const uint8_t* xrow = xs + (live ? m : 0) * pitch + 16 * piece;
    const int blocks = (V + 7) >> 3;
    for (int blk = blockIdx.x * kLmWaves + wave; blk < blocks; blk += gridDim.x * kLmWaves) {
        const int row = blk * 8 + (i >> 2);
        const uint16_t* wrow = w + static_cast<size_t>(row < V ? row : V - 1) * K + 8 * piece;
        f32x16 acc;
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[e] = 0.0f;
        for (int s0 = 0; s0 < steps; s0 += UNROLL) {
            u32x4 a[UNROLL];
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                const int s = s0 + u < steps ? s0 + u : steps - 1;
                a[u] = *reinterpret_cast<const u32x4*>(wrow + 64 * s);
            }
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                const int s = s0 + u;
                u32x4 b = *reinterpret_cast<const u32x4*>(xrow + 128 * (s < steps ? s : steps - 1));
                if (s >= steps || !live) b = u32x4{0u, 0u, 0u, 0u};
                acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a[u]), __builtin_bit_cast(bf16x8, b), acc, 0, 0, 0);
            }
        }
        // lane (column i, half hb) holds rows (e & 3) + 8 (e >> 2) + 4 hb: row 4 q + r with r = e & 3, q = 2 (e >> 2) + hb, i.e.
        // vocabulary row blk * 8 + q, pieces r (mod 4): its partial for batch row m is in column 4 m + r -- element r + 4 t
        // of the lane whose column has i % 4 == r
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            float part = (i & 3) == 0 ? acc[4 * t] : (i & 3) == 1 ? acc[4 * t + 1] : (i & 3) == 2 ? acc[4 * t + 2] : acc[4 * t + 3];
            part += dpp_permute<kDppSwapPairs>(part);
            part += dpp_permute<kDppSwapHalfQuads>(part);
            const int v = blk * 8 + 2 * t + hb;
            if ((i & 3) == 0 && live && v < V) logits[static_cast<size_t>(m) * V + v] = float_to_bf16_bits(part);
        }
    }
}

}  // namespace terna
