// Expands the compressed ternary format to a dense row-major bf16 [N][K] matrix of -1/0/+1.
// Same lane mapping as the small-M kernel: a wave takes one 16x64 band-tile, and a lane ends
// up with 8 weights of one row for each of its two bitmap bytes.
#pragma once

#include "decode_kernel.h"

namespace terna {

template <int WAVES>
__global__ __launch_bounds__(WAVES * 64) void terna_decompress_kernel(
    const uint64_t* __restrict__ bitmap, const int* __restrict__ tile_off,
    const uint16_t* __restrict__ median_off, const uint32_t* __restrict__ sign_words,
    uint16_t* __restrict__ w_dense, int N, int K)
{
    __shared__ uint2 lut[256];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    for (int e = tid; e < 256; e += WAVES * 64) lut[e] = make_lut_bf16(e);
    __syncthreads();

    const int band = blockIdx.x;
    const int gm = band >> 2, med = band & 3;
    const int ktiles = K >> 6;
    const int last_word = (tile_off[(N >> 6) * ktiles] >> 5) - 1;
    const LaneGeom q(lane);

    for (int gk = wave; gk < ktiles; gk += WAVES) {
        const int tile = gm * ktiles + gk;
        const uint64_t* bmp = bitmap + static_cast<size_t>(tile) * 64 + med * 16;
        const uint64_t scan_bm = bmp[q.i];
        const uint64_t bm[2] = {bmp[q.b0], bmp[q.b0 + 1]};
        int base = tile_off[tile];
        if (med) base += median_off[3 * tile + med - 1];
        uint32_t idx[2][2];
        band_tile_indices(q, scan_bm, bm, base, sign_words, last_word, idx);
        // value pair j of byte t sits at columns 16g + 4j + 2t, +1 of row 16*band + i
        uint32_t* row = reinterpret_cast<uint32_t*>(
            w_dense + static_cast<size_t>(band * 16 + q.i) * K + gk * 64 + q.g * 16);
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const uint2 lo = lut[idx[t][0]], hi = lut[idx[t][1]];
            row[0 + t] = lo.x;
            row[2 + t] = lo.y;
            row[4 + t] = hi.x;
            row[6 + t] = hi.y;
        }
    }
}

}  // namespace terna
