// Host-side producer of the compressed ternary weight format (no GPU work).
//
// The format is the one written by the reference's convert/convert_utils.py:52-228 and
// kernels/TernaSpMM.cu:282-439.  This encoder does not walk the matrix in the reference's
// loop nest; it computes, for every bit of every 8x8 bitmap, which original element it
// stands for:
//   bitmap b of tile T:  band = b / 16, g = (b / 4) % 4, sk = (b / 2) % 2, sm = b % 2
//   bit 8*r + c       :  row = 64*tm + 16*band + 8*sk + r
//                        col = 64*tk + 16*g + 4*(c / 2) + 2*sm + (c % 2)
// which folds the 16x16 block permutation (convert_utils.py:9-49) into the index math.
#include <cstdint>
#include <cstdlib>
#include <cstring>

#include "format_host.h"

namespace terna {

namespace {

inline float bf16_to_float(uint16_t h)
{
    uint32_t u = static_cast<uint32_t>(h) << 16;
    float f;
    std::memcpy(&f, &u, sizeof f);
    return f;
}

// `at(row, col)` returns <0, 0 or >0 for the element of the ORIGINAL matrix.
template <typename At>
int64_t encode_core(At at, int N, int K, uint64_t* bitmap, int* tile_off, uint16_t* median_off,
                    uint32_t* sign_words, int* max_padded_nnz)
{
    const int tiles_k = K / 64;
    int64_t pos = 0;                     // next free sign bit, always a multiple of 32 at tile start
    int64_t tile = 0;
    int max_nnz = 0;
    tile_off[0] = 0;
    for (int tm = 0; tm < N / 64; ++tm) {
        for (int tk = 0; tk < tiles_k; ++tk, ++tile) {
            const int64_t tile_start = pos;
            uint64_t word = 0;           // sign word being filled
            for (int b = 0; b < 64; ++b) {
                const int band = b >> 4, g = (b >> 2) & 3, sk = (b >> 1) & 1, sm = b & 1;
                if (b && (b & 15) == 0) median_off[3 * tile + band - 1] = static_cast<uint16_t>(pos - tile_start);
                const int row0 = 64 * tm + 16 * band + 8 * sk;
                const int col0 = 64 * tk + 16 * g + 2 * sm;
                uint64_t bits = 0;
                for (int r = 0; r < 8; ++r) {
                    for (int c = 0; c < 8; ++c) {
                        const int v = at(row0 + r, col0 + 4 * (c >> 1) + (c & 1));
                        if (v == 0) continue;
                        bits |= 1ull << (8 * r + c);
                        if (v < 0) word |= 1ull << (pos & 31);
                        if ((++pos & 31) == 0) {
                            sign_words[(pos >> 5) - 1] = static_cast<uint32_t>(word);
                            word = 0;
                        }
                    }
                }
                bitmap[tile * 64 + b] = bits;
            }
            if (pos & 31) {              // zero-pad the tile's stream to a whole word
                sign_words[pos >> 5] = static_cast<uint32_t>(word);
                pos = (pos | 31) + 1;
            }
            const int padded = static_cast<int>(pos - tile_start);
            if (padded > max_nnz) max_nnz = padded;
            tile_off[tile + 1] = static_cast<int>(pos);
        }
    }
    if (max_padded_nnz) *max_padded_nnz = max_nnz;
    return pos >> 5;
}

}  // namespace

int encode_sizes(int N, int K, int64_t* bitmap_len, int64_t* tile_off_len, int64_t* median_len,
                 int64_t* sign_words_capacity)
{
    if (N <= 0 || K <= 0 || N % 64 || K % 64) return -1;
    const int64_t nk = static_cast<int64_t>(N) * K;
    if (bitmap_len) *bitmap_len = nk / 64;
    if (tile_off_len) *tile_off_len = nk / 4096 + 1;
    if (median_len) *median_len = 3 * (nk / 4096);
    if (sign_words_capacity) *sign_words_capacity = nk / 32;
    return 0;
}

int64_t encode_i8(const int8_t* W, int N, int K, uint64_t* bitmap, int* tile_off, uint16_t* median_off,
                  uint32_t* sign_words)
{
    if (N <= 0 || K <= 0 || N % 64 || K % 64) return -1;
    const int64_t nk = static_cast<int64_t>(N) * K;
    for (int64_t e = 0; e < nk; ++e)
        if (W[e] < -1 || W[e] > 1) return -1;
    auto at = [=](int row, int col) -> int { return W[static_cast<int64_t>(row) * K + col]; };
    return encode_core(at, N, K, bitmap, tile_off, median_off, sign_words, nullptr);
}

int64_t encode_reordered_bf16(const uint16_t* A, int N, int K, uint64_t* bitmap, int* tile_off,
                              uint16_t* median_off, uint32_t* sign_words, int* max_padded_nnz)
{
    if (N <= 0 || K <= 0 || N % 64 || K % 64) return -1;
    // The caller hands over the matrix AFTER the 16x16 permutation; map original (row, col)
    // to where the permutation put it:  i' = (i&7) + 8*((k>>1)&1),  k' = 8*(i>>3) + 2*(k>>2) + (k&1).
    auto at = [=](int row, int col) -> int {
        const int i = row & 15, k = col & 15;
        const int ri = (i & 7) + 8 * ((k >> 1) & 1);
        const int rk = 8 * (i >> 3) + 2 * (k >> 2) + (k & 1);
        const float f = bf16_to_float(A[static_cast<int64_t>((row & ~15) + ri) * K + (col & ~15) + rk]);
        return f < 0.0f ? -1 : (f != 0.0f ? 1 : 0);
    };
    return encode_core(at, N, K, bitmap, tile_off, median_off, sign_words, max_padded_nnz);
}

void reorder_bf16(const uint16_t* W, uint16_t* out, int N, int K)
{
    for (int row = 0; row < N; ++row) {
        const int i = row & 15;
        for (int col = 0; col < K; ++col) {
            const int k = col & 15;
            const int ri = (i & 7) + 8 * ((k >> 1) & 1);
            const int rk = 8 * (i >> 3) + 2 * (k >> 2) + (k & 1);
            out[static_cast<int64_t>((row & ~15) + ri) * K + (col & ~15) + rk] = W[static_cast<int64_t>(row) * K + col];
        }
    }
}

}  // namespace terna
