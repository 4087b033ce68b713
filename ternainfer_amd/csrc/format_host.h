// Host-side encoder of the compressed ternary weight format (see format_host.cpp).
#pragma once
#include <cstdint>

namespace terna {

int encode_sizes(int N, int K, int64_t* bitmap_len, int64_t* tile_off_len, int64_t* median_len,
                 int64_t* sign_words_capacity);

// ORIGINAL int8 ternary matrix -> format arrays.  Returns sign words written, or -1.
int64_t encode_i8(const int8_t* W, int N, int K, uint64_t* bitmap, int* tile_off, uint16_t* median_off,
                  uint32_t* sign_words);

// Already permuted bf16 matrix -> format arrays.  Returns sign words written, or -1.
int64_t encode_reordered_bf16(const uint16_t* A, int N, int K, uint64_t* bitmap, int* tile_off,
                              uint16_t* median_off, uint32_t* sign_words, int* max_padded_nnz);

// The 16x16 block permutation on bf16 storage.
void reorder_bf16(const uint16_t* W, uint16_t* out, int N, int K);

}  // namespace terna
