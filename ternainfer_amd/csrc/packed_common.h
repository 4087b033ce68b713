// The load-time layout "P2" and its expansion to MFMA operands (gfx950).
//
// P2 is this library's own device layout of a ternary matrix; the reference has no counterpart.
// It is produced from the reference's compressed format by terna_repack_kernel (bit-exact,
// checked by round trip) either once at load time or, on the reference's prefill entry points,
// per call into the caller's workspace.  It costs 2 bits per weight (N*K/4 bytes, vs ~1.6 bits
// in the reference format) and buys a decode with no offsets, no popcounts and no LDS:
//
//   uint32 packed[N/16][K/64][64]
//   element [band][gk][4*i + g] : row 16*band + i, columns 64*gk + 16*g .. +15, 2 bits each
//                                 (bit0 = nonzero, bit1 = negative)
//   column j of the group       : byte j & 3, 2-bit field j >> 2, i.e. bit 8*(j&3) + 2*(j>>2).
//
// A 2-bit code in the top field of a byte IS the weight in two number formats at once:
//   as a signed byte        0x40 = +64, 0xC0 = -64, 0x00 = 0                  (int8 operand, times 64)
//   as a bf16 high byte     0x4000 = +2.0, 0xC000 = -2.0, 0x0000 = 0          (bf16 operand, times 2)
// and `(word << (6 - 2*q)) & 0xC0C0C0C0` puts the codes of columns 4q .. 4q+3 there, in natural column order -- the
// matching activation operand is a plain contiguous piece of the activation row.  For int8 that is the whole
// expansion (seven shift / mask operations per sixteen weights, no table); for bf16 two v_perm_b32 per four weights
// interleave the high bytes with zero low bytes into bf16 pairs.  The accumulators therefore hold a multiple of the
// true sum -- 64 times (int32; exact, and it fits for K < 2^31 / (64 * 128) = 262144) or twice (fp32; exact) -- and
// every consumer undoes it before the epilogue: `>> kI8WeightShift`, respectively `* kBf16WeightUndo`.
#pragma once

#include "decode_kernel.h"

namespace terna {

constexpr uint32_t kTopFieldMask = 0xC0C0C0C0u;  // the top field of every byte: an int8 weight times 64 / a bf16 high byte
constexpr int kI8WeightShift = 6;                // int8 accumulators hold the sum << 6
constexpr float kBf16WeightUndo = 0.5f;          // bf16-operand accumulators hold twice the sum
constexpr uint32_t kPair01 = 0x010C000Cu;        // [0, b0, 0, b1]: two bf16 with zero low bytes
constexpr uint32_t kPair23 = 0x030C020Cu;        // [0, b2, 0, b3]

// Eight bf16 weights (+-2 / 0), columns 8h .. 8h+7 of the group, from `t` = the packed word shifted LEFT by 4 - 4h
// (h = 0: word << 4, h = 1: the word itself): dword j holds columns 8h + 2j, 8h + 2j + 1.
__device__ __forceinline__ u32x4 expand_chunk_bf16(uint32_t t)
{
    const uint32_t hi0 = (t << 2) & kTopFieldMask;     // field 2h of every byte: columns 8h .. 8h+3
    const uint32_t hi1 = t & kTopFieldMask;            // field 2h + 1: columns 8h+4 .. 8h+7
    return u32x4{__builtin_amdgcn_perm(0u, hi0, kPair01), __builtin_amdgcn_perm(0u, hi0, kPair23),
                 __builtin_amdgcn_perm(0u, hi1, kPair01), __builtin_amdgcn_perm(0u, hi1, kPair23)};
}

// Sixteen int8 weights (+-64 / 0) of a packed word in column order: dword q holds columns 4q .. 4q+3.
// `mask`: kTopFieldMask, or 0 for a lane whose word stands for columns that do not exist (all weights zero).
__device__ __forceinline__ i32x4 expand_word_i8(uint32_t d, uint32_t mask = kTopFieldMask)
{
    return i32x4{static_cast<int>((d << 6) & mask), static_cast<int>((d << 4) & mask),
                 static_cast<int>((d << 2) & mask), static_cast<int>(d & mask)};
}

// Repack table: (nonzero nibble, next 4 sign bits of the stream) -> the nibble's four 2-bit codes
// where P2 wants them, up to a shift.  Bit cb of nibble hh of bitmap byte sm is column
// j = 4*(2hh + (cb>>1)) + 2sm + (cb&1) of the group: byte 2sm + (cb&1), field 2hh + (cb>>1).  The
// table holds byte (cb&1), field (cb>>1); the caller shifts by 16*sm + 4*hh.
__device__ __forceinline__ uint32_t make_lut_code(int e)
{
    const int nz = e >> 4, sg = e & 15;
    uint32_t r = 0;
    int used = 0;
#pragma unroll
    for (int cb = 0; cb < 4; ++cb) {
        if ((nz >> cb) & 1) {
            r |= (1u | (((sg >> used) & 1) << 1)) << (8 * (cb & 1) + 2 * (cb >> 1));
            ++used;
        }
    }
    return r;
}

// Fingerprint of a matrix in the reference format, computed by one wave: the total sign-bit count
// (tile_off[tiles]) and 64 words each from the start, the middle and the end of the bitmap array and from the start
// and the end of the sign stream, mixed per lane and folded over the wave.  A weight that was freed and replaced by
// another one at the same addresses differs in these 2.5 KB with all but negligible probability.  (Weights edited in
// place at a few positions are NOT what this detects.)
__device__ __forceinline__ unsigned long long fingerprint_mix(unsigned long long x)
{
    x ^= x >> 30;
    x *= 0xbf58476d1ce4e5b9ull;
    x ^= x >> 27;
    x *= 0x94d049bb133111ebull;
    return x ^ (x >> 31);
}
// `total` = tile_off[tiles] as it reads now.  The sign stream is sampled only when that equals the recorded length --
// the positions follow the length, and a stream that is shorter now must not be read past its end; a different length
// alone makes the fingerprint differ (the total is mixed in last).
__device__ __forceinline__ unsigned long long repack_fingerprint(const RepackGuard& g, int lane)
{
    const long long n_bm = static_cast<long long>(g.tiles) * 64;
    const int total = g.tile_off[g.tiles];
    const unsigned long long b0 = g.bitmap[lane], b1 = g.bitmap[n_bm / 2 - 32 + lane], b2 = g.bitmap[n_bm - 64 + lane];
    const int words = g.total_bits >> 5;
    unsigned long long s0 = 0, s1 = 0;
    if (total == g.total_bits && words > 0) {
        const int hi = words - 1;
        int tail = words - 64 + lane;
        tail = tail < 0 ? 0 : tail;
        s0 = g.sign_words[lane < hi ? lane : hi];
        s1 = g.sign_words[tail < hi ? tail : hi];
    }
    unsigned long long h = fingerprint_mix(b0 + 0x9e3779b97f4a7c15ull * (lane + 1));
    h ^= fingerprint_mix(b1 + 0xc2b2ae3d27d4eb4full * (lane + 65));
    h ^= fingerprint_mix(b2 + 0x165667b19e3779f9ull * (lane + 129));
    h ^= fingerprint_mix(((s0 << 32) | s1) + 0x27d4eb2f165667c5ull * (lane + 193));
    // Six exchange steps -- pairs, quads, eights (lane i <-> 7 - i), sixteens (i <-> 15 - i), the 16-lane rows, the halves --
    // with the data-parallel permutations of the VALU: an LDS-crossbar shuffle costs a hundred cycles a step, and the
    // workgroup that checks a cached copy must not outlast the ones that do the work.  Lane 0's value depends on all 64.
    uint32_t lo = static_cast<uint32_t>(h), hi32 = static_cast<uint32_t>(h >> 32);
    auto fold = [&](uint32_t partner_lo, uint32_t partner_hi) {
        lo += partner_lo * 0x85ebca6bu + 1u;                    // not symmetric: the lanes end up with different values
        hi32 ^= partner_hi;
    };
    auto dpp = [](uint32_t v, auto ctrl) {
        return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), decltype(ctrl)::value, 0xf, 0xf, true));
    };
    auto swap_rows = [](uint32_t v, bool halves) {              // the value of lane ^ 16 (lane ^ 32): see cross_row_reduce
        uint32_t a = v, b = v;
        if (halves) asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
        else asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
        return a ^ b ^ v;                                       // {a, b} = {own, partner}
    };
    fold(dpp(lo, std::integral_constant<int, 0xB1>{}), dpp(hi32, std::integral_constant<int, 0xB1>{}));      // quad_perm [1,0,3,2]
    fold(dpp(lo, std::integral_constant<int, 0x4E>{}), dpp(hi32, std::integral_constant<int, 0x4E>{}));      // quad_perm [2,3,0,1]
    fold(dpp(lo, std::integral_constant<int, 0x141>{}), dpp(hi32, std::integral_constant<int, 0x141>{}));    // row_half_mirror
    fold(dpp(lo, std::integral_constant<int, 0x140>{}), dpp(hi32, std::integral_constant<int, 0x140>{}));    // row_mirror
    fold(swap_rows(lo, false), swap_rows(hi32, false));
    fold(swap_rows(lo, true), swap_rows(hi32, true));
    return fingerprint_mix(((static_cast<unsigned long long>(hi32) << 32) | lo) ^ static_cast<unsigned long long>(static_cast<uint32_t>(total)));
}
// One wave: compare with the recorded fingerprint; on a mismatch report the copy's id in the host-visible words.
__device__ __forceinline__ void repack_guard_role(const RepackGuard& g, int lane)
{
    const unsigned long long want = *g.expect;          // requested together with the samples
    const unsigned long long now = repack_fingerprint(g, lane);
    if (lane == 0 && now != want) {
        volatile uint32_t* flags = g.stale;
        flags[1 + g.id % 1023u] = g.id;
        flags[0] = 1u;
    }
}

// Reference format -> P2.  One wave per 16x64 band-tile; lane (i, g) produces word 4*i + g.
template <int WAVES>
__global__ __launch_bounds__(WAVES * 64) void terna_repack_kernel(
    const uint64_t* __restrict__ bitmap, const int* __restrict__ tile_off,
    const uint16_t* __restrict__ median_off, const uint32_t* __restrict__ sign_words,
    uint32_t* __restrict__ packed, int N, int K)
{
    __shared__ uint32_t lut[256];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    for (int e = tid; e < 256; e += WAVES * 64) lut[e] = make_lut_code(e);
    __syncthreads();

    const int band = blockIdx.x;
    const int gm = band >> 2, med = band & 3;
    const int ktiles = K >> 6;
    const int last_word = (tile_off[(N >> 6) * ktiles] >> 5) - 1;
    const LaneGeom q(lane);

    for (int gk = wave; gk < ktiles; gk += WAVES) {
        const int tile = gm * ktiles + gk;
        const uint64_t* bmp = bitmap + static_cast<size_t>(tile) * 64 + med * 16;
        const uint64_t bm[2] = {bmp[q.b0], bmp[q.b0 + 1]};
        int base = tile_off[tile];
        if (med) base += median_off[3 * tile + med - 1];
        uint32_t win = 0;
        if (last_word >= 0) {
            const int wi = (base >> 5) + lane;
            win = sign_words[wi < last_word ? wi : last_word];
        }
        uint32_t idx[2][2];
        band_tile_indices_win(q, bm, base, win, idx);
        const uint32_t word = lut[idx[0][0]] | (lut[idx[0][1]] << 4) | (lut[idx[1][0]] << 16) | (lut[idx[1][1]] << 20);
        packed[(static_cast<size_t>(band) * ktiles + gk) * 64 + q.i * 4 + q.g] = word;
    }
}

}  // namespace terna
