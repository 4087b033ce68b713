// Small-M TernaSpMM kernel for gfx950: streams the compressed weight format once and
// multiplies it by a handful of activation rows.
//
// Work split.  One workgroup owns one 16-row band of W (a "median tile" row of the
// format, the smallest unit with its own sign-stream offset) over the whole K, for up
// to 16*MB batch rows.  Its WAVES wavefronts take the band's 64-column tiles round
// robin, accumulate in MFMA registers, and are summed through LDS in a fixed order.
// The scale epilogue and the bf16 store are fused behind that sum: one launch, no
// global workspace, no atomics, bit-reproducible.
//
// Lane mapping for one 16x64 band-tile (16 bitmaps b = 4*g + 2*sk + sm, bit = 8*r + c
// <-> row 8*sk + r, column 16*g + 4*(c>>1) + 2*sm + (c&1)):
//   lane L: i = L & 15 (W row inside the band, also the batch row of the B operand),
//           g = L >> 4 (16-column group).
//   One byte of a bitmap is 8 weights of one row, which is exactly one lane's share of a
//   16x16x32 MFMA A operand.  MFMA number t (t = sm = 0,1) therefore takes byte r = i&7
//   of bitmap 4g + 2(i>>3) + t.  The matching B operand is dwords t, 2+t, 4+t, 6+t of the
//   32 contiguous bytes X[m][64*gk + 16*g ..], so X needs no shuffling at all.
//   Sign bits: position of a lane's byte in the stream = tile offset + band offset
//   + popcounts of earlier bitmaps (16-lane DPP prefix scan) + popcount of the lower bytes.
//   The (nonzero nibble, next 4 sign bits) pair indexes a 256-entry LDS table that yields the
//   four bf16 (or int8) operand values in one read.
#pragma once

#include "terna_common.h"


namespace terna {

template <typename Act> struct ActTraits;

template <> struct ActTraits<uint16_t> {        // bf16 activations, fp32 accumulate
    using Acc = f32x4;
    using AccScalar = float;
    using Lut = u32x2;
    static constexpr int kXVecs = 2;             // 2 x 16 B = 16 bf16 per (row, 16-col group)
    __device__ static Lut make_lut(int e) { const uint2 v = make_lut_bf16(e); return u32x2{v.x, v.y}; }
};

template <> struct ActTraits<int8_t> {          // int8 activations, int32 accumulate
    using Acc = i32x4;
    using AccScalar = int;
    using Lut = uint32_t;
    static constexpr int kXVecs = 1;             // 16 B = 16 int8
    __device__ static Lut make_lut(int e) { return make_lut_i8(e); }
};

// Activations reach the MFMA B operand through a wave-private LDS slot.  The operand wants lane
// (m = L & 15, g = L >> 4) to hold 32 bytes of batch row m -- sixteen different rows in sixteen
// adjacent lanes, which a global load can only serve one cache line per lane.  So a wave loads
// its [16 rows][64 columns] slab the other way round (adjacent lanes walk along a row: 8 lanes per
// 128-byte row segment, fully coalesced), drops it into LDS with a padded row pitch, and reads
// it back in operand order; both LDS accesses are bank-conflict free.
template <typename Act> struct XSlab;
template <> struct XSlab<uint16_t> {              // bf16: a row segment is 128 B = 8 lanes x 16 B
    static constexpr int kPitch = 144, kLoads = 2;   // two loads: rows 0-7 and rows 8-15
    __device__ static int row_of(int lane, int h) { return 8 * h + (lane >> 3); }
    __device__ static int col_of(int lane) { return (lane & 7) * 8; }             // in elements
    __device__ static int write_off(int lane, int h) { return row_of(lane, h) * kPitch + (lane & 7) * 16; }
};
template <> struct XSlab<int8_t> {                // int8: a row segment is 64 B = 4 lanes x 16 B
    static constexpr int kPitch = 80, kLoads = 1;    // one load covers all 16 rows
    __device__ static int row_of(int lane, int) { return lane >> 2; }
    __device__ static int col_of(int lane) { return (lane & 3) * 16; }
    __device__ static int write_off(int lane, int) { return (lane >> 2) * kPitch + (lane & 3) * 16; }
};

__device__ __forceinline__ int row16_inclusive_scan(int v)
{
    // Inclusive prefix sum inside each row of 16 lanes: row_shr:n with bound_ctrl (zeros shifted in).
    v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, true);
    v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, true);
    v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, true);
    v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, true);
    return v;
}

// Per-lane constants of the band-tile mapping described at the top of this file.
struct LaneGeom {
    int i, g, sk, r, b0;
    uint32_t lo_mask, hi_mask;     // bits of a bitmap that precede byte r
    __device__ explicit LaneGeom(int lane)
    {
        i = lane & 15;
        g = lane >> 4;
        sk = i >> 3;
        r = i & 7;
        b0 = 4 * g + 2 * sk;       // bitmap for t = 0; t = 1 is the next one
        lo_mask = r >= 4 ? 0xffffffffu : ((1u << (8 * r)) - 1u);
        hi_mask = r > 4 ? ((1u << (8 * (r - 4))) - 1u) : 0u;
    }
};

// For one band-tile: the two bytes (t = 0, 1) of nonzero flags this lane owns and the four
// expansion-table indices that turn them into operand values.
//   scan_bm   bitmap (lane & 15) of the band-tile, bm[t] bitmap b0 + t
//   sign_base stream position (in bits) where the band-tile's signs start
__device__ __forceinline__ void band_tile_indices(const LaneGeom& q, uint64_t scan_bm, const uint64_t bm[2],
                                                  int sign_base, const uint32_t* __restrict__ sign_words,
                                                  int last_word, uint32_t idx[2][2])
{
    const int pc = __popcll(scan_bm);
    const int excl = row16_inclusive_scan(pc) - pc;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        const uint32_t lo = static_cast<uint32_t>(bm[t]);
        const uint32_t hi = static_cast<uint32_t>(bm[t] >> 32);
        const uint32_t nzb = ((q.r >= 4 ? hi : lo) >> (8 * (q.r & 3))) & 0xffu;
        const int below = __popc(lo & q.lo_mask) + __popc(hi & q.hi_mask);
        const int before = __builtin_amdgcn_ds_bpermute((q.b0 + t) << 2, excl);
        const int pos = sign_base + before + below;
        uint32_t w0 = 0, w1 = 0;
        if (nzb) {                          // a set bit guarantees pos>>5 is a valid word
            const int wi = pos >> 5;
            w0 = sign_words[wi];
            w1 = sign_words[wi < last_word ? wi + 1 : last_word];
        }
        const uint32_t sbits = __builtin_amdgcn_alignbit(w1, w0, pos & 31);
        const uint32_t n_lo = nzb & 15u;
        idx[t][0] = (n_lo << 4) | (sbits & 15u);
        idx[t][1] = (nzb & 0xf0u) | ((sbits >> __popc(n_lo)) & 15u);
    }
}

// Stream position (relative to the band-tile start) of bitmap 4g + 2sk for every lane, from
// nothing but the lane's own two bitmaps and three DPP moves:
//   lanes i and i^8 of a 16-lane row hold the two halves (sk = 0, 1) of 16-column group g, so
//   row_ror:8 hands each lane the other half's popcount; the group totals are then prefix-summed
//   across the four rows with row_bcast15 / row_bcast31, the cross-row steps of a wave scan.
__device__ __forceinline__ int band_tile_prefix(const LaneGeom& q, int pc_pair)
{
    const int other = __builtin_amdgcn_update_dpp(0, pc_pair, 0x128, 0xf, 0xf, false);     // row_ror:8
    const int group_total = pc_pair + other;
    int incl = group_total;
    incl += __builtin_amdgcn_update_dpp(0, incl, 0x142, 0xa, 0xf, false);                  // row_bcast15 -> rows 1,3
    incl += __builtin_amdgcn_update_dpp(0, incl, 0x143, 0xc, 0xf, false);                  // row_bcast31 -> rows 2,3
    return incl - group_total + (q.sk ? other : 0);
}

// For one band-tile: the two bytes (t = 0, 1) of nonzero flags this lane owns and the four
// expansion-table indices that turn them into operand values.  The sign bits come from a
// register-resident window: lane j of `win` holds sign word (sign_base >> 5) + j.  A band-tile has
// at most 1024 sign bits, so its stream lies inside words 0..32 of that window, and the window
// address depends only on the offset arrays, never on the bitmaps.
__device__ __forceinline__ void band_tile_indices_win(const LaneGeom& q, const uint64_t bm[2], int sign_base,
                                                      uint32_t win, uint32_t idx[2][2])
{
    uint32_t lo[2], hi[2];
    int pc[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        lo[t] = static_cast<uint32_t>(bm[t]);
        hi[t] = static_cast<uint32_t>(bm[t] >> 32);
        pc[t] = __popc(lo[t]) + __popc(hi[t]);
    }
    int before = band_tile_prefix(q, pc[0] + pc[1]) + (sign_base & 31);   // relative to the window start
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        const uint32_t nzb = ((q.r >= 4 ? hi[t] : lo[t]) >> (8 * (q.r & 3))) & 0xffu;
        const int pos = before + __popc(lo[t] & q.lo_mask) + __popc(hi[t] & q.hi_mask);   // <= 31 + 1024
        before += pc[t];
        const int wsel = (pos >> 5) << 2;
        const uint32_t w0 = __builtin_amdgcn_ds_bpermute(wsel, static_cast<int>(win));
        const uint32_t w1 = __builtin_amdgcn_ds_bpermute(wsel + 4, static_cast<int>(win));
        const uint32_t sbits = __builtin_amdgcn_alignbit(w1, w0, pos & 31);
        const uint32_t n_lo = nzb & 15u;
        idx[t][0] = (n_lo << 4) | (sbits & 15u);
        idx[t][1] = (nzb & 0xf0u) | ((sbits >> __popc(n_lo)) & 15u);
    }
}

// What a lane fetches for one band-tile before any arithmetic.
template <typename Act, int MB>
struct BandTileRaw {
    uint64_t bm[2];                         // bitmaps 4g + 2sk + t
    u32x4    x[MB][XSlab<Act>::kLoads];     // coalesced pieces of the activation slab
    uint32_t win;                           // sign word (sign_base >> 5) + L
    int      sign_base;                     // tile offset + band offset, in sign bits
};

// DEPTH = how many band-tiles ahead a wave keeps its global loads in flight.
template <typename Act, int WAVES, int MB, int DEPTH>
__global__ __launch_bounds__(WAVES * 64) void terna_decode_kernel(
    const Act* __restrict__ x, const uint64_t* __restrict__ bitmap, const int* __restrict__ tile_off,
    const uint16_t* __restrict__ median_off, const uint32_t* __restrict__ sign_words,
    uint16_t* __restrict__ out, int M, int N, int K, Epilogue ep)
{
    using T = ActTraits<Act>;
    using Acc = typename T::Acc;
    using Lut = typename T::Lut;
    constexpr int NBUF = DEPTH + 1;

    // One private copy of the 256-entry expansion table per wave: filling it needs no
    // workgroup barrier, and it happens while the first loads are in flight.
    __shared__ Lut lut_all[WAVES][256];
    __shared__ Acc red[WAVES][MB][64];
    using XS = XSlab<Act>;
    __shared__ __align__(16) uint8_t xslab_all[WAVES][MB][16 * XS::kPitch];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    Lut* lut = lut_all[wave];

    const int band = blockIdx.x;            // 16-row band of W
    const int gm = band >> 2, med = band & 3;
    const int m_base = blockIdx.y * (16 * MB);
    const int ktiles = K >> 6;
    const int last_word = (tile_off[(N >> 6) * ktiles] >> 5) - 1;   // index of the last sign word

    const LaneGeom q(lane);
    const int i = q.i, g = q.g, b0 = q.b0;

    // Coalesced activation pieces of this lane; rows past M are not loaded (their operand is zero
    // and their output column is never stored).
    const Act* xp[MB][XS::kLoads];
    bool x_ok[MB][XS::kLoads];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int h = 0; h < XS::kLoads; ++h) {
            const int m = m_base + mb * 16 + XS::row_of(lane, h);
            x_ok[mb][h] = m < M;
            xp[mb][h] = x + static_cast<size_t>(x_ok[mb][h] ? m : 0) * K + XS::col_of(lane);
        }

    Acc acc[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[mb] = Acc{0, 0, 0, 0};

    const int n0 = band * 16 + 4 * g;

    // This wave's band-tiles: gk = wave, wave + WAVES, ...  (cnt of them)
    const int cnt = ktiles > wave ? (ktiles - wave + WAVES - 1) / WAVES : 0;

    // Sign-stream start of band-tile number (c0 + lane) of this wave, held one per lane.
    // (No load sits inside a branch, here or below: the compiler waits for every outstanding load at the
    // join behind one, which would expose a memory round trip per band-tile.  Indices are clamped instead.)
    // Two steps, so that the offset-free loads of the first band-tiles can go out between the request and the
    // first use of the offsets.
    int base_glob = 0, base_part = 0;
    auto request_bases = [&](int c0) {
        const int j = c0 + lane;
        const int gk = wave + (j < cnt ? j : 0) * WAVES;
        const int tile = gm * ktiles + (gk < ktiles ? gk : ktiles - 1);
        base_glob = tile_off[tile];
        base_part = median_off[3 * tile + (med ? med - 1 : 0)];
    };
    auto finish_bases = [&](int c0) -> int { return c0 + lane < cnt ? base_glob + (med ? base_part : 0) : 0; };

    // Loads that need no offset: the band-tile's bitmaps and the activation slab.
    auto fetch_tile = [&](int j, BandTileRaw<Act, MB>& raw) {
        const int gk_raw = wave + j * WAVES;
        const int gk = gk_raw < ktiles ? gk_raw : ktiles - 1;        // past the end: the last one again, never used
        const int tile = gm * ktiles + gk;
        const uint64_t* bmp = bitmap + static_cast<size_t>(tile) * 64 + med * 16;
        raw.bm[0] = bmp[b0];
        raw.bm[1] = bmp[b0 + 1];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int h = 0; h < XS::kLoads; ++h)
                raw.x[mb][h] = x_ok[mb][h] ? *reinterpret_cast<const u32x4*>(xp[mb][h] + gk * 64) : u32x4{0u, 0u, 0u, 0u};
    };
    // The sign window: needs the band-tile's stream offset.
    // A matrix without nonzeros has no sign words at all: its (unused) window is read from the bitmaps.
    const uint32_t* sign_src = last_word >= 0 ? sign_words : reinterpret_cast<const uint32_t*>(bitmap);
    const int last_idx = last_word >= 0 ? last_word : 0;
    auto fetch_signs = [&](int base, BandTileRaw<Act, MB>& raw) {
        raw.sign_base = base;
        const int wi = (base >> 5) + lane;
        raw.win = sign_src[wi < last_idx ? wi : last_idx];
    };

    uint8_t* slab = xslab_all[wave][0];
    auto process = [&](const BandTileRaw<Act, MB>& cur) {
        // slab in (coalesced order), operands out (MFMA order); same wave, so LDS ordering suffices
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int h = 0; h < XS::kLoads; ++h)
                *reinterpret_cast<u32x4*>(slab + mb * (16 * XS::kPitch) + XS::write_off(lane, h)) = cur.x[mb][h];
        uint32_t idx[2][2];
        band_tile_indices_win(q, cur.bm, cur.sign_base, cur.win, idx);

        if constexpr (sizeof(Act) == 2) {
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const u32x2 a_lo = lut[idx[t][0]];
                const u32x2 a_hi = lut[idx[t][1]];
                const u32x4 a_bits = {a_lo.x, a_lo.y, a_hi.x, a_hi.y};
                const bf16x8 a = __builtin_bit_cast(bf16x8, a_bits);
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
                    const uint8_t* src = slab + mb * (16 * XS::kPitch) + i * XS::kPitch + g * 32;
                    const u32x4 x0 = *reinterpret_cast<const u32x4*>(src);
                    const u32x4 x1 = *reinterpret_cast<const u32x4*>(src + 16);
                    const u32x4 b_bits = t == 0 ? u32x4{x0.x, x0.z, x1.x, x1.z} : u32x4{x0.y, x0.w, x1.y, x1.w};
                    const bf16x8 b = __builtin_bit_cast(bf16x8, b_bits);
                    acc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[mb], 0, 0, 0);
                }
            }
        } else {
            // k order of the 16x16x64 operand: (t, c) -> column 4*(c>>1) + 2*t + (c&1)
            const i32x4 a = {static_cast<int>(lut[idx[0][0]]), static_cast<int>(lut[idx[0][1]]),
                             static_cast<int>(lut[idx[1][0]]), static_cast<int>(lut[idx[1][1]])};
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                const u32x4 xv = *reinterpret_cast<const u32x4*>(slab + mb * (16 * XS::kPitch) + i * XS::kPitch + g * 16);
                const i32x4 b = {   // dword j of xv = columns 4j .. 4j+3
                    static_cast<int>(__builtin_amdgcn_perm(xv.y, xv.x, 0x05040100u)),   // t=0, c=0..3
                    static_cast<int>(__builtin_amdgcn_perm(xv.w, xv.z, 0x05040100u)),   // t=0, c=4..7
                    static_cast<int>(__builtin_amdgcn_perm(xv.y, xv.x, 0x07060302u)),   // t=1, c=0..3
                    static_cast<int>(__builtin_amdgcn_perm(xv.w, xv.z, 0x07060302u))};  // t=1, c=4..7
                acc[mb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, acc[mb], 0, 0, 0);
            }
        }
    };

    // Ring of DEPTH + 1 register buffers, named one by one so that they stay in registers.
    static_assert(DEPTH == 1 || DEPTH == 2, "prefetch distance");
    BandTileRaw<Act, MB> ring0, ring1, ring2;
    int c0 = 0, vbase = 0, ccnt = 0;
    // One ring slot: start the loads of band-tile j + DEPTH into `pre`, then consume `cur`.
    auto slot = [&](int j, const BandTileRaw<Act, MB>& cur, BandTileRaw<Act, MB>& pre) {
        if (j < ccnt) {
            if (j + DEPTH < ccnt) {
                fetch_tile(c0 + j + DEPTH, pre);
                fetch_signs(__builtin_amdgcn_readlane(vbase, j + DEPTH), pre);
            }
            process(cur);
        }
    };
    // Start of a round: offset-free loads go out first so they overlap the offset fetch.
    auto prime = [&]() {
        request_bases(c0);
        fetch_tile(c0, ring0);
        if constexpr (DEPTH == 2) fetch_tile(c0 + 1, ring1);
        __builtin_amdgcn_sched_barrier(0);       // nothing that waits for the offsets moves above the requests
        vbase = finish_bases(c0);
        fetch_signs(__builtin_amdgcn_readlane(vbase, 0), ring0);
        if constexpr (DEPTH == 2) fetch_signs(__builtin_amdgcn_readlane(vbase, 1), ring1);
    };

    // Offsets come 64 band-tiles at a time (one per lane); K <= 4096 * WAVES needs one round.
    ccnt = cnt < 64 ? cnt : 64;
    prime();
    // Wave w finishes m-block w (and w + WAVES, ...): with the data loads in flight, fetch that block's scale
    // factors, so that no global load sits between the last MFMA and the store.
    EpilogueRaw eraw[(MB + WAVES - 1) / WAVES];
#pragma unroll
    for (int e = 0; e < (MB + WAVES - 1) / WAVES; ++e) {
        const int m = m_base + (wave + e * WAVES) * 16 + i;
        eraw[e] = load_epilogue_raw_flat<sizeof(Act) == 2>(ep, m < M ? m : M - 1, n0, N);
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) lut[lane + 64 * e] = T::make_lut(lane + 64 * e);
    while (ccnt > 0) {
        for (int j0 = 0; j0 < ccnt; j0 += NBUF) {
            if constexpr (DEPTH == 2) {
                slot(j0, ring0, ring2);
                slot(j0 + 1, ring1, ring0);
                slot(j0 + 2, ring2, ring1);
            } else {
                slot(j0, ring0, ring1);
                slot(j0 + 1, ring1, ring0);
            }
        }
        c0 += 64;
        ccnt = cnt - c0 < 64 ? cnt - c0 : 64;
        if (ccnt > 0) prime();
    }

    // Cross-wave sum in wave order, then the fused epilogue.  The accumulator layout of a
    // 16x16 MFMA: lane L holds output rows 4*(L>>4) .. +3 of column L & 15.
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) red[wave][mb][lane] = acc[mb];
    __syncthreads();
#pragma unroll
    for (int e = 0; e < (MB + WAVES - 1) / WAVES; ++e) {
        const int mb = wave + e * WAVES;
        if (mb >= MB) break;
        Acc sum = red[0][mb][lane];
#pragma unroll
        for (int w = 1; w < WAVES; ++w) sum += red[w][mb][lane];
        const int m = m_base + mb * 16 + i;
        if (m < M) {
            const EpilogueRegs eregs = finish_epilogue(ep, eraw[e]);
            uint16_t o[4];
#pragma unroll
            for (int v = 0; v < 4; ++v) o[v] = apply_epilogue<typename T::AccScalar>(ep.kind, eregs, v, sum[v]);
            const u32x2 packed = {o[0] | (static_cast<uint32_t>(o[1]) << 16), o[2] | (static_cast<uint32_t>(o[3]) << 16)};
            *reinterpret_cast<u32x2*>(out + static_cast<size_t>(m) * N + n0) = packed;
        }
    }
}

}  // namespace terna
