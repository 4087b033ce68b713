// Large-M TernaSpMM kernel for gfx950: a bf16 MFMA GEMM whose weight operand is decoded from
// the compressed ternary format on the fly, never stored densely in HBM.
//
//   out[m][n] = epilogue( sum_k X[m][k] * W[n][k] )
//
// Tiling.  One workgroup (4 waves) owns BN = 256 output features x BM = 64*MT batch rows and
// walks K in steps of 64 (one column of 64x64 format tiles).  Waves sit 2 (n) x 2 (m); each owns
// 128 x 32*MT outputs as 4 x MT accumulator tiles of v_mfma_f32_32x32x16_bf16 (W is the A
// operand, so a lane ends up with four consecutive output features of one batch row).
//
// LDS holds two stages of two operand tiles in "chunk" order: a chunk is the 16 bytes one lane
// feeds to one MFMA = 8 k-values of one row, and chunks are laid out [g][sm][row] with the row
// fastest, so that the 32 lanes of an operand read touch 512 contiguous bytes (no bank
// conflicts).  g = 16-column group, sm = which of its two interleaved 8-column sets:
//   chunk (row, g, sm) holds columns 16g + 4j + 2sm + {0,1}, j = 0..3 -- exactly the eight
//   weights of one bitmap byte of the format, so the decoder writes a chunk per expansion and
//   the activation loader splits each 32-byte group into its even and odd dwords.
// Every wave decodes 4 of the tile's 16 band-tiles and stages BM/4 activation rows per step,
// one step ahead of the MFMAs that consume them; global loads run two steps ahead.
#pragma once

#include "decode_kernel.h"

namespace terna {

constexpr int kPrefillBN = 256;

template <int MT>
struct PrefillSmem {
    static constexpr int BM = 64 * MT;
    static constexpr int PW = kPrefillBN * 16 + 16;   // bytes between chunk rows of the W tile (padded)
    static constexpr int PX = BM * 16 + 16;           // same for the X tile
    static constexpr int kStage = 8 * PW + 8 * PX;
    static constexpr int kLut = 2 * kStage;           // 256 x 8 B expansion table behind the stages
    static constexpr int kBytes = kLut + 2048;
};

// What a thread prefetches for one k-step: 4 band-tiles of W and its share of X.
template <typename Act, int MT>
struct PrefillRaw {
    static constexpr int XI = MT;                     // (row, group) activation items per thread
    uint64_t bm[4][2];
    uint32_t win[4];
    int      base[4];
    u32x4    x[XI][ActTraits<Act>::kXVecs];
};

// 16 int8 (one dword = 4 consecutive columns) -> the two bf16 chunks (sm = 0, 1) of the group.
// bf16(int8) is exact: the upper half of the float.
__device__ __forceinline__ void int8_group_to_chunks(const u32x4& v, u32x4& c0, u32x4& c1)
{
    const uint32_t d[4] = {v.x, v.y, v.z, v.w};
    uint32_t lo[4], hi[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        float f[4];
#pragma unroll
        for (int b = 0; b < 4; ++b)
            f[b] = static_cast<float>(static_cast<int>(static_cast<int8_t>((d[j] >> (8 * b)) & 0xff)));
        // columns 4j, 4j+1 -> set 0; 4j+2, 4j+3 -> set 1
        lo[j] = (__float_as_uint(f[0]) >> 16) | (__float_as_uint(f[1]) & 0xffff0000u);
        hi[j] = (__float_as_uint(f[2]) >> 16) | (__float_as_uint(f[3]) & 0xffff0000u);
    }
    c0 = u32x4{lo[0], lo[1], lo[2], lo[3]};
    c1 = u32x4{hi[0], hi[1], hi[2], hi[3]};
}

template <typename Act, int MT>
__global__ __launch_bounds__(256, 1) void terna_prefill_kernel(
    const Act* __restrict__ x, const uint64_t* __restrict__ bitmap, const int* __restrict__ tile_off,
    const uint16_t* __restrict__ median_off, const uint32_t* __restrict__ sign_words,
    uint16_t* __restrict__ out, Epilogue ep, int M, int N, int K)
{
    using T = ActTraits<Act>;
    using S = PrefillSmem<MT>;
    using Raw = PrefillRaw<Act, MT>;
    constexpr int BN = kPrefillBN, BM = S::BM, PW = S::PW, PX = S::PX;

    extern __shared__ __align__(16) uint8_t smem[];
    u32x2* lut = reinterpret_cast<u32x2*>(smem + S::kLut);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wn = wave & 1, wm = wave >> 1;
    const int n0 = blockIdx.x * BN, m0 = blockIdx.y * BM;
    const int ktiles = K >> 6;                       // host guarantees ktiles <= 128
    const int last_word = (tile_off[(N >> 6) * ktiles] >> 5) - 1;
    const int last_band = (N >> 4) - 1;

    {
        const uint2 e = make_lut_bf16(tid);
        lut[tid] = u32x2{e.x, e.y};
    }

    const LaneGeom q(lane);

    // ---- this wave's four band-tiles per step: bands 4*wave .. 4*wave+3 of the tile
    int band_med[4];
    const uint64_t* bm_ptr[4];                         // this lane's first bitmap of band u at k-step 0
    int vbase[4][2];                                   // sign-stream start of (band u, k-step lane / 64 + lane)
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        int band = (n0 >> 4) + 4 * wave + u;
        band = band < last_band ? band : last_band;    // a tile hanging over N re-decodes the last band; never stored
        const int gm = band >> 2;
        band_med[u] = band & 3;
        bm_ptr[u] = bitmap + (static_cast<size_t>(gm) * ktiles * 64 + band_med[u] * 16 + q.b0);
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int gk = 64 * h + lane;
            int base = 0;
            if (gk < ktiles) {
                const int tile = gm * ktiles + gk;
                base = tile_off[tile];
                if (band_med[u]) base += median_off[3 * tile + band_med[u] - 1];
            }
            vbase[u][h] = base;
        }
    }

    // ---- activation items of this thread: item = tid + 256*it -> (row = item / 4, group = item % 4)
    int x_lds[Raw::XI];                                // byte offset of the item's sm = 0 chunk in the X tile
    const Act* x_ptr[Raw::XI];
#pragma unroll
    for (int it = 0; it < Raw::XI; ++it) {
        const int item = tid + 256 * it;
        const int row = item >> 2, g = item & 3;
        x_lds[it] = (g * 2) * PX + row * 16;
        int m = m0 + row;
        m = m < M ? m : M - 1;
        x_ptr[it] = x + static_cast<size_t>(m) * K + g * 16;
    }

    // Global loads of k-step gk, one quarter (u) at a time.
    auto fetch_w = [&](int u, int gk, Raw& raw) {
        const uint64_t* bmp = bm_ptr[u] + static_cast<size_t>(gk) * 64;
        raw.bm[u][0] = bmp[0];
        raw.bm[u][1] = bmp[1];
        const int base = gk < 64 ? __builtin_amdgcn_readlane(vbase[u][0], gk & 63)
                                 : __builtin_amdgcn_readlane(vbase[u][1], gk & 63);
        raw.base[u] = base;
        uint32_t win = 0;
        if (last_word >= 0) {
            const int wi = (base >> 5) + lane;
            win = sign_words[wi < last_word ? wi : last_word];
        }
        raw.win[u] = win;
    };
    auto fetch_x = [&](int it, int gk, Raw& raw) {
        const u32x4* p = reinterpret_cast<const u32x4*>(x_ptr[it] + gk * 64);
#pragma unroll
        for (int v = 0; v < T::kXVecs; ++v) raw.x[it][v] = p[v];
    };

    // Decode one prefetched band-tile into stage `st` of the W tile.
    auto decode_w = [&](int u, const Raw& raw, int st) {
        uint8_t* ws = smem + st * S::kStage;
        uint32_t idx[2][2];
        band_tile_indices_win(q, raw.bm[u], raw.base[u], raw.win[u], idx);
        const int row = 16 * (4 * wave + u) + q.i;
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const u32x2 lo = lut[idx[t][0]], hi = lut[idx[t][1]];
            *reinterpret_cast<u32x4*>(ws + (q.g * 2 + t) * PW + row * 16) = u32x4{lo.x, lo.y, hi.x, hi.y};
        }
    };
    // Split one prefetched activation group into its two chunks in stage `st` of the X tile.
    auto stage_x = [&](int it, const Raw& raw, int st) {
        u32x4 c0, c1;
        if constexpr (sizeof(Act) == 2) {
            const u32x4 a = raw.x[it][0], b = raw.x[it][1];
            c0 = u32x4{a.x, a.z, b.x, b.z};
            c1 = u32x4{a.y, a.w, b.y, b.w};
        } else {
            int8_group_to_chunks(raw.x[it][0], c0, c1);
        }
        uint8_t* dst = smem + st * S::kStage + 8 * PW + x_lds[it];
        *reinterpret_cast<u32x4*>(dst) = c0;
        *reinterpret_cast<u32x4*>(dst + PX) = c1;
    };

    f32x16 acc[4][MT];
    {
        const f32x16 zero = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
            for (int b = 0; b < MT; ++b) acc[a][b] = zero;
    }

    const int kb = lane >> 5, l32 = lane & 31;
    struct Operands {
        bf16x8 a[4];
        bf16x8 b[MT];
    };
    const int a_off = kb * PW + (128 * wn + l32) * 16;            // + g*2*PW + a*512
    const int b_off = 8 * PW + kb * PX + (32 * MT * wm + l32) * 16;  // + g*2*PX + b*512
    auto load_operands = [&](int st, int g, Operands& r) {
        const uint8_t* base = smem + st * S::kStage;
#pragma unroll
        for (int a = 0; a < 4; ++a)
            r.a[a] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(base + a_off + g * 2 * PW + a * 512));
#pragma unroll
        for (int b = 0; b < MT; ++b)
            r.b[b] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(base + b_off + g * 2 * PX + b * 512));
    };
    auto mfma_block = [&](const Operands& r) {
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
            for (int b = 0; b < MT; ++b)
                acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(r.a[a], r.b[b], acc[a][b], 0, 0, 0);
    };

    // One k-step = four g-steps.  G-step j multiplies 16-column group j of stage `cur` while it
    // decodes band-tile j and stages activation item j of the NEXT k-step into stage `cur ^ 1`,
    // starts quarter j of the global loads two k-steps ahead, and reads the operands of group j+1.
    // The sched_group_barrier sequence asks the scheduler to deal those side jobs out between the
    // matrix instructions instead of in front of them.
    Raw raw;
    Operands ops;
    auto k_step = [&](int k, auto has_next, auto has_next2) {
        const int cur = k & 1;
        static_for<0, 4>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            Operands nxt;
            if constexpr (j < 3) load_operands(cur, j + 1, nxt);
            if constexpr (decltype(has_next)::value) {
                decode_w(j, raw, cur ^ 1);
                static_for<0, Raw::XI>([&](auto ic) {
                    constexpr int it = decltype(ic)::value;
                    if constexpr (it * (4 / MT) == j) stage_x(it, raw, cur ^ 1);
                });
            }
            if constexpr (decltype(has_next2)::value) {
                fetch_w(j, k + 2, raw);
                static_for<0, Raw::XI>([&](auto ic) {
                    constexpr int it = decltype(ic)::value;
                    if constexpr (it * (4 / MT) == j) fetch_x(it, k + 2, raw);
                });
            }
            mfma_block(ops);
#pragma unroll
            for (int r = 0; r < 4 * MT; ++r) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);               // one MFMA
                __builtin_amdgcn_sched_group_barrier(0x002, 16 / MT, 0);         // vector ALU
                __builtin_amdgcn_sched_group_barrier(0x100, MT >= 2 ? 1 : 3, 0); // LDS reads
                __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);               // LDS write
                __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);               // global read
            }
            if constexpr (j < 3) ops = nxt;
        });
        __syncthreads();
        if constexpr (decltype(has_next)::value) load_operands(cur ^ 1, 0, ops);
    };

    // ---- pipeline: global loads two k-steps ahead, decode one k-step ahead
    static_for<0, 4>([&](auto uc) { fetch_w(decltype(uc)::value, 0, raw); });
    static_for<0, Raw::XI>([&](auto ic) { fetch_x(decltype(ic)::value, 0, raw); });
    __syncthreads();                                  // expansion table ready
    static_for<0, 4>([&](auto uc) { decode_w(decltype(uc)::value, raw, 0); });
    static_for<0, Raw::XI>([&](auto ic) { stage_x(decltype(ic)::value, raw, 0); });
    if (ktiles > 1) {
        static_for<0, 4>([&](auto uc) { fetch_w(decltype(uc)::value, 1, raw); });
        static_for<0, Raw::XI>([&](auto ic) { fetch_x(decltype(ic)::value, 1, raw); });
    }
    __syncthreads();
    load_operands(0, 0, ops);
    int k = 0;
    for (; k + 2 < ktiles; ++k) k_step(k, std::true_type{}, std::true_type{});
    if (k + 1 < ktiles) {
        k_step(k, std::true_type{}, std::false_type{});
        ++k;
    }
    k_step(k, std::false_type{}, std::false_type{});

    // ---- epilogue: lane holds, per accumulator tile, column m = l32 and rows n = (v&3) + 8(v>>2) + 4kb
    EpilogueRegs e[MT];
    int m_of[MT];
    static_for<0, MT>([&](auto bc) {
        constexpr int b = decltype(bc)::value;
        m_of[b] = m0 + 32 * MT * wm + 32 * b + l32;
        e[b].s = ep.kind == EP_BF16 ? 1.0f : bf16_bits_to_float(ep.s[m_of[b] < M ? m_of[b] : M - 1]);
    });
    static_for<0, 16>([&](auto tc) {
        constexpr int a = decltype(tc)::value >> 2, vq = decltype(tc)::value & 3;
        const int n = n0 + 128 * wn + 32 * a + 8 * vq + 4 * kb;
        float wv[4];
        load_col_scales(ep, n < N ? n : N - 4, N, wv);
        static_for<0, MT>([&](auto bc) {
            constexpr int b = decltype(bc)::value;
            EpilogueRegs eb = e[b];
#pragma unroll
            for (int v = 0; v < 4; ++v) eb.w[v] = wv[v];
            uint16_t o[4];
#pragma unroll
            for (int v = 0; v < 4; ++v) o[v] = apply_epilogue<float>(ep.kind, eb, v, acc[a][b][4 * vq + v]);
            const u32x2 packed = {o[0] | (static_cast<uint32_t>(o[1]) << 16),
                                  o[2] | (static_cast<uint32_t>(o[3]) << 16)};
            if (m_of[b] < M && n < N)
                *reinterpret_cast<u32x2*>(out + static_cast<size_t>(m_of[b]) * N + n) = packed;
        });
    });
}

}  // namespace terna
