// Large-M TernaSpMM kernel on the P2 layout (see packed_common.h): a bf16 MFMA GEMM whose weight
// operand goes global memory -> registers -> matrix core, expanded by v_perm_b32, and never
// touches LDS.
//
//   out[m][n] = epilogue( sum_k X[m][k] * W2[n][k] / 2 ),   W2 = 2 W in {-2, 0, +2}
//
// Tiling.  One workgroup (4 waves) owns BN = 128*NA output features x BM = 32*MB batch rows and walks
// K in steps of 64.  The waves split the output features only: wave w owns rows 32*NA*w .. +32*NA-1 and
// ALL BM batch rows, i.e. NA x MB accumulator tiles of v_mfma_f32_32x32x16_bf16 with W as the A
// operand -- so every weight is expanded exactly once per workgroup, and one expansion (ten VALU
// ops) feeds MB matrix instructions.  A-operand lane (row = L%32, kb = L/32) of row-tile a needs,
// for 16-column group g, columns 8kb .. 8kb+7 of packed word (band, gk, i, g): the
// four words g = 0..3 of a row are adjacent, so one 16-byte load per row-tile and k-step brings
// everything the lane needs.  Only the activation tile goes through LDS (two stages, chunk order
// [g][half][row]: 16-byte pieces of 8 columns), staged one k-step ahead; B operands are read one
// group ahead of the MFMAs that use them; weight registers are refilled two k-steps ahead.
#pragma once

#include "packed_common.h"
#include "prefill_kernel.h"

namespace terna {

// 16 int8 -> 16 bf16 in column order (exact: the upper half of the float).
__device__ __forceinline__ void int8x16_to_bf16(const u32x4& v, u32x4& c0, u32x4& c1)
{
    const uint32_t d[4] = {v.x, v.y, v.z, v.w};
    uint32_t o[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        float f[4];
#pragma unroll
        for (int b = 0; b < 4; ++b)
            f[b] = static_cast<float>(static_cast<int>(static_cast<int8_t>((d[j] >> (8 * b)) & 0xff)));
        o[2 * j] = (__float_as_uint(f[0]) >> 16) | (__float_as_uint(f[1]) & 0xffff0000u);
        o[2 * j + 1] = (__float_as_uint(f[2]) >> 16) | (__float_as_uint(f[3]) & 0xffff0000u);
    }
    c0 = u32x4{o[0], o[1], o[2], o[3]};
    c1 = u32x4{o[4], o[5], o[6], o[7]};
}

// A wave's finished 32 batch rows x 32*NA features on their way to memory.  In the accumulator layout a lane holds
// four consecutive features of ONE batch row, so a direct store writes 8 bytes into each of 32 rows that lie N * 2
// bytes apart: 64 lanes, 32 memory segments, and the memory pipeline takes one step per segment.  Through this LDS
// tile the same block leaves as whole rows -- 16 bytes per lane, 4*NA consecutive lanes per row of 64*NA contiguous
// bytes -- in an eighth of the store instructions' pipeline steps (gate+up at M = 2048, same box: int8 76 -> 69 us, and
// 64 us with streaming stores; bf16 120 -> 117 us).
// Rows are 64*NA bytes with no padding; the 16-byte piece c of row r sits at position c ^ swizzle(r) so that both the
// 8-byte writes of 32 consecutive rows and the 16-byte reads of 4*NA-lane rows spread over all banks.
template <int NA>
struct OutTile {
    static constexpr int kRowBytes = 64 * NA;
    static constexpr int kBytes = 32 * kRowBytes;            // per wave
    static constexpr int kPieces = 4 * NA;                   // 16-byte pieces per row
    static constexpr int kRowsPerRead = 64 / kPieces;        // rows that one 64-lane, 16-byte read covers
    static constexpr int kReads = 32 / kRowsPerRead;
    __device__ static constexpr int swizzle(int row) { return (row >> (NA == 2 ? 1 : 2)) & (kPieces - 1); }
};

// Fused epilogue of one wave's NA x MB accumulator tiles (v_mfma_f32_32x32x16 layout: lane holds
// column m = L % 32 and rows n = (v&3) + 8(v>>2) + 4(L/32) of each tile).  A float accumulator is
// twice the true sum (weights were +-2; x0.5 is exact); an integer one is the sum times 64 (weights were +-64; >> 6 is exact).
// `tile`: this wave's OutTile<NA>::kBytes of LDS (results leave as whole rows; needs out and N * 2 to be multiples of
// 16 bytes), or nullptr (every lane stores its 8-byte pieces itself).
// One weight-group scale per 32-feature tile: always under the per-128-column rule of the prefill epilogue and with one
// group, otherwise when the group boundaries fall on multiples of 32.  (Host and device: the launcher picks a kernel by it.)
__host__ __device__ inline bool epilogue_scales_per_tile(const Epilogue& ep, int N)
{
    return ep.kind == EP_I8_PREFILL || ep.ws_num == 1 || (N == 3840 && ep.ws_num == 3) || (N / ep.ws_num) % 32 == 0;
}

// COLS = false leaves out the per-column path (scales that change inside a 32-feature tile): unrolled next to 64 - 128 live
// accumulators it spilled up to 88 registers, so every launch of the larger tiles carried scratch memory for a path that
// almost no call takes.  The launcher sends such calls to the 128 x 64 instantiation, which keeps the path.
template <int MB, int NA, typename AccV, bool COLS = true>
__device__ __forceinline__ void packed_prefill_epilogue(AccV (&acc)[NA][MB], uint16_t* __restrict__ out,
                                                        const Epilogue& ep, int M, int N, int n_wave, int m0, int lane,
                                                        uint8_t* tile = nullptr)
{
    using OT = OutTile<NA>;
    const int kb = lane >> 5, l32 = lane & 31;
    constexpr bool kFloatAcc = std::is_same<AccV, f32x16>::value;
    auto value = [&](auto ac, auto bc, int idx) {
        constexpr int a = decltype(ac)::value, b = decltype(bc)::value;
        if constexpr (kFloatAcc) return acc[a][b][idx] * kBf16WeightUndo;
        else return static_cast<float>(acc[a][b][idx] >> kI8WeightShift);
    };
    int m_of[MB];
    float s_of[MB];
    static_for<0, MB>([&](auto bc) {
        constexpr int b = decltype(bc)::value;
        m_of[b] = m0 + 32 * b + l32;
        s_of[b] = ep.kind == EP_BF16 ? 1.0f : bf16_bits_to_float(ep.s[m_of[b] < M ? m_of[b] : M - 1]);
    });
    // features 32a + 8vq + 4kb .. +3 of batch row 32b + l32
    const int tile_put = l32 * OT::kRowBytes + 8 * kb, tile_swz = OT::swizzle(l32);
    auto store4 = [&](int a, int b, int vq, float r0, float r1, float r2, float r3) {
        const u32x2 v = {pack_bf16x2(r0, r1), pack_bf16x2(r2, r3)};
        if (tile != nullptr) {
            *reinterpret_cast<u32x2*>(tile + tile_put + (((4 * a + vq) ^ tile_swz) << 4)) = v;
        } else {
            const int n = n_wave + 32 * a + 8 * vq + 4 * kb;
            if (m_of[b] < M && n < N) *reinterpret_cast<u32x2*>(out + static_cast<size_t>(m_of[b]) * N + n) = v;
        }
    };
    // after the last store4 of batch block b: its 32 rows leave the tile as rows
    auto flush = [&](int b) {
        if (tile == nullptr) return;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        const int piece = lane & (OT::kPieces - 1);
        const int n = n_wave + 8 * piece;
#pragma unroll
        for (int i = 0; i < OT::kReads; ++i) {
            const int row = i * OT::kRowsPerRead + lane / OT::kPieces;
            const u32x4 v = *reinterpret_cast<const u32x4*>(tile + row * OT::kRowBytes + ((piece ^ OT::swizzle(row)) << 4));
            const int m = m0 + 32 * b + row;
            // written once and read by a later launch: a streaming store keeps it from displacing the operands in L2
            if (m < M && n < N) __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(out + static_cast<size_t>(m) * N + n));
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    };

    // One weight-group scale per 32-feature tile whenever the group boundaries fall on multiples of
    // 32 (always for the per-128-column rule of the prefill epilogue): the per-element work is then
    // one multiply (bf16 family, prefill rule) or one divide and one multiply (decode rule), with
    // the same operations in the same order as apply_epilogue.
    const bool tile_groups = !COLS || epilogue_scales_per_tile(ep, N);
    if (tile_groups) {
        float w_of[NA];
        static_for<0, NA>([&](auto ac) {
            constexpr int a = decltype(ac)::value;
            int n_a = n_wave + 32 * a;
            n_a = n_a < N ? n_a : N - 4;
            const int g = ep.ws_num == 1 ? 0 : (ep.kind == EP_I8_PREFILL ? ws_group_prefill(n_a, N, ep.ws_num)
                                                                       : ws_group_decode(n_a, N, ep.ws_num));
            w_of[a] = ep.kind == EP_BF16 ? ep.scale[g] : bf16_bits_to_float(ep.ws[g]);
        });
        // Separate loops under a uniform branch: written as a select, the compiler evaluates the
        // IEEE division of the decode rule for every element of every kind.
        auto tiles = [&](auto&& element) {
            static_for<0, MB>([&](auto bc) {
                constexpr int b = decltype(bc)::value;
                static_for<0, NA>([&](auto ac) {
                    constexpr int a = decltype(ac)::value;
                    static_for<0, 4>([&](auto vc) {
                        constexpr int vq = decltype(vc)::value;
                        float r[4];
#pragma unroll
                        for (int v = 0; v < 4; ++v) r[v] = element(ac, bc, value(ac, bc, 4 * vq + v));
                        store4(a, b, vq, r[0], r[1], r[2], r[3]);
                    });
                });
                flush(b);
            });
        };
        if (ep.kind == EP_I8_DECODE) {
            tiles([&](auto ac, auto bc, float x) { return __fmul_rn(__fdiv_rn(x, s_of[decltype(bc)::value]), w_of[decltype(ac)::value]); });
        } else if (ep.kind == EP_I8_PREFILL) {
            float coeff[NA][MB];
#pragma unroll
            for (int a = 0; a < NA; ++a)
#pragma unroll
                for (int b = 0; b < MB; ++b) coeff[a][b] = s_of[b] != 0.0f ? __fdiv_rn(w_of[a], s_of[b]) : 0.0f;
            tiles([&](auto ac, auto bc, float x) { return __fmul_rn(x, coeff[decltype(ac)::value][decltype(bc)::value]); });
        } else {
            tiles([&](auto ac, auto, float x) { return __fmul_rn(x, w_of[decltype(ac)::value]); });
        }
        return;
    }
    // group boundaries inside a tile: per-column scales
    if constexpr (COLS) static_for<0, MB>([&](auto bc) {
        constexpr int b = decltype(bc)::value;
        static_for<0, 4 * NA>([&](auto tc) {
            constexpr int a = decltype(tc)::value >> 2, vq = decltype(tc)::value & 3;
            const int n = n_wave + 32 * a + 8 * vq + 4 * kb;
            float wv[4];
            load_col_scales(ep, n < N ? n : N - 4, N, wv);
            EpilogueRegs eb;
            eb.s = s_of[b];
#pragma unroll
            for (int v = 0; v < 4; ++v) eb.w[v] = wv[v];
            float r[4];
#pragma unroll
            for (int v = 0; v < 4; ++v)
                r[v] = bf16_bits_to_float(apply_epilogue<float>(ep.kind, eb, v, value(std::integral_constant<int, a>{}, bc, 4 * vq + v)));
            store4(a, b, vq, r[0], r[1], r[2], r[3]);
        });
        flush(b);
    });
}

// Raw accumulators of one wave into a [M][N] plane of split-K partial sums (same element order as the epilogue).
// `tile`: 4 KiB of LDS of this wave's own.  One 32 x 32 accumulator tile at a time goes through it and leaves as whole
// rows of 128 bytes (16 bytes per lane, 8 consecutive lanes per row), for the reason given at OutTile; the plane's rows
// are 16-byte aligned whenever split-K runs (N is a multiple of 4 and the scratch memory is aligned).  Piece p (16 bytes)
// of row r sits at position p ^ ((r >> 1) & 7): writes and reads are bank-conflict free.
constexpr int kPartialTileBytes = 32 * 128;
template <int MB, int NA, typename AccV, typename AccT>
__device__ __forceinline__ void packed_prefill_store_partial(AccV (&acc)[NA][MB], AccT* __restrict__ plane, int M, int N,
                                                             int n_wave, int m0, int lane, uint8_t* tile)
{
    typedef AccT V4 __attribute__((ext_vector_type(4)));
    static_assert(sizeof(AccT) == 4, "partial sums are 32-bit");
    const int kb = lane >> 5, l32 = lane & 31;
    const int put = l32 * 128, put_swz = (l32 >> 1) & 7;
    const int piece = lane & 7;
    static_for<0, NA>([&](auto ac) {
        constexpr int a = decltype(ac)::value;
        static_for<0, MB>([&](auto bc) {
            constexpr int b = decltype(bc)::value;
            static_for<0, 4>([&](auto vc) {
                constexpr int vq = decltype(vc)::value;          // features 8 vq + 4 kb .. +3 of row l32: piece 2 vq + kb
                *reinterpret_cast<V4*>(tile + put + (((2 * vq + kb) ^ put_swz) << 4)) =
                    V4{acc[a][b][4 * vq], acc[a][b][4 * vq + 1], acc[a][b][4 * vq + 2], acc[a][b][4 * vq + 3]};
            });
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            const int n = n_wave + 32 * a + 4 * piece;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int row = 8 * i + (lane >> 3);
                const V4 v = *reinterpret_cast<const V4*>(tile + row * 128 + ((piece ^ ((row >> 1) & 7)) << 4));
                const int m = m0 + 32 * b + row;
                if (m < M && n < N) __builtin_nontemporal_store(v, reinterpret_cast<V4*>(plane + static_cast<size_t>(m) * N + n));
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
        });
    });
}

template <int MB>
struct PackedPrefillSmem {
    static constexpr int BM = 32 * MB;
    static constexpr int PX = BM * 16 + 16;           // bytes between chunk rows of the X tile (padded)
    static constexpr int kStage = 8 * PX;
    static constexpr int kBytes = 2 * kStage;
};

template <typename Act, int MB, int NA>
__global__ __launch_bounds__(256, MB == 8 ? 1 : (MB == 3 ? 3 : 2)) void terna_prefill_packed_kernel(
    const Act* __restrict__ x, const uint32_t* __restrict__ packed, uint16_t* __restrict__ out,
    Epilogue ep, int M, int N, int K)
{
    using T = ActTraits<Act>;
    using S = PackedPrefillSmem<MB>;
    constexpr int BN = 128 * NA, BM = S::BM, PX = S::PX;
    static_assert(NA == 1 || NA == 2, "32 or 64 output features per wave");
    constexpr int XI = (BM + 63) / 64;                // (row, group) activation items per thread and k-step
    static_assert(MB == 2 || MB == 3 || MB == 4 || MB == 8, "batch tile of 64, 96, 128 or 256 rows");

    extern __shared__ __align__(16) uint8_t smem[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n0 = blockIdx.x * BN, m0 = blockIdx.y * BM;
    const int ktiles = K >> 6;
    const int last_band = (N >> 4) - 1;
    const int kb = lane >> 5, l32 = lane & 31;

    // ---- weight words of this lane: row-tile a -> band (n0/16 + 4*wave + 2a + l32/16), row i = l32 % 16
    const u32x4* w_ptr[NA];                            // running: advanced one k-step per fetch
#pragma unroll
    for (int a = 0; a < NA; ++a) {
        int band = (n0 >> 4) + 2 * NA * wave + 2 * a + (l32 >> 4);
        band = band < last_band ? band : last_band;   // a tile hanging over N re-reads the last band; never stored
        w_ptr[a] = reinterpret_cast<const u32x4*>(packed + (static_cast<size_t>(band) * ktiles) * 64 + (l32 & 15) * 4);
    }
    // ---- activation items of this thread: item = tid + 256*it -> (row = item / 4, group = item % 4)
    int x_lds[XI];
    const Act* x_ptr[XI];
#pragma unroll
    for (int it = 0; it < XI; ++it) {
        const int item = tid + 256 * it;
        int row = item >> 2;
        const int g = item & 3;
        row = row < BM ? row : BM - 1;                // 96-row tile: the spare half-item restages the last row
        x_lds[it] = (g * 2) * PX + row * 16;
        int m = m0 + row;
        m = m < M ? m : M - 1;
        x_ptr[it] = x + static_cast<size_t>(m) * K + g * 16;
    }

    struct RawW { u32x4 w[NA]; };                     // [a] -> words g = 0..3
    struct RawX { u32x4 x[XI][T::kXVecs]; };
    // Both fetches walk running pointers: one k-step is 16 u32x4 of weights and 64 activations.
    auto fetch_w = [&](RawW& r) {
#pragma unroll
        for (int a = 0; a < NA; ++a) {
            r.w[a] = *w_ptr[a];
            w_ptr[a] += 16;
        }
    };
    auto fetch_x = [&](RawX& r) {
#pragma unroll
        for (int it = 0; it < XI; ++it) {
            const u32x4* p = reinterpret_cast<const u32x4*>(x_ptr[it]);
#pragma unroll
            for (int v = 0; v < T::kXVecs; ++v) r.x[it][v] = p[v];
            x_ptr[it] += 64;
        }
    };
    auto stage_x = [&](const RawX& r, int st) {
#pragma unroll
        for (int it = 0; it < XI; ++it) {
            u32x4 c0, c1;                              // columns 16g .. 16g+7 and 16g+8 .. 16g+15 as bf16
            if constexpr (sizeof(Act) == 2) {
                c0 = r.x[it][0];
                c1 = r.x[it][1];
            } else {
                int8x16_to_bf16(r.x[it][0], c0, c1);
            }
            uint8_t* dst = smem + st * S::kStage + x_lds[it];
            *reinterpret_cast<u32x4*>(dst) = c0;
            *reinterpret_cast<u32x4*>(dst + PX) = c1;
        }
    };

    f32x16 acc[NA][MB];
    {
        const f32x16 zero = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int a = 0; a < NA; ++a)
#pragma unroll
            for (int b = 0; b < MB; ++b) acc[a][b] = zero;
    }

    const int b_off = kb * PX + l32 * 16;                    // + g*2*PX + b*512
    const int wshift = 4 - 4 * kb;                           // columns 8kb .. 8kb+7 of every word (left shift, see expand_chunk_bf16)

    struct BOps { bf16x8 b[MB]; };
    auto load_b = [&](int st, int g, BOps& r) {
        const uint8_t* xs = smem + st * S::kStage + b_off + g * 2 * PX;
#pragma unroll
        for (int b = 0; b < MB; ++b) r.b[b] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(xs + b * 512));
    };
    // One k-step: for each 16-column group g, expand the two A operands from registers and issue
    // 2*MB MFMAs against B operands that were read from LDS one group earlier.
    auto mma_step = [&](const RawW& rw, int st) {
        BOps bcur;
        load_b(st, 0, bcur);
        static_for<0, 4>([&](auto gc) {
            constexpr int g = decltype(gc)::value;
            BOps bnxt;
            if constexpr (g < 3) load_b(st, g + 1, bnxt);
#pragma unroll
            for (int a = 0; a < NA; ++a) {
                const bf16x8 af = __builtin_bit_cast(bf16x8, expand_chunk_bf16(rw.w[a][g] << wshift));
#pragma unroll
                for (int b = 0; b < MB; ++b)
                    acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af, bcur.b[b], acc[a][b], 0, 0, 0);
            }
            if constexpr (g < 3) bcur = bnxt;
        });
    };

    // ---- pipeline.  Two weight buffers: w0 serves even k-steps, w1 odd ones; each is refilled
    // for k + 2 as soon as step k has consumed it, so its loads have a whole k-step to land.
    // Activations: raw registers hold step k + 1 while LDS stage (k & 1) feeds the MFMAs of step k.
    RawW w0, w1;
    RawX x_raw;
    fetch_w(w0);
    fetch_x(x_raw);
    stage_x(x_raw, 0);
    if (ktiles > 1) {
        fetch_x(x_raw);                               // activations first: the loop waits for them before the weights
        fetch_w(w1);
    }
    __syncthreads();
    // k-step k with both look-aheads in range (k + 2 < ktiles)
    auto body_full = [&](int k, RawW& w) {
        stage_x(x_raw, (k + 1) & 1);
        fetch_x(x_raw);
        mma_step(w, k & 1);
        fetch_w(w);
        __syncthreads();
    };
    auto body_tail = [&](int k, RawW& w) {
        if (k + 1 < ktiles) stage_x(x_raw, (k + 1) & 1);
        if (k + 2 < ktiles) fetch_x(x_raw);
        mma_step(w, k & 1);
        if (k + 2 < ktiles) fetch_w(w);
        __syncthreads();
    };
    int k = 0;
    for (; k + 3 < ktiles; k += 2) {
        body_full(k, w0);
        body_full(k + 1, w1);
    }
    if (k < ktiles) body_tail(k++, w0);
    if (k < ktiles) body_tail(k++, w1);
    if (k < ktiles) body_tail(k++, w0);

    packed_prefill_epilogue<MB, NA>(acc, out, ep, M, N, n0 + 32 * NA * wave, m0, lane);
}

// ------------------------------------------------------------------------------------------------
// Variant (bf16 or int8 activations) whose activation tile goes global memory -> LDS directly
// (global_load_lds_dwordx4), with every load of the main loop issued and awaited by hand.
//
// Why by hand: the loop keeps two k-steps of loads in flight and each wait must leave exactly the
// younger ones outstanding; the counters are in-order, so that is one `s_waitcnt vmcnt(n)` with a
// known n per k-step -- folded into the step's only barrier.  Loads written as ordinary C++ get
// their waits from the compiler, which at loop headers settles for far stricter ones.
//
// Activation tile in LDS: three stages of BM rows x 128 bytes (one step = 64 bf16 or 128 int8), as 8
// pieces of 16 bytes; piece p of row r sits at position p ^ swizzle(r), so that the 16-byte
// operand reads of 32 consecutive rows spread over all banks.  One direct load writes 64 lanes x
// 16 bytes = 8 whole rows (lane = 8*row + position) and reads whole 128-byte lines from memory.
//
// Three stages: while step k multiplies out of stage k % 3, X(k+1) is landing in the next one and
// X(k+2) is issued into the third (see the step description inside the kernel).
constexpr int kXSwizzleShift = 1;
__device__ __forceinline__ constexpr int x_swizzle(int row) { return (row >> kXSwizzleShift) & 7; }

// LDS[lds_addr + 16*lane .. +15] <- global[sbase + voff .. +15]; completion is counted by vmcnt.
__device__ __forceinline__ void lds_dma_b128(const void* sbase, uint32_t voff, uint32_t lds_addr)
{
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(voff), "s"(sbase) : "memory");
}
// d <- global[sbase + voff .. +15] without a compiler-generated wait: d may be read only after a
// later wait_loads<>() and a landed(d).
__device__ __forceinline__ void global_load_b128_nowait(u32x4& d, const void* sbase, uint32_t voff)
{
    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(d) : "v"(voff), "s"(sbase) : "memory");
}
__device__ __forceinline__ void landed(u32x4& d) { asm volatile("" : "+v"(d)); }
template <int VM>
__device__ __forceinline__ void wait_loads_and_barrier()
{
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(VM) : "memory");
}

template <int MB>
struct PackedPrefillDmaSmem {
    static constexpr int BM = 32 * MB;
    static constexpr int kStages = 3;
    static constexpr int kStage = BM * 128;
    static constexpr int kBytes = kStages * kStage;
};

template <typename Act, int MB, int NA>
__global__ __launch_bounds__(256, MB * NA <= 4 ? 4 : (MB * NA <= 8 ? 2 : 1)) void terna_prefill_packed_dma_kernel(
    const Act* __restrict__ x, const uint32_t* __restrict__ packed, uint16_t* __restrict__ out,
    Epilogue ep, int M, int N, int K, int xcd_map, int splits, void* __restrict__ partial, int guard_on, RepackGuard guard)
{
    // guard_on: the launch runs on a cached copy of a caller's weight and carries one extra row of workgroups in y, the
    // first of which checks the copy's fingerprint next to the others (a launch of its own cost 1.5 - 2 us per call: 11 %
    // of a step at M = 256); the rest of that row leaves at once.
    const int tile_rows = static_cast<int>(gridDim.y) - (guard_on ? 1 : 0);
    if (guard_on && static_cast<int>(blockIdx.y) == tile_rows) {
        if (blockIdx.x == 0 && blockIdx.z == 0 && threadIdx.x < 64) repack_guard_role(guard, threadIdx.x);
        return;
    }
    using S = PackedPrefillDmaSmem<MB>;
    constexpr int BN = 128 * NA, BM = S::BM;
    // One step is 128 bytes of every activation row: 64 bf16 columns (one 64-column weight tile,
    // v_mfma_f32_32x32x16_bf16) or 128 int8 columns (two tiles, v_mfma_i32_32x32x32_i8; the lanes
    // of k-half kb take tile 2*step + kb whole, one 16-column word per MFMA).
    constexpr bool I8 = sizeof(Act) == 1;
    using AccV = typename std::conditional<I8, i32x16, f32x16>::type;
    static_assert(NA == 1 || NA == 2, "32 or 64 output features per wave");
    static_assert(MB == 2 || MB == 4, "batch tile of 64 or 128 rows (all stages below 64 KiB of LDS)");

    extern __shared__ __align__(16) uint8_t smem[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // Workgroup -> tile.  Workgroups go to the 8 XCDs round robin by their linear index, and each XCD
    // has its own L2: when the batch tiles divide by 8, XCD c gets batch tiles c*T/8 .. and walks
    // through them feature tile by feature tile, so its share of the activations (a few MB) stays in
    // its L2 and a weight tile is fetched once per XCD per pass instead of the activations being
    // streamed again for every feature tile.
    int n_tile = blockIdx.x, m_tile = blockIdx.y;
    if (xcd_map) {
        const int linear = blockIdx.y * gridDim.x + blockIdx.x;
        const int per_xcd = tile_rows >> 3;          // batch tiles per XCD
        const int xcd = linear & 7, idx = linear >> 3;
        m_tile = xcd * per_xcd + idx % per_xcd;
        n_tile = idx / per_xcd;
    }
    const int n0 = n_tile * BN, m0 = m_tile * BM;
    const int ktiles = K >> 6;
    const int steps = I8 ? (ktiles + 1) >> 1 : ktiles;
    // int8 with an odd tile count: in the last step the kb = 1 half has no tile.  Its loads are
    // pulled back onto the kb = 0 half's addresses (in bounds) and its weights are zeroed.
    const bool half_tail = I8 && (ktiles & 1);
    // Split-K (gridDim.z = splits > 1, partial != NULL): this workgroup walks the steps k_begin .. k_end - 1 only and
    // leaves its raw accumulators in partial[blockIdx.z][M][N]; terna_splitk_reduce_kernel sums the splits in order.
    const int k_begin = splits > 1 ? static_cast<int>(static_cast<long>(steps) * blockIdx.z / splits) : 0;
    const int k_end = splits > 1 ? static_cast<int>(static_cast<long>(steps) * (blockIdx.z + 1) / splits) : steps;
    const int last_band = (N >> 4) - 1;
    const int kb = lane >> 5, l32 = lane & 31;

    // ---- weights: row-tile a -> band (n0/16 + 2*NA*wave + 2a + l32/16), row l32 % 16; a tile is 256 bytes
    constexpr int kWStep = I8 ? 512 : 256;
    uint32_t w_off[NA];
#pragma unroll
    for (int a = 0; a < NA; ++a) {
        int band = (n0 >> 4) + 2 * NA * wave + 2 * a + (l32 >> 4);
        band = band < last_band ? band : last_band;   // a tile hanging over N re-reads the last band; never stored
        w_off[a] = static_cast<uint32_t>(band) * static_cast<uint32_t>(ktiles) * 256u + (l32 & 15) * 16 + (I8 ? kb * 256 : 0);
    }
    const uint8_t* w_base = reinterpret_cast<const uint8_t*>(packed);
    // ---- activations: direct load j of this wave fills rows 8*(wave + 4j) .. +7 of the stage
    uint32_t x_off[MB], x_tail[MB];
#pragma unroll
    for (int j = 0; j < MB; ++j) {
        const int row = 8 * (wave + 4 * j) + (lane >> 3);
        const int piece = (lane & 7) ^ x_swizzle(row);
        int m = m0 + row;
        m = m < M ? m : M - 1;
        x_off[j] = static_cast<uint32_t>(m) * static_cast<uint32_t>(K) * static_cast<uint32_t>(sizeof(Act)) + piece * 16;
        x_tail[j] = piece >= 4 ? 64 : 0;
    }
    const uint8_t* x_base = reinterpret_cast<const uint8_t*>(x);
    const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(smem)) + wave * 1024;

    // Stage of k-step kk is kk % 3, kept as running byte offsets (no division in the loop).
    auto next_stage = [](int st) { return st == 2 * S::kStage ? 0 : st + S::kStage; };
    auto issue_x = [&](int kk, int st) {
        const uint8_t* base = x_base + static_cast<size_t>(kk) * 128;
        const bool pull_back = half_tail && kk == steps - 1;
#pragma unroll
        for (int j = 0; j < MB; ++j)
            lds_dma_b128(base, pull_back ? x_off[j] - x_tail[j] : x_off[j], lds0 + st + j * 4096);
    };
    struct RawW { u32x4 w[NA]; };
    auto fetch_w = [&](RawW& r, int kk) {
        const uint8_t* base = w_base + static_cast<size_t>(kk) * kWStep;
        const bool pull_back = half_tail && kk == steps - 1;
#pragma unroll
        for (int a = 0; a < NA; ++a) global_load_b128_nowait(r.w[a], base, pull_back ? w_off[a] - kb * 256 : w_off[a]);
    };

    AccV acc[NA][MB];
#pragma unroll
    for (int a = 0; a < NA; ++a)
#pragma unroll
        for (int b = 0; b < MB; ++b)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[a][b][v] = 0;

    // B operand of (group g, tile b): row 32b + l32, piece 2g + kb (bf16: columns 16g + 8kb .. +7)
    // or 4kb + g (int8: columns 64kb + 16g .. +15); swizzle(32b + l32) == swizzle(l32)
    int b_off[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) b_off[g] = l32 * 128 + ((((I8 ? 4 * kb + g : 2 * g + kb)) ^ x_swizzle(l32)) * 16);
    const int wshift = 4 - 4 * kb;                           // bf16: columns 8kb .. 8kb+7 of every word (left shift, see expand_chunk_bf16)

    struct BOps { u32x4 b[MB]; };
    auto load_b = [&](int st, int g, BOps& r) {
        const uint8_t* stage = smem + st;
#pragma unroll
        for (int b = 0; b < MB; ++b) r.b[b] = *reinterpret_cast<const u32x4*>(stage + b_off[g] + b * 4096);
    };
    // One 16-column group: expand the NA weight operands and issue NA*MB MFMAs against `bcur`.
    uint32_t wmask = kTopFieldMask;                          // int8: 0 in the lanes without a tile (odd tile count, last step)
    auto mma_group = [&](const RawW& rw, auto gc, const BOps& bcur) {
        constexpr int g = decltype(gc)::value;
#pragma unroll
        for (int a = 0; a < NA; ++a) {
            if constexpr (I8) {
                const i32x4 af = expand_word_i8(rw.w[a][g], wmask);
#pragma unroll
                for (int b = 0; b < MB; ++b)
                    acc[a][b] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af, __builtin_bit_cast(i32x4, bcur.b[b]), acc[a][b], 0, 0, 0);
            } else {
                const bf16x8 af = __builtin_bit_cast(bf16x8, expand_chunk_bf16(rw.w[a][g] << wshift));
#pragma unroll
                for (int b = 0; b < MB; ++b)
                    acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af, __builtin_bit_cast(bf16x8, bcur.b[b]), acc[a][b], 0, 0, 0);
            }
        }
    };

    // A hand-issued load writes its registers (or LDS) whenever it lands, which the compiler does
    // not know: every one of them must be followed, on every path, by a wait that covers it
    // before its destination can be reused -- so none is issued for steps past the end.
    //
    // Step k, with its one barrier in the middle (so that the operand reads of the next group
    // are always in flight across it and across the step boundary):
    //   groups 0, 1                       operands of group g+1 are read while group g multiplies
    //   s_waitcnt vmcnt(NA); s_barrier    own part of X(k+1) landed; everybody is past step k-1
    //   issue X(k+2) -> stage (k+2) % 3   == stage of step k-1, which nobody reads any more
    //   groups 2, 3                       group 3 reads group 0 of step k+1
    //   issue W(k+2); s_waitcnt vmcnt(MB + NA)   W(k+1) landed; X(k+2), W(k+2) stay in flight
    // The scheduling fences keep the compiler from hoisting operand reads (8*MB registers if all
    // go to the top) or sinking MFMAs across the hand-placed waits.
    RawW w0, w1;
    BOps b_a, b_b;
    int st_mma = 0;                                          // stage of the step being multiplied
    int st_dma = 2 * S::kStage;                              // stage that the next direct load fills
    issue_x(k_begin, 0);
    fetch_w(w0, k_begin);
    if (k_end - k_begin > 1) {
        issue_x(k_begin + 1, S::kStage);
        fetch_w(w1, k_begin + 1);
        wait_loads_and_barrier<MB + NA>();
    } else {
        wait_loads_and_barrier<0>();
    }
    load_b(0, 0, b_a);
    auto body = [&](int k, RawW& w) {
        const bool more1 = k + 1 < k_end, more2 = k + 2 < k_end;        // uniform
        const int st_next = next_stage(st_mma);
#pragma unroll
        for (int a = 0; a < NA; ++a) landed(w.w[a]);
        wmask = (half_tail && k == steps - 1 && kb) ? 0u : kTopFieldMask;   // its loads were pulled onto the kb = 0 half's addresses
        __builtin_amdgcn_sched_barrier(0);
        load_b(st_mma, 1, b_b);
        mma_group(w, std::integral_constant<int, 0>{}, b_a);
        __builtin_amdgcn_sched_barrier(0);
        load_b(st_mma, 2, b_a);
        mma_group(w, std::integral_constant<int, 1>{}, b_b);
        __builtin_amdgcn_sched_barrier(0);
        if (more1) asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(NA) : "memory");
        if (more2) issue_x(k + 2, st_dma);
        __builtin_amdgcn_sched_barrier(0);
        load_b(st_mma, 3, b_b);
        mma_group(w, std::integral_constant<int, 2>{}, b_a);
        __builtin_amdgcn_sched_barrier(0);
        if (more1) load_b(st_next, 0, b_a);
        mma_group(w, std::integral_constant<int, 3>{}, b_b);
        __builtin_amdgcn_sched_barrier(0);
        if (more2) {
            fetch_w(w, k + 2);
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(MB + NA) : "memory");
        } else {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        __builtin_amdgcn_sched_barrier(0);
        st_mma = st_next;
        st_dma = next_stage(st_dma);
    };
    int k = k_begin;
    for (; k + 1 < k_end; k += 2) {
        body(k, w0);
        body(k + 1, w1);
    }
    if (k < k_end) body(k, w0);

    // Results (or split-K partial sums) leave as whole rows through a per-wave LDS tile; the tiles take the place of the
    // activation stages once every wave is done reading those.
    static_assert(4 * OutTile<NA>::kBytes <= S::kBytes && 4 * kPartialTileBytes <= S::kBytes, "output tiles fit in the activation stages");
    __syncthreads();
    if (partial != nullptr) {
        using AccT = typename std::conditional<I8, int, float>::type;
        packed_prefill_store_partial<MB, NA>(acc, static_cast<AccT*>(partial) + static_cast<size_t>(blockIdx.z) * M * N, M, N,
                                             n0 + 32 * NA * wave, m0, lane, smem + wave * kPartialTileBytes);
        return;
    }
    // ... for the final results whenever 16-byte stores can address the output
    const bool rows_ok = ((reinterpret_cast<uintptr_t>(out) | (static_cast<uintptr_t>(N) * 2)) & 15) == 0;
    packed_prefill_epilogue<MB, NA, AccV, MB == 2 && NA == 1>(acc, out, ep, M, N, n0 + 32 * NA * wave, m0, lane,
                                                                rows_ok ? smem + wave * OutTile<NA>::kBytes : nullptr);
}

// Second launch of a split-K call: out[m][n0 .. n0+3] = epilogue(sum over the splits, in split order, of partial[z][m][n]).
// AccT = int (int8 family: the sum is exact, so the result is that of the unsplit kernel bit for bit) or float (bf16
// family: weights were +-2, the sum is halved first, as in the unsplit epilogue).  One thread per four columns.
template <typename AccT>
__global__ __launch_bounds__(256) void terna_splitk_reduce_kernel(const AccT* __restrict__ partial, uint16_t* __restrict__ out,
                                                                  Epilogue ep, int M, int N, int splits, int guard_on, RepackGuard guard)
{
    // guard_on: the first workgroup of the grid checks the cached copy the planes were computed from (see the main kernel)
    if (guard_on && blockIdx.x == 0) {
        if (threadIdx.x < 64) repack_guard_role(guard, threadIdx.x);
        return;
    }
    typedef AccT V4 __attribute__((ext_vector_type(4)));
    const int quads = N >> 2;
    const long idx = (static_cast<long>(blockIdx.x) - (guard_on ? 1 : 0)) * 256 + threadIdx.x;
    if (idx >= static_cast<long>(M) * quads) return;
    const int m = static_cast<int>(idx / quads), n0 = static_cast<int>(idx - static_cast<long>(m) * quads) * 4;
    const size_t at = static_cast<size_t>(m) * N + n0, plane = static_cast<size_t>(M) * N;
    V4 sum = *reinterpret_cast<const V4*>(partial + at);
    for (int z = 1; z < splits; ++z) sum += *reinterpret_cast<const V4*>(partial + z * plane + at);
    const EpilogueRegs e = load_epilogue(ep, m, n0, N);
    uint16_t o[4];
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        if constexpr (std::is_same<AccT, float>::value) o[v] = apply_epilogue<float>(ep.kind, e, v, sum[v] * kBf16WeightUndo);
        else o[v] = apply_epilogue<int>(ep.kind, e, v, sum[v] >> kI8WeightShift);   // planes hold the sums << 6, like the accumulators
    }
    *reinterpret_cast<u32x2*>(out + at) = u32x2{o[0] | (static_cast<uint32_t>(o[1]) << 16), o[2] | (static_cast<uint32_t>(o[3]) << 16)};
}

}  // namespace terna
