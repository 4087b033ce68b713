// Multi-token attention over the padded KV cache: the prompt pass of a block (model.py:231-233, where the
// reference calls fmha.memory_efficient_attention_forward on the cache after rope_padded has written the new rows).
//
//   q      bf16 [B][H][T][D]          rotated queries of the T new tokens (ternaspmm_rope_kv_store's q_out)
//   cache  bf16 [B][KV][S][D]         keys / values; the new tokens' rows are already in their slots
//   pos    int64 [T]                  cache slot of new token t; it sees the slots 0 .. pos[t]
//                                     (per_seq != 0: [B][T], sequence b's token t sees 0 .. pos[b][t])
//   out    bf16 [B*T][H*D]            row b*T + t: softmax(scale * q K^T) V, head h in columns h*D ..
//
// One wave per (sequence, head, block of 16 queries), flash-attention style over blocks of 32 cache slots, both
// products on the matrix cores (v_mfma_f32_16x16x32_bf16) in the TRANSPOSED form, so that a score tile comes out of
// the first product in exactly the register layout the second one wants as its B operand:
//   S^T = K Q^T :  A = 16 keys x 32 dims (16 bytes of a key row per lane, straight from the cache),
//                  B = Q^T, held in registers for the whole kernel; lane L ends up with keys 4 (L >> 4) + v,
//                  v = 0 .. 3, of query L & 15 -- all of a lane's scores belong to ONE query, so the running
//                  maximum, the rescale factor and the running sum are per-lane scalars, completed over the
//                  four lanes of a query with two cross-lane exchanges;
//   O^T = V^T P^T: B = P^T: the eight probabilities a lane holds after two score tiles (bf16), as they are;
//                  the k index of this product is a POSITION, position 8g + e of lane group g = L >> 4 standing for
//                  key 4g + e (e < 4) or 16 + 4g + e - 4 of the block -- any one-to-one assignment of keys to
//                  positions works as long as A uses the same one;
//                  A = V^T: row d, those eight keys -- gathered as eight 2-byte reads from the value block staged
//                  in LDS (row pitch 2 D + 8 bytes: the four lane groups fall into disjoint banks).
// fp32 running maximum / sum / output, exp via v_exp_f32, probabilities as a sum of two bf16 terms in the second product.
#pragma once

#include "norm_quant_kernel.h"

namespace terna {

constexpr int kPrefillAttnKeys = 32;          // cache slots per block

// max / sum over the four lanes L, L ^ 16, L ^ 32, L ^ 48 (the four key groups of one query) with the row-swap
// permutations of the VALU: v_permlane16_swap exchanges the odd 16-lane rows of its first operand with the even rows of
// its second, v_permlane32_swap the upper half of the first with the lower half of the second -- applied to two copies
// of v, every lane ends up holding its own value and its partner's (measured: lanes of an even row get (a[L], a[L + 16]),
// of an odd row (b[L - 16], b[L])).  An LDS-crossbar shuffle costs a round trip of the order of a hundred cycles, and
// the running maximum needs two in sequence in every round.
// Written as asm statements: through the builtins the compiler took the two results of a swap for equal and dropped
// the operation between them.  The s_nop covers the wait states the instruction needs after a VALU write of its operands.
template <bool IS_MAX>
__device__ __forceinline__ float key_groups_reduce(float v)
{
    auto op = [](float a, float b) { return IS_MAX ? fmaxf(a, b) : a + b; };
    float a = v, b = v;
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
    v = op(a, b);
    a = v;
    b = v;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
    return op(a, b);
}

template <int D>
__global__ __launch_bounds__(64) void terna_prefill_attention_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ cache_k, const uint16_t* __restrict__ cache_v,
    const long long* __restrict__ pos, uint16_t* __restrict__ out, int T, int H, int KV, int S, float scale, int per_seq)
{
    // no multiply-add contraction: score * scale is rounded once and then used for the maximum and for the exponent;
    // both kernels of this file must round alike to give the same bits
#pragma clang fp contract(off)
    static_assert(D == 64 || D == 128, "head size");
    constexpr int DS = D / 32;                // 32-dimension slices of a row (first product)
    constexpr int DT = D / 16;                // 16-dimension tiles of the output (second product)
    constexpr int PITCH = 2 * D + 8;          // bytes between value rows in LDS
    __shared__ __align__(16) uint8_t vblk[kPrefillAttnKeys * PITCH];

    const int lane = threadIdx.x;
    const int qi = lane & 15, g = lane >> 4;
    const int t0 = blockIdx.x * 16, h = blockIdx.y, b = blockIdx.z;
    const int kvh = h / (H / KV);
    const int t = t0 + qi < T ? t0 + qi : T - 1;                     // rows past T repeat the last one and are not stored
    // prefix length of this lane's query, clamped to the cache (pos comes from device memory)
    long long p64 = pos[(per_seq ? b * T : 0) + t];
    p64 = p64 < 0 ? 0 : (p64 >= S ? S - 1 : p64);
    const int my_last = static_cast<int>(p64);                        // last visible slot
    int n_keys = my_last + 1;
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) n_keys = max(n_keys, __shfl_xor(n_keys, off));
    n_keys = __builtin_amdgcn_readfirstlane(n_keys);                  // largest prefix of the block's queries

    const uint16_t* qrow = q + ((static_cast<size_t>(b) * H + h) * T + t) * D;
    bf16x8 bq[DS];
#pragma unroll
    for (int ds = 0; ds < DS; ++ds) bq[ds] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(qrow + 32 * ds + 8 * g));
    const uint16_t* kbase = cache_k + (static_cast<size_t>(b) * KV + kvh) * S * D;
    const uint16_t* vbase = cache_v + (static_cast<size_t>(b) * KV + kvh) * S * D;

    f32x4 o[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[dt] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    float m_run = -1e30f, l_run = 0.0f;

    for (int k0 = 0; k0 < n_keys; k0 += kPrefillAttnKeys) {
        // ---- requests of the block: key pieces for the two score tiles, value rows for LDS
        u32x4 kr[2][DS];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            int key = k0 + 16 * j + qi;
            key = key < S ? key : S - 1;
#pragma unroll
            for (int ds = 0; ds < DS; ++ds) kr[j][ds] = *reinterpret_cast<const u32x4*>(kbase + static_cast<size_t>(key) * D + 32 * ds + 8 * g);
        }
        constexpr int VPR = D / 8;            // 16-byte vectors per value row
        constexpr int VL = kPrefillAttnKeys * VPR / 64;
        u32x4 vr[VL];
#pragma unroll
        for (int u = 0; u < VL; ++u) {
            const int idx = lane + 64 * u;
            const int key = k0 + idx / VPR;
            // slots past the block's largest prefix were never written (they may hold anything, NaN included, and
            // 0 * NaN would poison the product): read an in-range row instead and zero it
            const u32x4 row = *reinterpret_cast<const u32x4*>(vbase + static_cast<size_t>(key < n_keys ? key : 0) * D + (idx % VPR) * 8);
            vr[u] = key < n_keys ? row : u32x4{0u, 0u, 0u, 0u};
        }
        // ---- scores, transposed: lane = (query qi, keys 4g + v of tile j)
        f32x4 s[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            s[j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int ds = 0; ds < DS; ++ds)
                s[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, kr[j][ds]), bq[ds], s[j], 0, 0, 0);
        }
        float blk_max = -1e30f;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int key = k0 + 16 * j + 4 * g + v;
                s[j][v] = key <= my_last ? s[j][v] * scale : -1e30f;
                blk_max = fmaxf(blk_max, s[j][v]);
            }
        blk_max = key_groups_reduce<true>(blk_max);
        const float m_new = fmaxf(m_run, blk_max);
        const float alpha = __expf(m_run - m_new);
        float p[8], psum = 0.0f;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int key = k0 + 16 * j + 4 * g + v;
                const float e = key <= my_last ? __expf(s[j][v] - m_new) : 0.0f;
                p[4 * j + v] = e;
                psum += e;
            }
        l_run = __fmaf_rn(l_run, alpha, psum);        // this lane's keys only; the four key groups meet after the last block
        m_run = m_new;
        // probabilities as two bf16 terms (value = hi + lo to 16 bits): a single bf16 rounding of P is a relative error of
        // 2^-9 per term, which shows when large value channels nearly cancel; the second product runs once per term
        const u32x4 p_hi = pack_bf16x8(p);
        float hi_f[8], p_lo_f[8];
        unpack_bf16x8(p_hi, hi_f);
#pragma unroll
        for (int e = 0; e < 8; ++e) p_lo_f[e] = p[e] - hi_f[e];
        const bf16x8 bp = __builtin_bit_cast(bf16x8, p_hi), bp_lo = __builtin_bit_cast(bf16x8, pack_bf16x8(p_lo_f));
        // ---- value block through LDS (the previous block's reads are done: one wave, program order + the barrier)
        __syncthreads();
#pragma unroll
        for (int u = 0; u < VL; ++u) {
            const int idx = lane + 64 * u;
            *reinterpret_cast<u32x2*>(vblk + (idx / VPR) * PITCH + (idx % VPR) * 16) = u32x2{vr[u].x, vr[u].y};
            *reinterpret_cast<u32x2*>(vblk + (idx / VPR) * PITCH + (idx % VPR) * 16 + 8) = u32x2{vr[u].z, vr[u].w};
        }
        __syncthreads();
        // ---- O^T += V^T P^T: position 8g + e <-> key 4g + e (e < 4), 16 + 4g + e - 4 (e >= 4)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            const uint8_t* col = vblk + (16 * dt + qi) * 2;
            uint32_t w[4];
#pragma unroll
            for (int e2 = 0; e2 < 4; ++e2) {
                const int ka = (e2 < 2 ? 4 * g + 2 * e2 : 16 + 4 * g + 2 * (e2 - 2));
                const uint32_t lo = *reinterpret_cast<const uint16_t*>(col + ka * PITCH);
                const uint32_t hi = *reinterpret_cast<const uint16_t*>(col + (ka + 1) * PITCH);
                w[e2] = lo | (hi << 16);
            }
#pragma unroll
            for (int v = 0; v < 4; ++v) o[dt][v] *= alpha;
            const bf16x8 va = __builtin_bit_cast(bf16x8, u32x4{w[0], w[1], w[2], w[3]});
            o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va, bp, o[dt], 0, 0, 0);
            o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va, bp_lo, o[dt], 0, 0, 0);
        }
    }

    l_run = key_groups_reduce<false>(l_run);
    if (t0 + qi < T) {
        const float inv = 1.0f / l_run;
        uint16_t* orow = out + (static_cast<size_t>(b) * T + t) * (static_cast<size_t>(H) * D) + static_cast<size_t>(h) * D;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            const u32x2 pk = {pack_bf16x2(o[dt][0] * inv, o[dt][1] * inv), pack_bf16x2(o[dt][2] * inv, o[dt][3] * inv)};
            *reinterpret_cast<u32x2*>(orow + 16 * dt + 4 * g) = pk;
        }
    }
}


// ------------------------------------------------------------------------------------------------
// The same computation with the query heads of a kv head in one workgroup (grouped-query attention: H / KV = G heads
// read the same keys and values).  Wave w is head kvh * G + w over the same block of 16 queries; a block of 32 cache
// slots (64 with four or more heads per workgroup: two softmax steps per block) is fetched ONCE per workgroup,
// coalesced (16 bytes per lane, consecutive lanes on consecutive addresses), two blocks ahead of the one being
// multiplied, and shared through LDS (two buffers, one barrier per block):
//   * rows of a tile are 2 D + 16 bytes apart, so that the 16 rows a 16-byte operand read of the first product
//     touches (A = 16 keys x 32 dims) fall into different banks, and every operand address of a round is one
//     per-lane base plus a constant;
//   * the second product's A operand is V^T -- for one dim, eight keys -- which a row-major tile cannot give in one
//     read per lane.  ds_read_b64_tr_b16 can: within each 16 lanes, lane j supplies the address of 4 consecutive
//     16-bit elements and lane l receives element l % 4 of lanes l / 4, l / 4 + 4, l / 4 + 8, l / 4 + 12 (measured:
//     lane 4c + p gets {in[c][p], in[4 + c][p], in[8 + c][p], in[12 + c][p]}).  With lane j of group g pointing at
//     key 4g + j / 4, dims 4 (j % 4) .. +3 of a 16-dim tile, lane l ends up with dim l of keys 4g .. 4g + 3: two such
//     reads (one per 16-key score tile) are the eight keys of the operand, in the position order the probabilities
//     already have.  The one-wave kernel above gathers the same operand with eight 2-byte reads.
//   * blocks that every query of the workgroup sees whole run without the causal compares; the running output is
//     rescaled only in rounds where some lane's maximum moved (x 1.0 changes nothing: 32 multiplications saved in
//     most rounds once the maxima have settled).
// Arithmetic, order of the sums and therefore the bits of the result are those of the one-wave kernel.
// Workgroups are numbered from the last query block down: under a causal mask those have the most keys to walk.
typedef short s16x4 __attribute__((ext_vector_type(4)));

// d <- global[sbase + voff .. +15] with no compiler-generated wait: d may be read only after attn_wait_loads<N>() with
// N = the number of such loads issued after this one, followed by attn_landed(d).
__device__ __forceinline__ void attn_load_b128_nowait(u32x4& d, const void* sbase, uint32_t voff)
{
    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(d) : "v"(voff), "s"(sbase) : "memory");
}
__device__ __forceinline__ void attn_landed(u32x4& d) { asm volatile("" : "+v"(d)); }
template <int N>
__device__ __forceinline__ void attn_wait_loads() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }

template <int D, int G>
__global__ __launch_bounds__(64 * G) void terna_prefill_attention_group_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ cache_k, const uint16_t* __restrict__ cache_v,
    const long long* __restrict__ pos, uint16_t* __restrict__ out, int T, int H, int KV, int S, float scale, int per_seq)
{
#pragma clang fp contract(off)
    static_assert(D == 64 || D == 128, "head size");
    static_assert(G == 1 || G == 2 || G == 4 || G == 8, "query heads per kv head");
    constexpr int DS = D / 32;                 // 32-dimension slices of a row (first product)
    constexpr int DT = D / 16;                 // 16-dimension tiles of the output (second product)
    constexpr int KB = kPrefillAttnKeys;       // cache slots per softmax step (as in the one-wave kernel)
    constexpr int SUB = G >= 4 ? 2 : 1;        // softmax steps per round: fetch, move to LDS and barrier once per LB slots
    constexpr int LB = SUB * KB;               // cache slots per block in LDS
    constexpr int ROW = 2 * D;                 // bytes of a key / value row in the cache
    constexpr int PITCH = ROW + 16;            // ... and in LDS
    constexpr int PPR = D / 8;                 // 16-byte pieces per row
    constexpr int TILE = LB * PITCH;           // bytes of a key (or value) tile in LDS
    constexpr int PIECES = 2 * LB * PPR;       // pieces of a block: keys, then values
    constexpr int PT = PIECES / (64 * G);      // pieces per thread
    static_assert(PIECES % (64 * G) == 0 && PT >= 1, "a block divides over the workgroup");
    __shared__ __align__(16) uint8_t tiles[2][2 * TILE];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int qi = lane & 15, g = lane >> 4;
    const int t0 = (gridDim.x - 1 - blockIdx.x) * 16, kvh = blockIdx.y, b = blockIdx.z;
    const int h = kvh * G + wave;
    const int t = t0 + qi < T ? t0 + qi : T - 1;
    long long p64 = pos[(per_seq ? b * T : 0) + t];
    p64 = p64 < 0 ? 0 : (p64 >= S ? S - 1 : p64);
    const int my_last = static_cast<int>(p64);
    int n_keys = my_last + 1, n_full = my_last + 1;
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) {
        n_keys = max(n_keys, __shfl_xor(n_keys, off));
        n_full = min(n_full, __shfl_xor(n_full, off));
    }
    n_keys = __builtin_amdgcn_readfirstlane(n_keys);   // largest prefix of the block's queries; same in every wave
    n_full = __builtin_amdgcn_readfirstlane(n_full);   // smallest: slots below it are visible to every query

    const uint16_t* qrow = q + ((static_cast<size_t>(b) * H + h) * T + t) * D;
    bf16x8 bq[DS];
#pragma unroll
    for (int ds = 0; ds < DS; ++ds) bq[ds] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(qrow + 32 * ds + 8 * g));
    const uint16_t* kbase = cache_k + (static_cast<size_t>(b) * KV + kvh) * S * D;
    const uint16_t* vbase = cache_v + (static_cast<size_t>(b) * KV + kvh) * S * D;

    // this thread's pieces of a block: which tile (the same for a whole wave), which row, where in LDS
    int pc_row[PT], pc_lds[PT];
    uint32_t pc_off[PT], pc_piece[PT];        // byte offset inside a block / inside a row
    const uint16_t* pc_base[PT];
    bool pc_val[PT];
#pragma unroll
    for (int u = 0; u < PT; ++u) {
        const int idx = tid + 64 * G * u;
        const int which = __builtin_amdgcn_readfirstlane(idx / (LB * PPR)), rem = idx % (LB * PPR);
        const int row = rem / PPR, piece = rem % PPR;
        pc_row[u] = row;
        pc_val[u] = which != 0;
        pc_base[u] = which ? vbase : kbase;
        pc_piece[u] = piece * 16;
        pc_off[u] = row * ROW + piece * 16;
        pc_lds[u] = which * TILE + row * PITCH + piece * 16;
    }
    // Blocks travel global memory -> registers -> LDS; a block is requested two rounds before it is multiplied (one
    // round is shorter than a trip to memory) and moved into the free LDS buffer one round before.  The requests are
    // issued and awaited by hand: the load counter is in order, so "the block requested in the previous round has landed"
    // is one s_waitcnt vmcnt(n) with n = the loads issued since -- written as ordinary loads, the compiler waits for
    // everything at every round.
    struct Stage { u32x4 v[PT]; };
    // the block's first row goes into the (scalar) base address, so that a whole block costs no address arithmetic per
    // lane; only the last block of a prefix can reach past it, and there the row is pulled back in range
    auto fetch = [&](int k0, Stage& st) {
        if (k0 + LB <= n_keys) {                   // uniform
#pragma unroll
            for (int u = 0; u < PT; ++u) attn_load_b128_nowait(st.v[u], pc_base[u] + static_cast<size_t>(k0) * D, pc_off[u]);
        } else {
#pragma unroll
            for (int u = 0; u < PT; ++u) {
                const int key = k0 + pc_row[u];
                attn_load_b128_nowait(st.v[u], pc_base[u], static_cast<uint32_t>(key < n_keys ? key : n_keys - 1) * ROW + pc_piece[u]);
            }
        }
    };
    // Value slots past the block's largest prefix were never written (they may hold anything, NaN included, and 0 * NaN
    // would poison the product): the in-range row read in their place is zeroed.  Keys only need to be in range: their
    // scores are masked.  `younger`: whether a fetch() was issued after the one that filled `st`.
    auto commit = [&](Stage& st, int k0, int buf, bool younger) {
        if (younger) attn_wait_loads<PT>();
        else attn_wait_loads<0>();
#pragma unroll
        for (int u = 0; u < PT; ++u) attn_landed(st.v[u]);
        if (k0 + LB <= n_keys) {                   // uniform
#pragma unroll
            for (int u = 0; u < PT; ++u) *reinterpret_cast<u32x4*>(&tiles[buf][pc_lds[u]]) = st.v[u];
        } else {
#pragma unroll
            for (int u = 0; u < PT; ++u) {
                const bool dead = pc_val[u] && k0 + pc_row[u] >= n_keys;
                *reinterpret_cast<u32x4*>(&tiles[buf][pc_lds[u]]) = dead ? u32x4{0u, 0u, 0u, 0u} : st.v[u];
            }
        }
    };

    // operand addresses inside a block's tiles: one base per score tile j, the rest are constants
    int ka_base[2], va_base[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        ka_base[j] = (16 * j + qi) * PITCH + 16 * g;                               // + 64 ds: key 16j + qi, dims 32 ds + 8 g .. +7
        va_base[j] = TILE + (16 * j + 4 * g + (qi >> 2)) * PITCH + 8 * (qi & 3);   // + 32 dt: key 16j + 4g + qi / 4, dims 16 dt + 4 (qi % 4) .. +3
    }

    f32x4 o[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[dt] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    float m_run = -1e30f, l_run = 0.0f;

    // the queries must have landed before the first hand-issued request: a compiler-placed wait for them inside the
    // loop would count those requests as its own and drain them every time round
#pragma unroll
    for (int ds = 0; ds < DS; ++ds) asm volatile("" : "+v"(bq[ds]));
    Stage st0, st1;
    fetch(0, st0);
    if (LB < n_keys) fetch(LB, st1);
    commit(st0, 0, 0, LB < n_keys);
    __syncthreads();
    int buf = 0;

    // the KB slots at k0, which start at `tile` in the key tile of the current LDS buffer; MASKED: some query of the
    // workgroup does not see all of them
    auto multiply = [&](int k0, const uint8_t* tile, auto masked) {
        constexpr bool MASKED = decltype(masked)::value;
        // ---- scores, transposed: lane = (query qi, keys 4g + v of tile j)
        f32x4 s[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            s[j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int ds = 0; ds < DS; ++ds) {
                const bf16x8 ka = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(tile + ka_base[j] + 64 * ds));
                s[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka, bq[ds], s[j], 0, 0, 0);
            }
        }
        float blk_max = -1e30f;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int key = k0 + 16 * j + 4 * g + v;
                s[j][v] = (!MASKED || key <= my_last) ? s[j][v] * scale : -1e30f;
                blk_max = fmaxf(blk_max, s[j][v]);
            }
        blk_max = key_groups_reduce<true>(blk_max);
        const float m_new = fmaxf(m_run, blk_max);
        const float alpha = __expf(m_run - m_new);
        float p[8], psum = 0.0f;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int key = k0 + 16 * j + 4 * g + v;
                const float e = (!MASKED || key <= my_last) ? __expf(s[j][v] - m_new) : 0.0f;
                p[4 * j + v] = e;
                psum += e;
            }
        l_run = __fmaf_rn(l_run, alpha, psum);        // this lane's keys only; the four key groups meet after the last block
        m_run = m_new;
        // probabilities as two bf16 terms, as in the one-wave kernel
        const u32x4 p_hi = pack_bf16x8(p);
        float hi_f[8], p_lo_f[8];
        unpack_bf16x8(p_hi, hi_f);
#pragma unroll
        for (int e = 0; e < 8; ++e) p_lo_f[e] = p[e] - hi_f[e];
        const bf16x8 bp = __builtin_bit_cast(bf16x8, p_hi), bp_lo = __builtin_bit_cast(bf16x8, pack_bf16x8(p_lo_f));
        if (__any(alpha != 1.0f)) {
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int v = 0; v < 4; ++v) o[dt][v] *= alpha;
        }
        // ---- O^T += V^T P^T: position 8g + e <-> key 4g + e (e < 4), 16 + 4g + e - 4 (e >= 4)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            s16x4 half[2];
#pragma unroll
            for (int j = 0; j < 2; ++j)
                half[j] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(tile + va_base[j] + 32 * dt));
            const u32x2 h0 = __builtin_bit_cast(u32x2, half[0]), h1 = __builtin_bit_cast(u32x2, half[1]);
            const bf16x8 va = __builtin_bit_cast(bf16x8, u32x4{h0.x, h0.y, h1.x, h1.y});
            o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va, bp, o[dt], 0, 0, 0);
            o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va, bp_lo, o[dt], 0, 0, 0);
        }
    };
    // one round: the block at k0 is multiplied, KB slots at a time; `refill` (whose block is in LDS already) takes the
    // block two ahead, `next` (requested in the previous round) goes into the other buffer, which every wave stopped
    // reading before the barrier that ended the previous round.  All conditions are uniform over the workgroup.
    auto round = [&](int k0, Stage& refill, Stage& next) {
        if (k0 + 2 * LB < n_keys) fetch(k0 + 2 * LB, refill);
#pragma unroll
        for (int sub = 0; sub < SUB; ++sub) {
            const int ks = k0 + sub * KB;
            if (sub > 0 && ks >= n_keys) break;
            const uint8_t* tile = tiles[buf] + sub * KB * PITCH;
            if (ks + KB <= n_full) multiply(ks, tile, std::false_type{});
            else multiply(ks, tile, std::true_type{});
        }
        if (k0 + LB < n_keys) commit(next, k0 + LB, buf ^ 1, k0 + 2 * LB < n_keys);
        __syncthreads();
        buf ^= 1;
    };
    for (int k0 = 0; k0 < n_keys;) {
        round(k0, st0, st1);
        k0 += LB;
        if (k0 >= n_keys) break;
        round(k0, st1, st0);
        k0 += LB;
    }

    l_run = key_groups_reduce<false>(l_run);
    if (t0 + qi < T) {
        const float inv = 1.0f / l_run;
        uint16_t* orow = out + (static_cast<size_t>(b) * T + t) * (static_cast<size_t>(H) * D) + static_cast<size_t>(h) * D;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            const u32x2 pk = {pack_bf16x2(o[dt][0] * inv, o[dt][1] * inv), pack_bf16x2(o[dt][2] * inv, o[dt][3] * inv)};
            *reinterpret_cast<u32x2*>(orow + 16 * dt + 4 * g) = pk;
        }
    }
}

}  // namespace terna
