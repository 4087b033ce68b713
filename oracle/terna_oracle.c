/*
 * CPU oracle for the TernaSpMM path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the algorithms of the reference for the
 * ternary weight format and for the two linear-layer epilogues.  It is the
 * checker used by tests/, by __graft_entry__.smoke() and by bench.py's
 * cpu_baseline leg.  Nothing in the shipped library links, loads or calls it.
 *
 * Every function names the reference file:line it follows.  Parity status:
 *   oracle_reorder        pinned  (bijection + closed form + consumer simulation)
 *   oracle_compress       pinned  (closed-form tiles, invariants, consumer simulation)
 *   oracle_decode         pinned  (round trip, brute force)
 *   oracle_consumer_sim   pinned  (it IS the independent pin: it replays the reference
 *                                  kernel's lane-level fragment build and the published
 *                                  mma.m16n8k16 A-fragment layout)
 *   oracle_spmm_i8_*      pinned  (integer matmul is exact; x==1 gives row sums, the
 *                                  construction of the reference's tests/test_kernel.cu:81)
 *   oracle_spmm_bf16      pinned  (plain fp64 matmul)
 *   oracle_quant_input    pinned  (answers worked by hand: ties to even, scales that are exact,
 *   oracle_quant_input_mode        round down and round up in bf16, the all-zero row; one row on which the three
 *                                  modes give three different integers)
 *
 * Build: make -C oracle   (gcc -O2 -shared -fPIC)
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>

/* ---------------------------------------------------------------- bf16 helpers */

static float bf16_to_f32(uint16_t h)
{
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* round-to-nearest-even, the rounding of __float2bfloat16_rn
 * (used at Reduction_Kernel.cuh:60). */
static uint16_t f32_to_bf16_rn(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u)          /* NaN stays NaN */
        return (uint16_t)((u >> 16) | 0x0040u);
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}

uint16_t oracle_f32_to_bf16(float f) { return f32_to_bf16_rn(f); }
float    oracle_bf16_to_f32(uint16_t h) { return bf16_to_f32(h); }

/* ---------------------------------------------------------------- reorder
 * Follows kernels/TernaSpMM.cu:241-280 (reorder_WT_h) which is the same map as
 * convert/convert_utils.py:9-49 (reorder_weight).  Kept in the reference's
 * branch form on purpose: the numpy oracle holds the closed form, and a test
 * checks that both agree on all 256 positions of a 16x16 block. */
void oracle_reorder(const int8_t* w, int8_t* out, int N, int K)
{
    for (int rb = 0; rb < N; rb += 16)
        for (int kb = 0; kb < K; kb += 16)
            for (int i = 0; i < 16; ++i)
                for (int k = 0; k < 16; ++k) {
                    int di = i, dk;
                    if (i < 8) {                   /* upper half rows: TernaSpMM.cu:245-260 */
                        dk = (k + 1) / 2;
                        if (k & 2) { di += 8; dk -= 1; }
                    } else {                       /* lower half rows: TernaSpMM.cu:262-277 */
                        dk = (k + 1) / 2 + 8;
                        if ((k & 2) == 0) di -= 8; else dk -= 1;
                    }
                    out[(size_t)(rb + di) * K + kb + dk] = w[(size_t)(rb + i) * K + kb + k];
                }
}

/* ---------------------------------------------------------------- compress
 * Follows kernels/TernaSpMM.cu:282-439 (convert_reorderd) == convert/convert_utils.py:52-228
 * (compress_weight) with the fixed tile sizes the call sites pass
 * (tests/test_kernel.cu:255: 64,16,8,64,64,8).
 *
 * Input is the ALREADY REORDERED matrix.  Outputs are caller-allocated:
 *   bitmap      [N*K/64]            uint64
 *   tile_off    [N*K/4096 + 1]      int32   (sign-bit offsets, padded to 32 per tile)
 *   median_off  [3*N*K/4096]        uint16
 *   sign_words  [N*K/32] worst case uint32
 * Returns the number of sign words written (total padded count / 32), or -1. */
long oracle_compress(const int8_t* a, int N, int K,
                     uint64_t* bitmap, int32_t* tile_off, uint16_t* median_off,
                     uint32_t* sign_words)
{
    if (N % 64 || K % 64) return -1;
    long count = 0;                     /* running sign-bit count incl. padding  */
    long bm_i = 0, med_i = 0, tile_i = 0;
    tile_off[0] = 0;
    for (int tm = 0; tm < N / 64; ++tm)
        for (int tk = 0; tk < K / 64; ++tk) {
            long in_tile = 0;           /* unpadded count inside this 64x64 tile */
            for (int band = 0; band < 4; ++band) {              /* 16-row median tiles  */
                for (int kg = 0; kg < 8; kg += 2)                /* pairs of 8-col tiles */
                    for (int j = 0; j < 2; ++j)                  /* column-major 2x2:    */
                        for (int i = 0; i < 2; ++i) {            /* TernaSpMM.cu:351-354 */
                            int r0 = tm * 64 + band * 16 + i * 8;
                            int c0 = tk * 64 + (kg + j) * 8;
                            uint64_t bits = 0;
                            for (int r = 0; r < 8; ++r)
                                for (int c = 0; c < 8; ++c) {
                                    int8_t v = a[(size_t)(r0 + r) * K + c0 + c];
                                    if (v != 0) {
                                        bits |= 1ull << (r * 8 + c);          /* :372 */
                                        long pos = count + in_tile;
                                        if ((pos & 31) == 0) sign_words[pos >> 5] = 0;
                                        if (v < 0) sign_words[pos >> 5] |= 1u << (pos & 31); /* :412 */
                                        ++in_tile;
                                    }
                                }
                            bitmap[bm_i++] = bits;
                        }
                if (band < 3) median_off[med_i++] = (uint16_t)in_tile;        /* :390-394 */
            }
            long end = count + in_tile;
            while (end % 32) ++end;                              /* pad: :399-404 */
            /* a tile with zero nonzeros writes no word; a partially filled last
             * word was zero-initialised when its first bit was written, so the
             * padding bits read as 0 like the reference's pushed zeros */
            count = end;
            tile_off[++tile_i] = (int32_t)count;
        }
    return count / 32;
}

/* ---------------------------------------------------------------- decode
 * The reference has no host decoder; the meaning of the stream is fixed by its
 * consumer (kernels/src/SpMM/MatMulUtilities.cuh:79-114, 227-259 and
 * SpMM_Kernel.cuh:30-79, 263-269).  This walks the stream in encoder order and
 * undoes the reorder, giving the ORIGINAL (not reordered) ternary matrix.
 * Returns 0, or a negative code when a median offset disagrees with the
 * running count (-2) or a tile's padded length is inconsistent (-3). */
int oracle_decode(const uint64_t* bitmap, const int32_t* tile_off, const uint16_t* median_off,
                  const uint32_t* sign_words, int N, int K, int8_t* w)
{
    if (N % 64 || K % 64) return -1;
    memset(w, 0, (size_t)N * K);
    long tile = 0;
    for (int tm = 0; tm < N / 64; ++tm)
        for (int tk = 0; tk < K / 64; ++tk, ++tile) {
            long pos = tile_off[tile];
            for (int band = 0; band < 4; ++band) {
                if (band > 0 && pos - tile_off[tile] != median_off[3 * tile + band - 1]) return -2;
                for (int g = 0; g < 4; ++g)
                    for (int q = 0; q < 4; ++q) {
                        int sm = q & 1, sk = q >> 1;
                        uint64_t bits = bitmap[tile * 64 + band * 16 + g * 4 + q];
                        for (int b = 0; b < 64; ++b) {
                            if (!((bits >> b) & 1)) continue;
                            int neg = (sign_words[pos >> 5] >> (pos & 31)) & 1;
                            ++pos;
                            /* position in the reordered matrix */
                            int ri = sm * 8 + (b >> 3);         /* row inside 16x16 block */
                            int rk = sk * 8 + (b & 7);          /* col inside 16x16 block */
                            /* inverse of oracle_reorder */
                            int oi = (ri & 7) + 8 * (rk >> 3);
                            int ok = 4 * ((rk & 7) >> 1) + 2 * (ri >> 3) + (rk & 1);
                            int row = tm * 64 + band * 16 + oi;
                            int col = tk * 64 + g * 16 + ok;
                            w[(size_t)row * K + col] = neg ? -1 : 1;
                        }
                    }
            }
            long padded = tile_off[tile + 1] - tile_off[tile];
            long used = pos - tile_off[tile];
            if (padded < used || padded - used >= 32 || (padded & 31)) return -3;
        }
    return 0;
}

/* ---------------------------------------------------------------- consumer simulation
 * Replays what one 32-lane warp of the reference decode kernel does for one
 * 16-row band of one 64x64 tile (kernels/src/SpMM/MatMulUtilities.cuh:79-114):
 * lane L reads bits 2L and 2L+1 of four consecutive bitmaps per k16 step and
 * gathers expanded sign bytes (+1 / -1, MatMulUtilities.cuh:243-255) by popcount prefix.
 * The four bytes are a[i][j] of mma.sync.m16n8k16.s8 (MatMulUtilities.cuh:183), whose
 * published A-fragment layout for 8-bit types is:
 *     a[.][0] byte t -> A[row = L/4    ][k = 4*(L%4) + t]
 *     a[.][1] byte t -> A[row = L/4 + 8][k = 4*(L%4) + t]
 * The band start inside the tile is 0 for band 0, else median_off[3*tile+band-1]
 * (SpMM_Kernel.cuh:67-68, 94).  Output: the 16 x 64 block of W this band encodes,
 * in ORIGINAL coordinates, written to w16x64 (row-major, 64 columns). */
void oracle_consumer_sim(const uint64_t* bitmap, const int32_t* tile_off, const uint16_t* median_off,
                         const uint32_t* sign_words, long tile, int band, int8_t* w16x64)
{
    long tile_start = tile_off[tile];
    long nnz_pad = tile_off[tile + 1] - tile_start;
    /* expanded sign bytes of the whole tile: "smem_nnzs" */
    int8_t* vals = (int8_t*)malloc((size_t)(nnz_pad > 0 ? nnz_pad : 1));
    for (long t = 0; t < nnz_pad; ++t) {
        long p = tile_start + t;
        vals[t] = ((sign_words[p >> 5] >> (p & 31)) & 1) ? -1 : 1;
    }
    long band_start = band ? median_off[3 * tile + band - 1] : 0;
    const uint64_t* bm = bitmap + tile * 64 + band * 16;      /* smem_BitmapWarp */
    memset(w16x64, 0, 16 * 64);
    for (int lane = 0; lane < 32; ++lane) {
        long start = band_start;
        for (int i = 0; i < 4; ++i)                 /* k16 step                   */
            for (int j = 0; j < 2; ++j) {           /* register index a[i][j]     */
                int8_t byte[4] = {0, 0, 0, 0};
                for (int h = 0; h < 2; ++h) {       /* two bitmaps per register   */
                    uint64_t b = bm[i * 4 + j * 2 + h];
                    int sh = lane * 2;
                    int before = __builtin_popcountll(b & ((1ull << sh) - 1));
                    if ((b >> sh) & 1)       byte[2 * h]     = vals[start + before++];
                    if ((b >> (sh + 1)) & 1) byte[2 * h + 1] = vals[start + before];
                    start += __builtin_popcountll(b);
                }
                int row = lane / 4 + 8 * j;
                for (int t = 0; t < 4; ++t)
                    w16x64[row * 64 + i * 16 + 4 * (lane % 4) + t] = byte[t];
            }
    }
    free(vals);
}

/* ---------------------------------------------------------------- weight-scale group
 * Decode path: kernels/src/SpMM/Reduction_Kernel.cuh:46-54. */
int oracle_ws_group_decode(int col, int N, int ws_num)
{
    if (ws_num == 3 && N == 3840) {
        if (col < 2560) return 0;
        if (col < 2560 + 640) return 1;
        return 2;
    }
    return col / (N / ws_num);
}

/* Prefill path: kernels/src/GEMM/epilogue_visitor_scale_ws.h:135-148.  The group is
 * taken once per 128-column threadblock tile (gemm_scale_ws.h: ThreadblockShape
 * 128x128x64) from the tile's first column, and clamped to ws_num-1. */
int oracle_ws_group_prefill(int col, int N, int ws_num)
{
    int c0 = (col / 128) * 128;
    int k;
    if (N == 3840) {
        if (c0 < 2560) k = 0;
        else if (c0 < 2560 + 640) k = 1;
        else k = 2;
    } else {
        k = c0 / (N / ws_num);
    }
    return k < ws_num ? k : ws_num - 1;
}

/* ---------------------------------------------------------------- int8 linear
 * acc[m][n] = sum_k x[m][k] * w[n][k] in exact integers, then
 *   mode 0 (decode, M<=64 at TernaSpMM.cu:34): bf16_rn( (float(acc) / s[m]) * ws[g] )
 *          -- Reduction_Kernel.cuh:60
 *   mode 1 (prefill):  coeff = s[m]!=0 ? ws[g]/s[m] : 0;  bf16_rn( float(acc) * coeff )
 *          -- epilogue_visitor_scale_ws.h:188-205
 * s and ws are bf16 storage.  w is the decoded ternary matrix [N][K]. */
void oracle_spmm_i8(const int8_t* x, const int8_t* w, const uint16_t* s, const uint16_t* ws,
                    int ws_num, int M, int N, int K, int mode, uint16_t* out)
{
    for (int m = 0; m < M; ++m) {
        volatile float sm = bf16_to_f32(s[m]);
        for (int n = 0; n < N; ++n) {
            int32_t acc = 0;
            const int8_t* xr = x + (size_t)m * K;
            const int8_t* wr = w + (size_t)n * K;
            for (int k = 0; k < K; ++k) acc += (int32_t)xr[k] * wr[k];
            volatile float r;
            if (mode == 0) {
                volatile float wsv = bf16_to_f32(ws[oracle_ws_group_decode(n, N, ws_num)]);
                volatile float q = (float)acc / sm;
                r = q * wsv;
            } else {
                volatile float wsv = bf16_to_f32(ws[oracle_ws_group_prefill(n, N, ws_num)]);
                volatile float coeff = (sm != 0.0f) ? (wsv / sm) : 0.0f;
                r = (float)acc * coeff;
            }
            out[(size_t)m * N + n] = f32_to_bf16_rn(r);
        }
    }
}

/* ---------------------------------------------------------------- bf16 linear (fp64 golden)
 * ref[m][n] = scale[g(n)] * sum_k x[m][k] * w[n][k], all in double.
 * Group rule as on the decode path.  x is bf16 storage, scale is fp32. */
void oracle_spmm_bf16(const uint16_t* x, const int8_t* w, const float* scale, int ws_num,
                      int M, int N, int K, double* out)
{
    double* xd = (double*)malloc(sizeof(double) * (size_t)K);
    for (int m = 0; m < M; ++m) {
        for (int k = 0; k < K; ++k) xd[k] = (double)bf16_to_f32(x[(size_t)m * K + k]);
        for (int n = 0; n < N; ++n) {
            const int8_t* wr = w + (size_t)n * K;
            double pos = 0.0, neg = 0.0;
            for (int k = 0; k < K; ++k) {
                if (wr[k] > 0) pos += xd[k];
                else if (wr[k] < 0) neg += xd[k];
            }
            out[(size_t)m * N + n] =
                (pos - neg) * (double)scale[oracle_ws_group_decode(n, N, ws_num)];
        }
    }
}

/* ---------------------------------------------------------------- activation quantisation
 * model.py:120-123 (SpBitLinear.quant_input), with the one definition this build
 * fixes for the precision the reference leaves open: compute in fp32,
 * s = bf16_rn(127 / max(|x|, 1e-5)), and that rounded s is used both to quantise
 * and in the epilogue.  x is bf16 storage.  (The reference's eager mode multiplies
 * in the tensor's dtype and its compiled graph in fp32 with the unrounded quotient;
 * the known answers in tests/test_oracle_linear.py include a row on which the
 * three differ.) */
/* mode 0: the definition above.
 * `127 / tensor` in the reference's line is Tensor.__rtruediv__, which PyTorch evaluates as tensor.reciprocal() * 127:
 * mode 1: the method as the reference ships it, under @torch.compile -- one fused fp32 kernel with no intermediate
 *   rounding to bf16: the multiplier is t = fl32(fl32(1 / max(|x|, 1e-5)) * 127), UNROUNDED (product rounded to
 *   fp32, then to the nearest integer, ties to even); the returned s is bf16_rn(t).
 * mode 2: the same two lines in eager mode on a bf16 tensor -- every op rounds its result to bf16: the clamp floor
 *   is bf16_rn(1e-5), s = bf16_rn(bf16_rn(1 / max) * 127), the product x * s is rounded to bf16 before round(). */
void oracle_quant_input_mode(const uint16_t* x, int M, int K, int mode, int8_t* xq, uint16_t* s)
{
    const float floor_v = mode == 2 ? bf16_to_f32(f32_to_bf16_rn(1e-5f)) : 1e-5f;
    for (int m = 0; m < M; ++m) {
        float amax = 0.0f;
        for (int k = 0; k < K; ++k) {
            float v = fabsf(bf16_to_f32(x[(size_t)m * K + k]));
            if (v > amax) amax = v;
        }
        if (amax < floor_v) amax = floor_v;
        volatile float t;                                          /* volatile: rounded to fp32, no wider intermediate */
        if (mode == 0) {
            t = 127.0f / amax;
        } else {
            volatile float r = 1.0f / amax;
            if (mode == 2) r = bf16_to_f32(f32_to_bf16_rn(r));
            t = r * 127.0f;
        }
        uint16_t sb = f32_to_bf16_rn(t);
        float mul = mode == 1 ? t : bf16_to_f32(sb);
        s[m] = sb;
        for (int k = 0; k < K; ++k) {
            volatile float p = bf16_to_f32(x[(size_t)m * K + k]) * mul;
            float pr = p;
            if (mode == 2) pr = bf16_to_f32(f32_to_bf16_rn(pr));
            float q = nearbyintf(pr);
            if (q > 127.0f) q = 127.0f;
            if (q < -128.0f) q = -128.0f;
            xq[(size_t)m * K + k] = (int8_t)q;
        }
    }
}

void oracle_quant_input(const uint16_t* x, int M, int K, int8_t* xq, uint16_t* s)
{
    oracle_quant_input_mode(x, M, K, 0, xq, s);
}
