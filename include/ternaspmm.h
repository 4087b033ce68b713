/*
 * libternaspmm.so -- C ABI of the TernaSpMM path, MI355X (gfx950) build.
 *
 * The first eight symbols are the ones the reference library exports and that its
 * callers bind (model.py:21,76-89 through ctypes; tests/test_kernel.cu:51-76).  Names,
 * argument order and argument meaning are unchanged; "bf16" is 16-bit bfloat storage and
 * the stream argument is a hipStream_t (PyTorch-ROCm's stream.cuda_stream).  The symbols
 * after them are additions of this build and have no counterpart in the reference.
 *
 * Conventions shared by every compute entry point:
 *   - all pointers are device memory owned by the caller; `out` [M][N] row-major bf16 is
 *     fully overwritten.  Nothing is allocated, freed or synchronised on the call path -- with ONE exception, which
 *     is on by default: the repack cache behind the entry points that take the reference format (the section
 *     "Repack cache" below).  The first call that sees a weight allocates N*K/4 + 256 bytes of device memory
 *     (hipMalloc), runs two small launches and waits for the stream twice (hipStreamSynchronize); when the cache's
 *     byte limit is reached or a stale copy is dropped, a call may also hipFree (which waits for the device).  Later
 *     calls on that weight, every call during stream capture, and every call with TERNASPMM_REPACK_CACHE=0 in the
 *     environment (or after ternaspmm_repack_cache_enable(0)) only enqueue, as the reference does;
 *   - W is [N][K] ternary in the compressed format (bitmap / TileOffsets_global /
 *     TileOffsets_median / sign words), N % 64 == 0 and K % 64 == 0;
 *   - alignment: `out` at least 8 bytes (the kernels store four bf16 at a time); x, the scales and the format's
 *     arrays as their element types require.  16-byte aligned x and out (any torch / hipMalloc allocation) select
 *     the faster variants of the large-M kernels -- activations loaded straight into LDS, results stored as whole
 *     rows -- other pointers take slower variants (same bits for the int8 family, same tolerance for bf16);
 *   - calls only enqueue work on `stream` and are safe under stream capture;
 *   - on a HIP runtime error the library prints the error and exits the process, as the
 *     reference does (kernels/TernaSpMM.cu:15-22).
 */
#ifndef TERNASPMM_H
#define TERNASPMM_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef uint16_t terna_bf16;   /* bfloat16 storage                                   */
typedef void*    terna_stream; /* hipStream_t                                        */

/* ---- reference symbols ------------------------------------------------------------- */

/* kernels/TernaSpMM.cu:15 -- print and exit(1) if the runtime holds a pending error. */
void checkLastCudaError(int line);

/* kernels/TernaSpMM.cu:25 -- out = bf16( (x_q . W^T) scaled ), int8 activations.
 *   x       int8  [M][K] row-major (quantised activations)
 *   s       bf16  [M]    per-row activation scale (x_q = round(x*s))
 *   ws      bf16  [>=ws_num] weight-group scales, ws_num (1 .. 4) groups along N
 *   M <= 64 : epilogue bf16((acc / s[m]) * ws[g])        (Reduction_Kernel.cuh:60)
 *   M  > 64 : epilogue bf16(acc * (ws[g] / s[m])), 0 if s[m]==0, g per 128-column tile
 *                                                        (epilogue_visitor_scale_ws.h:135-205)
 *   `workspace` / SPLIT_K: the library writes at most what the reference itself writes there, so a buffer sized for
 *   the reference is large enough (model.py:34-42, tests/test_kernel.cu:331):
 *     - a call the reference serves by its decode path (M <= 64 here, any M on _decode):
 *       4 * M * N * SPLIT_K bytes, the reference's int32 partial planes (TernaSpMM_API.cuh:66-136);
 *     - a call it serves by its prefill path (M > 64 here, any M on _prefill): N * K bytes, the reference's dense
 *       int8 copy of the matrix (SpMM_Kernel.cuh:263-269, TernaSpMM_API.cuh:279-282).
 *   What for: split-K partial sums of the MFMA-tiled kernel (at most SPLIT_K planes of 4 * M * N bytes on the
 *   decode path) and, without a cached copy of the weight, a per-call transcode of the weights into its first
 *   N*K/4 bytes.  It is used only when it is non-NULL and 16-byte aligned; pass NULL to keep it untouched (the
 *   kernels then do without).  Small calls (the usual decode shapes) never touch it.  Nothing has to be preserved
 *   in it between calls; calls that share it must not overlap. */
void bitlinear_TernaSpMM(int8_t* x, uint64_t* bitmap, int* tile_offsets_global,
                         uint16_t* tile_offsets_median, uint32_t* sign_words,
                         terna_bf16* out, terna_bf16* s, terna_bf16* ws, int ws_num,
                         int M, int N, int K, int SPLIT_K, int32_t* workspace, terna_stream stream);

/* kernels/TernaSpMM.cu:79 -- as above, always the decode epilogue. */
void bitlinear_TernaSpMM_decode(int8_t* x, uint64_t* bitmap, int* tile_offsets_global,
                                uint16_t* tile_offsets_median, uint32_t* sign_words,
                                terna_bf16* out, terna_bf16* s, terna_bf16* ws, int ws_num,
                                int M, int N, int K, int SPLIT_K, int32_t* workspace, terna_stream stream);

/* kernels/TernaSpMM.cu:110 -- as above, always the prefill epilogue. */
void bitlinear_TernaSpMM_prefill(int8_t* x, uint64_t* bitmap, int* tile_offsets_global,
                                 uint16_t* tile_offsets_median, uint32_t* sign_words,
                                 terna_bf16* out, terna_bf16* s, terna_bf16* ws, int ws_num,
                                 int M, int N, int K, int SPLIT_K, int32_t* workspace, terna_stream stream);

/* kernels/TernaSpMM.cu:141 -- mode 0/1/2 = auto/prefill/decode; warm-up, event-timed loop,
 * prints "Shape(M=, N=, K=): %.2f us (avg over %d iters, warmup=%d)".  Synchronises. */
void bitlinear_TernaSpMM_benchmark(int mode, int warmup_iters, int bench_iters,
                                   int8_t* x, uint64_t* bitmap, int* tile_offsets_global,
                                   uint16_t* tile_offsets_median, uint32_t* sign_words,
                                   terna_bf16* out, terna_bf16* s, terna_bf16* ws, int ws_num,
                                   int M, int N, int K, int SPLIT_K, int32_t* workspace, terna_stream stream);

/* kernels/TernaSpMM.cu:241 -- host only: 16x16 block permutation of a bf16 [N][K] matrix. */
void reorder_WT_h(terna_bf16* W, terna_bf16* W_reordered, int N, int K);

/* kernels/TernaSpMM.cu:282 -- host only: encode an already reordered bf16 [N][K] matrix.
 * The tile-size arguments must be 64,16,8,64,64,8 (the only values the reference passes,
 * tests/test_kernel.cu:255); anything else returns -1.  Returns the number of 64x64 tiles.
 * *bitmap is pinned host memory (free with hipHostFree); the other three are malloc'd
 * (free with free()).  max_nnz_count is the reference's `int&`. */
int convert_reorderd(terna_bf16* A_h, int N, int K, int tile_N, int warp_subtile_N, int subtile_N,
                     int tile_K, int warp_subtile_K, int subtile_K,
                     uint64_t** bitmap, int** tile_offsets_global, uint16_t** tile_offsets_median,
                     uint32_t** sign_words, int* max_nnz_count);

/* kernels/TernaSpMM.cu:454 -- enqueue a kernel that spins for about `us` microseconds. */
void gpu_sleep(double us, terna_stream stream);

/* ---- additions of this build (no counterpart in the reference) ---------------------- */

/* bf16-activation family: out = bf16( (x . W^T) * scale[g(n)] ), fp32 accumulate.
 *   x bf16 [M][K], any M >= 1 (no padding rows needed); scale fp32 [ws_num];
 *   group rule of the decode path (Reduction_Kernel.cuh:46-54).
 * The plain symbol picks a kernel by M; _decode / _prefill force the small-M dot-product
 * kernel or the MFMA-tiled kernel.  workspace may be NULL; if given (16-byte aligned) it is used under the same
 * rule and within the same sizes as bitlinear_TernaSpMM's: 4 * M * N * SPLIT_K bytes for M <= 64 (and on _decode),
 * N * K bytes for M > 64 (and on _prefill) -- split-K partial sums, and the per-call transcode of a weight the cache
 * holds no copy of. */
void bitlinear_TernaSpMM_bf16(const terna_bf16* x, const uint64_t* bitmap, const int* tile_offsets_global,
                              const uint16_t* tile_offsets_median, const uint32_t* sign_words,
                              terna_bf16* out, const float* scale, int ws_num,
                              int M, int N, int K, int SPLIT_K, void* workspace, terna_stream stream);
void bitlinear_TernaSpMM_bf16_decode(const terna_bf16* x, const uint64_t* bitmap, const int* tile_offsets_global,
                                     const uint16_t* tile_offsets_median, const uint32_t* sign_words,
                                     terna_bf16* out, const float* scale, int ws_num,
                                     int M, int N, int K, int SPLIT_K, void* workspace, terna_stream stream);
void bitlinear_TernaSpMM_bf16_prefill(const terna_bf16* x, const uint64_t* bitmap, const int* tile_offsets_global,
                                      const uint16_t* tile_offsets_median, const uint32_t* sign_words,
                                      terna_bf16* out, const float* scale, int ws_num,
                                      int M, int N, int K, int SPLIT_K, void* workspace, terna_stream stream);

/* Host only: sizes of the four format arrays for an [N][K] matrix.  sign_words_capacity is
 * the worst case (all weights nonzero).  Returns 0, or -1 if N or K is not a multiple of 64. */
int ternaspmm_encode_sizes(int N, int K, int64_t* bitmap_len, int64_t* tile_offsets_global_len,
                           int64_t* tile_offsets_median_len, int64_t* sign_words_capacity);

/* Host only: reorder + encode an ORIGINAL (not reordered) ternary int8 [N][K] matrix into
 * caller-provided arrays of the sizes above.  Returns the number of sign words written
 * (= tile_offsets_global[last] / 32), or -1 on a bad shape or a value outside {-1,0,1}.
 * Output is bit-identical to reorder_weight + compress_weight (convert/convert_utils.py:9-228). */
int64_t ternaspmm_encode_i8(const int8_t* W, int N, int K, uint64_t* bitmap, int* tile_offsets_global,
                            uint16_t* tile_offsets_median, uint32_t* sign_words);

/* Device: expand the compressed format to a dense row-major bf16 [N][K] matrix of
 * {-1, 0, +1} on `stream` (load-time inspection and round-trip checks). */
void ternaspmm_decompress_bf16(const uint64_t* bitmap, const int* tile_offsets_global,
                               const uint16_t* tile_offsets_median, const uint32_t* sign_words,
                               terna_bf16* W_dense, int N, int K, terna_stream stream);

/* ---- load-time repack ("P2" layout, 2 bits per weight, N*K/4 bytes) ----------------------------
 * The reference format stays the on-disk and interchange format.  P2 is a device-side layout
 * this library can derive from it, bit-exactly, once at load time; its kernels need no offset
 * arrays and no sign-stream arithmetic.  Callers that keep to the reference entry points never
 * see it, except through the repack cache (below) and in that a large-M call on a weight without a cached copy
 * transcodes into `workspace` when one is given: N*K/4 bytes there, within the N*K bytes the reference's call site
 * guarantees (model.py:34-42). */

/* Bytes of a P2 buffer for an [N][K] matrix, or -1 if N or K is not a multiple of 64. */
int64_t ternaspmm_packed_bytes(int N, int K);

/* Device: reference format -> P2 into `packed` (16-byte aligned, ternaspmm_packed_bytes(N,K) bytes). */
void ternaspmm_repack(const uint64_t* bitmap, const int* tile_offsets_global, const uint16_t* tile_offsets_median,
                      const uint32_t* sign_words, void* packed, int N, int K, terna_stream stream);

/* bf16-activation linear on a P2 buffer.  route: 0 = the library picks the kernel (by measurement: the small-M kernel up
 * to 32 rows for matrices of more than 512 bands, up to 64 - 256 rows otherwise, depending on K, the activation type
 * and whether scratch memory for split-K is at hand), 1 = MFMA-tiled kernel, 2 = small-M kernel. */
void bitlinear_TernaSpMM_bf16_packed(const terna_bf16* x, const void* packed, terna_bf16* out, const float* scale,
                                     int ws_num, int M, int N, int K, int route, terna_stream stream);

/* int8-activation linear on a P2 buffer; arguments as bitlinear_TernaSpMM.  route: 0 = the reference's
 * rule (decode epilogue for M <= 64, prefill epilogue above), 1 = prefill epilogue, 2 = decode epilogue.  Which kernel
 * computes the sums is the library's choice (as above) and does not change the result: integer sums are exact. */
void bitlinear_TernaSpMM_packed(const int8_t* x, const void* packed, terna_bf16* out, const terna_bf16* s,
                                const terna_bf16* ws, int ws_num, int M, int N, int K, int route, terna_stream stream);

/* The two entry points above with scratch memory the library may use (may be NULL / 0: then they are the calls
 * above): `workspace` (16-byte aligned, workspace_bytes long) receives split-K partial sums when a large-M call has
 * few output tiles for the chip -- 4 * M * N bytes per split, up to 8 splits; the call then enqueues two launches
 * (partial products, then the sum in split order + epilogue; int8 results stay bit-exact).  Nothing has to be
 * preserved or initialised in it between calls; calls that share it must not overlap.
 * Kernel override for measurements: bitlinear_TernaSpMM_packed(_ws) also accepts route + 4 (small-M kernel at any M)
 * and route + 8 (MFMA-tiled kernel at any M); the low two bits keep selecting the epilogue rule. */
void bitlinear_TernaSpMM_bf16_packed_ws(const terna_bf16* x, const void* packed, terna_bf16* out, const float* scale,
                                        int ws_num, int M, int N, int K, int route, void* workspace,
                                        long long workspace_bytes, terna_stream stream);
void bitlinear_TernaSpMM_packed_ws(const int8_t* x, const void* packed, terna_bf16* out, const terna_bf16* s,
                                   const terna_bf16* ws, int ws_num, int M, int N, int K, int route, void* workspace,
                                   long long workspace_bytes, terna_stream stream);

/* ---- Fused prologue of a ternary linear (no counterpart in the reference's library) -----------------
 * One launch replaces the PyTorch / xformers / Inductor kernels the reference runs between two bitlinear
 * calls: the residual add and block norm (model.py:330, :334), the sub-norms (model.py:236, :280), the
 * gate squared_relu(x1) * x3 (model.py:279-280) and SpBitLinear.quant_input (model.py:120-123).  Per row:
 *   h = x, or bf16(x + residual) when residual != NULL (written to sum_out when that is non-NULL)
 *   y = bf16(h * rsqrt(mean(h^2) + eps) * weight)                       fp32 inside
 *   s = bf16(127 / max(max|y|, 1e-5)),  xq = clamp(rint(y * s), -128, 127)
 * y_out (bf16 [M][K]) and the pair xq_out (int8 [M][K]) / s_out (bf16 [M]) are each optional (NULL = not
 * written); xq_out / s_out feed bitlinear_TernaSpMM* directly.  K % 8 == 0, K <= 8192.  Only enqueues. */
void ternaspmm_rmsnorm_quant(const terna_bf16* x, const terna_bf16* residual, terna_bf16* sum_out,
                             const terna_bf16* weight, float eps, terna_bf16* y_out, int8_t* xq_out,
                             terna_bf16* s_out, int M, int K, terna_stream stream);

/* Which of the reference's evaluations of SpBitLinear.quant_input (model.py:120-123) the prologue kernels above and
 * below reproduce -- its two lines leave the intermediate precision to PyTorch, and the ways of running them differ on a
 * few percent of the int8 activations (by one step):
 *   0  s = bf16(127 / max(max|y|, 1e-5)) and q = rint(fp32(y * s)) with that ROUNDED s: quantiser and epilogue use one
 *      number (default);
 *   1  the method as shipped, under @torch.compile (one fused fp32 kernel, no intermediate rounding to bf16; `127 / t`
 *      on a tensor is t.reciprocal() * 127): q = rint(fp32(y * t)) with the UNROUNDED
 *      t = fp32(fp32(1 / max(max|y|, 1e-5)) * 127), s = bf16(t);
 *   2  the same lines in eager mode on bf16 tensors, every op rounded to bf16:
 *      s = bf16(bf16(1 / max(max|y|, bf16(1e-5))) * 127), q = rint(bf16(y * s)).
 * ternaspmm_quant_mode(mode) selects one for every later call of the process (a launch recorded in a graph keeps the
 * mode it was captured with) and returns the previous mode; any other value only queries.  Initial value:
 * TERNASPMM_QUANT_MODE in the environment, else 0.  The epilogue always divides by the published bf16 s. */
int ternaspmm_quant_mode(int mode);

/* Same with h = bf16(bf16(relu(x1)^2) * x3), x1 = x13[m][0:F], x3 = x13[m][F:2F] (x13 is the gate/up
 * linear's output, bf16 [M][2F]); the norm and the quantisation run over F columns. */
void ternaspmm_relu2_mul_rmsnorm_quant(const terna_bf16* x13, const terna_bf16* weight, float eps, terna_bf16* y_out,
                                       int8_t* xq_out, terna_bf16* s_out, int M, int F, terna_stream stream);

/* The same prologue inside the small-M linear: [residual add] -> RMSNorm -> quant_input -> ternary matmul ->
 * decode epilogue in ONE launch (x, residual, sum_out, norm_weight, eps as ternaspmm_rmsnorm_quant; packed, out,
 * ws, ws_num as bitlinear_TernaSpMM_packed).  xq_out / s_out are optional copies of the quantised activations
 * (NULL = not written).  sum_out must not alias x or residual (every workgroup reads both).  Supported: M <= 16
 * and K <= 3072 (K <= 2560 when N > 4096); without a residual, M <= 8 and N <= 4096 also K <= 8192 (the kernel of
 * ternaspmm_fused_linear's NORM prologue serves those).  Returns 1 when the launch was enqueued, 0 when the shape is
 * outside that range and nothing was done (no argument is read) -- the caller then runs ternaspmm_rmsnorm_quant +
 * bitlinear_TernaSpMM_packed.
 * Every workgroup repeats the prologue arithmetic (variants for 1, 2, 4, 8 and 16 rows: the lanes of a wave are spread
 * over the rows that exist), so the single launch pays for M = 1 (measured on MI355X: 5.2-5.6 us against 7.2-7.5 us
 * for the pair), still pays for M <= 4 and is no faster than the pair from M = 8 on. */
int bitlinear_TernaSpMM_packed_fused(const terna_bf16* x, const terna_bf16* residual, terna_bf16* sum_out,
                                     const terna_bf16* norm_weight, float eps, const void* packed, terna_bf16* out,
                                     const terna_bf16* ws, int ws_num, int8_t* xq_out, terna_bf16* s_out, int M,
                                     int N, int K, terna_stream stream);

/* Gated-FFN variant: h = bf16(bf16(relu(x1)^2) * x3) from x13 (bf16 [M][2F], as ternaspmm_relu2_mul_rmsnorm_quant),
 * norm and quantisation over F columns, then the [N][F] ternary linear.  Supported: M <= 4, N <= 4096, F <= 7168;
 * returns 0 otherwise (caller: ternaspmm_relu2_mul_rmsnorm_quant + bitlinear_TernaSpMM_packed). */
/* The O projection of a single-row decode step with the attention's deferred merge inside: as
 * bitlinear_TernaSpMM_packed_fused without a residual, but the activation row is formed from the partial results a
 * ternaspmm_rope_decode_attention_partial launch left (`partial`, `splits`; K = heads * head_dim) -- bit-identical to
 * ternaspmm_attention_merge followed by bitlinear_TernaSpMM_packed_fused.  M must be 1 (one sequence); returns 0
 * without doing anything for shapes outside what it supports (the caller then runs that pair). */
int bitlinear_TernaSpMM_packed_fused_attn(const float* partial, int splits, int head_dim, const terna_bf16* norm_weight, float eps,
                                          const void* packed, terna_bf16* out, const terna_bf16* ws, int ws_num,
                                          int8_t* xq_out, terna_bf16* s_out, int M, int N, int K, terna_stream stream);
int bitlinear_TernaSpMM_packed_fused_glu(const terna_bf16* x13, const terna_bf16* norm_weight, float eps,
                                         const void* packed, terna_bf16* out, const terna_bf16* ws, int ws_num,
                                         int8_t* xq_out, terna_bf16* s_out, int M, int N, int F, terna_stream stream);

/* ---- Chained small-M linears: producer-side norm statistics (no counterpart in the reference's library) ----------
 * The prologue above re-derives, in every workgroup, the two row statistics of the norm and of quant_input -- the sum
 * of h^2 and max |y| -- with two workgroup-wide reductions over K.  In a decode step the launch that PRODUCES h can
 * leave them instead: per row and per 16 (or more) columns a partial (sum of h^2, max |h * w|), w = the weights of
 * the norm that will read h (both are exact: products of two bf16 values).  The consumer adds / maximises the partials
 * of a row in a fixed order and continues element-wise:
 *     rstd = rsqrt(sum / K + eps);   y = bf16((h * w) * rstd);   max |y| = bf16(max|h * w| * rstd)   (exactly)
 * then s and xq as in ternaspmm_rmsnorm_quant (ternaspmm_quant_mode applies).  The norm output stays within one bf16
 * step of the float64 evaluation; (xq, s) can be published as before and the matmul on them is exact.
 *
 * ternaspmm_fused_linear: one launch = prologue -> ternary matmul on a P2 weight -> epilogue, M <= 8 rows.
 *   prologue  TERNASPMM_PROLOGUE_NORM       x = h bf16 [M][K]; statistics taken inside (as bitlinear_TernaSpMM_packed_fused)
 *             TERNASPMM_PROLOGUE_ATTENTION  x = the partial results of ternaspmm_rope_decode_attention_partial
 *                                           (attention_splits, head_dim; M = 1), merged inside, statistics taken inside
 *             TERNASPMM_PROLOGUE_STATS      x = h bf16 [M][K] with its partials stats_in fp32 [M][stats_count][2]
 *                                           (stats_count <= 448), as a producing epilogue or ternaspmm_row_stats left them
 *             TERNASPMM_PROLOGUE_QUANTISED  x = int8 [M][K] with its scales s_in bf16 [M] (ternaspmm_quant_from_stats,
 *                                           ternaspmm_rmsnorm_quant): no prologue; with TERNASPMM_EPILOGUE_RESIDUAL
 *                                           (M <= 16, any K the int8 kernels take) or TERNASPMM_EPILOGUE_GATE (M <= 16,
 *                                           K <= 6144).  From five rows on this pair -- the element-wise quantise launch,
 *                                           then the linear on its rows -- is the faster way to consume a producer's
 *                                           partials (measured, 2B shapes, 8 rows: 6706 against 6498 tokens/s for the
 *                                           norm kernels + plain linears, 6322 for the STATS prologue)
 *   epilogue  TERNASPMM_EPILOGUE_STORE      out bf16 [M][N] = the linear's output (decode rule, Reduction_Kernel.cuh:60)
 *             TERNASPMM_EPILOGUE_RESIDUAL   out bf16 [M][N] = bf16(residual + output): the residual stream after this
 *                                           linear (model.py:330, :334); stats_out fp32 [M][N/16][2] = its partials under
 *                                           next_norm_weight (bf16 [N]); raw_out (optional) also receives the output itself
 *             TERNASPMM_EPILOGUE_GATE       `packed` is a gate+up matrix whose bands were interleaved by
 *                                           ternaspmm_interleave_gate_up, ws = [scale of w1, scale of w3] (ws_num = 2);
 *                                           out bf16 [M][N/2] = bf16(bf16(relu(x1)^2) * x3) (model.py:279-280);
 *                                           stats_out fp32 [M][N/32][2] under next_norm_weight (bf16 [N/2], ffn_sub_norm)
 * Returns the number of partials per row written to stats_out (0 for TERNASPMM_EPILOGUE_STORE), or -1 when the
 * combination or the shape is not supported and nothing was enqueued (supported: K <= 2560 for every combination,
 * K <= 7168 for TERNASPMM_PROLOGUE_STATS with STORE / RESIDUAL, K <= 8192 for PROLOGUE_NORM, K <= 4096 for
 * PROLOGUE_ATTENTION; GATE needs PROLOGUE_STATS; PROLOGUE_NORM here only with EPILOGUE_RESIDUAL).  out must not alias x or
 * residual.  Only enqueues.  Every workgroup of a launch with a NORM / ATTENTION / STATS prologue repeats the norm +
 * quantisation of all M rows: measured on the 2B shapes that pays up to 4 rows; above, ternaspmm_quant_from_stats in front
 * of a PROLOGUE_QUANTISED launch (or of bitlinear_TernaSpMM_packed) consumes the producer's partials faster. */
enum { TERNASPMM_PROLOGUE_NORM = 0, TERNASPMM_PROLOGUE_ATTENTION = 1, TERNASPMM_PROLOGUE_STATS = 2, TERNASPMM_PROLOGUE_QUANTISED = 3 };
enum { TERNASPMM_EPILOGUE_STORE = 0, TERNASPMM_EPILOGUE_RESIDUAL = 1, TERNASPMM_EPILOGUE_GATE = 2 };
typedef struct ternaspmm_fused_linear_desc {
    int prologue, epilogue;
    int M, N, K;
    int ws_num;
    float eps;
    int stats_count;                  /* PROLOGUE_STATS */
    int attention_splits, head_dim;   /* PROLOGUE_ATTENTION */
    const void* x;
    const float* stats_in;
    const terna_bf16* norm_weight;    /* bf16 [K] */
    const void* packed;
    const terna_bf16* ws;
    terna_bf16* out;
    const terna_bf16* residual;       /* EPILOGUE_RESIDUAL: bf16 [M][N] */
    const terna_bf16* next_norm_weight;
    float* stats_out;
    terna_bf16* raw_out;              /* EPILOGUE_RESIDUAL, optional */
    int8_t* xq_out;                   /* optional pair: the quantised activations as published by the first workgroup */
    terna_bf16* s_out;
    const terna_bf16* s_in;           /* PROLOGUE_QUANTISED: bf16 [M], the scales that go with x = int8 [M][K] */
} ternaspmm_fused_linear_desc;
int ternaspmm_fused_linear(const ternaspmm_fused_linear_desc* desc, terna_stream stream);

/* Norm + quant_input of h bf16 [M][K] as a launch of its own, from partials a producer left: xq_out int8 [M][K], s_out bf16 [M]
 * -- the values the TERNASPMM_PROLOGUE_STATS prologue forms inside its launch (same order of additions), for row counts at
 * which every consuming workgroup repeating the element-wise work costs more than one more launch (measured on MI355X: the
 * down projection, K = 6912, from five rows on).  Returns 0 / -1.  Only enqueues. */
int ternaspmm_quant_from_stats(const terna_bf16* h, const float* stats, int stats_count, const terna_bf16* norm_weight, float eps,
                               int8_t* xq_out, terna_bf16* s_out, int M, int K, terna_stream stream);

/* Partials of a row block no producing epilogue wrote (the embedding rows in front of the first block): per row and per
 * 512 columns (sum of h^2, max |h * norm_weight|) -> stats_out fp32 [M][ternaspmm_row_stats_count(K)][2].  Returns that
 * count, or -1 (K not a multiple of 8).  Only enqueues. */
int ternaspmm_row_stats_count(int K);
int ternaspmm_row_stats(const terna_bf16* h, const terna_bf16* norm_weight, float* stats_out, int M, int K, terna_stream stream);

/* The inputs of a single-token step in one launch (the reference: the embedding lookup of model.py:367's tied matrix and
 * the rows of the RoPE table, two framework launches): x_out bf16 [B][K] = embedding[tokens[b]] (embedding bf16 [V][K]) with
 * its partials stats_out fp32 [B][ternaspmm_row_stats_count(K)][2] under norm_weight, exactly as ternaspmm_row_stats leaves
 * them, and rope_out fp32 [2][B][rope_half] = the cos rows, then the sin rows, of rope_table fp32 [S][2][rope_half] at
 * pos[b] (per_sequence) or pos[0] (tokens, pos: int64 in device memory; values outside their table are clamped).
 * K a multiple of 8, rope_half a multiple of 4 up to 512, 16-byte aligned tables and outputs.  Returns the partial count or
 * -1.  Only enqueues. */
int ternaspmm_step_inputs(const long long* tokens, const long long* pos, int per_sequence, const terna_bf16* embedding, int V, int K,
                          const float* rope_table, int S, int rope_half, const terna_bf16* norm_weight, terna_bf16* x_out,
                          float* stats_out, float* rope_out, int B, terna_stream stream);

/* Load time: band permutation of a P2 gate+up matrix [w1; w3] ([N][K], N = 2F) for TERNASPMM_EPILOGUE_GATE -- band 2j <-
 * rows 16j .. 16j+15 of w1, band 2j+1 <- the same rows of w3.  packed_out: N*K/4 bytes, not `packed`.  Returns 0 / -1. */
int ternaspmm_interleave_gate_up(const void* packed, void* packed_out, int N, int K, terna_stream stream);

/* ---- Attention-side kernels of a decode step (no counterpart in the reference's library) -----------
 * They stand where the reference calls xformers' rope_padded (model.py:218-229) and
 * fmha.memory_efficient_attention_forward (model.py:231-233).
 *
 * ternaspmm_rope_kv_store: rotary embedding of the q and k heads of the fused qkv linear's output
 * (bf16 [B*T][(H + 2*KV)*D], row b*T + t): pair j of a head -- dimensions (2j, 2j + 1) when `adjacent` is
 * non-zero (rope_padded's default and the order of the reference's checkpoints), (j, j + D/2) otherwise -- is
 * rotated by the angle whose cosine / sine is cos[t][j] / sin[t][j] (fp32 [T][D/2]); q goes to q_out
 * (bf16 [B][H][T][D]); k and v go into the caches (bf16 [B][KV][S][D]) at slot pos[t] (int64 [T], device memory).
 *
 * ternaspmm_decode_attention: one new token per sequence.  q bf16 [B][H][D]; head h reads kv head
 * h / (H/KV) at slots 0 .. pos[0]; out bf16 [B][H*D] = softmax(scale * q K^T) V.  D is 64 or 128,
 * S <= 8192.  Both only enqueue.
 *
 * Precondition on `pos` (device memory, which the host side of the call cannot inspect): 0 <= pos[t] < S.  A
 * position outside the cache writes no k / v row and the attention runs over the prefix clamped to [1, S]
 * slots: the result is then meaningless but every access stays inside the caller's buffers.
 *
 * `per_sequence` (every entry point of this group): 0 -- all sequences of the batch share the positions, `pos` is
 * int64 [T] and cos / sin are fp32 [T][D/2] (T = 1 for the single-token entry points); non-zero -- every sequence has
 * its own, `pos` is int64 [B][T] and cos / sin are fp32 [B][T][D/2]: sequences with different prefix lengths in one
 * batch, the kv_seqlen the reference hands to its attention bias (generate.py:253-262, 294).
 *
 * `workspace` (may be NULL): device memory of ternaspmm_attention_workspace_bytes(B, H, D) bytes, zero-filled by
 * the caller once before its first use.  With it the cache prefix of every head is split over up to 8 workgroups
 * (one CU streams a prefix at a few tens of GB/s, so few heads on the chip are bound by that); each leaves a partial
 * result in the workspace and the last to arrive merges them in a fixed order.  The kernel leaves the counters at
 * zero, so the same workspace serves every later call; calls that share one workspace must not overlap. */
long long ternaspmm_attention_workspace_bytes(int B, int H, int D);
void ternaspmm_rope_kv_store(const terna_bf16* qkv, const float* cos, const float* sin, const long long* pos,
                             int per_sequence, terna_bf16* q_out, terna_bf16* cache_k, terna_bf16* cache_v, int B, int T, int H,
                             int KV, int D, int S, int adjacent, terna_stream stream);
void ternaspmm_decode_attention(const terna_bf16* q, const terna_bf16* cache_k, const terna_bf16* cache_v,
                                const long long* pos, int per_sequence, terna_bf16* out, int B, int H, int KV, int D, int S,
                                float scale, void* workspace, terna_stream stream);
/* Several new tokens per sequence (the prompt pass): q bf16 [B][H][T][D] as ternaspmm_rope_kv_store leaves it, the
 * caches already holding the new tokens' rows; new token t sees the slots 0 .. pos[t] (int64 [T] shared by the
 * sequences, or [B][T] with `per_sequence`; clamped to the cache).  out bf16 [B*T][H*D], row b*T + t.  Stands for the same fmha call as
 * ternaspmm_decode_attention (model.py:231-233) at T > 1; flash-attention style, both products on the matrix cores,
 * no workspace.  D is 64 or 128, S <= 8192.  Only enqueues. */
void ternaspmm_prefill_attention(const terna_bf16* q, const terna_bf16* cache_k, const terna_bf16* cache_v,
                                 const long long* pos, int per_sequence, terna_bf16* out, int B, int T, int H, int KV, int D, int S,
                                 float scale, terna_stream stream);

/* ternaspmm_decode_attention for callers that cannot allocate or bring a workspace (code under HIP graph capture
 * that owns no buffers, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.
 * Same arguments, kernels and results as ternaspmm_decode_attention with a workspace, but the split-attention
 * scratch (arrival counters + partial results) is a static device array inside the library: about 1 MiB per GPU,
 * held until the process ends.  Limit: B * H <= 256 heads per call (D 64 or 128); beyond that the call prints an
 * error, does nothing and returns -1 (0 on success).  Calls no hipMalloc / hipFree.  Every call on one GPU shares
 * that GPU's array: calls that overlap on one GPU (two streams, two threads) race -- serialise them.  The first
 * call on a device looks the array's address up and enqueues a small clear of the counters on `stream`: it must
 * be made outside stream capture -- under capture that first call records nothing, prints an error and returns -1. */
int ternaspmm_decode_attention_static(const terna_bf16* q, const terna_bf16* cache_k, const terna_bf16* cache_v,
                                      const long long* pos, int per_sequence, terna_bf16* out, int B, int H, int KV, int D, int S,
                                      float scale, terna_stream stream);
/* Both of the above in one launch for T = 1: qkv bf16 [B][(H + 2*KV)*D], cos / sin fp32 [D/2] of the new
 * token's position ([B][D/2] with `per_sequence`); writes slot pos[0] (pos[b]) of the caches and out.  Results are bit-identical to
 * ternaspmm_rope_kv_store followed by ternaspmm_decode_attention. */
void ternaspmm_rope_decode_attention(const terna_bf16* qkv, const float* cos, const float* sin, const long long* pos,
                                     int per_sequence, terna_bf16* cache_k, terna_bf16* cache_v, terna_bf16* out, int B, int H, int KV,
                                     int D, int S, float scale, int adjacent, void* workspace, terna_stream stream);

/* ternaspmm_rope_decode_attention (always the unsplit launch) as a producer for the chained step: next to out it leaves,
 * per sequence and head, the partial statistics of the norm that reads the attention output (model.py:236
 * attn_sub_norm, norm_weight bf16 [H * D]): stats_out fp32 [B][H][2] = (sum of o^2, max |o * norm_weight|) over the
 * head's D columns of the stored bf16 row -- what ternaspmm_quant_from_stats (stats_count = H) or a
 * TERNASPMM_PROLOGUE_STATS launch adds up.  Returns H, or -1 for unsupported arguments (nothing enqueued). */
int ternaspmm_rope_decode_attention_stats(const terna_bf16* qkv, const float* cos, const float* sin, const long long* pos, int per_sequence,
                                          terna_bf16* cache_k, terna_bf16* cache_v, terna_bf16* out, int B, int H, int KV, int D, int S,
                                          float scale, int adjacent, const terna_bf16* norm_weight, float* stats_out, terna_stream stream);

/* ternaspmm_rope_decode_attention with up to six prefetch regions (no counterpart in the reference).  The attention
 * of a decode step occupies one CU per (sequence, head); this variant adds workgroups on the CUs that stay idle, which
 * read pf_bytes[r] bytes (at most 1 GiB) at pf_ptr[r] (16-byte aligned device memory) and discard them: the weights of the launches that
 * follow then start in the L2s / the last-level cache instead of HBM.  A region is cut into units of pf_unit_bytes[r]
 * (a multiple of 16) that are spread over the XCDs round robin -- for a P2 weight, what one workgroup of the consuming
 * kernel reads: bands per workgroup x K/64 x 256 bytes -- so that a unit lands in the L2 its consumer will use;
 * pf_unit_bytes[r] = 0 marks a small region (at most 1 MiB: norm weights, scales) that every workgroup of the
 * consumers reads and every XCD therefore fetches whole.
 * A region that breaks one of these rules is skipped; nothing is prefetched when the attention leaves fewer than 96
 * CUs idle (the few prefetching workgroups would outlast it).
 * pf_ptr / pf_bytes / pf_unit_bytes are host arrays of pf_count entries, read during the call.  Results are those of
 * ternaspmm_rope_decode_attention; nothing depends on where the prefetched bytes end up. */
void ternaspmm_rope_decode_attention_prefetch(const terna_bf16* qkv, const float* cos, const float* sin, const long long* pos,
                                              int per_sequence, terna_bf16* cache_k, terna_bf16* cache_v, terna_bf16* out, int B, int H, int KV,
                                              int D, int S, float scale, int adjacent, void* workspace,
                                              const void* const* pf_ptr, const long long* pf_bytes, const long long* pf_unit_bytes,
                                              int pf_count, terna_stream stream);

/* The single-token attention split over the cache WITHOUT the merge (no counterpart in the reference): as
 * ternaspmm_rope_decode_attention_prefetch, but the cache prefix of every head is spread over `splits` (1, 2, 4 or 8)
 * workgroups that leave their partial results -- unnormalised sums, score maxima, sums of numerators, fp32 -- in
 * `partial` (ternaspmm_attention_partial_bytes(B, H, D) bytes of device memory, no initialisation needed) and end;
 * the consumer of the attention output merges them in the next launch: ternaspmm_attention_merge (out bf16 [B][H*D],
 * the bits of the in-launch merge at the same split count) or bitlinear_TernaSpMM_packed_fused_attn, which merges
 * inside the O projection's prologue.  The launch boundary takes the place of the arrival counter and of the merging
 * workgroup's dependent reads, which cost the in-launch merge 5 - 6 us whatever the prefix length.
 * ternaspmm_attention_partial_splits(B, H, S): the split count the library recommends (a power of two; 1 when the
 * heads fill the chip anyway).  pf_ptr may be NULL with pf_count = 0.
 * Several sequences with 2 or 4 heads per kv head run one workgroup per (sequence, kv head, split): the heads of a kv
 * group read the same keys and values, which then cross from L2 into a CU once instead of once per head (same bits;
 * measured, 2B shape, caches of 1528 slots: 8 sequences 1.463 -> 1.351 ms per decode step, 6 sequences 1.405 -> 1.258).
 * ternaspmm_attention_partial_splits_kv(B, H, KV, S) is the recommendation for that form: it splits from 512 slots on. */
long long ternaspmm_attention_partial_bytes(int B, int H, int D);
int ternaspmm_attention_partial_splits(int B, int H, int S);
int ternaspmm_attention_partial_splits_kv(int B, int H, int KV, int S);   /* the same, knowing the kv heads: see below */
void ternaspmm_rope_decode_attention_partial(const terna_bf16* qkv, const float* cos, const float* sin, const long long* pos,
                                             int per_sequence, terna_bf16* cache_k, terna_bf16* cache_v, float* partial, int splits,
                                             int B, int H, int KV, int D, int S, float scale, int adjacent,
                                             const void* const* pf_ptr, const long long* pf_bytes, const long long* pf_unit_bytes,
                                             int pf_count, terna_stream stream);
void ternaspmm_attention_merge(const float* partial, int splits, terna_bf16* out, int B, int H, int D, terna_stream stream);
/* ternaspmm_attention_merge and the ternaspmm_rmsnorm_quant behind it (model.py:236 attn_sub_norm, :120-123 quant_input
 * of the O projection) in one launch, one workgroup per sequence: (xq_out int8 [B][H*D], s_out bf16 [B]) are the bits of
 * that pair; o_out (optional, bf16 [B][H*D]) receives the merged attention output.  For a step of several sequences,
 * whose O projection then takes the quantised rows (ternaspmm_fused_linear, TERNASPMM_PROLOGUE_QUANTISED) instead of
 * repeating merge, norm and quantisation in every workgroup.  H * D <= 4096, D = 64 or 128, splits 1, 2, 4 or 8;
 * returns 0, or -1 for anything else (nothing enqueued). */
int ternaspmm_attention_merge_rmsnorm_quant(const float* partial, int splits, const terna_bf16* norm_weight, float eps, terna_bf16* o_out,
                                            int8_t* xq_out, terna_bf16* s_out, int B, int H, int D, terna_stream stream);

/* The bookkeeping of one greedy decode step in one launch (generate.py:283-305: argmax, tokens[:, pos] = next_token,
 * the position counters): tok[b] = argmax(logits[b]) as above; if history != NULL and counters[1] < history_len,
 * history[b][counters[1]] = tok[b]; then counters[0] += 1 and counters[1] += 1 (counters int64 [2] = {cache slot of the
 * next token, number of tokens in the history}; NULL: step 0, nothing advanced).  Sixteen workgroups share a row.
 * state: ternaspmm_greedy_step_state_bytes(B) bytes of device memory, 8-byte aligned, zero-filled once by the caller
 * (every launch leaves its first 8 bytes zero again); launches that share a state must not overlap.  Only enqueues. */
size_t ternaspmm_greedy_step_state_bytes(int B);
void ternaspmm_greedy_step_bf16(const terna_bf16* logits, long long* tok, long long* history, int history_len,
                                long long* counters, void* state, int B, int V, terna_stream stream);

/* bf16 LM head of a decode step (F.linear on the tied embedding matrix, model.py:367, 449-455):
 * logits[m][v] = sum_k x[m][k] * w[v][k], fp32 accumulate, bf16 out.  x bf16 [M][K], M <= 16; w bf16 [V][K];
 * logits bf16 [M][V]; K a multiple of 32 with M * (2 K + 16) <= 160 KB; x and w 16-byte aligned.  An HBM-bound pass over w.
 * Only enqueues. */
void ternaspmm_lm_head_bf16(const terna_bf16* x, const terna_bf16* w, terna_bf16* logits, int M, int V, int K,
                            terna_stream stream);

/* Greedy sampling (torch.argmax over the logits, generate.py:283, 305): out[b] = index of the largest of
 * x[b][0 .. V-1] (bf16 [B][V]; out int64 [B]); ties go to the lowest index, NaN never wins.  Only enqueues. */
void ternaspmm_argmax_bf16(const terna_bf16* x, long long* out, int B, int V, terna_stream stream);

/* ---- Repack cache for unmodified call sites (on unless TERNASPMM_REPACK_CACHE=0 is in the environment) ----------
 * The reference-format entry points above (bitlinear_TernaSpMM*, bitlinear_TernaSpMM_bf16*) keep a device-side P2
 * copy of every weight they have seen -- keyed by device, the bitmap / sign / offset pointers and the shape -- and run
 * the P2 kernels from the second sight on.
 *   Cost in memory: N*K/4 + 256 bytes per weight seen (520 MB for the 120 matrices of a BitNet-2B model), up to a
 *     limit: by default an eighth of the device's memory, TERNASPMM_REPACK_CACHE_LIMIT_MB in the environment or
 *     ternaspmm_repack_cache_limit() change it.  At the limit the least recently used copies are released; a weight
 *     whose copy does not fit is served by the reference-format kernels.
 *   Cost in behaviour: the first sight of a weight allocates, repacks and waits for the stream (see the conventions
 *     at the top).  During stream capture nothing is allocated, released or waited for: a weight first seen there is
 *     served by the reference-format kernels -- warm up once before capturing, as generate.py:121-129 does.  A copy
 *     that a capture has used is never released behind the graph's back (not at the limit, not when it turns stale);
 *     only ternaspmm_repack_cache_clear() releases it: destroy such graphs before calling that.
 *   Stale copies: every launch on a cached copy re-checks a fingerprint of the caller's tensors (2.5 KB sampled from
 *     the bitmap and sign arrays + the sign-bit total) against the one recorded with the copy.  When weights were
 *     freed or replaced and other data sits at the same addresses, that launch reports it; the launch itself has
 *     already used the old copy and its output is invalid.  The next call into the library (outside capture) drops
 *     the copy, prints a warning (the first eight times) and continues: the weight gets a fresh copy at its next
 *     sight.  TERNASPMM_REPACK_CACHE_STRICT=1 makes that next call print an error and exit the process instead.  The
 *     check samples: it finds a replaced tensor, not a few weights edited in place.  Call
 *     ternaspmm_repack_cache_clear() after freeing, reloading or editing weights and the window never opens.
 * ternaspmm_repack_cache_clear(): releases every copy (waits for the device).
 * ternaspmm_repack_cache_enable(0 / 1): switches the cache off / on at run time, returns the previous setting (copies
 *   already made are kept until cleared).
 * ternaspmm_repack_cache_limit(bytes): sets the limit (bytes >= 0; a negative value only queries) and returns the
 *   previous one (-1: none set yet).  Copies beyond a lowered limit go at the next first sight.
 * ternaspmm_repack_cache_stats(out): out[0] copies held, [1] their bytes, [2] copies dropped as stale so far,
 *   [3] copies released at the limit so far, [4] bytes parked for captured graphs, [5] the limit (-1: none yet). */
void ternaspmm_repack_cache_clear(void);
int ternaspmm_repack_cache_enable(int on);
long long ternaspmm_repack_cache_limit(long long bytes);
void ternaspmm_repack_cache_stats(long long out[6]);

/* Host only, enqueues nothing: what a call of the reference-format entry points would do.  int8_activations:
 * 1 = bitlinear_TernaSpMM*, 0 = bitlinear_TernaSpMM_bf16*; route 0 / 1 / 2 = plain / _prefill / _decode symbol;
 * `workspace` as the call would pass it (only its alignment matters); cached: whether the weight has a cached P2
 * copy.  Returns the kernel: 0 small-M kernel on the reference format, 1 MFMA-tiled kernel decoding the reference
 * format on the fly, 2 per-call transcode into the workspace + MFMA-tiled P2 kernel, 3 small-M kernel on the cached
 * copy, 4 MFMA-tiled kernel on the cached copy; -1 for an unsupported shape.  *workspace_bytes_used (may be NULL):
 * the highest byte offset of `workspace` the call would write, 0 when it stays untouched -- never more than the
 * sizes documented at bitlinear_TernaSpMM. */
int ternaspmm_plan_reference_call(int int8_activations, int route, int M, int N, int K, int SPLIT_K,
                                  const void* workspace, int cached, long long* workspace_bytes_used);

/* ---- Calibration probes (no counterpart in the reference) ------------------------------------------------------
 * What the machine gives, measured by the same library in the same run as the kernels a benchmark prices:
 *   ternaspmm_probe_empty    enqueues an empty kernel (one wave): N of them in a captured graph, replayed, give the
 *                            cost of one graph kernel node -- the floor under every launch of a decode step;
 *   ternaspmm_probe_empty_shape  the same with a launch shape: `workgroups` of `threads` (a multiple of 64, at most 1024)
 *                            with `lds_bytes` (at most 64 KB) of LDS each and an empty body -- the floor under a
 *                            kernel of that shape (dispatch of its waves, LDS allocation, end of kernel).  0 / -1;
 *   ternaspmm_probe_read     streams `bytes` (16-byte aligned) through the chip and discards them: the read rate;
 *                            `sink` (16 bytes, may be NULL) is written practically never;
 *   ternaspmm_probe_read_grid  the same stream read by a given number of workgroups (1 .. 4096): the rate ONE CU sustains
 *                            (64 KB in flight per workgroup) and how it adds up.  0 / -1;
 *   ternaspmm_probe_copy     dst <- src, `bytes` each: the read + write rate;
 *   ternaspmm_probe_barrier  `rounds` device-wide synchronisations among `workgroups` co-resident workgroups (at most
 *                            one per CU, at most 256) through flags in `state` (ternaspmm_probe_barrier_state_bytes()
 *                            bytes, 16-byte aligned, zero-filled once; pass first_tag = 1 + the rounds run on it so
 *                            far): what a persistent kernel would pay between two dependent phases.  Every wait is
 *                            bounded; uint32 word 512 of `state` counts workgroups that gave up (0 after a good run).
 *                            Returns 0, or -1 when the arguments are refused.
 * All only enqueue; time them with events on `stream`. */
void ternaspmm_probe_empty(terna_stream stream);
int ternaspmm_probe_empty_shape(int workgroups, int threads, int lds_bytes, terna_stream stream);
void ternaspmm_probe_read(const void* src, long long bytes, void* sink, terna_stream stream);
int ternaspmm_probe_read_grid(const void* src, long long bytes, void* sink, int workgroups, terna_stream stream);
void ternaspmm_probe_copy(const void* src, void* dst, long long bytes, terna_stream stream);
size_t ternaspmm_probe_barrier_state_bytes(void);
int ternaspmm_probe_barrier(void* state, int workgroups, int rounds, unsigned first_tag, terna_stream stream);

/* Library version string, e.g. "ternaspmm-gfx950 0.1". */
const char* ternaspmm_version(void);

#ifdef __cplusplus
}
#endif
#endif /* TERNASPMM_H */
