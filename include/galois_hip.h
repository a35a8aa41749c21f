/*
 * galois_hip.h -- C ABI of the MI355X (gfx950) backend for galois's Q4_0 path.
 *
 * This is what a rewritten src/cuda.rs binds with `extern "C"` in place of
 * cudarc + galois_kernels + cuBLAS.  Plain pointers and sizes only.  Every
 * entry point cites the reference interface it replaces (paths relative to the
 * szuwgh/galois tree).
 *
 * Conventions
 *   - Every function returns a status: 0 = ok, negative = GALOIS_HIP_E_* (argument
 *     errors detected on the host before anything is launched), positive = the
 *     hipError_t that HIP reported.  Nothing aborts or throws across the boundary
 *     (the reference panics via todo!()/unwrap(), src/cuda.rs:305,611,805).
 *   - A context owns one device ordinal and one HIP stream (the reference uses
 *     cudarc's single default stream, src/cuda.rs:221-229).  All op entry points
 *     are asynchronous on that stream; only *_sync_copy and synchronize block.
 *     A context is thread-compatible: callers serialise access, as the
 *     reference's &mut dst borrow rules do.
 *   - Tensors are raw device pointers.  Q4_0 data keeps the reference's block
 *     bytes exactly (src/ggml_quants.rs:140-145, galois-kernels/src/matmul.cu:19-23):
 *     18 bytes per 32 weights = f16 scale d, then qs[16]; weight j is the low
 *     nibble of qs[j], weight j+16 the high nibble; value = (nibble - 8) * d.
 *   - Shapes are explicit int32/int64 (the reference passes usize where its
 *     kernels declare int, src/cuda.rs:1032 vs matmul.cu:45).
 */
#ifndef GALOIS_HIP_H
#define GALOIS_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Changes whenever the argument list of an exported function changes (2: n_table_rows of get_rows_q4_0,
 * head_major_n_ctx of the attention calls, galois_hip_abi_version / galois_hip_set_option and the panel calls added).  A binding compares
 * the value it was written against with galois_hip_abi_version() before its first call. */
#define GALOIS_HIP_ABI_VERSION 2

#define GALOIS_HIP_OK 0
#define GALOIS_HIP_E_NULL (-1)      /* a required pointer is NULL */
#define GALOIS_HIP_E_SHAPE (-2)     /* a dimension is <= 0, too large, or not a multiple the op needs */
#define GALOIS_HIP_E_ALIGN (-3)     /* a device pointer is not aligned as the op needs */
#define GALOIS_HIP_E_ORDINAL (-4)   /* no such device */
#define GALOIS_HIP_E_UNSUPPORTED (-5) /* the reference leaves this combination todo!() and so do we */
#define GALOIS_HIP_E_ARCH (-6)      /* the device is not gfx950 */
#define GALOIS_HIP_E_DEVICE_WAIT (-7) /* reported by synchronize / *_sync_copy: a workgroup of galois_hip_qkv_attn_decode_*
                                       * gave up a bounded wait for other workgroups of its launch.  The attention output of
                                       * that call is NaN, later launches on the context may have read stale vectors; the
                                       * status is reported once, the context is usable again afterwards */

typedef struct galois_hip_ctx galois_hip_ctx;
typedef struct galois_hip_event galois_hip_event;
typedef struct galois_hip_graph galois_hip_graph;

/* ---- device / stream / buffer layer -------------------------------------- */

/* GALOIS_HIP_ABI_VERSION of the library that was loaded (valid without a context; no counterpart in the reference,
 * whose kernels are looked up by name at run time, src/cuda.rs:304-307). */
int32_t galois_hip_abi_version(void);

/* CudaDevice::new(ordinal), src/cuda.rs:221-229: bind a device, create its stream. */
int32_t galois_hip_create(int32_t ordinal, galois_hip_ctx **out);
int32_t galois_hip_destroy(galois_hip_ctx *ctx);
/* init_cuda_function(&dev), src/kernels.rs:4-22.  Code objects are linked into
 * the library, so nothing is loaded; this checks the ABI version and that the
 * device can run them, and returns the number of kernels in *n_kernels. */
int32_t galois_hip_init_functions(galois_hip_ctx *ctx, int32_t abi_version, int32_t *n_kernels);
/* Per-context switches (no counterpart in the reference).  Unknown options return GALOIS_HIP_E_UNSUPPORTED.
 *   GEMV_F32_ARITHMETIC (0 / 1, default 0): galois_hip_dequantize_mul_mat_vec_q4_0 multiplies and adds in f32, weight by
 *     weight, as dequantize_mul_mat_vec_q4_0 does (matmul.cu:72-100), instead of the block-scaled fixed-point dot
 *     (same results within the 1e-4 bar; several times slower).  The grouped and fused launches are not affected.
 *   WAIT_SPIN_LIMIT (polls; 0 restores the default of 2^20, about a second) and WAIT_TARGET_BIAS (0 / 1): the bound
 *     of the waits inside galois_hip_qkv_attn_decode_* and an offset added to the count they wait for.  For tests of
 *     the give-up path only: with bias 1 every wait runs out, every kernel still ends normally, the call's output is
 *     NaN and the next synchronize returns GALOIS_HIP_E_DEVICE_WAIT. */
#define GALOIS_HIP_OPT_GEMV_F32_ARITHMETIC 1
#define GALOIS_HIP_OPT_WAIT_SPIN_LIMIT 2
#define GALOIS_HIP_OPT_WAIT_TARGET_BIAS 3
int32_t galois_hip_set_option(galois_hip_ctx *ctx, int32_t option, int32_t value);
/* Text of the last non-zero status on this context ("" if none); never NULL. */
const char *galois_hip_last_error(const galois_hip_ctx *ctx);
/* Name for a status code of this ABI (valid without a context). */
const char *galois_hip_status_string(int32_t status);
/* Device properties the harness prints: name/arch string, CU count, clocks (kHz), memory bytes. */
int32_t galois_hip_device_info(galois_hip_ctx *ctx, char *name, int32_t name_cap, char *arch,
                               int32_t arch_cap, int32_t *n_cu, int32_t *clock_khz,
                               int32_t *mem_clock_khz, int64_t *mem_bytes);

/* alloc_zeros::<T>(n), src/cuda.rs:723,757,926,1052,1066: zero-filled device memory. */
int32_t galois_hip_alloc_zeros(galois_hip_ctx *ctx, size_t bytes, void **out);
/* Drop of CudaSlice<T>. */
int32_t galois_hip_free(galois_hip_ctx *ctx, void *dptr);
/* htod_sync_copy, src/cuda.rs:234,250,274,281,288. */
int32_t galois_hip_htod_sync_copy(galois_hip_ctx *ctx, void *dst_dev, const void *src_host, size_t bytes);
/* dtoh_sync_copy_into, src/lib.rs:2217-2328: waits for the stream, then copies. */
int32_t galois_hip_dtoh_sync_copy(galois_hip_ctx *ctx, void *dst_host, const void *src_dev, size_t bytes);
/* cudaMemcpyAsync / cudaMemcpy2DAsync device-to-device, src/cuda.rs:335-371 (pitches in bytes). */
int32_t galois_hip_dtod_copy(galois_hip_ctx *ctx, void *dst_dev, const void *src_dev, size_t bytes);
int32_t galois_hip_dtod_copy_2d(galois_hip_ctx *ctx, void *dst_dev, size_t dpitch, const void *src_dev,
                                size_t spitch, size_t width_bytes, size_t height);
/* Stream synchronisation (implicit in the reference's to_cpu_tensor, src/lib.rs:2314).  This call and the two
 * *_sync_copy calls also report GALOIS_HIP_E_DEVICE_WAIT (above) for work that has finished. */
int32_t galois_hip_synchronize(galois_hip_ctx *ctx);

/* Timing on the context's stream (the reference has none: dead SystemTime pairs, src/op.rs:1392-1395). */
int32_t galois_hip_event_create(galois_hip_ctx *ctx, galois_hip_event **out);
int32_t galois_hip_event_record(galois_hip_ctx *ctx, galois_hip_event *ev);
int32_t galois_hip_event_elapsed_ms(galois_hip_ctx *ctx, galois_hip_event *start, galois_hip_event *stop,
                                    float *ms); /* synchronises on `stop` */
int32_t galois_hip_event_destroy(galois_hip_ctx *ctx, galois_hip_event *ev);

/* Stream capture (no counterpart in the reference, which launches every op of a decode step on its
 * own: src/cuda.rs:476-565).  Ops issued on the context between begin and end are recorded instead of
 * run; graph_launch replays them in order on the context's stream with the pointers and sizes they were
 * recorded with.  While a capture is open, calls that allocate, free or block return
 * GALOIS_HIP_E_UNSUPPORTED (a prefill matmul must have sized its workspace in an earlier eager call). */
int32_t galois_hip_graph_begin_capture(galois_hip_ctx *ctx);
int32_t galois_hip_graph_end_capture(galois_hip_ctx *ctx, galois_hip_graph **out);
int32_t galois_hip_graph_launch(galois_hip_ctx *ctx, galois_hip_graph *graph);
int32_t galois_hip_graph_destroy(galois_hip_ctx *ctx, galois_hip_graph *graph);

/* ---- Q4_0 format ----------------------------------------------------------- */

/* BlockQ4_0::from_f32 is todo!() in the reference (src/ggml_quants.rs:198-200); this is the
 * canonical ggml quantize_row_q4_0 whose output BlockQ4_0::to_f32 (src/ggml_quants.rs:209-228)
 * inverts: k floats -> k/32 blocks of 18 bytes.  k % 32 == 0.  Rows of a matrix are
 * quantized by one call over the whole contiguous buffer (blocks never straddle rows when
 * the row length is a multiple of 32). */
int32_t galois_hip_quantize_row_q4_0(galois_hip_ctx *ctx, const float *x, void *y, int64_t k);
/* BlockQ4_0::to_f32, src/ggml_quants.rs:209-228 (device twin dequantize_q4_0, matmul.cu:25-43). */
int32_t galois_hip_dequantize_row_q4_0(galois_hip_ctx *ctx, const void *x, float *y, int64_t k);

/* ---- the hot path --------------------------------------------------------- */

/* Decode GEMV.  Replaces the launch of dequantize_mul_mat_vec_q4_0
 * (src/cuda.rs:1011-1034 -> galois-kernels/src/matmul.cu:45-117), same argument
 * order: dst[row] = sum_col (q-8)*d * y[col], f32.  vx: nrows rows of ncols/32
 * Q4_0 blocks; ncols % 32 == 0; vx 2-byte aligned, y/dst 4-byte aligned.
 * The caller loops ne12*ne13 batch slices exactly as src/cuda.rs:1026-1034.
 * Arithmetic: when ncols % 64 == 0 and vx is 4-byte, y 8-byte aligned, the activations are rounded per block of 32 to
 * 18 bits below the block's largest one (blocks that this would leave too coarse carry a second, finer grid) and the
 * products are exact integer dots scaled in f32: within 1e-4 of the f64 dequantize-then-dot result (max error over
 * max |result|, and relative L2) for every input tested, with ONE stated exception -- a vector whose every block has its
 * largest activation below 2^-108 keeps 13 bits per block and stays within 5e-4.  Otherwise, and always when
 * GALOIS_HIP_OPT_GEMV_F32_ARITHMETIC is set, plain f32 multiply-add as in the reference kernel. */
int32_t galois_hip_dequantize_mul_mat_vec_q4_0(galois_hip_ctx *ctx, const void *vx, const float *y,
                                               float *dst, int32_t ncols, int32_t nrows);

/* Several decode GEMVs in one launch.  The reference launches one kernel per product and per
 * batch slice (the loop at src/cuda.rs:1026-1034) and one more for every op around it; on this
 * device a launch costs as much as streaming 15-20 MB of weights, so the products of a decode
 * step that do not depend on each other (q | k | v, gate | up) go out together and the row ops
 * next to them ride along:
 *   norm_weight != NULL: y is replaced by rms_norm(y, norm_eps) * norm_weight before the product
 *     (rms_norm_f32 + mul_f32, src/cuda.rs:1146-1215);
 *   vx_up != NULL: dst = silu(vx . y) * (vx_up . y), the SwiGLU pair (silu_f32 then mul_f32,
 *     src/cuda.rs:1665-1688, 1190-1215); vx_up has the shape of vx;
 *   residual != NULL: residual[row] is added to the result (add_f32, src/cuda.rs:1188-1244);
 *     residual may be dst.
 * A normalisation can also be split over two launches, so that the second fetches one vector instead of two and
 * waits for no reduction: the launch that produces a vector x (a plain product, usually with a residual) also writes
 *   dst_scaled[row] = dst[row] * scale_weight[row]  (x times the weight of the norm that follows), and
 *   sumsq_out[row / 16] = sum of dst[row]^2 over the 16 rows, ceil(nrows / 16) floats;
 * the launch that consumes it passes y = that dst_scaled and sumsq_in = that sumsq_out (ceil(ncols / 16) floats)
 * with norm_eps, and computes (vx . y) * rsqrt(sum(sumsq_in) / ncols + norm_eps), which is
 * vx . (rms_norm(x, norm_eps) * weight) up to rounding (the scalar is applied to both products of a pair).
 * dst_scaled and scale_weight go together; dst_scaled / sumsq_out need norm_weight, sumsq_in and vx_up NULL and at
 * most four products in the call; norm_weight and sumsq_in exclude each other.
 * Each product is what galois_hip_dequantize_mul_mat_vec_q4_0 computes.  1 <= n_items <= 8;
 * ncols % 64 == 0 and ncols <= 12288; matrices 4-byte aligned, y and norm_weight 8-byte aligned;
 * the products of a call all have a norm_weight, or all a sumsq_in, or none has either.  The items array is
 * read during the call only; unused pointer fields are NULL. */
typedef struct galois_hip_gemv_item {
    const void *vx;
    const void *vx_up;
    const float *y;
    const float *norm_weight;
    const float *residual;
    float *dst;
    int32_t ncols, nrows;
    float norm_eps;
    int32_t reserved;  /* 0 */
    float *dst_scaled;
    const float *scale_weight;
    float *sumsq_out;
    const float *sumsq_in;
} galois_hip_gemv_item;
int32_t galois_hip_dequantize_mul_mat_vec_q4_0_group(galois_hip_ctx *ctx, const galois_hip_gemv_item *items,
                                                     int32_t n_items);

/* Prefill matmul.  Replaces quantize_q8_1 + mul_mat_q4_0 (src/cuda.rs:1035-1136 ->
 * matmul.cu:133-174,452-504) with one call: Y[m*N + n] = sum_k deq(W)[n,k] * X[m*K + k]
 * (output layout of matmul.cu:359).  W tiles are dequantised to fp16 in LDS, X is
 * rounded to fp16, products accumulate in f32 on MFMA.  K % 32 == 0.  No Q8_1
 * scratch and no K padding (src/cuda.rs:1040-1068) are needed.  The fp16 copy of X lives in a workspace the context
 * owns and grows on demand (the call allocates when a larger one is needed; refused during a graph capture).  A large
 * product whose N leaves compute units idle (512 x 11008 x 4096 on 256 CUs) is computed as two shares of k that a
 * second launch adds: the f32 sums over k are then two chains instead of one, for the same operands on the same
 * device always the same way. */
int32_t galois_hip_mul_mat_q4_0_f32(galois_hip_ctx *ctx, const void *W, const float *X, float *Y,
                                    int32_t K, int32_t N, int32_t M);

/* The prefill matmul on activations that are ALREADY in the form its matrix instructions fetch ("the panel": fp16,
 * tiles of 16 rows x 32 columns, 1 KB each, tile (r16, c32) at (r16 * K/32 + c32) KB, inside a tile the eight
 * consecutive values k = c32*32 + g*8 .. of row r16*16 + r at (g * 16 + r) * 16 bytes; rows past M are zero), and
 * the producers that write it.  No counterpart in the reference, whose quantize_q8_1 pass (src/cuda.rs:1066-1087 ->
 * matmul.cu:133-174) runs inside every matmul call: galois_hip_mul_mat_q4_0_f32 likewise converts X on every call
 * (one launch, 5-6 us at 512 x 4096); a prefill graph that multiplies the same activations by several matrices
 * (q | k | v after the attention norm, gate | up after the FFN norm), or whose activations come out of a norm or a
 * SwiGLU anyway, writes the panel once, from the op that produces the activations, and hands it on:
 *   galois_hip_f16_panel_bytes: size of the panel of an M x K activation matrix (K % 256 == 0);
 *   galois_hip_f32_to_f16_panel: the conversion alone;
 *   galois_hip_rms_norm_mul_f16_panel: rms_norm_f32 + mul_f32 (src/cuda.rs:1146-1215) with the arithmetic of
 *     galois_hip_rms_norm_mul_f32, rounded to fp16 (nearest even) into the panel; ncols <= 16384;
 *   galois_hip_silu_mul_f16_panel: silu_f32 + mul_f32 (src/cuda.rs:1665-1688, 1190-1215) likewise;
 *   galois_hip_mul_mat_q4_0_f16_panel: Y_j[m*N_j + n] = sum_k deq(W_j)[n,k] * panel[m,k] for 1 to 4 matrices in ONE
 *     launch, each what galois_hip_mul_mat_q4_0_f32 computes from the f32 activations the panel was rounded from
 *     (bit for bit when the panel came from galois_hip_f32_to_f16_panel).  The matrices' column tiles are laid end to
 *     end, so q | k | v of a 4096-wide model fill the device at M = 512 where each alone leaves a third of it idle.
 *     W_j 16-byte aligned (rows of K/32 blocks), Y_j 4-byte, panel 16-byte aligned. */
typedef struct galois_hip_gemm_item {
    const void *W;
    float *Y;
    int32_t N;
    int32_t reserved; /* 0 */
} galois_hip_gemm_item;
int32_t galois_hip_f16_panel_bytes(int32_t K, int32_t M, int64_t *bytes);
int32_t galois_hip_f32_to_f16_panel(galois_hip_ctx *ctx, const float *x, void *panel, int32_t ncols, int32_t nrows);
int32_t galois_hip_rms_norm_mul_f16_panel(galois_hip_ctx *ctx, const float *x, const float *weight, void *panel,
                                          int32_t ncols, int32_t nrows, float eps);
int32_t galois_hip_silu_mul_f16_panel(galois_hip_ctx *ctx, const float *gate, const float *up, void *panel,
                                      int32_t ncols, int32_t nrows);
int32_t galois_hip_mul_mat_q4_0_f16_panel(galois_hip_ctx *ctx, const galois_hip_gemm_item *items, int32_t n_items,
                                          const void *panel, int32_t K, int32_t M);

/* rms_norm_f32 launch, src/cuda.rs:1146-1181 -> rms_norm.cu:13-49:
 * dst = x * rsqrt(mean(x^2) + eps) per row.  Unlike the reference (ne00 % 32 == 0
 * asserted at src/cuda.rs:1157) any ncols >= 1 is accepted. */
int32_t galois_hip_rms_norm_f32(galois_hip_ctx *ctx, const float *x, float *dst, int32_t ncols,
                                int32_t nrows, float eps);
/* Fusion of rms_norm_f32 with the broadcast mul_f32 that applies the norm weight
 * (src/cuda.rs:1190-1215 -> mul.cu:3-12): dst = rms_norm(x) * weight[col]. */
int32_t galois_hip_rms_norm_mul_f32(galois_hip_ctx *ctx, const float *x, const float *weight, float *dst,
                                    int32_t ncols, int32_t nrows, float eps);

/* rope_f32 launch, src/cuda.rs:1257-1297 -> rope.cu:3-28, same parameters (has_pos is
 * always true in the reference): adjacent pairs rotated by
 * pos[row / p_delta_rows] * freq_scale * theta_scale^(col/2).  ncols even. */
int32_t galois_hip_rope_f32(galois_hip_ctx *ctx, const float *x, float *dst, int32_t ncols, int32_t nrows,
                            const int32_t *pos, float freq_scale, int32_t p_delta_rows, float theta_scale);

/* soft_max_f32 launch, src/cuda.rs:1642-1663 -> softmax.cu:3-48: row softmax in f32,
 * -inf inputs are masked (exactly 0 out).  A row that is all -inf yields NaN as in the
 * reference kernel. */
int32_t galois_hip_soft_max_f32(galois_hip_ctx *ctx, const float *x, float *dst, int32_t ncols,
                                int32_t nrows);
/* Causal variant with the mask computed from indices instead of -inf inputs (the
 * reference has no mask op): row r keeps columns <= n_past + (r % rows_per_head),
 * other outputs are exactly 0 and their inputs are never read. */
int32_t galois_hip_soft_max_causal_f32(galois_hip_ctx *ctx, const float *x, float *dst, int32_t ncols,
                                       int32_t rows_per_head, int32_t nrows, int32_t n_past);

/* ---- around the hot path: the other ops of a LLaMA decode graph --------------------- */

/* add_f32 / mul_f32, src/cuda.rs:1188-1244 -> add.cu:3-12, mul.cu:3-12: dst[i] = x[i] (op) y[i % ky]
 * (row broadcast of a bias / norm weight; ky == kx is the plain elementwise case). */
int32_t galois_hip_add_f32(galois_hip_ctx *ctx, const float *x, const float *y, float *dst, int64_t kx, int64_t ky);
int32_t galois_hip_mul_f32(galois_hip_ctx *ctx, const float *x, const float *y, float *dst, int64_t kx, int64_t ky);
/* scale_f32, src/cuda.rs:1597-1638 -> scale.cu:1-11: dst = scale * x (the caller reads the scalar
 * out of its CPU tensor as CudaScale::f_g_c does). */
int32_t galois_hip_scale_f32(galois_hip_ctx *ctx, const float *x, float *dst, float scale, int64_t k);
/* silu_f32, src/cuda.rs:1665-1688 -> unary.cu:1-10: dst = x / (1 + exp(-x)). */
int32_t galois_hip_silu_f32(galois_hip_ctx *ctx, const float *x, float *dst, int64_t k);
/* Fusion of silu_f32 with the elementwise mul_f32 of SwiGLU: dst = silu(gate) * up. */
int32_t galois_hip_silu_mul_f32(galois_hip_ctx *ctx, const float *gate, const float *up, float *dst, int64_t k);
/* cpy_f32_f32 / cpy_f32_f16, src/cuda.rs:1382-1595 -> cpy.cu:79-156 (also galois_cont): element i of the
 * [ne00, ne01, *] source goes to element i of the [ne10, ne11, *] destination; nb* are BYTE strides as in
 * the reference's F32Dim / F16Dim (src/cuda.rs:1360-1380). */
int32_t galois_hip_cpy_f32(galois_hip_ctx *ctx, const void *x, void *dst, int32_t dst_is_f16, int64_t ne, int64_t ne00,
                           int64_t ne01, int64_t nb00, int64_t nb01, int64_t nb02, int64_t ne10, int64_t ne11,
                           int64_t nb10, int64_t nb11, int64_t nb12);
/* get_rows for a Q4_0 table: GetRows::f_q_x_f32, src/op.rs:2546-2571 (CPU-only in the reference; its GPU
 * arm is todo!(), src/op.rs:3281-3292): dst row i = to_f32(table row ids[i]), ncols % 32 == 0.  The table has
 * n_table_rows rows; the ids are read on the device, so an id outside 0 .. n_table_rows - 1 cannot be refused
 * here: its dst row is filled with NaN and nothing is read for it (the reference's slice index would panic). */
int32_t galois_hip_get_rows_q4_0(galois_hip_ctx *ctx, const void *table, const int32_t *ids, float *dst,
                                 int32_t ncols, int32_t nr, int32_t n_table_rows);
/* f32 x f32 batched matmul with galois's shape conventions; todo!() in the reference (src/cuda.rs:867-879,
 * src/op.rs:1624-1662).  a = [K, N, ne02] with element strides a_s0, a_s1, a_s2 (one of a_s0, a_s1 must
 * be 1, so permuted K/V-cache views work), b = [K, M, ne12] contiguous, dst = [N, M, ne12];
 * a is broadcast over ne12 / ne02 like the quantized path (src/op.rs:1473-1483). */
int32_t galois_hip_mul_mat_f32(galois_hip_ctx *ctx, const float *a, const float *b, float *dst, int32_t K, int32_t N,
                               int32_t M, int32_t ne02, int32_t ne12, int64_t a_s0, int64_t a_s1, int64_t a_s2);

/* The same with an f16 a (element strides count halfs): the (F16, F32) -> F32 arm of galois_matmul, which the
 * reference serves with cuBLAS gemm_ex on f16 operands with f16 accumulation and an f16 result
 * (CudaMatMul::f_x_y_y, src/cuda.rs:881-992 -> cuda_op_mul_mat_cublas, src/cuda.rs:698-757).  Here a is widened
 * exactly and sums are f32; with M > 1 and rows of a contiguous along K (K % 32 == 0, 16-byte aligned rows) the
 * product runs on the matrix cores with b rounded to f16 as the reference's convert_fp32_to_fp16 does (|b| above
 * 65504 becomes infinite there).  Everywhere else -- M == 1, K % 32 != 0, unaligned rows, a read along N -- b stays
 * f32, so the same operands multiplied at M == 1 (decode) and at M > 1 (prefill) differ by that rounding: at most
 * 2^-11 relative per element of b. */
int32_t galois_hip_mul_mat_f16_f32(galois_hip_ctx *ctx, const void *a, const float *b, float *dst, int32_t K, int32_t N,
                                   int32_t M, int32_t ne02, int32_t ne12, int64_t a_s0, int64_t a_s1, int64_t a_s2);

/* Attention of one decode step over an f32 KV cache in two launches instead of the nine of the op sequence
 * rope_custom(q), rope_custom(k), cpy(k -> cache), cpy(v -> cache), matmul(K^T, q), scale, soft_max, matmul(V, p)
 * (src/cuda.rs:1257-1356, 1382-1595, 698-782, 1597-1663), with the same arithmetic up to the order of f32 sums:
 *   q, k, v: this token's n_head * head_dim projections (not yet rotated); pos: its position (one int32 on the device,
 *   as rope_f32 takes it); rotation parameters as rope_f32 (mode 0, n_dims = head_dim);
 *   k_cache, v_cache: [n_ctx][n_head * head_dim] f32 (head_major_n_ctx == 0), or [n_head][head_major_n_ctx][head_dim]
 *   (head_major_n_ctx = the cache's capacity in positions, above n_past): a head's keys are then contiguous, 64 KB
 *   per workgroup instead of 128 pieces of 512 bytes, which this call alone streams 8 % faster (the launch that also
 *   carries q | k | v does not gain from it); results are bit-equal; the row of position n_past receives rope(k) and v;
 *   out[h * head_dim + d] = sum_l softmax_l(scale * rope(q)_h . K[l]_h) * V[l][h * head_dim + d] over l = 0 .. n_past.
 * head_dim 64 or 128; all pointers 16-byte aligned; partial results live in the context's scratch block, which bounds
 * n_head * ceil((n_past + 1) / 128) * (head_dim + 4) by 2^20. */
int32_t galois_hip_attn_decode_f32(galois_hip_ctx *ctx, const float *q, const float *k, const float *v, float *k_cache,
                                   float *v_cache, float *out, int32_t n_head, int32_t head_dim, int32_t n_past,
                                   const int32_t *pos, float freq_scale, float theta_scale, float scale, int32_t head_major_n_ctx);

/* galois_hip_attn_decode_f32 for callers that cannot allocate device memory or have it allocated on their behalf
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  Same arguments and bit-identical results; the partial results and per-head counters live in a static
 * device array of the library (1 MB + 4 KB, one copy per GPU, held until the process ends) instead of the block the
 * context allocated at creation, and the call allocates and frees nothing.  Limits (GALOIS_HIP_E_SHAPE beyond them):
 * n_head <= 1024 and n_head * ceil((n_past + 1) / 128) * (head_dim + 4) <= 262144, e.g. 32 heads of 128 up to
 * 7936 cached positions.  Every context on a GPU shares that GPU's array: calls that overlap on one GPU (two
 * contexts, two streams) race; calls on one context are ordered by its stream.  The counters are zero when the
 * library is loaded and every call returns them to zero. */
int32_t galois_hip_attn_decode_f32_static(galois_hip_ctx *ctx, const float *q, const float *k, const float *v,
                                          float *k_cache, float *v_cache, float *out, int32_t n_head, int32_t head_dim,
                                          int32_t n_past, const int32_t *pos, float freq_scale, float theta_scale,
                                          float scale, int32_t head_major_n_ctx);

/* The same with f16 caches, the form the reference keeps them in on the GPU (cpy_f32_f16 into the cache,
 * src/cuda.rs:1382-1595, then gemm_ex on F16 operands, src/cuda.rs:881-992): k_cache, v_cache are
 * [n_ctx][n_head * head_dim] f16; row n_past receives rope(k) and v rounded to nearest even, and this step's scores
 * and output use the rounded row, as a cpy followed by the matmuls would.  Half the cache bytes per step. */
int32_t galois_hip_attn_decode_f16kv(galois_hip_ctx *ctx, const float *q, const float *k, const float *v, void *k_cache,
                                     void *v_cache, float *out, int32_t n_head, int32_t head_dim, int32_t n_past,
                                     const int32_t *pos, float freq_scale, float theta_scale, float scale, int32_t head_major_n_ctx);

/* The q | k | v products of a decode step (three CudaMatMul launches, src/cuda.rs:1011-1034, with whatever
 * normalisation galois_hip_dequantize_mul_mat_vec_q4_0_group folds in) and the attention that consumes them
 * (galois_hip_attn_decode_f32 / _f16kv above) as ONE launch: qkv[0..2] are the three products, whose dst are the
 * q, k and v vectors of n_head * head_dim floats (written as by the group call, and read by the attention part).
 * The attention's workgroups follow the products' in the grid, request their cache rows while the last products
 * still stream, and wait -- bounded -- only for their own head's rows of q (k and v where position n_past lives);
 * should a wait ever run out, that head's whole output is NaN, the context's status word is set and the next synchronize
 * or *_sync_copy returns GALOIS_HIP_E_DEVICE_WAIT (once) after returning the counters to zero.  q, k, v and the appended cache rows equal those of the two
 * calls issued one after the other bit for bit (when the group call would run few rows in its 16-wave shape: up to the
 * order in which a normalising product adds its squares), the output up to the order of its f32 sums.  head_dim 128; the products are plain or normalising (no vx_up, residual, dst_scaled, sumsq_out); dst
 * 16-byte aligned; ncols <= 11776; otherwise the limits of both calls apply. */
int32_t galois_hip_qkv_attn_decode_f32(galois_hip_ctx *ctx, const galois_hip_gemv_item *qkv, float *k_cache,
                                       float *v_cache, float *out, int32_t n_head, int32_t head_dim, int32_t n_past,
                                       const int32_t *pos, float freq_scale, float theta_scale, float scale, int32_t head_major_n_ctx);
int32_t galois_hip_qkv_attn_decode_f16kv(galois_hip_ctx *ctx, const galois_hip_gemv_item *qkv, void *k_cache,
                                         void *v_cache, float *out, int32_t n_head, int32_t head_dim, int32_t n_past,
                                         const int32_t *pos, float freq_scale, float theta_scale, float scale, int32_t head_major_n_ctx);

/* One Q4_0 matrix against the panel with the residual stream added: Y = residual + W . panel (residual may be null),
 * Y and residual [M][N] f32 -- an output or down projection and the add that follows it (CudaMatMul then add_f32,
 * src/cuda.rs:1011-1034) as one call.  `workspace` is device memory the call may overwrite (16-byte aligned), or null:
 *   - with 2 * M * N floats of it, a matrix too narrow to give every compute unit a workgroup (N = 4096 at M = 512:
 *     86 tiles of 96 columns, or 172 of 48, for 256 CUs) is multiplied as two shares of k by 256 workgroups of 64
 *     columns, and the pass that adds the residual adds the two partial results as well (M = 512, 11008 -> 4096 with
 *     the residual: 70 -> 55 us);
 *   - Y may be the residual itself (the stream updated in place) when the workspace holds M * N floats or more.
 * The two shapes differ in the order of the f32 sums over k (one chain, or two halves added), i.e. by rounding only;
 * which one runs depends on shape, workspace and device alone, so a call repeats bit for bit.  One or two launches
 * (the product, then the adding pass when there is a residual or a second share). */
int32_t galois_hip_mul_mat_q4_0_f16_panel_add(galois_hip_ctx *ctx, const void *W, const void *panel, const float *residual,
                                              float *Y, int32_t K, int32_t N, int32_t M, void *workspace,
                                              int64_t workspace_bytes);

/* The gate and up projections of a feed-forward block and the SwiGLU between them and the down projection in one
 * launch: panel_out = the fp16 panel of silu(W_gate . x) * (W_up . x) ([N, M] operand, galois_hip_f16_panel_bytes(N, M)
 * bytes) for x given as `panel` ([K, M] operand) -- galois_hip_mul_mat_q4_0_f16_panel on the two matrices followed by
 * galois_hip_silu_mul_f16_panel (CudaMatMul x 2, silu_f32, mul_f32) without the two f32 results ever reaching memory:
 * a tile of the launch holds 48 columns of each matrix, so both products of an element meet in one wave's registers.
 * The products are the same bits as the two-call form's and the SwiGLU is the same expression; its compiled form may
 * fuse 1 + exp(-g) differently, so single elements can differ by one unit in the last place of fp16.  W_gate, W_up: [N rows][K / 32] Q4_0 blocks; K and N multiples of 256. */
int32_t galois_hip_mul_mat_q4_0_swiglu_f16_panel(galois_hip_ctx *ctx, const void *W_gate, const void *W_up, const void *panel,
                                                 void *panel_out, int32_t K, int32_t N, int32_t M);

/* The product of galois_hip_mul_mat_q4_0_f16_panel_add alone, as the shares of k it is computed in, for a caller whose
 * next op does the adding (galois_hip_add_rms_norm_mul_f16_panel below): *n_shares = 1 or 2 partial results [M][N] f32
 * at shares and shares + M * N, whose sum (in that order) is W . panel.  Two only when that pays for the shape
 * and shares_bytes holds 2 * M * N floats; shares_bytes must hold M * N. */
int32_t galois_hip_mul_mat_q4_0_f16_panel_shares(galois_hip_ctx *ctx, const void *W, const void *panel, float *shares,
                                                 int64_t shares_bytes, int32_t K, int32_t N, int32_t M, int32_t *n_shares);

/* sum_out = a (+ b) (+ c) (b, c may be null; added in that order), all [nrows][ncols] f32, and
 * rms_norm(sum_out, eps) * weight into the fp16 panel (as galois_hip_rms_norm_mul_f16_panel would write it from
 * sum_out): the adding pass behind an output / down projection (its one or two shares and the residual stream) and
 * the norm in front of the next product as one launch (add_f32 + rms_norm_f32 + mul_f32 of the reference,
 * src/cuda.rs:1146-1215).  sum_out may be one of a, b, c. */
int32_t galois_hip_add_rms_norm_mul_f16_panel(galois_hip_ctx *ctx, const float *a, const float *b, const float *c, float *sum_out,
                                              const float *weight, void *panel, int32_t ncols, int32_t nrows, float eps);

/* What a prefill does between its q | k | v products and its attention, one launch instead of two to four:
 * rope_custom (mode 0, n_dims = head_dim) of q and of k for n_tokens tokens -- rope_f32 twice, src/cuda.rs:1257-1356,
 * with the same arithmetic, q_out and the rotated k bit-equal to galois_hip_rope_f32's -- and the append of the rotated
 * k and (when v is given) of v to the cache rows of those tokens (cpy_f32_f32 / cpy_f32_f16, src/cuda.rs:1382-1595):
 *   q, k, v: [n_tokens][n_head * head_dim] f32; pos: the tokens' positions (int32, on the device);
 *   q_out: [n_tokens][n_head * head_dim] f32; k_rows, v_rows: the caches' rows of these tokens, contiguous
 *   [n_tokens][n_head * head_dim], f32 (kv_f16 = 0) or f16 rounded to nearest even (kv_f16 = 1).
 * v and v_rows are both null when the values are already in place (an f32 cache can take them from the product).
 * head_dim a multiple of 4 up to 256; 16-byte aligned tensors. */
int32_t galois_hip_rope_qk_append(galois_hip_ctx *ctx, const float *q, const float *k, const float *v, float *q_out, void *k_rows,
                                  void *v_rows, int32_t kv_f16, int32_t head_dim, int32_t n_head, int32_t n_tokens,
                                  const int32_t *pos, float freq_scale, float theta_scale);

/* Causal attention of n_tokens query rows over a KV cache in ONE launch: what a prefill issues per layer as
 * cpy(q -> [D, M, H]), matmul(K^T, q), scale, soft_max under the causal mask, matmul(V, p), cpy(-> [D, H, M])
 * (CudaMatMul src/cuda.rs:867-992, scale and soft_max src/cuda.rs:1597-1663 and 1257-1356, cpy src/cuda.rs:1382-1595),
 * without the scores ever reaching memory:
 *   q: [n_tokens][n_head * head_dim] f32, rotated; k_cache, v_cache: [>= n_past + n_tokens][n_head * head_dim] rows that
 *   already hold positions 0 .. n_past + n_tokens - 1 (this call appends nothing);
 *   row m of head h of the result = sum_l softmax_l(scale * q[m]_h . K[l]_h) V[l]_h over l = 0 .. n_past + m.
 * The result goes to out ([n_tokens][n_head * head_dim] f32) or to out_panel (the fp16 panel of that [n_head * head_dim,
 * n_tokens] operand, galois_hip_f16_panel_bytes(n_head * head_dim, n_tokens) bytes, ready for
 * galois_hip_mul_mat_q4_0_f16_panel): exactly one of the two is non-null.
 * Arithmetic: both products run on the matrix cores with fp16 operands and f32 sums, as the reference's gemm_ex on
 * converted operands does (convert_fp32_to_fp16, src/cuda.rs:881-992): q * scale * log2(e), the keys, the values and
 * the probabilities are rounded to fp16 (an f16 cache is read as it is), maxima, sums and the output accumulate in f32.
 * Against f64 arithmetic on the same inputs the result is within 2e-3 of the largest output magnitude for scores of a
 * few units (unit-variance q and k); rounding q and k moves a score by about 2^-11 of the size of its terms and the
 * exponential makes that a relative error of the probabilities, so scores of +-100 are held to 5e-3.
 * head_dim 128; all pointers 16-byte aligned. */
int32_t galois_hip_attn_prefill_f32(galois_hip_ctx *ctx, const float *q, const float *k_cache, const float *v_cache, float *out,
                                    void *out_panel, int32_t n_head, int32_t head_dim, int32_t n_tokens, int32_t n_past,
                                    float scale);
int32_t galois_hip_attn_prefill_f16kv(galois_hip_ctx *ctx, const float *q, const void *k_cache, const void *v_cache, float *out,
                                      void *out_panel, int32_t n_head, int32_t head_dim, int32_t n_tokens, int32_t n_past,
                                      float scale);

#ifdef __cplusplus
}
#endif
#endif /* GALOIS_HIP_H */
