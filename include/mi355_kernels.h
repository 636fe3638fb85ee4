/*
 * C ABI of the MI355X (gfx950) kernel library for llama.cpp's quantized-inference hot
 * path.  Plain pointers and sizes only.  All data pointers are DEVICE addresses unless a
 * parameter says "host".  `stream` is a hipStream_t passed as void* (NULL = default
 * stream).  Every entry point returns 0 on success or a negative MI355_ERR_* code and
 * launches asynchronously on `stream`; nothing here allocates device memory unless its
 * comment says so.
 *
 * Each entry point names the reference function it stands in for (paths relative to the
 * llama.cpp tree).  Element types use the reference's enum values
 * (ggml/include/ggml.h:351-392): F32 0, F16 1, Q4_0 2, Q4_1 3, Q5_0 6, Q5_1 7, Q8_0 8, Q8_1 9, Q4_K 12, Q5_K 13, Q6_K 14, IQ4_NL 20, IQ4_XS 23, I32 26.
 */
#ifndef MI355_KERNELS_H
#define MI355_KERNELS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI355_OK            0
#define MI355_ERR_ARG      -1   /* unsupported type, shape or alignment */
#define MI355_ERR_HIP      -2   /* a HIP runtime call failed; see mi355_last_error() */
#define MI355_ERR_WORKSPACE -3  /* workspace too small */

enum mi355_type {
    MI355_F32 = 0, MI355_F16 = 1, MI355_Q4_0 = 2, MI355_Q4_1 = 3, MI355_Q5_0 = 6, MI355_Q5_1 = 7, MI355_Q8_0 = 8, MI355_Q8_1 = 9,
    MI355_Q4_K = 12, MI355_Q5_K = 13, MI355_Q6_K = 14, MI355_IQ4_NL = 20, MI355_IQ4_XS = 23, MI355_I32 = 26,
};

/* Library / device ------------------------------------------------------------------ */

/* Version of this ABI (bumped on incompatible change). */
int mi355_abi_version(void);
/* Text of the last error on the calling thread ("" if none). */
const char *mi355_last_error(void);
/* Kernel launches this library has issued in this process so far (every entry point counts each of its launches, also while a
 * stream is being captured).  A host that fuses graph nodes reads it before and after a graph to report launches per graph. */
uint64_t mi355_launch_count(void);
/* 1 if `device` is a gfx950 GPU this library can run on, 0 if not, <0 on HIP error.
 * Counterpart of a backend's score function (ggml/src/ggml-backend-impl.h:212-214). */
int mi355_device_supported(int device);

/* Weight quantizers on the device (what `llama-quantize` runs per tensor without an importance matrix: ggml_quantize_chunk,
 * ggml/src/ggml.c:6410 -> quantize_row_q4_0_ref / q8_0_ref / q4_K_ref / q5_K_ref / q6_K_ref, ggml/src/ggml-quants.c:31-66, 194-217,
 * 1208-1278, 1395-1480, 1620-1688; q4_1 / q5_0 / q5_1 :68-192; quantize_iq4_nl / quantize_iq4_xs, :4573-4745: every weight type
 * of enum mi355_type).  x: DEVICE f32 [nrows][k], contiguous; y: DEVICE blocks in the REFERENCE byte layout
 * (nrows * k / block elements * block bytes; what a GGUF file holds and mi355_weights_scatter takes).  Bit for bit the reference's
 * bytes.  k a multiple of the type's block size; x 16-byte, y 4-byte aligned. */
int mi355_quantize_weights_supported(int type);
int mi355_quantize_weights(void *stream, int type, const float *x, void *y, int64_t k, int64_t nrows);

/* Weight storage -------------------------------------------------------------------- *
 * Quantized weight rows are kept in HBM in a per-row "device layout" that makes every
 * load a 16-byte aligned, coalesced access:
 *   Q4_K, Q5_K : unchanged (144- and 176-byte super-blocks are already 16-byte multiples)
 *   Q4_0, IQ4_NL : [nb x 16 B nibbles][nb x fp16 d]
 *   Q4_1 : [nb x 16 B nibbles][nb x {fp16 d, fp16 m}]
 *   Q5_0 : [nb x 16 B nibbles][nb x 4 B fifth bits][nb x fp16 d]
 *   Q5_1 : [nb x 16 B nibbles][nb x 4 B fifth bits][nb x {fp16 d, fp16 m}]
 *   Q8_0 : [nb x 32 B int8   ][nb x fp16 d]
 *   Q6_K : [nb x 128 B ql][nb x 64 B qh][nb x 16 B scales][nb x fp16 d]
 *   IQ4_XS : [nb x 128 B nibbles][nb x {fp16 d, u16 scales_h, 4 B scales_l}]
 * A row occupies exactly the same number of bytes as in the reference's block layout
 * (ggml/src/ggml-common.h:161-208, 279-290, 314-320, 399-412); the mapping is a byte
 * permutation inside each row.  These two entry points apply it / undo it for the byte
 * range [offset, offset+size) of a tensor of `nrows` rows of `k` elements, so partial
 * uploads and read-back return the reference's bytes
 * (ggml_backend_buffer_i::set_tensor / get_tensor, ggml/src/ggml-backend-impl.h:52-53).
 * `raw` holds only the `size` bytes of the range; `dev` is the base of the whole tensor. */
int mi355_weights_scatter(void *stream, int type, const void *raw, void *dev, int64_t k, int64_t nrows,
                          size_t offset, size_t size);
int mi355_weights_gather(void *stream, int type, const void *dev, void *raw, int64_t k, int64_t nrows,
                         size_t offset, size_t size);

/* Activation quantization ------------------------------------------------------------ *
 * quantize_row_q8_1_ref (ggml/src/ggml-quants.c:220-253), bit-exact: x is f32, row r at
 * x + r*x_stride (elements); y receives nrows * k/32 block_q8_1 (36 bytes each,
 * ggml/src/ggml-common.h:210-221), rows contiguous. */
int mi355_quantize_q8_1(void *stream, const float *x, void *y, int64_t k, int64_t nrows, int64_t x_stride);

/* Same quantizer writing the split layout the matrix kernels read:
 *   int8 q[nrows][k]  followed by  {float d; int32 sum_q;} ds[nrows][k/32]
 * where d is the fp16-rounded block scale widened to f32.  mi355_act_bytes() gives the size. */
size_t mi355_act_bytes(int64_t k, int64_t nrows);
int mi355_quantize_act(void *stream, const float *x, void *act, int64_t k, int64_t nrows, int64_t x_stride);

/* MUL_MAT --------------------------------------------------------------------------- *
 * ggml_compute_forward_mul_mat (ggml/src/ggml-cpu/ggml-cpu.c:7443-7635) for quantized
 * src0 and f32 src1:  dst[b*dst_stride + n] = sum_k W[n][k] * x[b*x_stride + k].
 * W: N rows of K elements of `type` in device layout.  x, dst f32.
 * Up to 4 activation rows (8 where the matrix-core kernels do not support the product) run the
 * bandwidth-bound GEMV (per-block integer dots of the weights against Q8_1 activations), up to 32
 * the weight-streaming matrix-core kernel (mi355_mul_mat_skinny), larger B the int8-MFMA tile kernels.
 * Q5_K (block_q5_K, ggml/src/ggml-common.h:296-308; ggml_vec_dot_q5_K_q8_K, ggml/src/ggml-cpu/ggml-cpu-quants.c:6859-7592) has the
 * GEMV for up to 8 rows, the super-block tile kernel on packed rows (mi355_mul_mat_q8k) for batches - what this entry
 * point runs above 32 rows; the per-32-block kernel mi355_mul_mat_q takes it too - and the wide-tile GEMM on tile images (mi355_kq_unpack_tiles + mi355_mul_mat_q8k_tiled) for callers that keep images.
 * Q4_1, Q5_0, Q5_1 and IQ4_NL (ggml/src/ggml-common.h:168-201, 399-404; ggml_vec_dot_q4_1_q8_1, _q5_0_q8_0, _q5_1_q8_1 and
 * _iq4_nl_q8_0, ggml/src/ggml-cpu/ggml-cpu-quants.c:2511, 2804, 3159, 11188) have the GEMV for up to 8 rows (also in the
 * launches that take several matrices or fuse an epilogue) and the per-32-block int8-MFMA tile kernel (mi355_mul_mat_q) beyond;
 * the weight-streaming kernel for 5..32 rows serves them too.
 * IQ4_XS (block_iq4_xs, ggml/src/ggml-common.h:406-412; ggml_vec_dot_iq4_xs_q8_K, ggml/src/ggml-cpu/ggml-cpu-quants.c:11381) runs on the
 * same three kernels as IQ4_NL, its block scales d * (ls - 32) taken from the super-block headers; from 256 rows on this entry point
 * runs it on mi355_mul_mat_q8k, and it has tile images for mi355_mul_mat_q8k_tiled.
 * `ws` is scratch of at least mi355_mul_mat_ws_bytes(K, B) bytes. */
size_t mi355_mul_mat_ws_bytes(int64_t K, int64_t B);
int mi355_mul_mat(void *stream, int type, const void *W, const float *x, float *dst, int64_t N, int64_t K, int64_t B,
                  int64_t x_stride, int64_t dst_stride, void *ws, size_t ws_bytes);

/* mi355_mul_mat for callers that cannot allocate device memory or bring a workspace (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  The workspace is an array of
 * mi355_mul_mat_static_max_ws() bytes (16 MiB) that lives inside the library, one copy per GPU that loads it, held until
 * the process ends; the call performs no hipMalloc / hipFree and calls no allocating library routine.  Products whose
 * quantized activation does not fit (mi355_mul_mat_ws_bytes(K, B) > the array, e.g. K = 14336 beyond B = 936) are rejected with
 * MI355_ERR_WORKSPACE.  Same result as mi355_mul_mat with a workspace of that size.  Every call on one GPU shares that
 * GPU's array: calls that overlap in time on one GPU (different streams or threads) race on it.
 * mi355_mul_mat_static_init() looks the array's device address up for the current device (the first lookup on a device may load
 * the code object and place the array); call it once per device at set-up, outside any stream capture.  A first
 * mi355_mul_mat_static call on a device makes the same lookup itself. */
size_t mi355_mul_mat_static_max_ws(void);
int mi355_mul_mat_static_init(void);
int mi355_mul_mat_static(void *stream, int type, const void *W, const float *x, float *dst, int64_t N, int64_t K, int64_t B,
                         int64_t x_stride, int64_t dst_stride);

/* The two halves of mi355_mul_mat for callers that reuse one quantized activation for
 * several weight matrices (Q/K/V or gate/up projections): `act` from mi355_quantize_act. */
int mi355_mul_mat_vec_q(void *stream, int type, const void *W, const void *act, float *dst, int64_t N, int64_t K,
                        int64_t B, int64_t dst_stride);
int mi355_mul_mat_q(void *stream, int type, const void *W, const void *act, float *dst, int64_t N, int64_t K, int64_t B,
                    int64_t dst_stride);
/* The same with a workspace for the split along K of products with few tiles (as mi355_mul_mat_q8k_ws): ws of
 * mi355_mul_mat_q_ws_bytes(N, K, B) bytes, 16-byte aligned; with less, or NULL, the product runs unsplit. */
size_t mi355_mul_mat_q_ws_bytes(int64_t N, int64_t K, int64_t B);
int mi355_mul_mat_q_ws(void *stream, int type, const void *W, const void *act, float *dst, int64_t N, int64_t K, int64_t B,
                       int64_t dst_stride, void *ws, size_t ws_bytes);

/* MUL_MAT for 1..32 activation rows as one weight-streaming launch on the int8 matrix cores (every weight type; K a
 * multiple of 256; 16-byte aligned rows: mi355_mul_mat_skinny_supported says whether a product qualifies).  Same operands
 * as mi355_mul_mat_vec_q (`act` from mi355_quantize_act) plus an optional residual added to the result (may alias dst).
 * It is what mi355_mul_mat uses between the batch-1 kernels and the tile kernels (ggml's MUL_MAT with src1->ne[1] of
 * 5..32, ggml_compute_forward_mul_mat, ggml/src/ggml-cpu/ggml-cpu.c:7380-7560).  `ws` of mi355_mul_mat_skinny_ws_bytes
 * bytes lets products with few rows split K over several groups; with less, or NULL, one group walks the whole of K. */
int mi355_mul_mat_skinny_supported(int type, const void *W, int64_t K, int64_t B);
size_t mi355_mul_mat_skinny_ws_bytes(int64_t N, int64_t K, int64_t B);
int mi355_mul_mat_skinny(void *stream, int type, const void *W, const void *act, float *dst, const float *residual, int64_t N,
                         int64_t K, int64_t B, int64_t dst_stride, void *ws, size_t ws_bytes);

/* The same product for 33..128 activation rows on Q4_K weights (ggml_compute_forward_mul_mat with ggml_vec_dot_q4_K_q8_K,
 * ggml-cpu.c:7443-7635, ggml-cpu-quants.c:6817-6848): weights streamed once, packed; the 6-bit sub-block scales folded into two
 * int8 operand planes so that the matrix cores accumulate whole super-blocks in int32 - the CPU path's own integer sums.
 * act: tile images of the B activation rows (mi355_quantize_act_q8k_tiled: quantize_row_q8_K_ref levels, scales and sums).
 * Products with few 32-row tiles run as slices of K when `ws` has mi355_mul_mat_mid_ws_bytes(N, K, B) bytes (may be NULL / 0:
 * one slice).  dst = W x act (+ residual, which may alias dst). */
int mi355_mul_mat_mid_supported(int type, const void *W, int64_t K, int64_t B);
size_t mi355_mul_mat_mid_ws_bytes(int64_t N, int64_t K, int64_t B);
int mi355_mul_mat_mid(void *stream, int type, const void *W, const void *act, float *dst, const float *residual, int64_t N, int64_t K, int64_t B,
                      int64_t dst_stride, void *ws, size_t ws_bytes);

/* K-quant (Q4_K, Q6_K; Q5_K and IQ4_XS on the 64 x 128 form of the kernel) tile GEMM with the activation format ggml-cpu uses for these weight
 * types: one f32 scale per 256 elements (quantize_row_q8_K_ref, ggml/src/ggml-quants.c:2479-2516;
 * vec_dot_type of type_traits_cpu, ggml/src/ggml-cpu/ggml-cpu.c:252-417), so the integer
 * sub-scales fold into the int8 operands and the sums of a whole super-block stay integer
 * (ggml_vec_dot_q4_K_q8_K / ggml_vec_dot_q6_K_q8_K, ggml/src/ggml-cpu/ggml-cpu-quants.c:6817-6848,
 * 8262-8283).  `act` layout: int8 q[nrows][k]; float d[nrows][k/256] (16-byte padded);
 * fp16 bs[nrows][k/256][16] = {bsum_j & 63, bsum_j >> 6} of the eight 32-element sub-blocks.
 * The levels and d are bit-identical to block_q8_K. */
size_t mi355_act_q8k_bytes(int64_t k, int64_t nrows);
int mi355_quantize_act_q8k(void *stream, const float *x, void *act, int64_t k, int64_t nrows, int64_t x_stride);
int mi355_mul_mat_q8k(void *stream, int type, const void *W, const void *act, float *dst, int64_t N, int64_t K, int64_t B,
                      int64_t dst_stride);
/* Same product with the ADD that follows it in the graph (the residual after wo and ffn_down, src/llama.cpp:1566, :1609) done in
 * the epilogue: dst[b][n] = W[n] . x[b] + residual[b][n].  residual has dst's shape and stride and may be dst itself. */
int mi355_mul_mat_q8k_add(void *stream, int type, const void *W, const void *act, float *dst, const float *residual, int64_t N, int64_t K,
                          int64_t B, int64_t dst_stride);

/* The same product with a workspace for the split along K: a launch with few tiles (N/64 x B/128 < 384, e.g. any matrix at batch
 * 64 or the 1024-row wk/wv at batch 512) is cut into up to 8 slices of >= 4 super-blocks that run side by side, their partial
 * sums land in ws and a second launch adds them in fixed order (plus the residual).  ws: mi355_mul_mat_q8k_ws_bytes(N, K, B) bytes,
 * 16-byte aligned (0 = this shape is not split); with less, or NULL, the product runs unsplit (then bit-identical to
 * mi355_mul_mat_q8k_add, otherwise equal up to f32 summation order).  mi355_mul_mat uses whatever its own workspace holds beyond
 * mi355_mul_mat_ws_bytes(K, B) for this.  No counterpart in the reference (its CPU path splits rows over threads). */
size_t mi355_mul_mat_q8k_ws_bytes(int64_t N, int64_t K, int64_t B);
int mi355_mul_mat_q8k_ws(void *stream, int type, const void *W, const void *act, float *dst, const float *residual, int64_t N, int64_t K,
                         int64_t B, int64_t dst_stride, void *ws, size_t ws_bytes);

/* Second, unpacked copy of K-quant weights for the tile GEMM: the two int8 planes whose weighted sum R*hi + lo is the integer
 * sub-scale times the level (sc*n for Q4_K with R = 8, sc*(l-32) for Q6_K with R = 64; dequantize_row_q4_K / _q6_K,
 * ggml/src/ggml-quants.c:1280-1302, 1690-1719), 2 bytes per weight: int8 hi[rows][K], int8 lo[rows][K], then 48 bytes per
 * (row, super-block): the eight sub-block mins as f16, the same times 64 as f16, and {d, dmin} as f32 (Q6_K: only d).
 * Written once per weight matrix (K % 256 == 0, rows 16-byte aligned as for mi355_mul_mat_q8k); mi355_mul_mat_q8k_planes then
 * streams the planes straight into LDS and computes exactly what mi355_mul_mat_q8k_add computes (same integer sums, same f32
 * arithmetic, bit-identical dst) without touching the packed rows.  It pays for Q6_K, whose unpack costs the most vector
 * instructions per weight (about 1.35x the in-kernel-unpack rate at batch 512); for Q4_K the two run at the same speed, so
 * callers keep planes for Q6_K matrices only.  No counterpart in the reference, which unpacks in its mmq tile loaders
 * (ggml/src/ggml-cuda/mmq.cuh load_tiles_q6_K). */
size_t mi355_kq_planes_bytes(int64_t rows, int64_t K);
int mi355_kq_unpack_planes(void *stream, int type, const void *W, void *planes, int64_t rows, int64_t K);
int mi355_mul_mat_q8k_planes(void *stream, int type, const void *planes, const void *act, float *dst, const float *residual, int64_t N,
                             int64_t K, int64_t B, int64_t dst_stride);
/* ... with the split-along-K workspace of mi355_mul_mat_q8k_ws (same slices, so still bit-identical to it) */
int mi355_mul_mat_q8k_planes_ws(void *stream, int type, const void *planes, const void *act, float *dst, const float *residual, int64_t N,
                                int64_t K, int64_t B, int64_t dst_stride, void *ws, size_t ws_bytes);

/* Wide-tile form of the K-quant tile GEMM (128 weight rows x 128 activation rows per 512-thread group).  Both operands are
 * *tile images*: an int8 matrix cut into tiles of 16 rows x 64 elements = 1 KiB, stored [row block][k block], each tile byte
 * for byte what the kernel keeps in LDS, so that one wave-wide global-to-LDS transfer moves a tile.
 *   activations: mi355_quantize_act_q8k_tiled - same levels, scales and sub-block sums as mi355_quantize_act_q8k
 *                (quantize_row_q8_K_ref, ggml/src/ggml-quants.c:2479-2516), mi355_act_q8k_tiled_bytes(k, nrows) bytes;
 *   weights:     mi355_kq_unpack_tiles - the two int8 planes of mi355_kq_unpack_planes (dequantize_row_q4_K / _q6_K,
 *                ggml/src/ggml-quants.c:1280-1302, 1690-1719) plus per-super-block d, dmin and mins, written once per
 *                weight matrix, mi355_kq_tiles_bytes(type, rows, K) bytes (about 2 bytes per weight).  Also Q5_K
 *                (dequantize_row_q5_K, :1482-1507): sub-block scale times level 0..31 = 16 * hi + lo; and IQ4_XS
 *                (dequantize_row_iq4_xs, :2454-2475): (ls - 32) times the table value = 64 * hi + lo, no minima (the Q6_K form).
 * mi355_mul_mat_q8k_tiled computes what mi355_mul_mat_q8k_add computes (same integer sums: ggml_vec_dot_q4_K_q8_K /
 * ggml_vec_dot_q6_K_q8_K, ggml/src/ggml-cpu/ggml-cpu-quants.c:6817-6848, 8262-8283; f32 summation order may differ), and for
 * Q5_K / IQ4_XS the integer sums of ggml_vec_dot_q5_K_q8_K (:7539-7592) / ggml_vec_dot_iq4_xs_q8_K (:11381 ff.).
 * ws: optional workspace of mi355_mul_mat_q8k_tiled_ws_bytes(N, K, B) bytes for the split along K of products with few
 * tiles (NULL or too small: unsplit).  No counterpart in the reference (its CUDA backend unpacks in the tile loaders,
 * ggml/src/ggml-cuda/mmq.cuh). */
size_t mi355_act_q8k_tiled_bytes(int64_t k, int64_t nrows);
int mi355_quantize_act_q8k_tiled(void *stream, const float *x, void *act, int64_t k, int64_t nrows, int64_t x_stride);
size_t mi355_kq_tiles_bytes(int type, int64_t rows, int64_t K);
int mi355_kq_unpack_tiles(void *stream, int type, const void *W, void *tiles, int64_t rows, int64_t K);
size_t mi355_mul_mat_q8k_tiled_ws_bytes(int64_t N, int64_t K, int64_t B);
int mi355_mul_mat_q8k_tiled(void *stream, int type, const void *tiles, const void *act, float *dst, const float *residual, int64_t N,
                            int64_t K, int64_t B, int64_t dst_stride, void *ws, size_t ws_bytes);
/* The same product followed by the RMS norm of its rows: dst as above, then y[b] = rms_norm(dst[b]) * norm_w and act_out = the
 * tile image of y (mi355_act_q8k_tiled_bytes(N, B) bytes) - MUL_MAT(wo / ffn_down) -> ADD(residual) -> RMS_NORM -> MUL(norm weight)
 * of llm_build_kv / llm_build_ffn / the next layer's llm_build_norm (src/llama.cpp:1566, :1609, :175-198), whose readers are
 * K-quant products on tile images.  When the product is cut along K (few tiles: a 4096-row matrix at batch 512) the launch that adds
 * the slices and the residual also normalises and quantizes the row it has just formed; otherwise the norm is a launch of its own.
 * Same bits as mi355_mul_mat_q8k_tiled followed by mi355_rms_norm_mul_quant_q8k_tiled.  N a multiple of 256; y may be NULL. */
int mi355_mul_mat_q8k_tiled_norm(void *stream, int type, const void *tiles, const void *act, float *dst, const float *residual, int64_t N,
                                 int64_t K, int64_t B, int64_t dst_stride, void *ws, size_t ws_bytes, const float *norm_w, float eps, float *y,
                                 int64_t y_stride, void *act_out);
/* One launch for up to three matrices of the same K-quant type that consume the same activation image (gate and up of llm_build_ffn,
 * src/llama.cpp:280-320; Q, K and V of a layer where their types agree): their tiles fill the compute units together (gate + up at
 * batch 512: 896 tiles = 3.5 rounds on 256 compute units instead of two launches of 2 rounds; Q + K + V: 192 tiles in one round
 * instead of three launches cut along K and their three sum launches).  Each matrix computes exactly what
 * mi355_mul_mat_q8k_tiled computes for it alone without a workspace.  A single matrix is handled as by mi355_mul_mat_q8k_tiled
 * (ws: mi355_mul_mat_q8k_tiled_multi_ws_bytes(n_mats, Ns, K, B) bytes, 0 for more than one matrix).  residual: as above, per matrix. */
typedef struct mi355_tiled_mat {
    const void *tiles;      /* mi355_kq_unpack_tiles image of the matrix */
    float *dst;             /* [B][dst_stride] */
    const float *residual;  /* may be NULL; may be dst; same stride as dst */
    int64_t N;              /* rows of the matrix */
    int64_t dst_stride;     /* floats between two rows of dst, >= N */
} mi355_tiled_mat;
size_t mi355_mul_mat_q8k_tiled_multi_ws_bytes(int n_mats, const int64_t *Ns, int64_t K, int64_t B);
int mi355_mul_mat_q8k_tiled_multi(void *stream, int type, int n_mats, const mi355_tiled_mat *mats, const void *act, int64_t K, int64_t B,
                                  void *ws, size_t ws_bytes);
/* The same launch for matrices of different K-quant types (types[i] of mats[i]): llama-quantize's Q4_K_M mix gives attn_v and ffn_down
 * Q6_K in half of the layers (src/llama-quant.cpp:122-340), and a lone Q6_K V product is 32 tiles at batch 512 - cut along K and
 * summed by a second launch after the Q + K launch, or 32 more tiles inside that launch, which leaves compute units free.  The planes of
 * the three types differ only in the radix between them (8, 16, 64), taken per matrix; Q6_K images carry zero minima.  Every matrix
 * gets the bits of its own mi355_mul_mat_q8k_tiled launch without a workspace.  No split along K. */
int mi355_mul_mat_q8k_tiled_mixed(void *stream, int n_mats, const int *types, const mi355_tiled_mat *mats, const void *act, int64_t K, int64_t B);
/* Q, K and V of a prompt batch in that launch, with what llm_build_kv does to them next in its epilogue (src/llama.cpp:1514-1560:
 * ggml_rope_ext on Q and K, ggml_cpy of K and V into the f16 cache views): mats[0] = Q, dst = the rotated q, f32 [B][N_q]; mats[1] = K
 * and mats[2] = V, dst = base of the f16 cache, element (cell, head, d) at cells[b] * nb1 + head * nb2 + 2 * d (dst_stride unused).
 * ROPE in its adjacent-pair mode (mode 0, ggml_compute_forward_rope_f32, ggml/src/ggml-cpu/ggml-cpu.c:9390-9470): the two elements of
 * a pair are neighbouring rows of the matrix, hence neighbouring lanes of the result.  rope_table: {cos, sin} per (token, pair), T x D/2
 * float pairs written by mi355_rope_table once per batch (positions and frequencies do not depend on the layer).  Same bits as
 * mi355_mul_mat_q8k_tiled_mixed followed by mi355_rope_kv_store.  N_q, N_k = N_v multiples of D; no residual. */
int mi355_rope_table(void *stream, const int32_t *pos, const float *freq_factors, float *table, int64_t T, int64_t D, int n_dims, int n_ctx_orig,
                     float freq_base, float freq_scale, float ext_factor, float attn_factor, float beta_fast, float beta_slow);
int mi355_mul_mat_q8k_tiled_qkv_rope(void *stream, const int *types, const mi355_tiled_mat *mats, const void *act, int64_t K, int64_t B,
                                     const float *rope_table, const int32_t *cells, int64_t D, int n_dims, size_t k_nb1, size_t k_nb2, size_t v_nb1,
                                     size_t v_nb2);

/* Up to four weight matrices that consume the same quantized activation (the Q/K/V and the
 * gate/up projections of llm_build_kv / llm_build_ffn, src/llama.cpp:1514-1533, :200-330) in ONE
 * launch, each optionally adding a residual in its epilogue (the ggml_add that follows the wo and
 * ffn_down products, src/llama.cpp:1566, :1609): dst_i[b][n] = W_i[n] . x[b] (+ residual_i[b][n]).
 * residual has dst's shape and stride and may alias dst.  B <= 8; up to 32 where every matrix qualifies for
 * mi355_mul_mat_skinny, which this call then uses from five activation rows on (one launch per matrix). */
typedef struct mi355_gemv_mat {
    int          type;        /* weight type of this matrix */
    const void  *W;           /* N rows x K, device layout */
    int64_t      N;
    float       *dst;
    int64_t      dst_stride;
    const float *residual;    /* NULL for none */
} mi355_gemv_mat;
int mi355_mul_mat_vec_q_multi(void *stream, int n_mats, const mi355_gemv_mat *mats, const void *act, int64_t K, int64_t B);
/* mi355_mul_mat_mid for up to three matrices of the type that share the activation image (Q, K and V; gate and up of
 * llm_build_kv / llm_build_ffn, src/llama.cpp:1514-1533, :280-320) as one launch: their 32-row tiles fill the compute units together and
 * the small ones (1024 rows: 32 groups) do not pay a launch and a slice-sum launch of their own.  The slices along K are chosen for the
 * launch as a whole; ws of mi355_mul_mat_mid_multi_ws_bytes(n_mats, Ns, K, B) bytes (NULL / less: one slice).  Every matrix gets the
 * integer sums of its own mi355_mul_mat_mid call (f32 summation order follows the number of slices). */
/* mi355_mul_mat_mid followed by the RMS norm of its rows, as mi355_mul_mat_q8k_tiled_norm does for the wide-tile GEMM (same operands,
 * same bits as the product followed by mi355_rms_norm_mul_quant_q8k_tiled; the launch that adds a cut product's slices carries the
 * norm).  ws: mi355_mul_mat_mid_ws_bytes(N, K, B). */
int mi355_mul_mat_mid_norm(void *stream, int type, const void *W, const void *act, float *dst, const float *residual, int64_t N, int64_t K, int64_t B,
                           int64_t dst_stride, void *ws, size_t ws_bytes, const float *norm_w, float eps, float *y, int64_t y_stride, void *act_out);
size_t mi355_mul_mat_mid_multi_ws_bytes(int n_mats, const int64_t *Ns, int64_t K, int64_t B);
int mi355_mul_mat_mid_multi(void *stream, int type, int n_mats, const mi355_gemv_mat *mats, const void *act, int64_t K, int64_t B, void *ws,
                            size_t ws_bytes);

/* Integer sub-block dots, for parity checking the kernels' inner products bit-for-bit
 * against ggml_vec_dot_q4_0_q8_0 / q8_0_q8_0 / q4_K_q8_K / q5_K_q8_K / q6_K_q8_K
 * (ggml/src/ggml-cpu/ggml-cpu-quants.c:2492-2506, 3919-3927, 6817-6848, 7539-7592, 8262-8283).
 * a: ONE activation row in the split layout written by mi355_quantize_act (the same bytes
 * the GEMV reads).  out: int32 [N][k/g], g = 32 (16 for Q6_K); the weight level has its
 * fixed offset removed (Q4_0: nibble-8, Q6_K: q-32, Q4_K: nibble, Q5_K: level 0..31). */
int mi355_block_dots_q8_1(void *stream, int type, const void *W, const void *a, int32_t *out, int64_t N, int64_t K);

/* MUL_MAT_ID ------------------------------------------------------------------------ *
 * ggml_compute_forward_mul_mat_id (ggml/src/ggml-cpu/ggml-cpu.c:7717-7895; semantics
 * ggml/src/ggml.c:2723-2759): as = n_expert matrices of N rows x K in device layout, back
 * to back; b f32 [K, nb1, T] contiguous; ids int32, element (e,t) at ids[t*ids_stride + e];
 * dst f32 [N, n_used, T] contiguous.  dst[:,e,t] = as[ids[e,t]] . b[:, e % nb1, t].
 * Expert bucketing is done on the device (no host synchronisation).
 * ws: at least mi355_mul_mat_id_ws_bytes(...) bytes. */
size_t mi355_mul_mat_id_ws_bytes(int64_t K, int64_t n_expert, int64_t n_used, int64_t nb1, int64_t T);
int mi355_mul_mat_id(void *stream, int type, const void *as, const float *b, const int32_t *ids, int64_t ids_stride,
                     float *dst, int64_t N, int64_t K, int64_t n_expert, int64_t n_used, int64_t nb1, int64_t T,
                     void *ws, size_t ws_bytes);

/* mi355_mul_mat_id for many (token, expert slot) pairs and Q4_K / Q5_K / Q6_K / IQ4_XS experts: the slots are sorted by expert on the
 * device (the row grouping of ggml_compute_forward_mul_mat_id, ggml/src/ggml-cpu/ggml-cpu.c:7805-7820, mmid_row_mapping
 * :7639-7644) and one tile launch walks all experts, so every expert's matrix is read once.  `act` holds the nb1*T rows
 * of b in the mi355_quantize_act_q8k layout; route_ws: at least mi355_mul_mat_id_q8k_route_bytes(...) bytes, 16-byte
 * aligned.  At most 256 experts; mi355_mul_mat_id picks this path from 32 slots on. */
size_t mi355_mul_mat_id_q8k_route_bytes(int64_t n_expert, int64_t n_used, int64_t T);
int mi355_mul_mat_id_q8k(void *stream, int type, const void *as, const void *act, const int32_t *ids, int64_t ids_stride, float *dst,
                         int64_t N, int64_t K, int64_t n_expert, int64_t n_used, int64_t nb1, int64_t T, void *route_ws,
                         size_t route_ws_bytes);

/* The same for experts of the per-32-block types (Q4_0, Q4_1, Q5_0, Q5_1, IQ4_NL, Q8_0): the routed form of mi355_mul_mat_q's tile
 * kernel on 128-slot column tiles.  `act` holds the nb1*T rows of b in the mi355_quantize_act (Q8_1) layout; route_ws as above.
 * K a multiple of 128, expert rows 16-byte aligned, at most 256 experts (mi355_mul_mat_id_q_supported); mi355_mul_mat_id picks
 * this path from 32 slots on. */
int mi355_mul_mat_id_q_supported(int type, const void *as, int64_t N, int64_t K, int64_t n_expert);
int mi355_mul_mat_id_q(void *stream, int type, const void *as, const void *act, const int32_t *ids, int64_t ids_stride, float *dst,
                       int64_t N, int64_t K, int64_t n_expert, int64_t n_used, int64_t nb1, int64_t T, void *route_ws,
                       size_t route_ws_bytes);

/* MUL_MAT_ID with many slots on the wide-tile kernel (ggml_compute_forward_mul_mat_id, ggml-cpu.c:7717-7895; K-quants only).
 * expert_tiles: the experts' tile images (mi355_kq_unpack_tiles of each expert's N x K matrix), expert e at
 * expert_tiles + e * expert_tiles_bytes.  b: the f32 activations [T][nb1][K] (16-byte aligned, rows K apart); they are
 * quantized per 256 elements like mi355_quantize_act_q8k, gathered in expert order into one image with 128 rows per column tile.
 * dst f32 [T][n_used][N].  ws: mi355_mul_mat_id_q8k_tiled_ws_bytes(...) bytes, 16-byte aligned.  Results equal those of
 * mi355_mul_mat_q8k_tiled on each expert's rows. */
size_t mi355_mul_mat_id_q8k_tiled_ws_bytes(int64_t K, int64_t n_expert, int64_t n_used, int64_t T);
int mi355_mul_mat_id_q8k_tiled(void *stream, int type, const void *expert_tiles, size_t expert_tiles_bytes, const float *b, const int32_t *ids,
                               int64_t ids_stride, float *dst, int64_t N, int64_t K, int64_t n_expert, int64_t n_used, int64_t nb1, int64_t T,
                               void *ws, size_t ws_bytes);

/* Second half of mi355_mul_mat_id: `act` holds the nb1*T rows of b quantized by
 * mi355_quantize_act (row t*nb1 + j). */
int mi355_mul_mat_id_vec(void *stream, int type, const void *as, const void *act, const int32_t *ids, int64_t ids_stride,
                         float *dst, int64_t N, int64_t K, int64_t n_expert, int64_t n_used, int64_t nb1, int64_t T);

/* FLASH_ATTN_EXT -------------------------------------------------------------------- *
 * ggml_compute_forward_flash_attn_ext_f16 (ggml/src/ggml-cpu/ggml-cpu.c:10916-11129).
 * q f32 [D, Nq, Hq] with byte strides q_nb1 (query) and q_nb2 (head); k, v f16
 * [D, Nkv, Hkv] with byte strides *_nb1 (kv cell) and *_nb2 (kv head); mask f16
 * [Nkv, >=Nq] contiguous rows of mask_nb1 bytes, or NULL; dst f32 [D, Hq, Nq]
 * contiguous.  Hq % Hkv == 0 (grouped-query).  -inf mask entries are skipped.
 * D must be 64, 80, 96, 112, 128 or 256.  ws: mi355_flash_attn_ws_bytes(...) bytes. */
size_t mi355_flash_attn_ws_bytes(int64_t D, int64_t Nq, int64_t Nkv, int64_t Hq);
int mi355_flash_attn_ext(void *stream, const float *q, const void *k, const void *v, const void *mask, float *dst,
                         int64_t D, int64_t Nq, int64_t Nkv, int64_t Hq, int64_t Hkv, size_t q_nb1, size_t q_nb2,
                         size_t k_nb1, size_t k_nb2, size_t v_nb1, size_t v_nb2, size_t mask_nb1, float scale,
                         float max_bias, float logit_softcap, void *ws, size_t ws_bytes);

/* Same, and also writes the Q8_1 quantization of dst (one activation row of Hq*D elements per
 * query, layout of mi355_quantize_act) for the attention-output projection that follows it in
 * llm_build_kv (src/llama.cpp:157-199), saving that MUL_MAT's separate quantization pass.
 * act may be NULL; D % 32 == 0 is required otherwise. */
int mi355_flash_attn_ext_quant(void *stream, const float *q, const void *k, const void *v, const void *mask, float *dst,
                         int64_t D, int64_t Nq, int64_t Nkv, int64_t Hq, int64_t Hkv, size_t q_nb1, size_t q_nb2,
                         size_t k_nb1, size_t k_nb2, size_t v_nb1, size_t v_nb2, size_t mask_nb1, float scale,
                         float max_bias, float logit_softcap, void *ws, size_t ws_bytes, void *act);

/* Glue operators -------------------------------------------------------------------- *
 * A strided f32/f16/i32 operand: up to 4 dimensions, ne[] elements, nb[] byte strides
 * (the fields of struct ggml_tensor, ggml/include/ggml.h:576-608). */
typedef struct mi355_tensor {
    void   *data;
    int     type;
    int64_t ne[4];
    size_t  nb[4];
} mi355_tensor;

/* ggml_compute_forward_rms_norm_f32 (ggml-cpu.c:7015-7061); rows along ne[0], row strides honoured */
int mi355_rms_norm(void *stream, const mi355_tensor *src, const mi355_tensor *dst, float eps);
/* ggml_compute_forward_{add,sub,mul,div}_f32 (ggml-cpu.c:4067-4140, 5142-5305): src1 broadcast over src0. op: 0 add 1 sub 2 mul 3 div */
int mi355_bin_bcast(void *stream, int op, const mi355_tensor *src0, const mi355_tensor *src1, const mi355_tensor *dst);
/* ggml_compute_forward_unary (ggml-cpu.c:6646-6683 for silu).  op: ggml_unary_op value
 * (ggml/include/ggml.h:530-547); supported: ABS SGN NEG STEP TANH ELU RELU SIGMOID GELU GELU_QUICK SILU HARDSWISH HARDSIGMOID EXP */
int mi355_unary(void *stream, int op, const mi355_tensor *src, const mi355_tensor *dst);
/* ggml_compute_forward_scale_f32 (ggml-cpu.c:8158) */
int mi355_scale(void *stream, const mi355_tensor *src, const mi355_tensor *dst, float s);
/* ggml_compute_forward_dup (CPY/CONT/DUP, ggml-cpu.c:3519-3830): f32<->f16, f32->f32, f16->f16, i32->i32; any strides, same element count */
int mi355_cpy(void *stream, const mi355_tensor *src, const mi355_tensor *dst);
/* KV-cache store: dst[:, rows[i], j] = convert(src[:, i, j]); src f32 [ne0, n, ne2], rows int32 [n] in DEVICE memory,
 * dst f32/f16 [ne0, *, ne2].  Same result as the CPY into a view of the cache at row kv_head that llm_build_kv_store
 * emits (src/llama.cpp:157-199; ggml_compute_forward_dup_f32, ggml-cpu.c:3519-3830), with the row taken from device
 * memory so that a captured launch sequence does not change as the cache fills. */
int mi355_set_rows(void *stream, const mi355_tensor *src, const int32_t *rows, const mi355_tensor *dst);
/* ggml_compute_forward_get_rows (ggml-cpu.c:8464-8590): src f32/f16 rows, or whole quantized rows (Q4_0, Q4_1, Q5_0, Q5_1, IQ4_NL, IQ4_XS, Q8_0, Q4_K, Q5_K, Q6_K in the
 * device row layout, nb[1] = row bytes; dequantize_row_*, ggml-quants.c:255-273, 349-363, 1280-1302, 1482-1507, 1690-1719), ids i32
 * [n, b2, b3]; dst f32 */
int mi355_get_rows(void *stream, const mi355_tensor *src, const mi355_tensor *ids, const mi355_tensor *dst);
/* ggml_compute_forward_soft_max_f32 (ggml-cpu.c:8959-9055): mask f32 or f16 or NULL */
int mi355_soft_max(void *stream, const mi355_tensor *src, const mi355_tensor *mask, const mi355_tensor *dst, float scale,
                   float max_bias);
/* ggml_compute_forward_rope_f32 (ggml-cpu.c:9366-9549): mode 0 (adjacent pairs) and 2 (NeoX); pos i32 [ne2]; freq_factors f32 or NULL */
int mi355_rope(void *stream, const mi355_tensor *src, const int32_t *pos, const float *freq_factors,
               const mi355_tensor *dst, int n_dims, int mode, int n_ctx_orig, float freq_base, float freq_scale,
               float ext_factor, float attn_factor, float beta_fast, float beta_slow);
/* ggml_compute_forward_sum_rows_f32 (ggml-cpu.c:5678) */
int mi355_sum_rows(void *stream, const mi355_tensor *src, const mi355_tensor *dst);
/* ggml_compute_forward_argsort_f32 (ggml-cpu.c:10857): order 0 ascending, 1 descending; ne[0] <= 1024 */
int mi355_argsort(void *stream, const mi355_tensor *src, const mi355_tensor *dst, int order);
/* Fused node sequences --------------------------------------------------------------- *
 * Each does the work of the consecutive graph nodes named, with the same arithmetic; where the
 * consumer is a quantized MUL_MAT the Q8_1 activation (split layout of mi355_quantize_act,
 * quantize_row_q8_1_ref arithmetic) is produced in the same pass.  y and act are optional (NULL). */

/* llm_build_norm: RMS_NORM then MUL by the norm weight (src/llama.cpp:1499-1503; ggml-cpu.c:7015-7061, 5142-5211).
 * x f32 rows of k (row stride x_stride elements), w f32 [k] or NULL, y f32 rows (y_stride). k <= 16384. */
int mi355_rms_norm_mul_quant(void *stream, const float *x, int64_t x_stride, const float *w, float *y, int64_t y_stride,
                             void *act, int64_t k, int64_t nrows, float eps);
/* The same for the FFN norm of a mixture-of-experts layer, continued with the router of llm_build_moe_ffn (src/llama.cpp:438-468):
 * logits f32 [nrows][n_expert] = MUL_MAT(W f32 [n_expert] rows of k, stride w_stride elements; y), probs = SOFT_MAX(logits), order i32
 * [nrows][n_expert] = ARGSORT(descending).  Same bits as mi355_rms_norm_mul_quant, mi355_mul_mat_f and mi355_moe_route one after the
 * other.  k <= 4096, a few rows, n_expert <= 64; W 16-byte aligned. */
int mi355_rms_norm_mul_quant_router(void *stream, const float *x, int64_t x_stride, const float *w, float *y, int64_t y_stride, void *act, int64_t k,
                                    int64_t nrows, float eps, const float *W, int64_t w_stride, float *logits, float *probs, int32_t *order,
                                    int64_t n_expert);
/* llm_build_ffn LLM_FFN_SILU + LLM_FFN_PAR: UNARY(SILU)(gate) then MUL by up (src/llama.cpp:280-320; ggml-cpu.c:6646-6683). */
int mi355_swiglu_quant(void *stream, const float *gate, const float *up, int64_t in_stride, float *y, int64_t y_stride, void *act,
                       int64_t k, int64_t nrows);
/* The two sequences above with `act` in the per-super-block layout of mi355_quantize_act_q8k (what the K-quant tile GEMM reads);
 * k must be a multiple of 256.  Same levels, scales and sums as quantizing y with mi355_quantize_act_q8k. */
int mi355_rms_norm_mul_quant_q8k(void *stream, const float *x, int64_t x_stride, const float *w, float *y, int64_t y_stride,
                                 void *act, int64_t k, int64_t nrows, float eps);
int mi355_swiglu_quant_q8k(void *stream, const float *gate, const float *up, int64_t in_stride, float *y, int64_t y_stride, void *act,
                           int64_t k, int64_t nrows);
/* ... and with `act` as the tile images of mi355_quantize_act_q8k_tiled (what mi355_mul_mat_q8k_tiled reads) */
int mi355_rms_norm_mul_quant_q8k_tiled(void *stream, const float *x, int64_t x_stride, const float *w, float *y, int64_t y_stride,
                                       void *act, int64_t k, int64_t nrows, float eps);
int mi355_swiglu_quant_q8k_tiled(void *stream, const float *gate, const float *up, int64_t in_stride, float *y, int64_t y_stride, void *act,
                                 int64_t k, int64_t nrows);
/* ROPE(q), ROPE(k), CPY(k -> K cache), CPY(v -> V cache) of build_llama + llm_build_kv_store (src/llama.cpp:1535-1548, :157-199;
 * ggml-cpu.c:9366-9549, 3519-3830).  q f32 [T][H][D] is rotated in place; k, v f32 [T][HK][D] are read; the f16 caches are addressed
 * as cell*nb1 + head*nb2 + 2*d with the cell of token t taken from cells[t] and its rope position from pos[t] (both DEVICE int32). */
int mi355_rope_kv_store(void *stream, float *q, const float *k, const float *v, void *kcache, void *vcache, const int32_t *pos,
                        const int32_t *cells, const float *freq_factors, int64_t T, int64_t H, int64_t HK, int64_t D, size_t k_nb1,
                        size_t k_nb2, size_t v_nb1, size_t v_nb2, int n_dims, int mode, int n_ctx_orig, float freq_base, float freq_scale,
                        float ext_factor, float attn_factor, float beta_fast, float beta_slow);
/* The same launch with typed caches (what llm_build_kv_store builds with -ctk / -ctv q8_0, q4_0: CPY f32 -> Q8_0 / Q4_0,
 * ggml_compute_forward_dup_f32, ggml-cpu.c:3519-3830, via quantize_row_q8_0_ref / quantize_row_q4_0_ref, ggml-quants.c:194-218, 39-72;
 * bit-identical to mi355_cpy_f32_quant of the rotated rows).  For an f16 cache (type MI355_F16) kcache / k_a / k_b are the view's
 * data, nb1 and nb2 as above; for MI355_Q8_0 / MI355_Q4_0 kcache is the data of the tensor that owns the cache memory, k_a the
 * index (blocks of 32, plain ggml addressing) of cell 0's first block within it and k_b its blocks per row in the device row
 * layout (0: plain ggml blocks); token t's rows go to blocks k_a + cells[t] * HK * D / 32 ...  Likewise for V.  A quantized
 * cache takes mode 0 (adjacent pairs) and D % 32 == 0. */
int mi355_rope_kv_store_typed(void *stream, float *q, const float *k, const float *v, int type_k, void *kcache, int64_t k_a, int64_t k_b, int type_v,
                              void *vcache, int64_t v_a, int64_t v_b, const int32_t *pos, const int32_t *cells, const float *freq_factors, int64_t T,
                              int64_t H, int64_t HK, int64_t D, int n_dims, int mode, int n_ctx_orig, float freq_base, float freq_scale,
                              float ext_factor, float attn_factor, float beta_fast, float beta_slow);
/* Up to three weight matrices on one quantized activation whose finished rows go through the nodes that follow the projections in
 * build_llama (src/llama.cpp:1514-1548; llm_build_kv_store :157-199): ROPE (ggml-cpu.c:9366-9549, adjacent-pair mode only) and / or
 * CPY to an f16 tensor such as a KV-cache view (ggml-cpu.c:3519-3830).  A wave owns output rows 2i and 2i+1, i.e. one rotation pair.
 *   MI355_EPI_STORE       dst f32 [B][dst_stride]                          plain product
 *   MI355_EPI_ROPE        dst f32 [B][dst_stride], rows = [head][head_dim]  rotated by pos[b]
 *   MI355_EPI_ROPE_CACHE  dst f16 at cells[b]*nb1 + head*nb2 + 2*d          rotated, then converted
 *   MI355_EPI_CACHE       dst f16 at cells[b]*nb1 + head*nb2 + 2*d          converted
 *   MI355_EPI_ROPE_QCACHE / MI355_EPI_QCACHE   the same two with a Q8_0 / Q4_0 destination (CPY f32 -> quantized, ggml_compute_forward_dup_f32, ggml-cpu.c:3519-3830, via
 *                         quantize_row_q8_0_ref / quantize_row_q4_0_ref, ggml-quants.c:194-218, 39-72; bit-identical to
 *                         mi355_cpy_f32_quant of the rotated row): dst = data of the tensor that owns the cache memory, dst_stride =
 *                         MI355_Q8_0 or MI355_Q4_0, nb1 = index (in blocks of 32, plain ggml addressing) of cell 0's first block
 *                         within that tensor, nb2 = the owner's blocks per row when it is kept in the device row layout (0: plain
 *                         ggml blocks); row b of the product becomes blocks nb1 + cells[b]*N/32 ... of the owner.  N % 32 == 0.
 * pos / cells: DEVICE int32 [B].  B <= 4; 16-byte aligned weight rows. */
enum { MI355_EPI_STORE = 0, MI355_EPI_ROPE = 1, MI355_EPI_ROPE_CACHE = 2, MI355_EPI_CACHE = 3, MI355_EPI_ROPE_QCACHE = 4, MI355_EPI_QCACHE = 5 };
typedef struct mi355_gemv_rope_mat {
    int          type;
    const void  *W;           /* N rows x K, device layout */
    int64_t      N;           /* a whole number of heads unless the epilogue is MI355_EPI_STORE */
    int          epilogue;
    void        *dst;
    int64_t      dst_stride;  /* f32 elements between activation rows (STORE, ROPE); the cache type (ROPE_QCACHE, QCACHE) */
    int64_t      nb1, nb2;    /* bytes per cell and per head (ROPE_CACHE, CACHE); first block and blocks per row (ROPE_QCACHE, QCACHE) */
} mi355_gemv_rope_mat;
typedef struct mi355_rope_desc {
    const int32_t *pos;
    const int32_t *cells;
    const float   *freq_factors;   /* [n_dims/2] or NULL */
    int64_t        head_dim;
    int            n_dims, mode, n_ctx_orig;
    float          freq_base, freq_scale, ext_factor, attn_factor, beta_fast, beta_slow;
} mi355_rope_desc;
int mi355_mul_mat_vec_q_rope(void *stream, int n_mats, const mi355_gemv_rope_mat *mats, const void *act, int64_t K, int64_t B,
                             const mi355_rope_desc *rope);

/* The same launch for ONE activation row that is still to be normalised: RMS_NORM(x) -> MUL(norm_w) -> Q8_1 (llm_build_norm,
 * src/llama.cpp:1506-1511; ggml-cpu.c:6741-6805) done by every group for itself, then the products and epilogues of
 * mi355_mul_mat_vec_q_rope.  Bit-identical to mi355_rms_norm_mul_quant followed by mi355_mul_mat_vec_q_rope; neither the
 * normalised f32 row nor its Q8_1 form is written to memory.  K <= 4096 and a multiple of 1024; x, norm_w 16-byte aligned. */
int mi355_rms_norm_mul_mat_vec_q_rope(void *stream, const float *x, const float *norm_w, float eps, int n_mats, const mi355_gemv_rope_mat *mats,
                                      int64_t K, const mi355_rope_desc *rope);

/* The Q, K and V projections of build_llama (src/llama.cpp:1514-1533) in ONE bandwidth-bound launch whose epilogue does what the graph
 * does next: ROPE(q) into q f32 [B][H][D]; ROPE(k) and CPY into the f16 K cache; CPY(v) into the f16 V cache (src/llama.cpp:1535-1548,
 * llm_build_kv_store :157-199; ggml-cpu.c:9366-9549, 3519-3830).  wq/wk/wv: device-layout rows of K (16-byte aligned rows required);
 * act from mi355_quantize_act / mi355_rms_norm_mul_quant (B <= 4 rows).  Cache addressing and pos/cells as in mi355_rope_kv_store.
 * Only the adjacent-pair rope mode (mode 0) is fused: a wave owns output rows 2i and 2i+1. */
int mi355_qkv_rope_store(void *stream, int type_q, const void *wq, int type_k, const void *wk, int type_v, const void *wv, const void *act,
                         float *q, void *kcache, void *vcache, const int32_t *pos, const int32_t *cells, const float *freq_factors,
                         int64_t K, int64_t B, int64_t H, int64_t HK, int64_t D, size_t k_nb1, size_t k_nb2, size_t v_nb1, size_t v_nb2,
                         int n_dims, int mode, int n_ctx_orig, float freq_base, float freq_scale, float ext_factor, float attn_factor,
                         float beta_fast, float beta_slow);

/* The same for ONE activation row, with the RMS_NORM -> MUL(norm weights) -> Q8_1 that precedes the projections in build_llama
 * (llm_build_norm, src/llama.cpp:1506-1511; ggml_compute_forward_rms_norm_f32, ggml-cpu.c:6741-6805) done by every group for
 * itself into its LDS copy of the activation: one launch less per decoded token and layer, bit-identical to
 * mi355_rms_norm_mul_quant followed by mi355_qkv_rope_store.  x: the f32 layer input (K elements), K <= 4096 and a multiple of
 * 1024; x and norm_w 16-byte aligned. */
int mi355_rms_norm_qkv_rope_store(void *stream, const float *x, const float *norm_w, float eps, int type_q, const void *wq, int type_k,
                                  const void *wk, int type_v, const void *wv, float *q, void *kcache, void *vcache, const int32_t *pos,
                                  const int32_t *cells, const float *freq_factors, int64_t K, int64_t H, int64_t HK, int64_t D, size_t k_nb1,
                                  size_t k_nb2, size_t v_nb1, size_t v_nb2, int n_dims, int mode, int n_ctx_orig, float freq_base,
                                  float freq_scale, float ext_factor, float attn_factor, float beta_fast, float beta_slow);

/* The gate and up projections of llm_build_ffn (LLM_FFN_SILU, LLM_FFN_PAR; src/llama.cpp:280-320) in ONE bandwidth-bound launch that
 * also performs UNARY(SILU)(gate), MUL by up and the Q8_1 quantization the ffn_down product needs (ggml-cpu.c:6646-6683, 5142-5211;
 * quantize_row_q8_1_ref).  gate/up: f32 [B][out_stride] receive the raw products; act_out: mi355_quantize_act layout of B rows of N.
 * counters: N/32 zero-initialised DEVICE words that the launch leaves zero (the group that completes a 32-row block finishes it).
 * B <= 4, N % 32 == 0, 16-byte aligned weight rows. */
int mi355_ffn_gate_up_swiglu(void *stream, int type_gate, const void *w_gate, int type_up, const void *w_up, const void *act, float *gate,
                             float *up, int64_t out_stride, void *act_out, unsigned *counters, int64_t N, int64_t K, int64_t B);

/* The same for the experts of a mixture-of-experts layer (llm_build_moe_ffn, src/llama.cpp:417-538): MUL_MAT_ID(up experts),
 * MUL_MAT_ID(gate experts), UNARY(SILU), MUL and the Q8_1 rows the MUL_MAT_ID of the down experts reads, in one launch
 * (ggml_compute_forward_mul_mat_id, ggml-cpu.c:7717-7894, per slot as mi355_mul_mat_id_vec; same bits as that call twice followed by
 * mi355_swiglu_quant).  as_gate / as_up: n_expert stacked matrices of N rows in the device layout, both of `type`; act: the
 * mi355_quantize_act form of src1 (nb1 * T rows of K); slot t * n_used + e reads expert ids[t * ids_stride + e] and activation row
 * t * nb1 + e % nb1.  gate / up: f32 [T * n_used][N], the raw products; act_out: mi355_quantize_act layout of T * n_used rows of N.
 * N % 32 == 0, K % 64 == 0, 16-byte aligned weight rows. */
int mi355_moe_gate_up_swiglu(void *stream, int type, const void *as_gate, const void *as_up, const void *act, const int32_t *ids, int64_t ids_stride,
                             float *gate, float *up, void *act_out, int64_t N, int64_t K, int64_t n_expert, int64_t n_used, int64_t nb1, int64_t T);
/* 1 when mi355_moe_gate_up_swiglu takes these expert stacks (the shape limits above and 16-byte aligned rows), else 0; no counterpart
 * in the reference (a caller's pre-check, like ggml_backend_dev_supports_op for one launch form). */
int mi355_moe_gate_up_swiglu_supported(int type, const void *as_gate, const void *as_up, int64_t N, int64_t K);



/* Quantized KV cache (llama.cpp's -ctk / -ctv q8_0, q4_0).
 * Where a block lives: with row_blocks = 0 blocks sit where ggml puts them (block g of a tensor at g * block bytes from its data).
 * A tensor kept in the device row layout of mi355_weights_scatter (all levels of a row, then the row's scales) is addressed through
 * the tensor that owns the memory: `base` = its data, row_blocks = blocks per row of THAT tensor; block g is then block
 * g % row_blocks of row g / row_blocks, whatever view (1-D for the store, [D, cells, heads] for attention) is in use.
 * cpy_f32_quant: CPY of contiguous f32 into n/32 consecutive Q8_0 / Q4_0 blocks starting at block dst_first_block - what
 *   llm_build_kv_store (src/llama.cpp:157-199) does to k_cur / v_cur; the bytes of quantize_row_q8_0_ref / quantize_row_q4_0_ref
 *   (ggml/src/ggml-quants.c:39-72, 194-218; ggml-cpu.c:3519-3830 converts row by row with the type's from_float).
 * flash_attn_ext_kv: mi355_flash_attn_ext_quant over K and V of type MI355_F16, MI355_Q8_0 or MI355_Q4_0 each (ggml-cpu.c:10997-11003,
 *   11040-11099).  k / v point at the first row in plain ggml addressing (row of (cell, head) at cell * nb1 + head * nb2); k_base /
 *   v_base = data of the owning tensor (NULL: k / v themselves).  Quantized rows are expanded to f16 (d * level) in an image at the
 *   end of the workspace and the f16 kernels run on the image; the reference instead quantizes q to Q8_0 and takes integer dots,
 *   so results agree to the tolerance of the op (NMSE 5e-4), not to the bit.  ws: 256-byte aligned, at least
 *   mi355_flash_attn_kv_ws_bytes.  D % 32 == 0. */
int mi355_cpy_f32_quant(void *stream, int type, const float *src, void *dst_base, int64_t dst_first_block, int64_t dst_row_blocks, int64_t n);
/* CPY between contiguous f32 rows and a VIEW of a Q8_0 / Q4_0 tensor whose rows start on block boundaries, in either direction: what
 * the K-shift of a quantized cache does around its ROPE (llama_kv_cache_unified::build_rope_shift, src/llama-kv-cache.cpp: ggml_cast
 * of the [head_dim, heads, cells] view of the cache to f32, ggml_rope_ext_inplace, ggml_cpy back; ggml-cpu.c:3519-3830 with the
 * type's to_float / from_float).  f32: ne[0] x ne[1] x ne[2] x ne[3] contiguous floats; element (i0, i1, i2, i3) lies in block
 * q_first_block + i0 / 32 + i1 * stride_blocks[0] + i2 * stride_blocks[1] + i3 * stride_blocks[2] of the tensor that owns the
 * memory (q_base, q_row_blocks as in mi355_cpy_f32_quant).  to_f32 = 1 dequantizes (dequantize_row_q8_0 / q4_0), 0 quantizes
 * (quantize_row_q8_0_ref / q4_0_ref).  ne[0] % 32 == 0. */
/* CPY of n_blocks consecutive blocks (in plain ggml addressing) of a Q8_0 / Q4_0 tensor to consecutive blocks of another tensor of
 * the same type - the row copies of build_defrag (src/llama.cpp:1215-1300) on a quantized cache; base / first_block / row_blocks
 * per side as in mi355_cpy_f32_quant. */
int mi355_cpy_quant_blocks(void *stream, int type, const void *src_base, int64_t src_first_block, int64_t src_row_blocks, void *dst_base,
                           int64_t dst_first_block, int64_t dst_row_blocks, int64_t n_blocks);
int mi355_cpy_quant_view(void *stream, int type, int to_f32, float *f32, void *q_base, int64_t q_first_block, int64_t q_row_blocks, const int64_t *ne,
                         const int64_t *stride_blocks);
size_t mi355_flash_attn_kv_ws_bytes(int64_t D, int64_t Nq, int64_t Nkv, int64_t Hq, int64_t Hkv, int type_k, int type_v);
int mi355_flash_attn_ext_kv(void *stream, const float *q, const void *k, int type_k, const void *k_base, int64_t k_row_blocks, const void *v,
                            int type_v, const void *v_base, int64_t v_row_blocks, const void *mask, float *dst, int64_t D, int64_t Nq, int64_t Nkv,
                            int64_t Hq, int64_t Hkv, size_t q_nb1, size_t q_nb2, size_t k_nb1, size_t k_nb2, size_t v_nb1, size_t v_nb2,
                            size_t mask_nb1, float scale, float max_bias, float logit_softcap, void *ws, size_t ws_bytes, void *act);

/* Mixture-of-experts glue of llm_build_moe_ffn (src/llama.cpp:417-530), each call the work of the consecutive graph nodes named,
 * writing every tensor those nodes write, bit-identical to running them one by one.  All operands contiguous.
 * moe_route: SOFT_MAX (no mask, scale 1) then ARGSORT descending: logits f32 [T][n_expert] -> probs f32, order i32 (ties by index;
 *   ggml-cpu.c:8959-9055, 10857).  n_expert <= 64.
 * moe_weights: GET_ROWS of the selected experts' probabilities, SUM_ROWS, DIV (ggml-cpu.c:8590, 5678, 5236-5305):
 *   ids i32 [T][ids_stride] (first n_used of each row) -> raw f32 [T][n_used], sum f32 [T], norm f32 [T][n_used].
 * moe_combine: MUL by the weights, the ADD chain over the expert slots and optionally the residual ADD that follows
 *   (ggml-cpu.c:5142-5211, 4067-4140): experts f32 [T][n_used][n_embd], weights f32 [T][n_used] -> scaled (same shape, may be
 *   NULL when nothing else reads it), out f32 [T][n_embd] = sum_e scaled[t][e] (+ residual[t]). */
int mi355_moe_route(void *stream, const float *logits, float *probs, int32_t *order, int64_t n_expert, int64_t T);
int mi355_moe_weights(void *stream, const float *probs, const int32_t *ids, int64_t ids_stride, float *raw, float *sum, float *norm,
                      int64_t n_expert, int64_t n_used, int64_t T);
int mi355_moe_combine(void *stream, const float *experts, const float *weights, float *scaled, const float *residual, float *out,
                      int64_t n_embd, int64_t n_used, int64_t T);
/* moe_weights and moe_combine in one launch (a few tokens): the same outputs with the same bits.  raw, sum and norm may be NULL (all
 * three) when nothing else reads the weights; nothing the launch writes may overlap probs or ids. */
int mi355_moe_weights_combine(void *stream, const float *probs, const int32_t *ids, int64_t ids_stride, float *raw, float *sum, float *norm,
                              int64_t n_expert, const float *experts, float *scaled, const float *residual, float *out, int64_t n_embd, int64_t n_used,
                              int64_t T);

/* MUL_MAT with f32 or f16 src0 and f32 src1 (router / small dense matrices): dst[b][n] = sum_k W[n][k] x[b][k], strides honoured, ne2/ne3 broadcast */
int mi355_mul_mat_f(void *stream, const mi355_tensor *src0, const mi355_tensor *src1, const mi355_tensor *dst);

#ifdef __cplusplus
}
#endif
#endif /* MI355_KERNELS_H */
