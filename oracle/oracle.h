/*
 * CPU oracle for the quantized-inference hot path.  TEST INFRASTRUCTURE ONLY:
 * nothing in the shipped library calls into this file.  Every function restates,
 * in plain scalar C, an algorithm of the reference (ggerganov/llama.cpp); the
 * reference file:line each one follows is given at its definition in oracle.c.
 *
 * Tensor element types use the reference's enum values (ggml/include/ggml.h:351-392).
 */
#ifndef ORACLE_H
#define ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum orc_type {
    ORC_F32  = 0,
    ORC_F16  = 1,
    ORC_Q4_0 = 2,
    ORC_Q4_1 = 3,
    ORC_Q5_0 = 6,
    ORC_Q5_1 = 7,
    ORC_Q8_0 = 8,
    ORC_Q8_1 = 9,
    ORC_Q4_K = 12,
    ORC_Q5_K = 13,
    ORC_Q6_K = 14,
    ORC_Q8_K = 15,
    ORC_IQ4_NL = 20,
    ORC_IQ4_XS = 23,
};

/* IEEE binary16 <-> binary32, round to nearest even */
uint16_t orc_f32_to_f16(float f);
float    orc_f16_to_f32(uint16_t h);
void     orc_f32_to_f16_row(const float *x, uint16_t *y, int64_t n);
void     orc_f16_to_f32_row(const uint16_t *x, float *y, int64_t n);

/* block geometry: elements per block, bytes per block, bytes per row of k elements */
int    orc_block_elems(int type);
size_t orc_block_bytes(int type);
size_t orc_row_bytes(int type, int64_t k);

/* row quantizers / dequantizers; return 0 on success, -1 for an unknown type */
int orc_quantize(int type, const float *x, void *y, int64_t nrows, int64_t k);
int orc_dequantize(int type, const void *x, float *y, int64_t nrows, int64_t k);

/* Integer dots of weight sub-blocks against Q8_1 activation blocks.
 * W: nrows rows of k elements of `type`; a: one activation row of k/32 block_q8_1.
 * Granule g = 32 for Q4_0/Q8_0/Q4_K, 16 for Q6_K.  out[r*(k/g) + j] = sum over the
 * j-th granule of row r of  wq * aq, where wq is the stored integer level with its
 * fixed offset removed (Q4_0: nibble-8, Q8_0: q, Q4_K: nibble, Q6_K: q6-32). */
int orc_block_dots_q8_1(int type, const void *W, const void *a, int64_t nrows, int64_t k, int32_t *out);

/* dst[b*N + n] = sum_k W[n,k] * x[b*K + k]
 *  _cpu : the reference CPU pipeline: activations quantized to the type's vec_dot
 *         partner (Q8_0 for Q4_0/Q8_0, Q8_K for Q4_K/Q6_K), scalar vec_dot.
 *  _q8_1: the device formulation: activations quantized to Q8_1, exact integer
 *         sub-block dots, scale algebra accumulated in double.
 *  _f64 : dequantize(W) . x in double, no activation quantization. */
int orc_mul_mat_cpu (int type, const void *W, const float *x, float *dst, int64_t N, int64_t K, int64_t B);
int orc_mul_mat_q8_1(int type, const void *W, const float *x, float *dst, int64_t N, int64_t K, int64_t B);
int orc_mul_mat_f64 (int type, const void *W, const float *x, float *dst, int64_t N, int64_t K, int64_t B);

/* MUL_MAT_ID: as = n_expert matrices [N,K] of `type` (contiguous), b f32 [K, nb1, T],
 * ids int32 [n_used, T] with row stride ids_stride (in int32 elements),
 * dst f32 [N, n_used, T];  dst[:,e,t] = as[ids[e,t]] . b[:, e % nb1, t]   (q8_1 formulation) */
int orc_mul_mat_id_q8_1(int type, const void *as, const float *b, const int32_t *ids, int64_t ids_stride,
                        float *dst, int64_t N, int64_t K, int64_t n_expert, int64_t n_used, int64_t nb1, int64_t T);

/* FLASH_ATTN_EXT.  q f32 [D, Nq, Hq] (contiguous in that order), k,v f16 [D, Nkv, Hkv],
 * mask f16 [Nkv, Nq_pad] or NULL, dst f32 [D, Hq, Nq].
 *  _cpu : restates the reference CPU kernel (q rounded to f16, f16 V accumulator).
 *  _f64 : textbook softmax(q k^T * scale + mask) v in double. */
void orc_flash_attn_cpu(const float *q, const uint16_t *k, const uint16_t *v, const uint16_t *mask,
                        float *dst, int64_t D, int64_t Nq, int64_t Nkv, int64_t Hq, int64_t Hkv,
                        float scale, float max_bias, float softcap);
/* _kv_cpu : the same kernel over a typed KV cache (ORC_F16, ORC_Q8_0, ORC_Q4_0 for K and V independently); k, v hold
 *  [Hkv][Nkv] rows of D elements in the type's block layout.  Returns 0, or -1 for an unsupported type / D. */
int orc_flash_attn_kv_cpu(const float *q, const void *k, int type_k, const void *v, int type_v, const uint16_t *mask,
                          float *dst, int64_t D, int64_t Nq, int64_t Nkv, int64_t Hq, int64_t Hkv,
                          float scale, float max_bias, float softcap);
void orc_flash_attn_f64(const float *q, const uint16_t *k, const uint16_t *v, const uint16_t *mask,
                        float *dst, int64_t D, int64_t Nq, int64_t Nkv, int64_t Hq, int64_t Hkv,
                        float scale, float max_bias, float softcap);

/* glue ops (contiguous f32 rows unless said otherwise) */
void orc_rms_norm(const float *x, float *y, int64_t ncols, int64_t nrows, float eps);
void orc_silu(const float *x, float *y, int64_t n);
void orc_soft_max(const float *x, const float *mask_f32, float *y, int64_t ncols, int64_t nrows, float scale);
/* mode 0 = adjacent pairs ("norm"), 2 = NeoX pairs (i, i+n_dims/2) */
void orc_rope(const float *x, const int32_t *pos, const float *freq_factors, float *y,
              int64_t ne0, int64_t n_heads, int64_t n_tokens, int n_dims, int mode,
              float freq_base, float freq_scale, float ext_factor, float attn_factor,
              float beta_fast, float beta_slow, int n_ctx_orig);
void orc_argsort(const float *x, int32_t *idx, int64_t ncols, int64_t nrows, int descending);

#ifdef __cplusplus
}
#endif
#endif /* ORACLE_H */
