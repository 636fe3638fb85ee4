// Thin C entry points that run single operators on the REFERENCE's own CPU backend
// (libggml-base / libggml-cpu compiled from the reference sources by oracle/Makefile).
// Test infrastructure only: used by tests/ to check the C restatement in oracle.c and
// the HIP kernels, and by bench.py's cpu_baseline leg.  Nothing shipped links this.
//
// Every function builds a one-node graph exactly as tests/test-backend-ops.cpp does
// (build_graph, :1936-1983 for MUL_MAT, :2003-2035 for MUL_MAT_ID, :3148-3180 for
// FLASH_ATTN_EXT) and computes it with ggml_backend_graph_compute on the CPU backend.

#include <ggml.h>
#include <ggml-alloc.h>
#include <ggml-backend.h>
#include <ggml-cpu.h>

#include <chrono>
#include <cstdint>
#include <cstring>
#include <vector>

extern "C" {
// reference quantizers that are exported from libggml-base (ggml/src/ggml-quants.h)
void quantize_row_q8_1_ref(const float * x, void * y, int64_t k);
void quantize_row_q8_0_ref(const float * x, void * y, int64_t k);
void quantize_row_q8_K_ref(const float * x, void * y, int64_t k);
}

namespace {

// The fp16->fp32 lookup table of the reference is filled by the first ggml_init
// (ggml/src/ggml.c:1385-1402); quantizers and dequantizers read it, so make sure it
// exists before any entry point runs.
struct table_init {
    table_init() {
        ggml_init_params ip = { ggml_tensor_overhead(), nullptr, true };
        ggml_free(ggml_init(ip));
    }
} g_table_init;

struct cpu_graph {
    ggml_context * ctx = nullptr;
    ggml_backend_t backend = nullptr;
    ggml_backend_buffer_t buf = nullptr;

    explicit cpu_graph(int n_threads) {
        ggml_init_params ip = { ggml_tensor_overhead() * 64 + ggml_graph_overhead(), nullptr, true };
        ctx = ggml_init(ip);
        backend = ggml_backend_cpu_init();
        ggml_backend_cpu_set_n_threads(backend, n_threads > 0 ? n_threads : 1);
    }
    ~cpu_graph() {
        if (buf) ggml_backend_buffer_free(buf);
        if (backend) ggml_backend_free(backend);
        if (ctx) ggml_free(ctx);
    }
    bool alloc() {
        buf = ggml_backend_alloc_ctx_tensors(ctx, backend);
        return buf != nullptr;
    }
    // returns seconds per run (averaged over `reps` timed runs after one untimed run when reps > 0)
    double run(ggml_tensor * out, int reps) {
        ggml_cgraph * gf = ggml_new_graph(ctx);
        ggml_build_forward_expand(gf, out);
        ggml_backend_graph_compute(backend, gf);
        if (reps <= 0) return 0.0;
        auto t0 = std::chrono::steady_clock::now();
        for (int i = 0; i < reps; i++) ggml_backend_graph_compute(backend, gf);
        auto t1 = std::chrono::steady_clock::now();
        return std::chrono::duration<double>(t1 - t0).count() / reps;
    }
};

} // namespace

extern "C" {

int64_t ref_type_size(int type) { return (int64_t) ggml_type_size((ggml_type) type); }
int64_t ref_blck_size(int type) { return ggml_blck_size((ggml_type) type); }
int64_t ref_row_size(int type, int64_t k) { return (int64_t) ggml_row_size((ggml_type) type, k); }

// ggml_quantize_chunk (ggml/src/ggml.c:6410), no importance matrix
int64_t ref_quantize(int type, const float * src, void * dst, int64_t nrows, int64_t k) {
    return (int64_t) ggml_quantize_chunk((ggml_type) type, src, dst, 0, nrows, k, nullptr);
}

int ref_dequantize(int type, const void * src, float * dst, int64_t n) {
    const ggml_type_traits * tt = ggml_get_type_traits((ggml_type) type);
    if (!tt || !tt->to_float) return -1;
    tt->to_float(src, dst, n);
    return 0;
}

void ref_quantize_row_q8_1(const float * x, void * y, int64_t k) { quantize_row_q8_1_ref(x, y, k); }
void ref_quantize_row_q8_0(const float * x, void * y, int64_t k) { quantize_row_q8_0_ref(x, y, k); }
void ref_quantize_row_q8_K(const float * x, void * y, int64_t k) { quantize_row_q8_K_ref(x, y, k); }

void ref_fp32_to_fp16_row(const float * x, uint16_t * y, int64_t n) { ggml_fp32_to_fp16_row(x, (ggml_fp16_t *) y, n); }
void ref_fp16_to_fp32_row(const uint16_t * x, float * y, int64_t n) { ggml_fp16_to_fp32_row((const ggml_fp16_t *) x, y, n); }

// MUL_MAT: W [K,N] of `type`, x f32 [K,B], dst f32 [N,B].  Returns seconds/run when reps>0.
double ref_mul_mat(int type, const void * W, const float * x, float * dst, int64_t N, int64_t K, int64_t B,
                   int n_threads, int reps) {
    cpu_graph g(n_threads);
    ggml_tensor * a = ggml_new_tensor_2d(g.ctx, (ggml_type) type, K, N);
    ggml_tensor * b = ggml_new_tensor_2d(g.ctx, GGML_TYPE_F32, K, B);
    ggml_tensor * out = ggml_mul_mat(g.ctx, a, b);
    if (!g.alloc()) return -1.0;
    ggml_backend_tensor_set(a, W, 0, ggml_nbytes(a));
    ggml_backend_tensor_set(b, x, 0, ggml_nbytes(b));
    double t = g.run(out, reps);
    ggml_backend_tensor_get(out, dst, 0, ggml_nbytes(out));
    return t;
}

// MUL_MAT_ID: as [K,N,n_expert], b f32 [K,nb1,T], ids i32 [n_used,T] taken as a view of an
// [n_expert,T] tensor (row stride n_expert), dst f32 [N,n_used,T].
double ref_mul_mat_id(int type, const void * as, const float * b, const int32_t * ids_full, float * dst, int64_t N,
                      int64_t K, int64_t n_expert, int64_t n_used, int64_t nb1, int64_t T, int n_threads, int reps) {
    cpu_graph g(n_threads);
    ggml_tensor * ta = ggml_new_tensor_3d(g.ctx, (ggml_type) type, K, N, n_expert);
    ggml_tensor * tb = ggml_new_tensor_3d(g.ctx, GGML_TYPE_F32, K, nb1, T);
    ggml_tensor * ti = ggml_new_tensor_2d(g.ctx, GGML_TYPE_I32, n_expert, T);
    ggml_tensor * tv = n_used != n_expert ? ggml_view_2d(g.ctx, ti, n_used, T, ti->nb[1], 0) : ti;
    ggml_tensor * out = ggml_mul_mat_id(g.ctx, ta, tb, tv);
    if (!g.alloc()) return -1.0;
    ggml_backend_tensor_set(ta, as, 0, ggml_nbytes(ta));
    ggml_backend_tensor_set(tb, b, 0, ggml_nbytes(tb));
    ggml_backend_tensor_set(ti, ids_full, 0, ggml_nbytes(ti));
    double t = g.run(out, reps);
    ggml_backend_tensor_get(out, dst, 0, ggml_nbytes(out));
    return t;
}

// FLASH_ATTN_EXT: q f32 [D,Nq,Hq], k,v f16 [D,Nkv,Hkv], mask f16 [Nkv, Nq_pad] or NULL,
// dst f32 [D,Hq,Nq].
double ref_flash_attn(const float * q, const uint16_t * k, const uint16_t * v, const uint16_t * mask, float * dst,
                      int64_t D, int64_t Nq, int64_t Nkv, int64_t Hq, int64_t Hkv, int64_t Nq_pad, float scale,
                      float max_bias, float softcap, int n_threads, int reps) {
    cpu_graph g(n_threads);
    ggml_tensor * tq = ggml_new_tensor_3d(g.ctx, GGML_TYPE_F32, D, Nq, Hq);
    ggml_tensor * tk = ggml_new_tensor_3d(g.ctx, GGML_TYPE_F16, D, Nkv, Hkv);
    ggml_tensor * tv = ggml_new_tensor_3d(g.ctx, GGML_TYPE_F16, D, Nkv, Hkv);
    ggml_tensor * tm = mask ? ggml_new_tensor_2d(g.ctx, GGML_TYPE_F16, Nkv, Nq_pad) : nullptr;
    ggml_tensor * out = ggml_flash_attn_ext(g.ctx, tq, tk, tv, tm, scale, max_bias, softcap);
    ggml_flash_attn_ext_set_prec(out, GGML_PREC_F32);
    if (!g.alloc()) return -1.0;
    ggml_backend_tensor_set(tq, q, 0, ggml_nbytes(tq));
    ggml_backend_tensor_set(tk, k, 0, ggml_nbytes(tk));
    ggml_backend_tensor_set(tv, v, 0, ggml_nbytes(tv));
    if (tm) ggml_backend_tensor_set(tm, mask, 0, ggml_nbytes(tm));
    double t = g.run(out, reps);
    ggml_backend_tensor_get(out, dst, 0, ggml_nbytes(out));
    return t;
}

// FLASH_ATTN_EXT over a typed KV cache: k, v are [D, Nkv, Hkv] tensors of type_k / type_v (f16 or a quantized type).
double ref_flash_attn_kv(const float * q, const void * k, int type_k, const void * v, int type_v, const uint16_t * mask, float * dst,
                         int64_t D, int64_t Nq, int64_t Nkv, int64_t Hq, int64_t Hkv, int64_t Nq_pad, float scale,
                         float max_bias, float softcap, int n_threads, int reps) {
    cpu_graph g(n_threads);
    ggml_tensor * tq = ggml_new_tensor_3d(g.ctx, GGML_TYPE_F32, D, Nq, Hq);
    ggml_tensor * tk = ggml_new_tensor_3d(g.ctx, (ggml_type) type_k, D, Nkv, Hkv);
    ggml_tensor * tv = ggml_new_tensor_3d(g.ctx, (ggml_type) type_v, D, Nkv, Hkv);
    ggml_tensor * tm = mask ? ggml_new_tensor_2d(g.ctx, GGML_TYPE_F16, Nkv, Nq_pad) : nullptr;
    ggml_tensor * out = ggml_flash_attn_ext(g.ctx, tq, tk, tv, tm, scale, max_bias, softcap);
    ggml_flash_attn_ext_set_prec(out, GGML_PREC_F32);
    if (!g.alloc()) return -1.0;
    ggml_backend_tensor_set(tq, q, 0, ggml_nbytes(tq));
    ggml_backend_tensor_set(tk, k, 0, ggml_nbytes(tk));
    ggml_backend_tensor_set(tv, v, 0, ggml_nbytes(tv));
    if (tm) ggml_backend_tensor_set(tm, mask, 0, ggml_nbytes(tm));
    double t = g.run(out, reps);
    ggml_backend_tensor_get(out, dst, 0, ggml_nbytes(out));
    return t;
}

// CPY of contiguous f32 rows of k elements into a tensor of `type` (what llm_build_kv_store does with a quantized cache):
// the CPU backend's own conversion (its from_float, which may round differently from quantize_row_*_ref on SIMD builds).
int ref_cpy_f32_to(int type, const float * x, void * y, int64_t k, int64_t nrows, int n_threads) {
    cpu_graph g(n_threads);
    ggml_tensor * a = ggml_new_tensor_2d(g.ctx, GGML_TYPE_F32, k, nrows);
    ggml_tensor * b = ggml_new_tensor_2d(g.ctx, (ggml_type) type, k, nrows);
    ggml_tensor * out = ggml_cpy(g.ctx, a, b);
    if (!g.alloc()) return -1;
    ggml_backend_tensor_set(a, x, 0, ggml_nbytes(a));
    g.run(out, 0);
    ggml_backend_tensor_get(b, y, 0, ggml_nbytes(b));
    return 0;
}

int ref_rms_norm(const float * x, float * y, int64_t ncols, int64_t nrows, float eps, int n_threads) {
    cpu_graph g(n_threads);
    ggml_tensor * a = ggml_new_tensor_2d(g.ctx, GGML_TYPE_F32, ncols, nrows);
    ggml_tensor * out = ggml_rms_norm(g.ctx, a, eps);
    if (!g.alloc()) return -1;
    ggml_backend_tensor_set(a, x, 0, ggml_nbytes(a));
    g.run(out, 0);
    ggml_backend_tensor_get(out, y, 0, ggml_nbytes(out));
    return 0;
}

int ref_silu(const float * x, float * y, int64_t n, int n_threads) {
    cpu_graph g(n_threads);
    ggml_tensor * a = ggml_new_tensor_1d(g.ctx, GGML_TYPE_F32, n);
    ggml_tensor * out = ggml_silu(g.ctx, a);
    if (!g.alloc()) return -1;
    ggml_backend_tensor_set(a, x, 0, ggml_nbytes(a));
    g.run(out, 0);
    ggml_backend_tensor_get(out, y, 0, ggml_nbytes(out));
    return 0;
}

int ref_soft_max(const float * x, const float * mask, float * y, int64_t ncols, int64_t nrows, float scale,
                 int n_threads) {
    cpu_graph g(n_threads);
    ggml_tensor * a = ggml_new_tensor_2d(g.ctx, GGML_TYPE_F32, ncols, nrows);
    ggml_tensor * m = mask ? ggml_new_tensor_2d(g.ctx, GGML_TYPE_F32, ncols, nrows) : nullptr;
    ggml_tensor * out = ggml_soft_max_ext(g.ctx, a, m, scale, 0.0f);
    if (!g.alloc()) return -1;
    ggml_backend_tensor_set(a, x, 0, ggml_nbytes(a));
    if (m) ggml_backend_tensor_set(m, mask, 0, ggml_nbytes(m));
    g.run(out, 0);
    ggml_backend_tensor_get(out, y, 0, ggml_nbytes(out));
    return 0;
}

int ref_rope(const float * x, const int32_t * pos, const float * freq_factors, float * y, int64_t ne0, int64_t n_heads,
             int64_t n_tokens, int n_dims, int mode, float freq_base, float freq_scale, float ext_factor,
             float attn_factor, float beta_fast, float beta_slow, int n_ctx_orig, int n_threads) {
    cpu_graph g(n_threads);
    ggml_tensor * a = ggml_new_tensor_3d(g.ctx, GGML_TYPE_F32, ne0, n_heads, n_tokens);
    ggml_tensor * p = ggml_new_tensor_1d(g.ctx, GGML_TYPE_I32, n_tokens);
    ggml_tensor * f = freq_factors ? ggml_new_tensor_1d(g.ctx, GGML_TYPE_F32, n_dims / 2) : nullptr;
    ggml_tensor * out = ggml_rope_ext(g.ctx, a, p, f, n_dims, mode, n_ctx_orig, freq_base, freq_scale, ext_factor,
                                      attn_factor, beta_fast, beta_slow);
    if (!g.alloc()) return -1;
    ggml_backend_tensor_set(a, x, 0, ggml_nbytes(a));
    ggml_backend_tensor_set(p, pos, 0, ggml_nbytes(p));
    if (f) ggml_backend_tensor_set(f, freq_factors, 0, ggml_nbytes(f));
    g.run(out, 0);
    ggml_backend_tensor_get(out, y, 0, ggml_nbytes(out));
    return 0;
}

int ref_argsort(const float * x, int32_t * idx, int64_t ncols, int64_t nrows, int descending, int n_threads) {
    cpu_graph g(n_threads);
    ggml_tensor * a = ggml_new_tensor_2d(g.ctx, GGML_TYPE_F32, ncols, nrows);
    ggml_tensor * out = ggml_argsort(g.ctx, a, descending ? GGML_SORT_ORDER_DESC : GGML_SORT_ORDER_ASC);
    if (!g.alloc()) return -1;
    ggml_backend_tensor_set(a, x, 0, ggml_nbytes(a));
    g.run(out, 0);
    ggml_backend_tensor_get(out, idx, 0, ggml_nbytes(out));
    return 0;
}

} // extern "C"
