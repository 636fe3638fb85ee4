"""ctypes bindings for the CPU checkers used by the tests.

`oracle`  : oracle/liboracle.so   - this repository's plain-C restatement of the reference.
`ref`     : oracle/_ref/libref_driver.so - entry points that run the reference's own CPU
            backend (built from the reference sources by oracle/Makefile); None when absent.

Test infrastructure only.
"""
import ctypes as C
import os

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

F32, F16, Q4_0, Q8_0, Q8_1, Q4_K, Q5_K, Q6_K, Q8_K, I32 = 0, 1, 2, 8, 9, 12, 13, 14, 15, 26
Q4_1, Q5_0, Q5_1, IQ4_NL, IQ4_XS = 3, 6, 7, 20, 23
WEIGHT_TYPES = {"q4_0": Q4_0, "q8_0": Q8_0, "q4_K": Q4_K, "q5_K": Q5_K, "q6_K": Q6_K, "q4_1": Q4_1, "q5_0": Q5_0, "q5_1": Q5_1,
                "iq4_nl": IQ4_NL, "iq4_xs": IQ4_XS}
BLOCK = {F32: (1, 4), F16: (1, 2), Q4_0: (32, 18), Q8_0: (32, 34), Q8_1: (32, 36), Q4_K: (256, 144), Q5_K: (256, 176),
         Q6_K: (256, 210), Q8_K: (256, 292), Q4_1: (32, 20), Q5_0: (32, 22), Q5_1: (32, 24), IQ4_NL: (32, 18), IQ4_XS: (256, 136)}

_p = C.c_void_p
_i64 = C.c_int64
_f = C.c_float
_int = C.c_int


def row_bytes(t, k):
    be, bb = BLOCK[t]
    assert k % be == 0
    return k // be * bb


def _ptr(a):
    return None if a is None else a.ctypes.data_as(_p)


def _load(path):
    return C.CDLL(path) if os.path.exists(path) else None


oracle = _load(os.path.join(ROOT, "oracle", "liboracle.so"))
ref = _load(os.path.join(ROOT, "oracle", "_ref", "libref_driver.so"))

if oracle is not None:
    oracle.orc_f32_to_f16.restype = C.c_uint16
    oracle.orc_f32_to_f16.argtypes = [_f]
    oracle.orc_f16_to_f32.restype = _f
    oracle.orc_f16_to_f32.argtypes = [C.c_uint16]
    oracle.orc_row_bytes.restype = C.c_size_t
    oracle.orc_row_bytes.argtypes = [_int, _i64]
    for name in ("orc_quantize", "orc_dequantize"):
        getattr(oracle, name).restype = _int
        getattr(oracle, name).argtypes = [_int, _p, _p, _i64, _i64]
    oracle.orc_block_dots_q8_1.restype = _int
    oracle.orc_block_dots_q8_1.argtypes = [_int, _p, _p, _i64, _i64, _p]
    for name in ("orc_mul_mat_cpu", "orc_mul_mat_q8_1", "orc_mul_mat_f64"):
        getattr(oracle, name).restype = _int
        getattr(oracle, name).argtypes = [_int, _p, _p, _p, _i64, _i64, _i64]
    oracle.orc_mul_mat_id_q8_1.restype = _int
    oracle.orc_mul_mat_id_q8_1.argtypes = [_int, _p, _p, _p, _i64, _p, _i64, _i64, _i64, _i64, _i64, _i64]
    for name in ("orc_flash_attn_cpu", "orc_flash_attn_f64"):
        getattr(oracle, name).restype = None
        getattr(oracle, name).argtypes = [_p, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _f, _f, _f]
    oracle.orc_rms_norm.argtypes = [_p, _p, _i64, _i64, _f]
    oracle.orc_flash_attn_kv_cpu.restype = _int
    oracle.orc_flash_attn_kv_cpu.argtypes = [_p, _p, _int, _p, _int, _p, _p, _i64, _i64, _i64, _i64, _i64, _f, _f, _f]
    oracle.orc_silu.argtypes = [_p, _p, _i64]
    oracle.orc_soft_max.argtypes = [_p, _p, _p, _i64, _i64, _f]
    oracle.orc_rope.argtypes = [_p, _p, _p, _p, _i64, _i64, _i64, _int, _int, _f, _f, _f, _f, _f, _f, _int]
    oracle.orc_argsort.argtypes = [_p, _p, _i64, _i64, _int]
    oracle.orc_f32_to_f16_row.argtypes = [_p, _p, _i64]
    oracle.orc_f16_to_f32_row.argtypes = [_p, _p, _i64]

if ref is not None:
    ref.ref_row_size.restype = _i64
    ref.ref_row_size.argtypes = [_int, _i64]
    ref.ref_quantize.restype = _i64
    ref.ref_quantize.argtypes = [_int, _p, _p, _i64, _i64]
    ref.ref_dequantize.restype = _int
    ref.ref_dequantize.argtypes = [_int, _p, _p, _i64]
    for name in ("ref_quantize_row_q8_1", "ref_quantize_row_q8_0", "ref_quantize_row_q8_K"):
        getattr(ref, name).restype = None
        getattr(ref, name).argtypes = [_p, _p, _i64]
    ref.ref_fp32_to_fp16_row.argtypes = [_p, _p, _i64]
    ref.ref_fp16_to_fp32_row.argtypes = [_p, _p, _i64]
    ref.ref_mul_mat.restype = C.c_double
    ref.ref_mul_mat.argtypes = [_int, _p, _p, _p, _i64, _i64, _i64, _int, _int]
    ref.ref_mul_mat_id.restype = C.c_double
    ref.ref_mul_mat_id.argtypes = [_int, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _i64, _int, _int]
    if hasattr(ref, "ref_flash_attn_kv"):
        ref.ref_flash_attn_kv.restype = C.c_double
        ref.ref_flash_attn_kv.argtypes = [_p, _p, _int, _p, _int, _p, _p, _i64, _i64, _i64, _i64, _i64, _i64, _f, _f, _f, _int, _int]
        ref.ref_cpy_f32_to.restype = _int
        ref.ref_cpy_f32_to.argtypes = [_int, _p, _p, _i64, _i64, _int]
    ref.ref_flash_attn.restype = C.c_double
    ref.ref_flash_attn.argtypes = [_p, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _i64, _f, _f, _f, _int, _int]
    ref.ref_rms_norm.argtypes = [_p, _p, _i64, _i64, _f, _int]
    ref.ref_silu.argtypes = [_p, _p, _i64, _int]
    ref.ref_soft_max.argtypes = [_p, _p, _p, _i64, _i64, _f, _int]
    ref.ref_rope.argtypes = [_p, _p, _p, _p, _i64, _i64, _i64, _int, _int, _f, _f, _f, _f, _f, _f, _int, _int]
    ref.ref_argsort.argtypes = [_p, _p, _i64, _i64, _int, _int]


# ---------------------------------------------------------------- numpy-level helpers
def f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def quantize(lib_kind, t, x):
    """x: float32 [nrows, k] -> uint8 [nrows, row_bytes]"""
    x = f32(x)
    nrows, k = x.shape
    out = np.zeros((nrows, row_bytes(t, k)), dtype=np.uint8)
    if lib_kind == "oracle":
        assert oracle.orc_quantize(t, _ptr(x), _ptr(out), nrows, k) == 0
    else:
        if t == Q8_1:
            for r in range(nrows):
                ref.ref_quantize_row_q8_1(_ptr(x[r]), _ptr(out[r]), k)
        elif t == Q8_K:
            for r in range(nrows):
                ref.ref_quantize_row_q8_K(_ptr(x[r]), _ptr(out[r]), k)
        else:
            assert ref.ref_quantize(t, _ptr(x), _ptr(out), nrows, k) == out.size
    return out


def quantize_mt(lib_kind, t, x, threads=16):
    """quantize() over row chunks on `threads` host threads (the C calls release the interpreter lock): whole 8B-model matrices"""
    from concurrent.futures import ThreadPoolExecutor
    x = f32(x)
    n = x.shape[0]
    step = max(64, (n + 4 * threads - 1) // (4 * threads))
    with ThreadPoolExecutor(max_workers=threads) as ex:
        parts = list(ex.map(lambda i: quantize(lib_kind, t, x[i:i + step]), range(0, n, step)))
    return np.concatenate(parts)


def dequantize(lib_kind, t, q, k):
    q = np.ascontiguousarray(q, dtype=np.uint8)
    nrows = q.shape[0]
    out = np.zeros((nrows, k), dtype=np.float32)
    if lib_kind == "oracle":
        assert oracle.orc_dequantize(t, _ptr(q), _ptr(out), nrows, k) == 0
    else:
        assert ref.ref_dequantize(t, _ptr(q), _ptr(out), nrows * k) == 0
    return out


def block_dots(t, W, act, k):
    """W uint8 [N,row_bytes], act uint8 [row_bytes(Q8_1)] -> int32 [N, k/granule]"""
    g = 16 if t == Q6_K else 32
    N = W.shape[0]
    out = np.zeros((N, k // g), dtype=np.int32)
    assert oracle.orc_block_dots_q8_1(t, _ptr(W), _ptr(act), N, k, _ptr(out)) == 0
    return out


def mul_mat(kind, t, W, x, n_threads=4):
    """W uint8 [N,row_bytes], x f32 [B,K] -> f32 [B,N].  kind: cpu|q8_1|f64|ref"""
    x = f32(x)
    B, K = x.shape
    N = W.shape[0]
    out = np.zeros((B, N), dtype=np.float32)
    W = np.ascontiguousarray(W)
    if kind == "ref":
        assert ref.ref_mul_mat(t, _ptr(W), _ptr(x), _ptr(out), N, K, B, n_threads, 0) >= 0
    else:
        fn = getattr(oracle, "orc_mul_mat_" + kind)
        assert fn(t, _ptr(W), _ptr(x), _ptr(out), N, K, B) == 0
    return out


def flash_attn(kind, q, k, v, mask, scale, max_bias=0.0, softcap=0.0, n_threads=4):
    """q f32 [Hq,Nq,D]; k,v f16-bits uint16 [Hkv,Nkv,D]; mask uint16 [Nq_pad,Nkv] or None -> f32 [Nq,Hq,D]"""
    Hq, Nq, D = q.shape
    Hkv, Nkv, _ = k.shape
    q = f32(q)
    k = np.ascontiguousarray(k, dtype=np.uint16)
    v = np.ascontiguousarray(v, dtype=np.uint16)
    out = np.zeros((Nq, Hq, D), dtype=np.float32)
    if mask is not None:
        mask = np.ascontiguousarray(mask, dtype=np.uint16)
    if kind == "ref":
        nq_pad = mask.shape[0] if mask is not None else Nq
        assert ref.ref_flash_attn(_ptr(q), _ptr(k), _ptr(v), _ptr(mask), _ptr(out), D, Nq, Nkv, Hq, Hkv, nq_pad, scale,
                                  max_bias, softcap, n_threads, 0) >= 0
    else:
        getattr(oracle, "orc_flash_attn_" + kind)(_ptr(q), _ptr(k), _ptr(v), _ptr(mask), _ptr(out), D, Nq, Nkv, Hq,
                                                   Hkv, scale, max_bias, softcap)
    return out


F16 = 1


def kv_rows(t, x):
    """f32 [Hkv, Nkv, D] -> the cache bytes of type t (f16 bits as uint8, or quantized blocks by the reference-pinned quantizer)"""
    x = f32(x)
    if t == F16:
        return np.ascontiguousarray(x.astype(np.float16)).view(np.uint8).reshape(x.shape[0], x.shape[1], -1)
    H, N, D = x.shape
    return quantize("oracle", t, x.reshape(H * N, D)).reshape(H, N, -1)


def flash_attn_kv(kind, q, k, type_k, v, type_v, mask, scale, max_bias=0.0, softcap=0.0, n_threads=4):
    """q f32 [Hq,Nq,D]; k, v uint8 [Hkv,Nkv,row bytes] of type_k / type_v (see kv_rows); mask uint16 or None -> f32 [Nq,Hq,D]"""
    Hq, Nq, D = q.shape
    Hkv, Nkv = k.shape[0], k.shape[1]
    q = f32(q)
    k = np.ascontiguousarray(k, dtype=np.uint8)
    v = np.ascontiguousarray(v, dtype=np.uint8)
    out = np.zeros((Nq, Hq, D), dtype=np.float32)
    if mask is not None:
        mask = np.ascontiguousarray(mask, dtype=np.uint16)
    if kind == "ref":
        nq_pad = mask.shape[0] if mask is not None else Nq
        assert ref.ref_flash_attn_kv(_ptr(q), _ptr(k), type_k, _ptr(v), type_v, _ptr(mask), _ptr(out), D, Nq, Nkv, Hq, Hkv, nq_pad, scale,
                                     max_bias, softcap, n_threads, 0) >= 0
    else:
        assert oracle.orc_flash_attn_kv_cpu(_ptr(q), _ptr(k), type_k, _ptr(v), type_v, _ptr(mask), _ptr(out), D, Nq, Nkv, Hq, Hkv, scale,
                                            max_bias, softcap) == 0
    return out


def nmse(a, b):
    """normalised mean squared error as in tests/test-backend-ops.cpp:175-188 (b is the reference)"""
    a = np.asarray(a, dtype=np.float64).ravel()
    b = np.asarray(b, dtype=np.float64).ravel()
    den = float(np.sum(b * b))
    num = float(np.sum((a - b) ** 2))
    return num / den if den > 0 else num


def f16_bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).astype(np.float16).view(np.uint16)
