"""Python view of the MI355X kernel library (ctypes over include/mi355_kernels.h).

PyTorch is used only to own device memory and streams; every operator below goes through
the C ABI of libmi355_kernels.so.  There is no CPU fallback: loading fails loudly when the
library has not been built.
"""
import ctypes as C
import os

from . import build as _build

F32, F16, Q4_0, Q8_0, Q8_1, Q4_K, Q5_K, Q6_K, I32 = 0, 1, 2, 8, 9, 12, 13, 14, 26
Q4_1, Q5_0, Q5_1, IQ4_NL, IQ4_XS = 3, 6, 7, 20, 23
WEIGHT_TYPES = {"q4_0": Q4_0, "q8_0": Q8_0, "q4_K": Q4_K, "q5_K": Q5_K, "q6_K": Q6_K, "q4_1": Q4_1, "q5_0": Q5_0, "q5_1": Q5_1,
                "iq4_nl": IQ4_NL, "iq4_xs": IQ4_XS}
BLOCK = {F32: (1, 4), F16: (1, 2), I32: (1, 4), Q4_0: (32, 18), Q8_0: (32, 34), Q8_1: (32, 36), Q4_K: (256, 144), Q5_K: (256, 176),
         Q6_K: (256, 210), Q4_1: (32, 20), Q5_0: (32, 22), Q5_1: (32, 24), IQ4_NL: (32, 18), IQ4_XS: (256, 136)}

_p, _i64, _sz, _f, _int = C.c_void_p, C.c_int64, C.c_size_t, C.c_float, C.c_int


class TiledMat(C.Structure):
    """struct mi355_tiled_mat"""
    _fields_ = [("tiles", _p), ("dst", _p), ("residual", _p), ("N", _i64), ("dst_stride", _i64)]


class GemvMat(C.Structure):
    """struct mi355_gemv_mat"""
    _fields_ = [("type", _int), ("W", _p), ("N", _i64), ("dst", _p), ("dst_stride", _i64), ("residual", _p)]


class GemvRopeMat(C.Structure):
    """struct mi355_gemv_rope_mat"""
    _fields_ = [("type", _int), ("W", _p), ("N", _i64), ("epilogue", _int), ("dst", _p), ("dst_stride", _i64), ("nb1", _i64), ("nb2", _i64)]


class RopeDesc(C.Structure):
    """struct mi355_rope_desc"""
    _fields_ = [("pos", _p), ("cells", _p), ("freq_factors", _p), ("head_dim", _i64), ("n_dims", _int), ("mode", _int), ("n_ctx_orig", _int),
                ("freq_base", _f), ("freq_scale", _f), ("ext_factor", _f), ("attn_factor", _f), ("beta_fast", _f), ("beta_slow", _f)]


EPI_STORE, EPI_ROPE, EPI_ROPE_CACHE, EPI_CACHE, EPI_ROPE_QCACHE, EPI_QCACHE = range(6)


class Tensor(C.Structure):
    """struct mi355_tensor"""
    _fields_ = [("data", _p), ("type", _int), ("ne", _i64 * 4), ("nb", _sz * 4)]


_SIGNATURES = {
    "mi355_abi_version": (_int, []),
    "mi355_last_error": (C.c_char_p, []),
    "mi355_launch_count": (C.c_uint64, []),
    "mi355_device_supported": (_int, [_int]),
    "mi355_quantize_weights_supported": (_int, [_int]),
    "mi355_quantize_weights": (_int, [_p, _int, _p, _p, _i64, _i64]),
    "mi355_weights_scatter": (_int, [_p, _int, _p, _p, _i64, _i64, _sz, _sz]),
    "mi355_weights_gather": (_int, [_p, _int, _p, _p, _i64, _i64, _sz, _sz]),
    "mi355_quantize_q8_1": (_int, [_p, _p, _p, _i64, _i64, _i64]),
    "mi355_act_bytes": (_sz, [_i64, _i64]),
    "mi355_quantize_act": (_int, [_p, _p, _p, _i64, _i64, _i64]),
    "mi355_mul_mat_ws_bytes": (_sz, [_i64, _i64]),
    "mi355_mul_mat": (_int, [_p, _int, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _p, _sz]),
    "mi355_mul_mat_static_max_ws": (_sz, []),
    "mi355_mul_mat_static_init": (_int, []),
    "mi355_mul_mat_static": (_int, [_p, _int, _p, _p, _p, _i64, _i64, _i64, _i64, _i64]),
    "mi355_mul_mat_vec_q": (_int, [_p, _int, _p, _p, _p, _i64, _i64, _i64, _i64]),
    "mi355_mul_mat_q": (_int, [_p, _int, _p, _p, _p, _i64, _i64, _i64, _i64]),
    "mi355_mul_mat_q_ws_bytes": (_sz, [_i64, _i64, _i64]),
    "mi355_mul_mat_q_ws": (_int, [_p, _int, _p, _p, _p, _i64, _i64, _i64, _i64, _p, _sz]),
    "mi355_mul_mat_skinny_supported": (_int, [_int, _p, _i64, _i64]),
    "mi355_mul_mat_skinny_ws_bytes": (_sz, [_i64, _i64, _i64]),
    "mi355_mul_mat_skinny": (_int, [_p, _int, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _p, _sz]),
    "mi355_mul_mat_mid_supported": (_int, [_int, _p, _i64, _i64]),
    "mi355_mul_mat_mid_ws_bytes": (_sz, [_i64, _i64, _i64]),
    "mi355_mul_mat_mid": (_int, [_p, _int, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _p, _sz]),
    "mi355_mul_mat_mid_norm": (_int, [_p, _int, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _p, _sz, _p, _f, _p, _i64, _p]),
    "mi355_mul_mat_mid_multi_ws_bytes": (_sz, [_int, _p, _i64, _i64]),
    "mi355_mul_mat_mid_multi": (_int, [_p, _int, _int, _p, _p, _i64, _i64, _p, _sz]),
    "mi355_act_q8k_bytes": (_sz, [_i64, _i64]),
    "mi355_quantize_act_q8k": (_int, [_p, _p, _p, _i64, _i64, _i64]),
    "mi355_mul_mat_q8k": (_int, [_p, _int, _p, _p, _p, _i64, _i64, _i64, _i64]),
    "mi355_kq_planes_bytes": (_sz, [_i64, _i64]),
    "mi355_kq_unpack_planes": (_int, [_p, _int, _p, _p, _i64, _i64]),
    "mi355_mul_mat_q8k_planes": (_int, [_p, _int, _p, _p, _p, _p, _i64, _i64, _i64, _i64]),
    "mi355_mul_mat_q8k_planes_ws": (_int, [_p, _int, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _p, _sz]),
    "mi355_mul_mat_q8k_ws_bytes": (_sz, [_i64, _i64, _i64]),
    "mi355_mul_mat_q8k_ws": (_int, [_p, _int, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _p, _sz]),
    "mi355_mul_mat_q8k_add": (_int, [_p, _int, _p, _p, _p, _p, _i64, _i64, _i64, _i64]),
    "mi355_act_q8k_tiled_bytes": (_sz, [_i64, _i64]),
    "mi355_quantize_act_q8k_tiled": (_int, [_p, _p, _p, _i64, _i64, _i64]),
    "mi355_kq_tiles_bytes": (_sz, [_int, _i64, _i64]),
    "mi355_kq_unpack_tiles": (_int, [_p, _int, _p, _p, _i64, _i64]),
    "mi355_mul_mat_id_q8k_tiled_ws_bytes": (_sz, [_i64, _i64, _i64, _i64]),
    "mi355_mul_mat_id_q8k_tiled": (_int, [_p, _int, _p, _sz, _p, _p, _i64, _p, _i64, _i64, _i64, _i64, _i64, _i64, _p, _sz]),
    "mi355_mul_mat_q8k_tiled_ws_bytes": (_sz, [_i64, _i64, _i64]),
    "mi355_mul_mat_q8k_tiled": (_int, [_p, _int, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _p, _sz]),
    "mi355_mul_mat_q8k_tiled_mixed": (_int, [_p, _int, _p, _p, _p, _i64, _i64]),
    "mi355_rope_table": (_int, [_p, _p, _p, _p, _i64, _i64, _int, _int, _f, _f, _f, _f, _f, _f]),
    "mi355_mul_mat_q8k_tiled_qkv_rope": (_int, [_p, _p, _p, _p, _i64, _i64, _p, _p, _i64, _int, _sz, _sz, _sz, _sz]),
    "mi355_mul_mat_q8k_tiled_norm": (_int, [_p, _int, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _p, _sz, _p, _f, _p, _i64, _p]),
    "mi355_mul_mat_q8k_tiled_multi_ws_bytes": (_sz, [_int, _p, _i64, _i64]),
    "mi355_mul_mat_q8k_tiled_multi": (_int, [_p, _int, _int, _p, _p, _i64, _i64, _p, _sz]),
    "mi355_mul_mat_vec_q_multi": (_int, [_p, _int, _p, _p, _i64, _i64]),
    "mi355_rms_norm_mul_quant_router": (_int, [_p, _p, _i64, _p, _p, _i64, _p, _i64, _i64, _f, _p, _i64, _p, _p, _p, _i64]),
    "mi355_rms_norm_mul_quant": (_int, [_p, _p, _i64, _p, _p, _i64, _p, _i64, _i64, _f]),
    "mi355_swiglu_quant": (_int, [_p, _p, _p, _i64, _p, _i64, _p, _i64, _i64]),
    "mi355_rms_norm_mul_quant_q8k": (_int, [_p, _p, _i64, _p, _p, _i64, _p, _i64, _i64, _f]),
    "mi355_swiglu_quant_q8k": (_int, [_p, _p, _p, _i64, _p, _i64, _p, _i64, _i64]),
    "mi355_rms_norm_mul_quant_q8k_tiled": (_int, [_p, _p, _i64, _p, _p, _i64, _p, _i64, _i64, _f]),
    "mi355_swiglu_quant_q8k_tiled": (_int, [_p, _p, _p, _i64, _p, _i64, _p, _i64, _i64]),
    "mi355_rope_kv_store": (_int, [_p, _p, _p, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _sz, _sz, _sz, _sz, _int, _int, _int,
                            _f, _f, _f, _f, _f, _f]),
    "mi355_rope_kv_store_typed": (_int, [_p, _p, _p, _p, _int, _p, _i64, _i64, _int, _p, _i64, _i64, _p, _p, _p, _i64, _i64, _i64, _i64, _int, _int, _int,
                                  _f, _f, _f, _f, _f, _f]),
    "mi355_moe_gate_up_swiglu_supported": (_int, [_int, _p, _p, _i64, _i64]),
    "mi355_moe_gate_up_swiglu": (_int, [_p, _int, _p, _p, _p, _p, _i64, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _i64]),
    "mi355_ffn_gate_up_swiglu": (_int, [_p, _int, _p, _int, _p, _p, _p, _p, _i64, _p, _p, _i64, _i64, _i64]),
    "mi355_mul_mat_vec_q_rope": (_int, [_p, _int, _p, _p, _i64, _i64, _p]),
    "mi355_rms_norm_mul_mat_vec_q_rope": (_int, [_p, _p, _p, _f, _int, _p, _i64, _p]),
    "mi355_qkv_rope_store": (_int, [_p, _int, _p, _int, _p, _int, _p, _p, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64,
                                    _sz, _sz, _sz, _sz, _int, _int, _int, _f, _f, _f, _f, _f, _f]),
    "mi355_rms_norm_qkv_rope_store": (_int, [_p, _p, _p, _f, _int, _p, _int, _p, _int, _p, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _i64,
                                             _sz, _sz, _sz, _sz, _int, _int, _int, _f, _f, _f, _f, _f, _f]),
    "mi355_block_dots_q8_1": (_int, [_p, _int, _p, _p, _p, _i64, _i64]),
    "mi355_mul_mat_id_ws_bytes": (_sz, [_i64, _i64, _i64, _i64, _i64]),
    "mi355_mul_mat_id": (_int, [_p, _int, _p, _p, _p, _i64, _p, _i64, _i64, _i64, _i64, _i64, _i64, _p, _sz]),
    "mi355_mul_mat_id_q8k_route_bytes": (_sz, [_i64, _i64, _i64]),
    "mi355_mul_mat_id_q8k": (_int, [_p, _int, _p, _p, _p, _i64, _p, _i64, _i64, _i64, _i64, _i64, _i64, _p, _sz]),
    "mi355_moe_route": (_int, [_p, _p, _p, _p, _i64, _i64]),
    "mi355_moe_weights": (_int, [_p, _p, _p, _i64, _p, _p, _p, _i64, _i64, _i64]),
    "mi355_moe_weights_combine": (_int, [_p, _p, _p, _i64, _p, _p, _p, _i64, _p, _p, _p, _p, _i64, _i64, _i64]),
    "mi355_moe_combine": (_int, [_p, _p, _p, _p, _p, _p, _i64, _i64, _i64]),
    "mi355_mul_mat_id_q_supported": (_int, [_int, _p, _i64, _i64, _i64]),
    "mi355_mul_mat_id_q": (_int, [_p, _int, _p, _p, _p, _i64, _p, _i64, _i64, _i64, _i64, _i64, _i64, _p, _sz]),
    "mi355_mul_mat_id_vec": (_int, [_p, _int, _p, _p, _p, _i64, _p, _i64, _i64, _i64, _i64, _i64, _i64]),
    "mi355_flash_attn_ws_bytes": (_sz, [_i64, _i64, _i64, _i64]),
    "mi355_flash_attn_ext": (_int, [_p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _sz, _sz, _sz, _sz, _sz, _sz,
                                    _sz, _f, _f, _f, _p, _sz]),
    "mi355_flash_attn_ext_quant": (_int, [_p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _sz, _sz, _sz, _sz, _sz, _sz,
                                          _sz, _f, _f, _f, _p, _sz, _p]),
    "mi355_cpy_f32_quant": (_int, [_p, _int, _p, _p, _i64, _i64, _i64]),
    "mi355_cpy_quant_view": (_int, [_p, _int, _int, _p, _p, _i64, _i64, _p, _p]),
    "mi355_cpy_quant_blocks": (_int, [_p, _int, _p, _i64, _i64, _p, _i64, _i64, _i64]),
    "mi355_flash_attn_kv_ws_bytes": (_sz, [_i64, _i64, _i64, _i64, _i64, _int, _int]),
    "mi355_flash_attn_ext_kv": (_int, [_p, _p, _p, _int, _p, _i64, _p, _int, _p, _i64, _p, _p, _i64, _i64, _i64, _i64, _i64, _sz, _sz, _sz, _sz,
                                       _sz, _sz, _sz, _f, _f, _f, _p, _sz, _p]),
    "mi355_rms_norm": (_int, [_p, C.POINTER(Tensor), C.POINTER(Tensor), _f]),
    "mi355_bin_bcast": (_int, [_p, _int, C.POINTER(Tensor), C.POINTER(Tensor), C.POINTER(Tensor)]),
    "mi355_unary": (_int, [_p, _int, C.POINTER(Tensor), C.POINTER(Tensor)]),
    "mi355_scale": (_int, [_p, C.POINTER(Tensor), C.POINTER(Tensor), _f]),
    "mi355_cpy": (_int, [_p, C.POINTER(Tensor), C.POINTER(Tensor)]),
    "mi355_set_rows": (_int, [_p, C.POINTER(Tensor), _p, C.POINTER(Tensor)]),
    "mi355_get_rows": (_int, [_p, C.POINTER(Tensor), C.POINTER(Tensor), C.POINTER(Tensor)]),
    "mi355_soft_max": (_int, [_p, C.POINTER(Tensor), C.POINTER(Tensor), C.POINTER(Tensor), _f, _f]),
    "mi355_rope": (_int, [_p, C.POINTER(Tensor), _p, _p, C.POINTER(Tensor), _int, _int, _int, _f, _f, _f, _f, _f, _f]),
    "mi355_sum_rows": (_int, [_p, C.POINTER(Tensor), C.POINTER(Tensor)]),
    "mi355_argsort": (_int, [_p, C.POINTER(Tensor), C.POINTER(Tensor), _int]),
    "mi355_mul_mat_f": (_int, [_p, C.POINTER(Tensor), C.POINTER(Tensor), C.POINTER(Tensor)]),
}

_lib = None


def lib_path():
    return _build.kernels_lib_path()


def load():
    """dlopen libmi355_kernels.so (already-built file only; see build.build_kernels)."""
    global _lib
    if _lib is None:
        path = lib_path()
        if not os.path.exists(path):
            raise RuntimeError("%s is missing: run `python __graft_entry__.py` (build()) first" % path)
        lib = C.CDLL(path)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(lib, name)   # AttributeError if the library lacks a declared symbol
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


class Mi355Error(RuntimeError):
    pass


def check(rc):
    if rc != 0:
        raise Mi355Error("mi355 error %d: %s" % (rc, load().mi355_last_error().decode()))


def row_bytes(t, k):
    be, bb = BLOCK[t]
    assert k % be == 0
    return k // be * bb


# ---------------------------------------------------------------- torch-facing helpers
def _stream():
    import torch
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None else None


_TORCH_TYPES = None


def tensor_desc(t):
    """mi355_tensor for a torch tensor; ggml order: ne[0] is the fastest (last torch) dimension."""
    import torch
    global _TORCH_TYPES
    if _TORCH_TYPES is None:
        _TORCH_TYPES = {torch.float32: F32, torch.float16: F16, torch.int32: I32}
    d = Tensor()
    d.data = t.data_ptr()
    d.type = _TORCH_TYPES[t.dtype]
    shape = list(t.shape)[::-1]
    strides = [s * t.element_size() for s in t.stride()][::-1]
    assert len(shape) <= 4
    for i in range(4):
        d.ne[i] = shape[i] if i < len(shape) else 1
        d.nb[i] = strides[i] if i < len(shape) else (d.nb[i - 1] * d.ne[i - 1] if i > 0 else t.element_size())
    return d


def upload_weights(t, raw):
    """raw: torch.uint8 CUDA tensor [nrows, row_bytes] in the reference block layout -> device layout copy"""
    import torch
    nrows, rb = raw.shape
    k = rb // BLOCK[t][1] * BLOCK[t][0]
    out = torch.empty_like(raw)
    check(load().mi355_weights_scatter(_stream(), t, _ptr(raw), _ptr(out), k, nrows, 0, raw.numel()))
    return out


def download_weights(t, dev):
    import torch
    nrows, rb = dev.shape
    k = rb // BLOCK[t][1] * BLOCK[t][0]
    out = torch.empty_like(dev)
    check(load().mi355_weights_gather(_stream(), t, _ptr(dev), _ptr(out), k, nrows, 0, dev.numel()))
    return out


def quantize_weights(t, x):
    """x: f32 CUDA tensor [nrows, k] -> uint8 [nrows, row_bytes] in the reference block layout (the reference quantizer's bytes)"""
    import torch
    x = x.contiguous()
    nrows, k = x.shape
    y = torch.empty((nrows, row_bytes(t, k)), dtype=torch.uint8, device=x.device)
    check(load().mi355_quantize_weights(_stream(), t, _ptr(x), _ptr(y), k, nrows))
    return y


def quantize_q8_1(x):
    """x f32 [nrows, k] -> uint8 [nrows, k/32*36] (block_q8_1)"""
    import torch
    nrows, k = x.shape
    y = torch.empty((nrows, k // 32 * 36), dtype=torch.uint8, device=x.device)
    check(load().mi355_quantize_q8_1(_stream(), _ptr(x), _ptr(y), k, nrows, x.stride(0)))
    return y


def quantize_act(x):
    import torch
    nrows, k = x.shape
    ws = torch.empty(load().mi355_act_bytes(k, nrows), dtype=torch.uint8, device=x.device)
    check(load().mi355_quantize_act(_stream(), _ptr(x), _ptr(ws), k, nrows, x.stride(0)))
    return ws


def quantize_act_q8k(x):
    """x f32 [nrows, k] -> workspace in the per-super-block layout (int8 levels, f32 d per 256, fp16 sub-block sums)"""
    import torch
    nrows, k = x.shape
    ws = torch.empty(load().mi355_act_q8k_bytes(k, nrows), dtype=torch.uint8, device=x.device)
    check(load().mi355_quantize_act_q8k(_stream(), _ptr(x), _ptr(ws), k, nrows, x.stride(0)))
    return ws


def quantize_act_q8k_tiled(x):
    """x f32 [nrows, k] -> the tile-image form of the per-super-block activation quantization"""
    import torch
    nrows, k = x.shape
    ws = torch.empty(load().mi355_act_q8k_tiled_bytes(k, nrows), dtype=torch.uint8, device=x.device)
    check(load().mi355_quantize_act_q8k_tiled(_stream(), _ptr(x), _ptr(ws), k, nrows, x.stride(0)))
    return ws


def kq_unpack_tiles(t, W):
    """W: device-layout uint8 [N, row_bytes] (Q4_K / Q5_K / Q6_K / IQ4_XS) -> tile images of its two int8 planes + per-super-block scales"""
    import torch
    N, rb = W.shape
    K = rb // BLOCK[t][1] * BLOCK[t][0]
    tiles = torch.empty(load().mi355_kq_tiles_bytes(t, N, K), dtype=torch.uint8, device=W.device)
    check(load().mi355_kq_unpack_tiles(_stream(), t, _ptr(W), _ptr(tiles), N, K))
    return tiles


def mul_mat_q8k_tiled_multi(t, tiles_list, act, Ns, K, B, dsts=None, residuals=None):
    """one launch of the wide-tile K-quant GEMM for up to three matrices of type t (a list: one type per matrix) that share `act`
    -> list of f32 [B, N_i]"""
    import torch
    n = len(tiles_list)
    dev = tiles_list[0].device
    if dsts is None:
        dsts = [torch.empty((B, Ni), dtype=torch.float32, device=dev) for Ni in Ns]
    arr = (TiledMat * n)()
    for i in range(n):
        arr[i].tiles, arr[i].dst, arr[i].N, arr[i].dst_stride = tiles_list[i].data_ptr(), dsts[i].data_ptr(), Ns[i], dsts[i].stride(0)
        arr[i].residual = residuals[i].data_ptr() if residuals is not None and residuals[i] is not None else None
    if isinstance(t, (list, tuple)):
        check(load().mi355_mul_mat_q8k_tiled_mixed(_stream(), n, (C.c_int * n)(*t), arr, _ptr(act), K, B))
        return dsts
    ns = (C.c_int64 * n)(*Ns)
    nws = load().mi355_mul_mat_q8k_tiled_multi_ws_bytes(n, ns, K, B)
    ws = torch.empty(max(nws, 16), dtype=torch.uint8, device=dev)
    check(load().mi355_mul_mat_q8k_tiled_multi(_stream(), t, n, arr, _ptr(act), K, B, _ptr(ws) if nws else None, nws))
    return dsts


def mul_mat_q8k_tiled(t, tiles, act, N, K, B, residual=None, split=True, dst=None):
    """the wide-tile K-quant GEMM: tiles from kq_unpack_tiles, act from quantize_act_q8k_tiled -> f32 [B, N]"""
    import torch
    if dst is None:
        dst = torch.empty((B, N), dtype=torch.float32, device=tiles.device)
    nws = load().mi355_mul_mat_q8k_tiled_ws_bytes(N, K, B) if split else 0
    ws = torch.empty(max(nws, 16), dtype=torch.uint8, device=tiles.device)
    check(load().mi355_mul_mat_q8k_tiled(_stream(), t, _ptr(tiles), _ptr(act), _ptr(dst), _ptr(residual) if residual is not None else None,
                                         N, K, B, dst.stride(0), _ptr(ws) if nws else None, nws))
    return dst


def mul_mat_q8k_tiled_norm(t, tiles, act, N, K, B, norm_w, eps, residual=None, split=True, dst=None):
    """the wide-tile K-quant GEMM (+ residual) followed by RMS_NORM * norm_w of its rows -> (dst f32 [B, N], y f32 [B, N], tile image of y)"""
    import torch
    if dst is None:
        dst = torch.empty((B, N), dtype=torch.float32, device=tiles.device)
    y = torch.empty((B, N), dtype=torch.float32, device=tiles.device)
    img = torch.zeros(load().mi355_act_q8k_tiled_bytes(N, B), dtype=torch.uint8, device=tiles.device)
    nws = load().mi355_mul_mat_q8k_tiled_ws_bytes(N, K, B) if split else 0
    ws = torch.empty(max(nws, 16), dtype=torch.uint8, device=tiles.device)
    check(load().mi355_mul_mat_q8k_tiled_norm(_stream(), t, _ptr(tiles), _ptr(act), _ptr(dst), _ptr(residual) if residual is not None else None,
                                              N, K, B, dst.stride(0), _ptr(ws) if nws else None, nws, _ptr(norm_w), eps, _ptr(y), y.stride(0), _ptr(img)))
    return dst, y, img


def mul_mat(t, W, x, ws=None, split=True):
    """W: device-layout uint8 [N, row_bytes]; x f32 [B, K] -> f32 [B, N].  split: also give the workspace the room that lets a
    product with few tiles run as slices along K"""
    import torch
    B, K = x.shape
    N = W.shape[0]
    need = load().mi355_mul_mat_ws_bytes(K, B)
    if split:
        need += max(load().mi355_mul_mat_q_ws_bytes(N, K, B), load().mi355_mul_mat_q8k_ws_bytes(N, K, B), load().mi355_mul_mat_skinny_ws_bytes(N, K, B),
                    load().mi355_mul_mat_mid_ws_bytes(N, K, B))
    if ws is None or ws.numel() < need:
        ws = torch.empty(need, dtype=torch.uint8, device=x.device)
    dst = torch.empty((B, N), dtype=torch.float32, device=x.device)
    check(load().mi355_mul_mat(_stream(), t, _ptr(W), _ptr(x), _ptr(dst), N, K, B, x.stride(0), N, _ptr(ws), ws.numel()))
    return dst


def mul_mat_static(t, W, x, dst):
    """mi355_mul_mat on the library's own per-GPU scratch array: the call allocates nothing (dst comes from the caller)"""
    B, K = x.shape
    N = W.shape[0]
    check(load().mi355_mul_mat_static(_stream(), t, _ptr(W), _ptr(x), _ptr(dst), N, K, B, x.stride(0), dst.stride(0)))
    return dst


def mul_mat_skinny(t, W, x, residual=None, split=True):
    """The weight-streaming matrix-core product for 1..32 activation rows (every weight type): W device layout [N, row_bytes],
    x f32 [B, K] -> f32 [B, N] (+ residual [B, N]).  split: give it the workspace that lets few rows run as slices along K"""
    import torch
    B, K = x.shape
    N = W.shape[0]
    act = quantize_act(x)
    nws = load().mi355_mul_mat_skinny_ws_bytes(N, K, B) if split else 0
    ws = torch.empty(max(nws, 16), dtype=torch.uint8, device=x.device)
    dst = torch.empty((B, N), dtype=torch.float32, device=x.device)
    check(load().mi355_mul_mat_skinny(_stream(), t, _ptr(W), _ptr(act), _ptr(dst), _ptr(residual) if residual is not None else None,
                                      N, K, B, N, _ptr(ws) if nws else None, nws))
    return dst


def mul_mat_mid(t, W, x, residual=None, split=True):
    """The weight-streaming matrix-core product for 33..128 activation rows (Q4_K): W device layout [N, row_bytes], x f32 [B, K]
    -> f32 [B, N] (+ residual [B, N]).  split: give it the workspace that lets few rows run as slices along K"""
    import torch
    B, K = x.shape
    N = W.shape[0]
    act = quantize_act_q8k_tiled(x)
    nws = load().mi355_mul_mat_mid_ws_bytes(N, K, B) if split else 0
    ws = torch.empty(max(nws, 16), dtype=torch.uint8, device=x.device)
    dst = torch.empty((B, N), dtype=torch.float32, device=x.device)
    check(load().mi355_mul_mat_mid(_stream(), t, _ptr(W), _ptr(act), _ptr(dst), _ptr(residual) if residual is not None else None,
                                   N, K, B, N, _ptr(ws) if nws else None, nws))
    return dst


def mul_mat_mid_multi(t, Ws, x, residuals=None, split=True):
    """mul_mat_mid for up to three matrices on one activation in one launch -> list of f32 [B, N_i]"""
    import torch
    B, K = x.shape
    n = len(Ws)
    act = quantize_act_q8k_tiled(x)
    Ns = [W.shape[0] for W in Ws]
    dsts = [torch.empty((B, N), dtype=torch.float32, device=x.device) for N in Ns]
    arr = (GemvMat * n)()
    for i in range(n):
        arr[i].type, arr[i].W, arr[i].N, arr[i].dst, arr[i].dst_stride = t, Ws[i].data_ptr(), Ns[i], dsts[i].data_ptr(), Ns[i]
        arr[i].residual = residuals[i].data_ptr() if residuals is not None and residuals[i] is not None else None
    nws = load().mi355_mul_mat_mid_multi_ws_bytes(n, (C.c_int64 * n)(*Ns), K, B) if split else 0
    ws = torch.empty(max(nws, 16), dtype=torch.uint8, device=x.device)
    check(load().mi355_mul_mat_mid_multi(_stream(), t, n, arr, _ptr(act), K, B, _ptr(ws) if nws else None, nws))
    return dsts


def block_dots(t, W, x_row):
    """integer granule dots of every row of W against the Q8_1 quantization of x_row (f32 [K])"""
    import torch
    K = x_row.numel()
    N = W.shape[0]
    act = quantize_act(x_row.reshape(1, K))
    g = 16 if t == Q6_K else 32
    out = torch.empty((N, K // g), dtype=torch.int32, device=W.device)
    check(load().mi355_block_dots_q8_1(_stream(), t, _ptr(W), _ptr(act), _ptr(out), N, K))
    return out


def mul_mat_id(t, as_dev, b, ids, n_used):
    """as_dev uint8 [n_expert, N, row_bytes] device layout; b f32 [T, nb1, K]; ids int32 [T, >=n_used] (row-strided)
    -> f32 [T, n_used, N]"""
    import torch
    n_expert, N, _ = as_dev.shape
    T, nb1, K = b.shape
    need = load().mi355_mul_mat_id_ws_bytes(K, n_expert, n_used, nb1, T)
    ws = torch.empty(need, dtype=torch.uint8, device=b.device)
    dst = torch.empty((T, n_used, N), dtype=torch.float32, device=b.device)
    check(load().mi355_mul_mat_id(_stream(), t, _ptr(as_dev), _ptr(b), _ptr(ids), ids.stride(0), _ptr(dst), N, K,
                                  n_expert, n_used, nb1, T, _ptr(ws), ws.numel()))
    return dst


def kq_unpack_expert_tiles(t, as_dev):
    """as_dev uint8 [n_expert, N, row_bytes] device layout -> uint8 [n_expert, tile image bytes]: every expert's tile images"""
    import torch
    n_expert, N, rb = as_dev.shape
    K = rb // BLOCK[t][1] * BLOCK[t][0]
    per = (load().mi355_kq_tiles_bytes(t, N, K) + 255) // 256 * 256
    out = torch.empty((n_expert, per), dtype=torch.uint8, device=as_dev.device)
    for e in range(n_expert):
        check(load().mi355_kq_unpack_tiles(_stream(), t, _ptr(as_dev[e]), _ptr(out[e]), N, K))
    return out


def mul_mat_id_tiled(t, expert_tiles, N, b, ids, n_used):
    """expert_tiles from kq_unpack_expert_tiles; b f32 [T, nb1, K]; ids int32 [T, >=n_used] (row-strided) -> f32 [T, n_used, N]"""
    import torch
    n_expert = expert_tiles.shape[0]
    T, nb1, K = b.shape
    need = load().mi355_mul_mat_id_q8k_tiled_ws_bytes(K, n_expert, n_used, T)
    ws = torch.empty(need, dtype=torch.uint8, device=b.device)
    dst = torch.empty((T, n_used, N), dtype=torch.float32, device=b.device)
    check(load().mi355_mul_mat_id_q8k_tiled(_stream(), t, _ptr(expert_tiles), expert_tiles.stride(0), _ptr(b), _ptr(ids), ids.stride(0), _ptr(dst), N, K,
                                            n_expert, n_used, nb1, T, _ptr(ws), ws.numel()))
    return dst


def flash_attn_ext(q, k, v, mask, scale, max_bias=0.0, softcap=0.0, quantized=False, workspace=True):
    """q f32 [Hq, Nq, D] (any head/row strides), k,v f16 [Hkv, Nkv, D], mask f16 [>=Nq, Nkv] or None -> f32 [Nq, Hq, D]
    (quantized=True: also returns the Q8_1 activation workspace of the output rows)"""
    import torch
    Hq, Nq, D = q.shape
    Hkv, Nkv, _ = k.shape
    assert q.stride(2) == 1 and k.stride(2) == 1 and v.stride(2) == 1
    need = load().mi355_flash_attn_ws_bytes(D, Nq, Nkv, Hq)
    ws = torch.empty(min(need, 1 << 28) if workspace else 0, dtype=torch.uint8, device=q.device)   # none: no kv splits, no mask pre-pass
    dst = torch.empty((Nq, Hq, D), dtype=torch.float32, device=q.device)
    args = (_stream(), _ptr(q), _ptr(k), _ptr(v), _ptr(mask), _ptr(dst), D, Nq, Nkv, Hq, Hkv,
            q.stride(1) * 4, q.stride(0) * 4, k.stride(1) * 2, k.stride(0) * 2,
            v.stride(1) * 2, v.stride(0) * 2, mask.stride(0) * 2 if mask is not None else 0,
            scale, max_bias, softcap, _ptr(ws) if workspace else None, ws.numel())
    if quantized:
        act = torch.empty(load().mi355_act_bytes(Hq * D, Nq), dtype=torch.uint8, device=q.device)
        check(load().mi355_flash_attn_ext_quant(*args, _ptr(act)))
        return dst, act
    check(load().mi355_flash_attn_ext(*args))
    return dst
