"""Writes the small golden fixtures under tests/golden/ from the REFERENCE's own quantizers and CPU
backend (oracle/_ref, built from the reference sources by oracle/Makefile).  Run in the build
container (`python tests/golden/make_fixtures.py`); the fixtures are data only: seeded inputs and
the reference's outputs for them, so the oracle can be pinned where the reference is absent.

  quant_<type>.npz   : x f32 [4,512]; q = reference quantization bytes; dq = reference dequantization
  q8_1_special.npz   : hand-made blocks (zeros, single +-amax, .5 ties) and quantize_row_q8_1_ref bytes
  mul_mat_<type>.npz : W bytes [48,512], x f32 [3,512], y = reference CPU MUL_MAT output
  flash_attn.npz     : q,k,v,mask for D=64, Nq=3, Nkv=40, Hq=4, Hkv=2 and the reference CPU output
  flash_attn_alibi_softcap.npz : 6 query heads over 3 kv heads, the reference CPU outputs with max_bias = 8 and with logit_softcap = 10
  flash_attn_kv_types.npz : D=64, 4 query heads over 2 kv heads; reference CPU outputs for K and V each of f16, Q8_0, Q4_0
  glue.npz           : inputs/outputs of RMS_NORM, SOFT_MAX, ROPE (modes 0 and 2), SILU, ARGSORT
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import orc  # noqa: E402


def main():
    assert orc.ref is not None, "build oracle/_ref first (make -C oracle ref refdriver)"
    rng = np.random.default_rng(20240607)
    K = 512
    first_types = [(n, t) for n, t in orc.WEIGHT_TYPES.items() if n in ("q4_0", "q8_0", "q4_K", "q6_K")]   # the stream below was laid out for these
    for name, t in first_types + [("q8_1", orc.Q8_1), ("q8_K", orc.Q8_K)]:
        x = (rng.standard_normal((4, K)) * (0.02 if name not in ("q8_1", "q8_K") else 1.0)).astype(np.float32)
        x[0, :32] = 0
        q = orc.quantize("ref", t, x)
        out = {"x": x, "q": q}
        if t not in (orc.Q8_1, orc.Q8_K):
            out["dq"] = orc.dequantize("ref", t, q, K)
        np.savez_compressed(os.path.join(HERE, "quant_%s.npz" % name), **out)

    sp = np.zeros((1, 32 * 5), dtype=np.float32)
    sp[0, 32 + 5] = -3.25
    sp[0, 64:96] = np.concatenate([[127.0], np.arange(31) - 15 + 0.5])
    sp[0, 96:128] = 1e-30
    sp[0, 128:160] = np.linspace(-7e4, 7e4, 32)
    np.savez_compressed(os.path.join(HERE, "q8_1_special.npz"), x=sp, q=orc.quantize("ref", orc.Q8_1, sp))

    for name, t in first_types:
        W = orc.quantize("ref", t, (rng.standard_normal((48, K)) * 0.02).astype(np.float32))
        x = rng.standard_normal((3, K)).astype(np.float32)
        np.savez_compressed(os.path.join(HERE, "mul_mat_%s.npz" % name), W=W, x=x, y=orc.mul_mat("ref", t, W, x))

    # weight types added later draw from a generator of their own, so that the files above keep their contents
    for seed, (name, t) in enumerate([(n, t) for n, t in orc.WEIGHT_TYPES.items() if (n, t) not in first_types]):
        r2 = np.random.default_rng(20240610 + seed)
        x = (r2.standard_normal((4, K)) * 0.02).astype(np.float32)
        x[0, :32] = 0
        q = orc.quantize("ref", t, x)
        np.savez_compressed(os.path.join(HERE, "quant_%s.npz" % name), x=x, q=q, dq=orc.dequantize("ref", t, q, K))
        W = orc.quantize("ref", t, (r2.standard_normal((48, K)) * 0.02).astype(np.float32))
        xa = r2.standard_normal((3, K)).astype(np.float32)
        np.savez_compressed(os.path.join(HERE, "mul_mat_%s.npz" % name), W=W, x=xa, y=orc.mul_mat("ref", t, W, xa))

    D, Nq, Nkv, Hq, Hkv = 64, 3, 40, 4, 2
    q = rng.standard_normal((Hq, Nq, D)).astype(np.float32)
    k = rng.standard_normal((Hkv, Nkv, D)).astype(np.float16)
    v = rng.standard_normal((Hkv, Nkv, D)).astype(np.float16)
    mask = rng.uniform(-1, 1, (64, Nkv)).astype(np.float32)
    mask[:, 30:] = -np.inf
    mask[1, 5] = -np.inf
    mask = mask.astype(np.float16)
    y = orc.flash_attn("ref", q, k.view(np.uint16), v.view(np.uint16), mask.view(np.uint16), 0.125)
    np.savez_compressed(os.path.join(HERE, "flash_attn.npz"), q=q, k=k.view(np.uint16), v=v.view(np.uint16), mask=mask.view(np.uint16),
                        y=y, scale=np.float32(0.125))
    # the ALiBi (max_bias > 0: per-head slopes on the mask) and logit soft-cap branches of the same kernel; 6 heads make
    # n_head_log2 = 4 < n_head, so both slope formulas are exercised
    Hq2, Hkv2 = 6, 3
    rng2 = np.random.default_rng(20240608)   # its own stream: the fixtures below keep their inputs
    q2 = rng2.standard_normal((Hq2, Nq, D)).astype(np.float32)
    k2 = rng2.standard_normal((Hkv2, Nkv, D)).astype(np.float16)
    v2 = rng2.standard_normal((Hkv2, Nkv, D)).astype(np.float16)
    y_alibi = orc.flash_attn("ref", q2, k2.view(np.uint16), v2.view(np.uint16), mask.view(np.uint16), 0.125, max_bias=8.0)
    y_cap = orc.flash_attn("ref", q2, k2.view(np.uint16), v2.view(np.uint16), mask.view(np.uint16), 0.125, softcap=10.0)
    np.savez_compressed(os.path.join(HERE, "flash_attn_alibi_softcap.npz"), q=q2, k=k2.view(np.uint16), v=v2.view(np.uint16),
                        mask=mask.view(np.uint16), y_alibi=y_alibi, y_softcap=y_cap, scale=np.float32(0.125), max_bias=np.float32(8.0),
                        softcap=np.float32(10.0))

    # a quantized KV cache: every pairing of f16, Q8_0 and Q4_0 for K and V (q is quantized to Q8_0 for a quantized K, V rows are
    # dequantized into an f32 accumulator)
    rng3 = np.random.default_rng(20240609)
    D3, Nq3, Nkv3, Hq3, Hkv3 = 64, 3, 40, 4, 2
    q3 = rng3.standard_normal((Hq3, Nq3, D3)).astype(np.float32)
    kf3 = rng3.standard_normal((Hkv3, Nkv3, D3)).astype(np.float32)
    vf3 = rng3.standard_normal((Hkv3, Nkv3, D3)).astype(np.float32)
    out3 = {"q": q3, "kf": kf3, "vf": vf3, "mask": mask.view(np.uint16), "scale": np.float32(0.125)}
    for tk in (orc.F16, orc.Q8_0, orc.Q4_0):
        for tv in (orc.F16, orc.Q8_0, orc.Q4_0):
            out3["y_%d_%d" % (tk, tv)] = orc.flash_attn_kv("ref", q3, orc.kv_rows(tk, kf3), tk, orc.kv_rows(tv, vf3), tv, mask.view(np.uint16), 0.125)
    np.savez_compressed(os.path.join(HERE, "flash_attn_kv_types.npz"), **out3)

    g = {}
    x = rng.standard_normal((5, 96)).astype(np.float32)
    y = np.zeros_like(x)
    orc.ref.ref_rms_norm(orc._ptr(x), orc._ptr(y), 96, 5, 1e-5, 2)
    g["rms_x"], g["rms_y"] = x, y.copy()
    m = rng.standard_normal((5, 96)).astype(np.float32)
    orc.ref.ref_soft_max(orc._ptr(x), orc._ptr(m), orc._ptr(y), 96, 5, 0.7, 2)
    g["sm_mask"], g["sm_y"] = m, y.copy()
    orc.ref.ref_silu(orc._ptr(x), orc._ptr(y), x.size, 2)
    g["silu_y"] = y.copy()
    xr = rng.standard_normal((6, 4, 64)).astype(np.float32)
    pos = np.array([0, 1, 7, 100, 2047, 4095], dtype=np.int32)
    for mode in (0, 2):
        yr = np.zeros_like(xr)
        orc.ref.ref_rope(orc._ptr(xr), orc._ptr(pos), None, orc._ptr(yr), 64, 4, 6, 32, mode, 500000.0, 1.0, 0.0, 1.0, 32.0, 1.0, 8192, 2)
        g["rope_y%d" % mode] = yr
    ff = (1 + rng.uniform(0, 1, 16)).astype(np.float32)
    yr = np.zeros_like(xr)
    orc.ref.ref_rope(orc._ptr(xr), orc._ptr(pos), orc._ptr(ff), orc._ptr(yr), 64, 4, 6, 32, 0, 10000.0, 0.5, 1.0, 1.0, 32.0, 1.0, 4096, 2)
    g["rope_x"], g["rope_pos"], g["rope_ff"], g["rope_y_yarn"] = xr, pos, ff, yr
    a = np.stack([rng.permutation(24) for _ in range(4)]).astype(np.float32)
    idx = np.zeros((4, 24), dtype=np.int32)
    orc.ref.ref_argsort(orc._ptr(a), orc._ptr(idx), 24, 4, 1, 2)
    g["argsort_x"], g["argsort_desc"] = a, idx
    np.savez_compressed(os.path.join(HERE, "glue.npz"), **g)
    print("fixtures written to", HERE)


if __name__ == "__main__":
    main()
