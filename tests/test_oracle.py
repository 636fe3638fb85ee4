"""Pins the CPU oracle (oracle/oracle.c) without a GPU:
  * against the golden fixtures under tests/golden/ (outputs of the reference's own quantizers and
    CPU backend on seeded inputs),
  * against the reference build itself where oracle/_ref exists,
  * against what the mathematics fixes: closed-form special cases, brute force on the integer
    levels, dequantize-then-dot in double, textbook softmax attention with repeated kv heads."""
import os

import numpy as np
import pytest

import orc

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
ALL_Q = list(orc.WEIGHT_TYPES.items()) + [("q8_1", orc.Q8_1), ("q8_K", orc.Q8_K)]
needs_ref = pytest.mark.skipif(orc.ref is None, reason="oracle/_ref not built (needs the llama.cpp tree)")


def gold(name):
    return np.load(os.path.join(GOLD, name))


def test_oracle_library_present():
    assert orc.oracle is not None, "build oracle/liboracle.so (make -C oracle oracle)"


# ------------------------------------------------------------------ fp16
def test_f16_round_trip_and_rounding():
    halves = np.arange(65536, dtype=np.uint16)
    f = np.zeros(65536, dtype=np.float32)
    orc.oracle.orc_f16_to_f32_row(orc._ptr(halves), orc._ptr(f), 65536)
    ref = halves.view(np.float16).astype(np.float32)
    ok = np.isnan(ref) | (f.view(np.uint32) == ref.view(np.uint32))
    assert ok.all()
    fin = np.isfinite(ref)
    back = np.zeros(65536, dtype=np.uint16)
    orc.oracle.orc_f32_to_f16_row(orc._ptr(f), orc._ptr(back), 65536)
    assert np.array_equal(back[fin], halves[fin])                       # exact values survive
    # ties between neighbouring halves go to the even one; numpy's float16 cast is IEEE RNE too
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(100000).astype(np.float32) * s for s in (1e-8, 1e-6, 1e-3, 1, 300, 7e4)] +
                       [((f[:-1].astype(np.float64) + f[1:].astype(np.float64)) / 2).astype(np.float32)[fin[:-1] & fin[1:]]])
    x = np.ascontiguousarray(x[np.isfinite(x)])
    got = np.zeros(x.size, dtype=np.uint16)
    orc.oracle.orc_f32_to_f16_row(orc._ptr(x), orc._ptr(got), x.size)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(got, want)


@needs_ref
def test_f16_vs_reference():
    rng = np.random.default_rng(1)
    x = np.ascontiguousarray(np.concatenate([rng.standard_normal(50000).astype(np.float32) * s for s in (1e-7, 1e-4, 1, 1e3, 1e5)]))
    a = np.zeros(x.size, dtype=np.uint16)
    b = np.zeros(x.size, dtype=np.uint16)
    orc.oracle.orc_f32_to_f16_row(orc._ptr(x), orc._ptr(a), x.size)
    orc.ref.ref_fp32_to_fp16_row(orc._ptr(x), orc._ptr(b), x.size)
    assert np.array_equal(a, b)


# ------------------------------------------------------------------ quantizers
@pytest.mark.parametrize("name,t", ALL_Q)
def test_quantizers_match_golden(name, t):
    g = gold("quant_%s.npz" % name)
    q = orc.quantize("oracle", t, g["x"])
    assert np.array_equal(q, g["q"])
    if "dq" in g:
        assert np.array_equal(orc.dequantize("oracle", t, g["q"], g["x"].shape[1]).view(np.uint32), g["dq"].view(np.uint32))


@needs_ref
@pytest.mark.parametrize("name,t", ALL_Q)
@pytest.mark.parametrize("scale", [0.02, 1.0, 300.0])
def test_quantizers_match_reference_bytes(name, t, scale):
    rng = np.random.default_rng(int(scale * 100) + t)
    x = (rng.standard_normal((6, 1024)) * scale).astype(np.float32)
    x[1, 256:512] = 0
    x[2] = rng.uniform(-scale, scale, 1024)
    assert np.array_equal(orc.quantize("oracle", t, x), orc.quantize("ref", t, x))


def test_q8_1_special_cases():
    g = gold("q8_1_special.npz")
    q = orc.quantize("oracle", orc.Q8_1, g["x"])
    assert np.array_equal(q, g["q"])
    blocks = q.reshape(-1, 36)
    assert not blocks[0].any()                                           # zero block: d = 0, s = 0, q = 0
    b1 = blocks[1]
    assert b1[4 + 5].view(np.int8) == -127 and np.count_nonzero(b1[4:]) == 1   # single -amax -> level -127
    assert b1[:2].view(np.float16)[0] == np.float16(3.25 / 127)
    lv = blocks[2][4:].view(np.int8)                                     # d = 1: .5 ties round away from zero
    want = np.concatenate([[127], np.where(np.arange(31) - 15 + 0.5 > 0, np.arange(31) - 15 + 1, np.arange(31) - 15)])
    assert np.array_equal(lv, want.astype(np.int8))
    # s = fp16(d * sum q)
    d = blocks[2][:2].view(np.float16)[0].astype(np.float32)
    assert blocks[2][2:4].view(np.float16)[0] == np.float16(np.float32(lv.astype(np.int32).sum()) * np.float32(127.0 / 127))
    assert d == 1.0


@pytest.mark.parametrize("name,t", list(orc.WEIGHT_TYPES.items()))
def test_round_trip_error_within_reference_threshold(name, t):
    """tests/test-quantize-fns.cpp:17-35: data 0.1 + 2cos(i + offset), RMSE of quantize->dequantize <= 0.002"""
    n = 4096
    x = (0.1 + 2.0 * np.cos(np.arange(n) + 0.0)).astype(np.float32)[None, :]
    q = orc.quantize("oracle", t, x)
    dq = orc.dequantize("oracle", t, q, n)
    rmse = np.sqrt(np.sum((dq - x) ** 2)) / n
    assert rmse <= 0.002


# ------------------------------------------------------------------ integer dots / mul_mat
def _levels(t, W, K):
    """integer level of every weight element with its fixed offset removed, via float dequantization with unit scales
    is not possible for K-quants, so recompute from the byte layout independently of oracle.c"""
    N = W.shape[0]
    if t == orc.Q4_0:
        b = W.reshape(N, K // 32, 18)[:, :, 2:]
        return np.concatenate([(b & 15).astype(np.int32) - 8, (b >> 4).astype(np.int32) - 8], axis=2).reshape(N, K)
    if t == orc.Q8_0:
        return W.reshape(N, K // 32, 34)[:, :, 2:].view(np.int8).astype(np.int32).reshape(N, K)
    if t in (orc.Q4_1, orc.IQ4_NL):
        b = W.reshape(N, K // 32, orc.BLOCK[t][1])[:, :, -16:]
        n = np.concatenate([(b & 15), (b >> 4)], axis=2).astype(np.int32).reshape(N, K)
        return n if t == orc.Q4_1 else np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], dtype=np.int32)[n]
    if t in (orc.Q5_0, orc.Q5_1):
        blk = W.reshape(N, K // 32, orc.BLOCK[t][1])
        b = blk[:, :, -16:]
        qh = np.ascontiguousarray(blk[:, :, -20:-16]).view("<u4")                        # [N, nb, 1]: bit j = fifth bit of element j
        bits = ((qh >> np.arange(32, dtype=np.uint32).reshape(1, 1, 32)) & 1).astype(np.int32)
        n = np.concatenate([(b & 15), (b >> 4)], axis=2).astype(np.int32) + 16 * bits
        return (n - (16 if t == orc.Q5_0 else 0)).reshape(N, K)
    if t == orc.IQ4_XS:
        b = W.reshape(N, K // 256, 136)[:, :, 8:].reshape(N, K // 32, 16)
        n = np.concatenate([(b & 15), (b >> 4)], axis=2).astype(np.int32).reshape(N, K)
        return np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], dtype=np.int32)[n]
    if t == orc.Q4_K:
        qs = W.reshape(N, K // 256, 144)[:, :, 16:].reshape(N, K // 256, 4, 32)
        return np.concatenate([(qs & 15), (qs >> 4)], axis=3).astype(np.int32).reshape(N, K)
    if t == orc.Q5_K:
        blk = W.reshape(N, K // 256, 176)
        qs = blk[:, :, 48:].reshape(N, K // 256, 4, 32)
        qh = blk[:, :, 16:48].reshape(N, K // 256, 1, 32)
        g = np.arange(4, dtype=np.uint8).reshape(1, 1, 4, 1)
        lo = (qs & 15) | (((qh >> (2 * g)) & 1) << 4)        # sub-block 2g: bit 2g of qh
        hi = (qs >> 4) | (((qh >> (2 * g + 1)) & 1) << 4)    # sub-block 2g + 1: bit 2g + 1
        return np.concatenate([lo, hi], axis=3).astype(np.int32).reshape(N, K)
    blk = W.reshape(N, K // 256, 210)
    ql = blk[:, :, :128].reshape(N, -1, 2, 64)
    qh = blk[:, :, 128:192].reshape(N, -1, 2, 32)
    q1 = (ql[..., :32] & 15) | ((qh & 3) << 4)
    q2 = (ql[..., 32:] & 15) | (((qh >> 2) & 3) << 4)
    q3 = (ql[..., :32] >> 4) | (((qh >> 4) & 3) << 4)
    q4 = (ql[..., 32:] >> 4) | (((qh >> 6) & 3) << 4)
    return (np.concatenate([q1, q2, q3, q4], axis=3).astype(np.int32) - 32).reshape(N, K)


@pytest.mark.parametrize("name,t", list(orc.WEIGHT_TYPES.items()))
def test_block_dots_brute_force(name, t):
    rng = np.random.default_rng(5)
    N, K = 7, 1024
    W = rng.integers(0, 256, (N, orc.row_bytes(t, K)), dtype=np.uint8)
    x = rng.standard_normal((1, K)).astype(np.float32)
    a = orc.quantize("oracle", orc.Q8_1, x)
    aq = a.reshape(K // 32, 36)[:, 4:].view(np.int8).astype(np.int32).reshape(K)
    g = 16 if t == orc.Q6_K else 32
    want = (_levels(t, W, K) * aq[None, :]).reshape(N, K // g, g).sum(axis=2)
    assert np.array_equal(orc.block_dots(t, W, a[0], K), want.astype(np.int32))


@pytest.mark.parametrize("name,t", list(orc.WEIGHT_TYPES.items()))
def test_mul_mat_matches_golden_and_f64(name, t):
    g = gold("mul_mat_%s.npz" % name)
    W, x, y = g["W"], g["x"], g["y"]
    cpu = orc.mul_mat("cpu", t, W, x)
    assert orc.nmse(cpu, y) < 1e-10                     # same algorithm as the reference CPU path (SIMD summation order aside)
    dev = orc.mul_mat("q8_1", t, W, x)
    assert orc.nmse(dev, y) <= 5e-4                     # the device formulation differs only by activation format
    f64 = orc.mul_mat("f64", t, W, x)
    assert orc.nmse(dev, f64) <= 5e-4 and orc.nmse(cpu, f64) <= 5e-4
    # linearity in x for the exact path
    f2 = orc.mul_mat("f64", t, W, 2 * x)
    assert orc.nmse(f2, 2 * f64) < 1e-12


@needs_ref
@pytest.mark.parametrize("name,t", list(orc.WEIGHT_TYPES.items()))
def test_mul_mat_vs_reference_cpu(name, t):
    rng = np.random.default_rng(9)
    W = orc.quantize("ref", t, (rng.standard_normal((96, 2048)) * 0.02).astype(np.float32))
    x = rng.standard_normal((4, 2048)).astype(np.float32)
    r = orc.mul_mat("ref", t, W, x)
    assert orc.nmse(orc.mul_mat("cpu", t, W, x), r) < 1e-10
    assert orc.nmse(orc.mul_mat("q8_1", t, W, x), r) <= 5e-4


def test_mul_mat_id_reduces_to_mul_mat():
    rng = np.random.default_rng(10)
    t, N, K, E, U, T = orc.Q4_K, 16, 512, 4, 2, 3
    W = orc.quantize("oracle", t, (rng.standard_normal((E * N, K)) * 0.02).astype(np.float32))
    b = rng.standard_normal((T, 1, K)).astype(np.float32)
    ids = np.stack([rng.permutation(E) for _ in range(T)]).astype(np.int32)
    out = np.zeros((T, U, N), dtype=np.float32)
    assert orc.oracle.orc_mul_mat_id_q8_1(t, orc._ptr(W), orc._ptr(b), orc._ptr(ids), E, orc._ptr(out), N, K, E, U, 1, T) == 0
    for tt in range(T):
        for e in range(U):
            ex = ids[tt, e]
            want = orc.mul_mat("q8_1", t, W[ex * N:(ex + 1) * N], b[tt])
            assert np.array_equal(out[tt, e], want[0])


# ------------------------------------------------------------------ flash attention
def test_flash_attn_golden_and_textbook():
    g = gold("flash_attn.npz")
    q, k, v, mask, y = g["q"], g["k"], g["v"], g["mask"], g["y"]
    scale = float(g["scale"])
    cpu = orc.flash_attn("cpu", q, k, v, mask, scale)
    f64 = orc.flash_attn("f64", q, k, v, mask, scale)
    assert orc.nmse(cpu, y) < 1e-6                      # same algorithm; the f16 accumulator makes it order sensitive
    assert orc.nmse(f64, y) <= 5e-4
    # textbook form in numpy, kv heads repeated over their query heads (grouped-query attention)
    kf = k.view(np.float16).astype(np.float64)
    vf = v.view(np.float16).astype(np.float64)
    mf = mask.view(np.float16).astype(np.float64)
    Hq, Nq, D = q.shape
    rep = Hq // kf.shape[0]
    out = np.zeros((Nq, Hq, D))
    for h in range(Hq):
        s = q[h].astype(np.float64) @ kf[h // rep].T * scale + mf[:Nq]
        p = np.exp(s - s.max(axis=1, keepdims=True))
        p /= p.sum(axis=1, keepdims=True)
        out[:, h] = p @ vf[h // rep]
    assert orc.nmse(f64, out) < 1e-12


def test_flash_attn_alibi_and_softcap_golden():
    """the ALiBi slopes (ggml-cpu.c:10979-10995: m0 / m1 powers by head index) and the logit soft-cap (tanh) of the oracle against
    outputs of the reference build, and against the textbook form with the slope / cap written out"""
    g = gold("flash_attn_alibi_softcap.npz")
    q, k, v, mask, scale = g["q"], g["k"], g["v"], g["mask"], float(g["scale"])
    Hq, Nq, D = q.shape
    kf, vf = k.view(np.float16).astype(np.float64), v.view(np.float16).astype(np.float64)
    mf = mask.view(np.float16).astype(np.float64)
    rep = Hq // kf.shape[0]
    for key, max_bias, softcap in (("y_alibi", float(g["max_bias"]), 0.0), ("y_softcap", 0.0, float(g["softcap"]))):
        cpu = orc.flash_attn("cpu", q, k, v, mask, scale, max_bias, softcap)
        f64 = orc.flash_attn("f64", q, k, v, mask, scale, max_bias, softcap)
        assert orc.nmse(cpu, g[key]) < 1e-6
        assert orc.nmse(f64, g[key]) <= 5e-4
        n2 = 1 << int(np.floor(np.log2(Hq)))
        m0, m1 = 2.0 ** (-max_bias / n2), 2.0 ** (-max_bias / 2.0 / n2)
        out = np.zeros((Nq, Hq, D))
        for h in range(Hq):
            slope = 1.0 if max_bias == 0.0 else (m0 ** (h + 1) if h < n2 else m1 ** (2 * (h - n2) + 1))
            s = q[h].astype(np.float64) @ kf[h // rep].T * scale
            if softcap != 0.0:
                s = softcap * np.tanh(s / softcap)
            s = s + slope * mf[:Nq]
            p = np.exp(s - s.max(axis=1, keepdims=True))
            p /= p.sum(axis=1, keepdims=True)
            out[:, h] = p @ vf[h // rep]
        assert orc.nmse(f64, out) < 1e-10


def test_flash_attn_quantized_kv_golden():
    """the oracle over a Q8_0 / Q4_0 KV cache (q quantized to Q8_0 and integer block dots for a quantized K, f32 accumulator over
    dequantized rows for a quantized V; ggml-cpu.c:10997-11003, 11040-11099) against committed outputs of the reference build, and
    against the textbook form on the dequantized cache (which the q quantization leaves ~2e-5 away)"""
    g = gold("flash_attn_kv_types.npz")
    q, kf, vf, mask, scale = g["q"], g["kf"], g["vf"], g["mask"], float(g["scale"])
    Hq, Nq, D = q.shape
    Hkv, Nkv = kf.shape[0], kf.shape[1]
    mf = mask.view(np.float16).astype(np.float64)
    for tk in (orc.F16, orc.Q8_0, orc.Q4_0):
        for tv in (orc.F16, orc.Q8_0, orc.Q4_0):
            k, v = orc.kv_rows(tk, kf), orc.kv_rows(tv, vf)
            got = orc.flash_attn_kv("cpu", q, k, tk, v, tv, mask, scale)
            assert orc.nmse(got, g["y_%d_%d" % (tk, tv)]) < 1e-6, (tk, tv)

            def deq(a, t):
                if t == orc.F16:
                    return a.view(np.float16).astype(np.float64).reshape(Hkv, Nkv, D)
                return orc.dequantize("oracle", t, a.reshape(Hkv * Nkv, -1), D).reshape(Hkv, Nkv, D).astype(np.float64)
            kd, vd = deq(k, tk), deq(v, tv)
            out = np.zeros((Nq, Hq, D))
            for h in range(Hq):
                s = q[h].astype(np.float64) @ kd[h // 2].T * scale + mf[:Nq]
                p = np.exp(s - s.max(axis=1, keepdims=True))
                out[:, h] = (p / p.sum(axis=1, keepdims=True)) @ vd[h // 2]
            assert orc.nmse(got, out) < 2e-4, (tk, tv)
    # with f16 K and V it is the kernel of orc_flash_attn_cpu
    k16, v16 = orc.kv_rows(orc.F16, kf), orc.kv_rows(orc.F16, vf)
    a = orc.flash_attn_kv("cpu", q, k16, orc.F16, v16, orc.F16, mask, scale)
    b = orc.flash_attn("cpu", q, k16.view(np.uint16).reshape(Hkv, Nkv, D), v16.view(np.uint16).reshape(Hkv, Nkv, D), mask, scale)
    assert np.array_equal(a, b)


# ------------------------------------------------------------------ glue ops
def test_glue_golden():
    g = gold("glue.npz")
    x = g["rms_x"]
    y = np.zeros_like(x)
    orc.oracle.orc_rms_norm(orc._ptr(x), orc._ptr(y), x.shape[1], x.shape[0], 1e-5)
    assert orc.nmse(y, g["rms_y"]) < 1e-12
    want = x / np.sqrt((x.astype(np.float64) ** 2).mean(axis=1, keepdims=True) + 1e-5)
    assert orc.nmse(y, want) < 1e-12
    m = g["sm_mask"]
    orc.oracle.orc_soft_max(orc._ptr(x), orc._ptr(m), orc._ptr(y), x.shape[1], x.shape[0], 0.7)
    assert orc.nmse(y, g["sm_y"]) < 1e-10
    assert np.allclose(y.sum(axis=1), 1.0, atol=1e-6)
    orc.oracle.orc_silu(orc._ptr(x), orc._ptr(y), x.size)
    assert orc.nmse(y, g["silu_y"]) < 1e-10
    xr, pos = g["rope_x"], g["rope_pos"]
    yr = np.zeros_like(xr)
    for mode in (0, 2):
        orc.oracle.orc_rope(orc._ptr(xr), orc._ptr(pos), None, orc._ptr(yr), 64, 4, 6, 32, mode, 500000.0, 1.0, 0.0, 1.0, 32.0, 1.0, 8192)
        assert orc.nmse(yr, g["rope_y%d" % mode]) < 1e-12
        assert np.array_equal(yr[:, :, 32:], xr[:, :, 32:])             # dims beyond n_dims pass through
        assert np.allclose((yr ** 2).sum(axis=2), (xr ** 2).sum(axis=2), rtol=1e-5)   # rotations keep the norm
        assert np.array_equal(yr[0], xr[0])                               # position 0 is the identity
    ff = g["rope_ff"]
    orc.oracle.orc_rope(orc._ptr(xr), orc._ptr(pos), orc._ptr(ff), orc._ptr(yr), 64, 4, 6, 32, 0, 10000.0, 0.5, 1.0, 1.0, 32.0, 1.0, 4096)
    assert orc.nmse(yr, g["rope_y_yarn"]) < 1e-12
    a = g["argsort_x"]
    idx = np.zeros(a.shape, dtype=np.int32)
    orc.oracle.orc_argsort(orc._ptr(a), orc._ptr(idx), a.shape[1], a.shape[0], 1)
    assert np.array_equal(idx, g["argsort_desc"])
    assert np.array_equal(idx, np.argsort(-a, axis=1).astype(np.int32))
