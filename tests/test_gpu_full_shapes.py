"""GPU parity at the full Llama-3-8B / Mixtral-8x7B operator shapes: the launch code picks its kernel instantiation from the
size of the product (rows per wave from 8192 / 32768 rows on, the activation copied to LDS from 1536 groups on), so the
instantiations that serve the real models are only reached by products of the real size.  Every case holds a 512-row slice from
each end of the matrix to the oracle's exact-integer formulation (NMSE < 1e-9: only f32 summation order remains) and EVERY output
to the reference CPU backend (NMSE <= 5e-4, tests/test-backend-ops.cpp:1916)."""
import ctypes as C

import numpy as np
import pytest

import orc

pytestmark = pytest.mark.gpu

MAIN = (orc.Q4_0, orc.Q8_0, orc.Q4_K, orc.Q6_K)
TYPES = list(orc.WEIGHT_TYPES.items())


def _t(dev, a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def _weights(rng, t, N, K, std=0.02):
    assert orc.ref is not None, "the reference build (oracle/_ref) is the whole-output check of these tests"
    Wf = rng.standard_normal((N, K), dtype=np.float32) * np.float32(std)
    return orc.quantize_mt("ref", t, Wf)


def _gemv(dev, t, Wd, x):
    """mi355_mul_mat_vec_q on the Q8_1 quantization of x: f32 [B, K] -> f32 [B, N]"""
    import torch
    import mi355
    B, K = x.shape
    N = Wd.shape[0]
    act = mi355.quantize_act(_t(dev, x))
    dst = torch.full((B, N), float("nan"), dtype=torch.float32, device=dev)
    mi355.check(mi355.load().mi355_mul_mat_vec_q(None, t, Wd.data_ptr(), act.data_ptr(), dst.data_ptr(), N, K, B, N))
    torch.cuda.synchronize()
    return dst.cpu().numpy()


def _check_slices(got, t, Wq, x, tol=1e-9):
    """both ends of the matrix against the oracle's integer dots with f64 scale algebra"""
    N = Wq.shape[0]
    n = min(512, N)
    assert orc.nmse(got[:, :n], orc.mul_mat("q8_1", t, Wq[:n], x)) < tol
    assert orc.nmse(got[:, N - n:], orc.mul_mat("q8_1", t, Wq[N - n:], x)) < tol


@pytest.mark.parametrize("name,t", TYPES)
@pytest.mark.parametrize("N,K", [(14336, 4096), (4096, 14336), (128256, 4096)])
def test_gemv_llama8b_shapes(dev, name, t, N, K):
    """ffn_gate / ffn_up, ffn_down and the output projection at batch 1..8 through mi355_mul_mat_vec_q (the four path types at
    every batch, the further types at batch 1 and 8)"""
    import mi355
    rng = np.random.default_rng(N + K + t)
    Wq = _weights(rng, t, N, K)
    Wd = mi355.upload_weights(t, _t(dev, Wq))
    for B in ((1, 2, 3, 4, 8) if t in MAIN else (1, 8)):
        x = rng.standard_normal((B, K)).astype(np.float32)
        got = _gemv(dev, t, Wd, x)
        assert np.isfinite(got).all(), B
        _check_slices(got, t, Wq, x)
        assert orc.nmse(got, orc.mul_mat("ref", t, Wq, x, n_threads=16)) <= 5e-4, B


@pytest.mark.parametrize("tg,tu", [(orc.Q4_K, orc.Q4_K), (orc.Q4_K, orc.Q6_K), (orc.Q4_0, orc.Q8_0), (orc.Q5_K, orc.IQ4_NL)])
def test_gate_up_one_launch_llama8b(dev, tg, tu):
    """ffn_gate + ffn_up of an 8B llama (2 x 14336 x 4096) as one launch of mi355_mul_mat_vec_q_multi, batch 1..4: the launch a
    decoded token makes once per layer; every matrix also equals its own single-matrix launch bit for bit"""
    import torch
    import mi355
    lib = mi355.load()
    N, K = 14336, 4096
    rng = np.random.default_rng(tg * 31 + tu)
    Wq = [_weights(rng, t, N, K) for t in (tg, tu)]
    Wd = [mi355.upload_weights(t, _t(dev, W)) for t, W in zip((tg, tu), Wq)]
    for B in (1, 2, 4):
        x = rng.standard_normal((B, K)).astype(np.float32)
        act = mi355.quantize_act(_t(dev, x))
        outs = [torch.full((B, N), float("nan"), dtype=torch.float32, device=dev) for _ in range(2)]
        arr = (mi355.GemvMat * 2)()
        for i, t in enumerate((tg, tu)):
            arr[i].type, arr[i].W, arr[i].N, arr[i].dst, arr[i].dst_stride, arr[i].residual = t, Wd[i].data_ptr(), N, outs[i].data_ptr(), N, None
        mi355.check(lib.mi355_mul_mat_vec_q_multi(None, 2, arr, act.data_ptr(), K, B))
        torch.cuda.synchronize()
        for i, t in enumerate((tg, tu)):
            got = outs[i].cpu().numpy()
            _check_slices(got, t, Wq[i], x)
            assert orc.nmse(got, orc.mul_mat("ref", t, Wq[i], x, n_threads=16)) <= 5e-4
            if B < 4:   # a single matrix at batch 4 goes to the matrix-core kernel: other summation order
                assert np.array_equal(got, _gemv(dev, t, Wd[i], x))


@pytest.mark.parametrize("t", [orc.Q4_K, orc.Q6_K, orc.Q4_0])
def test_gate_up_swiglu_one_launch_llama8b(dev, t):
    """ffn_gate + ffn_up + SiLU * up + Q8_1 of an 8B llama layer in one launch (mi355_ffn_gate_up_swiglu; a group owns a 32-row block
    of both matrices): gate and up hold the bits of the two-matrix product launch, the activation the bits of SiLU * up + Q8_1 as
    their own launch, and the products match the oracle and the reference CPU backend"""
    import torch
    import mi355
    lib = mi355.load()
    N, K = 14336, 4096
    rng = np.random.default_rng(100 + t)
    Wq = [_weights(rng, t, N, K) for _ in range(2)]
    Wd = [mi355.upload_weights(t, _t(dev, W)) for W in Wq]
    tickets = torch.zeros(N // 32 + 1, dtype=torch.int32, device=dev)
    for B in (1, 2, 4):
        x = rng.standard_normal((B, K)).astype(np.float32)
        act = mi355.quantize_act(_t(dev, x))
        g0, u0 = (torch.full((B, N), float("nan"), dtype=torch.float32, device=dev) for _ in range(2))
        arr = (mi355.GemvMat * 2)()
        for i, out in enumerate((g0, u0)):
            arr[i].type, arr[i].W, arr[i].N, arr[i].dst, arr[i].dst_stride, arr[i].residual = t, Wd[i].data_ptr(), N, out.data_ptr(), N, None
        mi355.check(lib.mi355_mul_mat_vec_q_multi(None, 2, arr, act.data_ptr(), K, B))
        a0 = torch.zeros(lib.mi355_act_bytes(N, B), dtype=torch.uint8, device=dev)
        mi355.check(lib.mi355_swiglu_quant(None, g0.data_ptr(), u0.data_ptr(), N, None, 0, a0.data_ptr(), N, B))
        g1, u1 = (torch.full((B, N), float("nan"), dtype=torch.float32, device=dev) for _ in range(2))
        a1 = torch.zeros_like(a0)
        mi355.check(lib.mi355_ffn_gate_up_swiglu(None, t, Wd[0].data_ptr(), t, Wd[1].data_ptr(), act.data_ptr(), g1.data_ptr(), u1.data_ptr(), N,
                                                 a1.data_ptr(), tickets.data_ptr(), N, K, B))
        torch.cuda.synchronize()
        assert torch.equal(g1, g0) and torch.equal(u1, u0) and torch.equal(a1, a0), B
        for out, W in ((g1, Wq[0]), (u1, Wq[1])):
            got = out.cpu().numpy()
            _check_slices(got, t, W, x)
            assert orc.nmse(got, orc.mul_mat("ref", t, W, x, n_threads=16)) <= 5e-4


@pytest.mark.parametrize("tq,tk,tv", [(orc.Q4_K, orc.Q4_K, orc.Q6_K), (orc.Q4_K, orc.Q4_K, orc.Q4_K), (orc.Q4_0, orc.Q4_0, orc.Q8_0)])
def test_norm_qkv_rope_store_llama8b(dev, tq, tk, tv):
    """attention norm + Q/K/V + ROPE + cache store of an 8B llama layer (d 4096, 32 / 8 heads of 128) in one launch: bit-identical to
    norm, products, ROPE and SET_ROWS as separate launches, and q / the cache rows against the oracle's arithmetic"""
    import torch
    import mi355
    lib = mi355.load()
    K, H, HK, D, n_ctx = 4096, 32, 8, 128, 64
    rng = np.random.default_rng(tq + 7 * tv)
    x = rng.standard_normal((1, K)).astype(np.float32)
    nw = (1 + 0.1 * rng.standard_normal(K)).astype(np.float32)
    Wq = [_weights(rng, t, N, K, 0.05) for t, N in ((tq, H * D), (tk, HK * D), (tv, HK * D))]
    Ws = [mi355.upload_weights(t, _t(dev, W)) for t, W in zip((tq, tk, tv), Wq)]
    xd, nwd = _t(dev, x), _t(dev, nw)
    pos, cells = _t(dev, np.array([37], dtype=np.int32)), _t(dev, np.array([11], dtype=np.int32))
    rope = (D, 0, 8192, 500000.0, 1.0, 0.0, 1.0, 32.0, 1.0)

    def caches():
        return (torch.zeros(n_ctx, HK, D, dtype=torch.float16, device=dev), torch.zeros(n_ctx, HK, D, dtype=torch.float16, device=dev))

    # separate launches
    y = torch.empty(1, K, device=dev)
    act = torch.zeros(lib.mi355_act_bytes(K, 1), dtype=torch.uint8, device=dev)
    mi355.check(lib.mi355_rms_norm_mul_quant(None, xd.data_ptr(), K, nwd.data_ptr(), y.data_ptr(), K, act.data_ptr(), K, 1, 1e-5))
    outs = [torch.zeros(1, W.shape[0], device=dev) for W in Ws]
    arr = (mi355.GemvMat * 3)()
    for i, (t, W, out) in enumerate(zip((tq, tk, tv), Ws, outs)):
        arr[i].type, arr[i].W, arr[i].N, arr[i].dst, arr[i].dst_stride, arr[i].residual = t, W.data_ptr(), out.shape[1], out.data_ptr(), out.shape[1], None
    mi355.check(lib.mi355_mul_mat_vec_q_multi(None, 3, arr, act.data_ptr(), K, 1))
    plain = [o.cpu().numpy().copy() for o in outs]
    kc0, vc0 = caches()
    mi355.check(lib.mi355_rope_kv_store(None, outs[0].data_ptr(), outs[1].data_ptr(), outs[2].data_ptr(), kc0.data_ptr(), vc0.data_ptr(), pos.data_ptr(),
                                        cells.data_ptr(), None, 1, H, HK, D, kc0.stride(0) * 2, kc0.stride(1) * 2, vc0.stride(0) * 2, vc0.stride(1) * 2, *rope))
    # one launch
    q1 = torch.zeros(1, H * D, device=dev)
    kc1, vc1 = caches()
    mi355.check(lib.mi355_rms_norm_qkv_rope_store(None, xd.data_ptr(), nwd.data_ptr(), 1e-5, tq, Ws[0].data_ptr(), tk, Ws[1].data_ptr(), tv, Ws[2].data_ptr(),
                                                  q1.data_ptr(), kc1.data_ptr(), vc1.data_ptr(), pos.data_ptr(), cells.data_ptr(), None, K, H, HK, D,
                                                  kc1.stride(0) * 2, kc1.stride(1) * 2, vc1.stride(0) * 2, vc1.stride(1) * 2, *rope))
    torch.cuda.synchronize()
    assert torch.equal(q1, outs[0]) and torch.equal(kc1, kc0) and torch.equal(vc1, vc0)
    # the products against the oracle on the normalised row the device produced, then its ROPE
    yn = y.cpu().numpy()
    for t, W, p in zip((tq, tk, tv), Wq, plain):
        assert orc.nmse(p, orc.mul_mat("q8_1", t, W, yn)) < 1e-9
        assert orc.nmse(p, orc.mul_mat("ref", t, W, yn, n_threads=16)) <= 5e-4
    qr = np.zeros((1, H, D), dtype=np.float32)
    posn = np.array([37], dtype=np.int32)
    orc.oracle.orc_rope(orc._ptr(np.ascontiguousarray(plain[0].reshape(1, H, D))), orc._ptr(posn), None, orc._ptr(qr), D, H, 1, D, 0, 500000.0, 1.0, 0.0, 1.0, 32.0, 1.0, 8192)
    assert orc.nmse(q1.cpu().numpy().reshape(1, H, D), qr) < 1e-7
    assert np.array_equal(vc1.cpu().numpy()[11].reshape(-1), plain[2].reshape(-1).astype(np.float16))
    assert kc1.cpu().numpy()[11].any() and not kc1.cpu().numpy()[:11].any()


@pytest.mark.parametrize("name,t", [(n, t) for n, t in TYPES if t in MAIN])
@pytest.mark.parametrize("B", [64, 512])
def test_mul_mat_4096x4096_batches(dev, name, t, B):
    """the attention-output shape of BASELINE config 1 at batch 64 and 512, whole output against the reference CPU backend"""
    import mi355
    N = K = 4096
    rng = np.random.default_rng(B + t)
    Wq = _weights(rng, t, N, K)
    Wd = mi355.upload_weights(t, _t(dev, Wq))
    x = rng.standard_normal((B, K)).astype(np.float32)
    got = mi355.mul_mat(t, Wd, _t(dev, x)).cpu().numpy()
    kind = "cpu" if t in (orc.Q4_K, orc.Q6_K) else "q8_1"     # K-quant batches compute in the CPU path's Q8_K activation format
    assert orc.nmse(got[:24, :64], orc.mul_mat(kind, t, Wq[:64], x[:24])) < 1e-9
    assert orc.nmse(got[B - 3:, N - 9:], orc.mul_mat(kind, t, Wq[N - 9:], x[B - 3:])) < 1e-9
    assert orc.nmse(got, orc.mul_mat("ref", t, Wq, x, n_threads=16)) <= 5e-4


@pytest.mark.parametrize("N,K", [(14336, 4096), (4096, 14336)])
@pytest.mark.parametrize("T", [1, 512])
def test_mul_mat_id_mixtral_shapes(dev, N, K, T):
    """MUL_MAT_ID at the expert shapes of BASELINE config 4: 8 experts of 14336 x 4096 (gate / up) and 4096 x 14336 (down) in Q4_K,
    2 used per token, one decoded token (per-slot GEMV) and a 512-token prompt (routed tile GEMM); semantics of
    tests/test-backend-ops.cpp:4089-4119, every output against the reference CPU backend"""
    import torch
    import mi355
    t, n_expert, n_used = orc.Q4_K, 8, 2
    rng = np.random.default_rng(N + T)
    Wq = _weights(rng, t, n_expert * N, K)
    nb1 = 1 if N > K else n_used                  # gate / up broadcast the token's row over its slots, down has a row per slot
    b = rng.standard_normal((T, nb1, K)).astype(np.float32)
    ids_full = np.stack([rng.permutation(n_expert) for _ in range(T)]).astype(np.int32)
    Wd = mi355.upload_weights(t, _t(dev, Wq)).reshape(n_expert, N, -1)
    idd = _t(dev, ids_full)[:, :n_used]
    got = mi355.mul_mat_id(t, Wd, _t(dev, b), idd, n_used).cpu().numpy()
    assert np.isfinite(got).all()
    cpu = np.zeros((T, n_used, N), dtype=np.float32)
    assert orc.ref.ref_mul_mat_id(t, orc._ptr(Wq), orc._ptr(b), orc._ptr(ids_full), orc._ptr(cpu), N, K, n_expert, n_used, nb1, T, 16, 0) >= 0
    assert orc.nmse(got, cpu) <= 5e-4           # tests/test-backend-ops.cpp:2001
    # the exact-integer form on a slice of rows from both ends of every expert the tokens use
    kind = "cpu" if T * n_used >= 32 else "q8_1"   # routed tiles compute in the CPU path's Q8_K format, per-slot GEMVs in Q8_1
    for ex in range(n_expert):
        where = [(tt, e) for tt in range(min(T, 64)) for e in range(n_used) if ids_full[tt, e] == ex]
        if not where:
            continue
        rows = np.stack([b[tt, e % nb1] for tt, e in where])
        for lo in (0, N - 48):
            want = orc.mul_mat(kind, t, Wq[ex * N + lo:ex * N + lo + 48], rows)
            have = np.stack([got[tt, e, lo:lo + 48] for tt, e in where])
            assert orc.nmse(have, want) < 1e-9, (ex, lo)


def test_decode_attention_32768_cells_unscaled(dev):
    """BASELINE config 2's longest decode shape exactly as stated (q ~ N(0,1), 32768 cells, 32 / 8 heads of 128): held to the
    textbook form in f64.  (The reference CPU backend's own f16 accumulator is 6.7e-4 from exact on this input, above the operator
    tolerance, so the comparison with it uses scaled queries in test_gpu_flash_attn.py.)"""
    import mi355
    rng = np.random.default_rng(32769)
    Nkv, Hq, Hkv, D = 32768, 32, 8, 128
    q = rng.standard_normal((Hq, 1, D)).astype(np.float32)
    k = rng.standard_normal((Hkv, Nkv, D)).astype(np.float16)
    v = rng.standard_normal((Hkv, Nkv, D)).astype(np.float16)
    mask = np.zeros((64, Nkv), dtype=np.float16)
    scale = 1.0 / np.sqrt(D)
    got = mi355.flash_attn_ext(_t(dev, q), _t(dev, k), _t(dev, v), _t(dev, mask), scale).cpu().numpy()     # [1, 32, 128]
    qh = q.astype(np.float16).astype(np.float64)
    full = np.empty((1, Hq, D))
    for h in range(Hq):
        s_ = qh[h] @ k[h // 4].astype(np.float64).T * scale
        p = np.exp(s_ - s_.max(axis=1, keepdims=True))
        full[:, h] = (p / p.sum(axis=1, keepdims=True)) @ v[h // 4].astype(np.float64)
    assert orc.nmse(got, full) < 1e-5


def test_runner_full_width_decode_equals_node_sequence(dev):
    """two layers at the full width of an 8B llama (d 4096, ffn 14336, 32 / 8 heads, vocabulary 128256): the decode launch sequence
    (7 launches per layer, the instantiations the timed step uses) against the node-for-node sequence"""
    import torch
    from mi355 import llama_graph as lg
    cfg = lg.LlamaConfig(n_layer=2, n_ctx=256)
    w = lg.LlamaWeights(cfg, dev, seed=3)
    run = lg.LlamaRunner(w, max_tokens=16)
    emb = torch.randn(16, cfg.n_embd, generator=torch.Generator().manual_seed(5)).pin_memory()
    run.set_inputs(emb, 0, 9, 256)
    run.forward_nodes(9, 256)                      # a short prompt fills the cache
    for pos0 in (9, 10):
        run.set_inputs(emb[pos0:], pos0, 1, 256)
        a = run.forward_nodes(1, 256).cpu().numpy().copy()
        run.set_inputs(emb[pos0:], pos0, 1, 256)
        b = run.forward(1, 256).cpu().numpy().copy()
        assert np.isfinite(a).all() and a.shape == (1, cfg.n_vocab)
        # the same integer dots and f32 chains per row in both sequences; the SILU node uses the library's expf and division, the
        # SiLU * up launch the hardware's exp and reciprocal forms, so a few activation levels of ffn_down's input differ
        assert orc.nmse(b, a) < 1e-6
