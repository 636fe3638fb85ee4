"""GPU parity of activation quantization, integer block dots, GEMV and the MFMA GEMM against
the CPU oracle (and, where it has been built, the reference's own CPU backend)."""
import numpy as np
import pytest

import orc

pytestmark = pytest.mark.gpu

TYPES = list(orc.WEIGHT_TYPES.items())


def _weights(rng, t, N, K, kind="oracle"):
    Wf = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    return orc.quantize("ref" if (kind == "ref" and orc.ref is not None) else "oracle", t, Wf)


def _to_dev(dev, a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


@pytest.mark.parametrize("K", [32, 256, 4096, 14336])
@pytest.mark.parametrize("dist", ["normal", "uniform", "special"])
def test_quantize_q8_1_bit_exact(dev, K, dist):
    import mi355
    rng = np.random.default_rng(7 + K)
    nrows = 5
    if dist == "normal":
        x = rng.standard_normal((nrows, K)).astype(np.float32)
    elif dist == "uniform":
        x = rng.uniform(-1, 1, (nrows, K)).astype(np.float32)
    else:
        x = rng.standard_normal((nrows, K)).astype(np.float32)
        x[0, :32] = 0.0                      # all-zero block: d = 0, q = 0, s = 0
        x[1, :32] = 0.0
        x[1, 5] = -3.25                      # single -amax: that level is exactly -127
        x[2, :32] = np.concatenate([[127.0], np.arange(31) - 15 + 0.5])   # d = 1: x*id lands on .5 ties (away from zero)
        x[3, :32] = 1e-30                    # tiny but non-zero scale
        x[4, :32] = 65504.0 * 100            # d overflows fp16 -> inf in the d field
    got = mi355.quantize_q8_1(_to_dev(dev, x)).cpu().numpy()
    want = orc.quantize("oracle", orc.Q8_1, x)
    assert np.array_equal(got, want)
    if orc.ref is not None:
        assert np.array_equal(got, orc.quantize("ref", orc.Q8_1, x))


@pytest.mark.parametrize("name,t", TYPES)
@pytest.mark.parametrize("K", [256, 2048, 4096])
def test_weight_layout_round_trip(dev, name, t, K):
    """scatter (upload) then gather (read-back) returns the reference's bytes, also for partial ranges"""
    import torch
    import mi355
    rng = np.random.default_rng(11)
    N = 9
    raw = rng.integers(0, 256, (N, orc.row_bytes(t, K)), dtype=np.uint8)
    d_raw = _to_dev(dev, raw)
    d_dev = mi355.upload_weights(t, d_raw)
    back = mi355.download_weights(t, d_dev).cpu().numpy()
    assert np.array_equal(back, raw)
    # partial range, not block aligned
    lib = mi355.load()
    total = raw.size
    off, size = 37, total - 101
    part = torch.zeros(size, dtype=torch.uint8, device=dev)
    mi355.check(lib.mi355_weights_gather(None, t, d_dev.data_ptr(), part.data_ptr(), K, N, off, size))
    torch.cuda.synchronize()
    assert np.array_equal(part.cpu().numpy(), raw.reshape(-1)[off:off + size])
    d2 = torch.zeros_like(d_dev)
    mi355.check(lib.mi355_weights_scatter(None, t, d_raw.reshape(-1)[:off].contiguous().data_ptr(), d2.data_ptr(), K, N, 0, off))
    mi355.check(lib.mi355_weights_scatter(None, t, d_raw.reshape(-1)[off:].contiguous().data_ptr(), d2.data_ptr(), K, N, off, total - off))
    torch.cuda.synchronize()
    assert torch.equal(d2, d_dev)


@pytest.mark.parametrize("name,t", TYPES)
@pytest.mark.parametrize("K", [2048, 4096, 14336])
def test_block_dots_bit_exact(dev, name, t, K):
    import mi355
    rng = np.random.default_rng(3)
    N = 33
    Wq = _weights(rng, t, N, K)
    x = rng.standard_normal((1, K)).astype(np.float32)
    Wd = mi355.upload_weights(t, _to_dev(dev, Wq))
    got = mi355.block_dots(t, Wd, _to_dev(dev, x)[0]).cpu().numpy()
    want = orc.block_dots(t, Wq, orc.quantize("oracle", orc.Q8_1, x)[0], K)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("name,t", TYPES)
@pytest.mark.parametrize("N,K", [(4096, 4096), (1024, 14336), (257, 2048), (16, 256)])
@pytest.mark.parametrize("B", [1, 2, 3, 5, 8])
def test_gemv_matches_oracle(dev, name, t, N, K, B):
    import mi355
    rng = np.random.default_rng(N + K + B)
    Nt = min(N, 512)     # the oracle is scalar C: check a slice of rows exactly, all rows through the reference below
    Wq = _weights(rng, t, N, K, "ref")
    x = rng.standard_normal((B, K)).astype(np.float32)
    Wd = mi355.upload_weights(t, _to_dev(dev, Wq))
    got = mi355.mul_mat(t, Wd, _to_dev(dev, x)).cpu().numpy()
    want = orc.mul_mat("q8_1", t, Wq[:Nt], x)
    # same integer dots, f32 vs f64 scale algebra: only summation-order noise remains
    assert orc.nmse(got[:, :Nt], want) < 1e-9
    cpu = orc.mul_mat("ref", t, Wq, x) if orc.ref is not None else orc.mul_mat("cpu", t, Wq[:Nt], x)
    assert orc.nmse(got[:, :cpu.shape[1]], cpu) <= 5e-4      # tests/test-backend-ops.cpp:1916


@pytest.mark.parametrize("K", [256, 4096, 14336])
@pytest.mark.parametrize("dist", ["normal", "special"])
def test_quantize_q8k_bit_exact(dev, K, dist):
    """levels and scale equal block_q8_K of the reference; the sub-block sums are its bsums pairwise"""
    import mi355
    rng = np.random.default_rng(11 + K)
    nrows = 6
    x = rng.standard_normal((nrows, K)).astype(np.float32)
    if dist == "special":
        x[0, :256] = 0.0                       # all-zero super-block: d = 0, levels 0
        x[1, :256] = 0.0
        x[1, 77] = 2.5                         # single +amax: its level is exactly -127 and d is negative
        x[2, 3] = 9.0
        x[2, 200] = -9.0                       # equal magnitudes: the first one decides the sign of the scale
        x[3, :256] = -1e-30
        x[4, :256] = 0.0
        x[4, 0] = -127.0                       # scale exactly 1: the values below are exact .5 ties (round half to even)
        x[4, 1:202] = np.arange(-100, 101) + 0.5
    got = mi355.quantize_act_q8k(_to_dev(dev, x)).cpu().numpy()
    nsb = K // 256
    q = got[:nrows * K].view(np.int8).reshape(nrows, nsb, 256)
    d = got[nrows * K:nrows * K + nrows * nsb * 4].view(np.float32).reshape(nrows, nsb)
    off = (nrows * K + nrows * nsb * 4 + 15) // 16 * 16
    bs = got[off:off + nrows * nsb * 32].view(np.float16).reshape(nrows, nsb, 16).astype(np.int64)
    for kind in ["oracle"] + (["ref"] if orc.ref is not None else []):
        want = orc.quantize(kind, orc.Q8_K, x).reshape(nrows, nsb, 292)
        wd = np.ascontiguousarray(want[:, :, :4]).view(np.float32).reshape(nrows, nsb)
        wq = want[:, :, 4:260].view(np.int8)
        assert np.array_equal(d.view(np.uint32), wd.view(np.uint32))
        assert np.array_equal(q, wq)
        sums = wq.astype(np.int64).reshape(nrows, nsb, 8, 32).sum(axis=3)
        assert np.array_equal(64 * bs[:, :, 8:] + bs[:, :, :8], sums)
        assert bs[:, :, :8].min() >= 0 and bs[:, :, :8].max() <= 63


@pytest.mark.parametrize("name,t", TYPES)
@pytest.mark.parametrize("N,K,B", [(512, 4096, 64), (384, 2048, 512), (130, 1024, 33), (4096, 4096, 9), (128, 14336, 100)])
def test_mmq_matches_oracle(dev, name, t, N, K, B):
    import mi355
    rng = np.random.default_rng(N * 3 + K + B)
    Wq = _weights(rng, t, N, K, "ref")
    x = rng.standard_normal((B, K)).astype(np.float32)
    Wd = mi355.upload_weights(t, _to_dev(dev, Wq))
    got = mi355.mul_mat(t, Wd, _to_dev(dev, x)).cpu().numpy()
    Nt, Bt = min(N, 64), min(B, 24)
    skinny = B <= 32 and K % 256 == 0 and (t != orc.Q6_K or K % 2048 == 0)   # up to 32 activation rows: the weight-streaming kernel, Q8_1 activations
    if B > 8 and not skinny and (t in (orc.Q4_K, orc.Q5_K) or (t == orc.Q6_K and K % 2048 == 0) or
                                 (t == orc.IQ4_XS and B >= 256 and K % 512 == 0)):   # Q6_K / IQ4_XS rows are 16-byte aligned only then
        # K-quants take the activation format of the CPU path (one scale per 256): integer sums are the
        # CPU's own (ggml-cpu-quants.c:6817-6848, 8262-8283), only the f32 summation order differs
        want = orc.mul_mat("cpu", t, Wq[:Nt], x[:Bt])
    else:
        want = orc.mul_mat("q8_1", t, Wq[:Nt], x[:Bt])
    # Q4_1 / Q5_1 batches add "m * d_x * sum(q)" through fp16 operands (fp16 d_x * sum(q) is the `s` field the reference's own dot
    # uses); Q5_K batches on packed rows subtract "dmin * m * d_x * sum(q)" the same way
    assert orc.nmse(got[:Bt, :Nt], want) < (1e-6 if (B > 8 and t in (orc.Q4_1, orc.Q5_1, orc.Q5_K)) else 1e-9)
    if orc.ref is not None:
        cpu = orc.mul_mat("ref", t, Wq, x)
        assert orc.nmse(got, cpu) <= 5e-4


@pytest.mark.parametrize("name,t", TYPES)
@pytest.mark.parametrize("N,K,B", [(100, 256, 5), (257, 1024, 8), (4096, 4096, 13), (1024, 14336, 17), (64, 3584, 24), (333, 2048, 32), (4096, 4096, 1),
                                   (77, 6144, 9)])
@pytest.mark.parametrize("split", [False, True])
def test_skinny_matches_oracle(dev, name, t, N, K, B, split):
    """the weight-streaming matrix-core kernel for a few activation rows: ragged row and batch counts, K that does not divide
    evenly over the four waves, with and without slices along K, with a residual"""
    import mi355
    if t == orc.Q6_K and K % 2048 != 0:
        pytest.skip("Q6_K rows are 16-byte aligned only when K is a multiple of 2048")
    if t == orc.IQ4_XS and K % 512 != 0:
        pytest.skip("IQ4_XS rows (136 bytes per super-block) are 16-byte aligned only when K is a multiple of 512")
    rng = np.random.default_rng(N * 5 + K + B)
    Wq = _weights(rng, t, N, K, "ref")
    x = rng.standard_normal((B, K)).astype(np.float32)
    res = rng.standard_normal((B, N)).astype(np.float32)
    Wd = mi355.upload_weights(t, _to_dev(dev, Wq))
    got = mi355.mul_mat_skinny(t, Wd, _to_dev(dev, x), split=split).cpu().numpy()
    got_res = mi355.mul_mat_skinny(t, Wd, _to_dev(dev, x), residual=_to_dev(dev, res), split=split).cpu().numpy()
    assert np.array_equal(got_res, got + res)
    Nt, Bt = min(N, 64), min(B, 24)
    want = orc.mul_mat("q8_1", t, Wq[:Nt], x[:Bt])
    assert orc.nmse(got[:Bt, :Nt], want) < 1e-9      # exact integer dots; f32 against f64 scale algebra
    if orc.ref is not None:
        assert orc.nmse(got, orc.mul_mat("ref", t, Wq, x)) <= 5e-4      # tests/test-backend-ops.cpp:1916


@pytest.mark.parametrize("N,K,B", [(100, 256, 33), (257, 1024, 64), (4096, 4096, 50), (1024, 14336, 100), (64, 3584, 128), (333, 2048, 96), (77, 6144, 65),
                                   (130, 512, 20), (4096, 4096, 128), (512, 4096, 40)])
@pytest.mark.parametrize("split", [False, True])
def test_mid_matches_oracle(dev, N, K, B, split):
    """the weight-streaming matrix-core kernel for 33..128 activation rows on Q4_K (sub-block scales folded into two int8 operand
    planes): the CPU path's integer sums (ggml-cpu-quants.c:6817-6848) - ragged row and batch counts, both activation halves, K that
    does not divide evenly over the four waves, with and without slices along K, with a residual"""
    import mi355
    t = orc.Q4_K
    rng = np.random.default_rng(N * 5 + K + B)
    Wq = _weights(rng, t, N, K, "ref")
    x = rng.standard_normal((B, K)).astype(np.float32)
    res = rng.standard_normal((B, N)).astype(np.float32)
    Wd = mi355.upload_weights(t, _to_dev(dev, Wq))
    got = mi355.mul_mat_mid(t, Wd, _to_dev(dev, x), split=split).cpu().numpy()
    got_res = mi355.mul_mat_mid(t, Wd, _to_dev(dev, x), residual=_to_dev(dev, res), split=split).cpu().numpy()
    assert np.array_equal(got_res, got + res)
    Nt = min(N, 48)
    assert orc.nmse(got[:, :Nt], orc.mul_mat("cpu", t, Wq[:Nt], x)) < 1e-9          # every activation row, the first weight rows
    assert orc.nmse(got[B - 9:, N - 40:], orc.mul_mat("cpu", t, Wq[N - 40:], x[B - 9:])) < 1e-9
    if orc.ref is not None:
        assert orc.nmse(got, orc.mul_mat("ref", t, Wq, x)) <= 5e-4      # tests/test-backend-ops.cpp:1916
    if B > 32:   # mi355_mul_mat takes this kernel for 33..128 rows
        assert np.array_equal(mi355.mul_mat(t, Wd, _to_dev(dev, x), split=split).cpu().numpy(), got)


@pytest.mark.parametrize("N,K,B,split", [(4096, 4096, 128, True), (4096, 14336, 64, True), (2048, 1024, 100, True), (4096, 4096, 128, False), (8192, 2048, 50, True)])
def test_mid_norm_equals_product_then_norm(dev, N, K, B, split):
    """the 33..128-row product (+ residual) -> RMS_NORM -> MUL(weight) -> tile image as one call: the bits of the product followed by
    the norm launch, in the row, in the normalised row and in the image"""
    import torch
    import mi355
    lib = mi355.load()
    t = orc.Q4_K
    rng = np.random.default_rng(N + K + B)
    xd = _to_dev(dev, rng.standard_normal((B, K)).astype(np.float32))
    act = mi355.quantize_act_q8k_tiled(xd)
    Wd = mi355.upload_weights(t, _to_dev(dev, _weights(rng, t, N, K, "ref")))
    res = _to_dev(dev, rng.standard_normal((B, N)).astype(np.float32))
    nw = _to_dev(dev, rng.standard_normal(N).astype(np.float32))
    want_x = mi355.mul_mat_mid(t, Wd, xd, residual=res, split=split)
    want_y = torch.empty((B, N), dtype=torch.float32, device=dev)
    want_img = torch.zeros(lib.mi355_act_q8k_tiled_bytes(N, B), dtype=torch.uint8, device=dev)
    mi355.check(lib.mi355_rms_norm_mul_quant_q8k_tiled(None, want_x.data_ptr(), N, nw.data_ptr(), want_y.data_ptr(), N, want_img.data_ptr(), N, B, 1e-5))
    got_x = torch.empty((B, N), dtype=torch.float32, device=dev)
    got_y = torch.empty((B, N), dtype=torch.float32, device=dev)
    got_img = torch.zeros_like(want_img)
    nws = lib.mi355_mul_mat_mid_ws_bytes(N, K, B) if split else 0
    ws = torch.empty(max(nws, 16), dtype=torch.uint8, device=dev)
    mi355.check(lib.mi355_mul_mat_mid_norm(None, t, Wd.data_ptr(), act.data_ptr(), got_x.data_ptr(), res.data_ptr(), N, K, B, N, ws.data_ptr() if nws else None, nws,
                                           nw.data_ptr(), 1e-5, got_y.data_ptr(), N, got_img.data_ptr()))
    torch.cuda.synchronize()
    assert np.array_equal(got_x.cpu().numpy(), want_x.cpu().numpy())
    assert np.array_equal(got_y.cpu().numpy(), want_y.cpu().numpy())
    assert np.array_equal(got_img.cpu().numpy(), want_img.cpu().numpy())


@pytest.mark.parametrize("Ns,K,B", [((4096, 1024, 1024), 4096, 128), ((14336, 14336), 4096, 64), ((100, 257, 64), 2048, 100), ((2048, 512), 1024, 40)])
@pytest.mark.parametrize("split", [False, True])
def test_mid_multi_equals_single_launches(dev, Ns, K, B, split):
    """up to three Q4_K matrices on one activation in one launch of the 33..128-row kernel: without slices every matrix has the bits of
    its own launch; with slices (chosen for the launch as a whole) the same integer sums in another f32 order; residuals per matrix"""
    import mi355
    t = orc.Q4_K
    rng = np.random.default_rng(sum(Ns) + K + B)
    x = rng.standard_normal((B, K)).astype(np.float32)
    Wq = [_weights(rng, t, N, K, "ref") for N in Ns]
    Wd = [mi355.upload_weights(t, _to_dev(dev, W)) for W in Wq]
    res = [_to_dev(dev, rng.standard_normal((B, N)).astype(np.float32)) if i != 1 else None for i, N in enumerate(Ns)]
    xd = _to_dev(dev, x)
    alone = [mi355.mul_mat_mid(t, W, xd, split=False).cpu().numpy() for W in Wd]
    multi = [o.cpu().numpy() for o in mi355.mul_mat_mid_multi(t, Wd, xd, split=split)]
    with_res = [o.cpu().numpy() for o in mi355.mul_mat_mid_multi(t, Wd, xd, residuals=res, split=split)]
    for i, N in enumerate(Ns):
        if not split:
            assert np.array_equal(multi[i], alone[i])
        assert orc.nmse(multi[i], alone[i]) < 1e-12
        assert np.array_equal(with_res[i], multi[i] + res[i].cpu().numpy() if res[i] is not None else multi[i])
        Nt = min(N, 40)
        assert orc.nmse(multi[i][:, :Nt], orc.mul_mat("cpu", t, Wq[i][:Nt], x)) < 1e-9
        assert orc.nmse(multi[i][B - 5:, N - 7:], orc.mul_mat("cpu", t, Wq[i][N - 7:], x[B - 5:])) < 1e-9


@pytest.mark.parametrize("name,t", TYPES)
@pytest.mark.parametrize("N,K", [(14336, 4096), (4096, 14336)])
def test_mmq_llama8b_ffn_shapes(dev, name, t, N, K):
    """the FFN products of an 8B llama (gate/up 14336 x 4096, down 4096 x 14336) at batch 64 and 512, whole: every output against
    the reference CPU backend (NMSE <= 5e-4, tests/test-backend-ops.cpp:1916), a 64 x 24 corner and the last rows/columns against
    the oracle's integer arithmetic; the K-quants additionally through their tile images"""
    import mi355
    rng = np.random.default_rng(N + K + t)
    Wq = _weights(rng, t, N, K, "ref")
    Wd = mi355.upload_weights(t, _to_dev(dev, Wq))
    kq = t in (orc.Q4_K, orc.Q5_K, orc.Q6_K, orc.IQ4_XS)
    tiles = mi355.kq_unpack_tiles(t, Wd) if kq else None
    for B in (64, 512):
        x = rng.standard_normal((B, K)).astype(np.float32)
        xd = _to_dev(dev, x)
        got = mi355.mul_mat(t, Wd, xd).cpu().numpy()
        # K-quants (IQ4_XS from 256 rows on) compute in the CPU path's Q8_K format, the others in Q8_1
        kind = "cpu" if (kq and (t != orc.IQ4_XS or B >= 256)) else "q8_1"
        corner = orc.mul_mat(kind, t, Wq[:64], x[:24])
        edge = orc.mul_mat(kind, t, Wq[N - 9:], x[B - 3:])
        tol = 1e-6 if t in (orc.Q4_1, orc.Q5_1, orc.Q5_K) else 1e-9    # the block minimum meets fp16(d_x * sum(q)), as in the reference's dot
        assert orc.nmse(got[:24, :64], corner) < tol
        assert orc.nmse(got[B - 3:, N - 9:], edge) < tol
        assert orc.ref is not None, "the reference build (oracle/_ref) is the whole-output check of this test"
        want = orc.mul_mat("ref", t, Wq, x, n_threads=16)
        assert orc.nmse(got, want) <= 5e-4
        if kq:
            act = mi355.quantize_act_q8k_tiled(xd)
            wide = mi355.mul_mat_q8k_tiled(t, tiles, act, N, K, B).cpu().numpy()
            assert orc.nmse(wide, want) <= 5e-4
            if kind == "cpu":
                assert orc.nmse(wide[:24, :64], corner) < 1e-9
                assert orc.nmse(wide[B - 3:, N - 9:], edge) < 1e-9
                assert orc.nmse(wide, got) < 1e-12      # same integer sums in both tile kernels
            else:
                assert orc.nmse(wide[:24, :64], orc.mul_mat("cpu", t, Wq[:64], x[:24])) < 1e-9


@pytest.mark.parametrize("name,t", [(n, t) for n, t in TYPES if t in (orc.Q4_K, orc.Q6_K)])
@pytest.mark.parametrize("N,K,B", [(256, 4096, 64), (130, 1024, 33)])
def test_mmq_q8_1_path_for_k_quants(dev, name, t, N, K, B):
    """the per-32-block tile kernel stays reachable for K-quants through mi355_mul_mat_q"""
    import mi355
    import torch
    rng = np.random.default_rng(N + K + B)
    Wq = _weights(rng, t, N, K)
    x = rng.standard_normal((B, K)).astype(np.float32)
    Wd = mi355.upload_weights(t, _to_dev(dev, Wq))
    act = mi355.quantize_act(_to_dev(dev, x))
    dst = torch.empty((B, N), dtype=torch.float32, device=dev)
    mi355.check(mi355.load().mi355_mul_mat_q(None, t, Wd.data_ptr(), act.data_ptr(), dst.data_ptr(), N, K, B, N))
    torch.cuda.synchronize()
    tol = 1e-6 if t == orc.Q4_K else 1e-9    # Q4_K adds its min term through fp16 operands
    assert orc.nmse(dst.cpu().numpy()[:24, :64], orc.mul_mat("q8_1", t, Wq[:64], x[:24])) < tol


@pytest.mark.parametrize("name,t", TYPES)
def test_unaligned_rows_fallback(dev, name, t):
    """K for which the device-layout rows are not 16-byte multiples (byte-load kernel)"""
    import mi355
    rng = np.random.default_rng(5)
    be = orc.BLOCK[t][0]
    K = be * 3
    for B in (1, 12, 40):
        Wq = _weights(rng, t, 19, K)
        x = rng.standard_normal((B, K)).astype(np.float32)
        Wd = mi355.upload_weights(t, _to_dev(dev, Wq))
        got = mi355.mul_mat(t, Wd, _to_dev(dev, x)).cpu().numpy()
        # Q4_K rows are always aligned, so B > 32 takes the super-block tile kernel and the CPU's activation format
        # (5..32 rows: the weight-streaming kernel with Q8_1 activations)
        want = orc.mul_mat("cpu" if (t in (orc.Q4_K, orc.Q5_K) and B > 32) else "q8_1", t, Wq, x)
        # Q5_K rows are always aligned too: its batches run the per-32-block tile kernel, whose minimum term goes through fp16 operands
        assert orc.nmse(got, want) < (1e-6 if (t == orc.Q5_K and B > 8) else 1e-9)


KQ_TYPES = [(n, t) for n, t in TYPES if t in (orc.Q4_K, orc.Q6_K)]
TILED_TYPES = [(n, t) for n, t in TYPES if t in (orc.Q4_K, orc.Q5_K, orc.Q6_K, orc.IQ4_XS)]   # types with tile images for the wide-tile GEMM


def _tile_off(row, k, K):
    """byte offset of element (row, k) in a tile image (16 rows x 64 elements per 1 KiB tile, chunk c of row r at c ^ ((r >> 2) & 3))"""
    r, c = row & 15, (k >> 4) & 3
    return ((row >> 4) * (K >> 6) + (k >> 6)) * 1024 + r * 64 + ((c ^ ((r >> 2) & 3)) << 4) + (k & 15)


@pytest.mark.parametrize("K,B", [(256, 5), (4096, 33), (14336, 130)])
def test_quantize_q8k_tiled_bit_exact(dev, K, B):
    """the tile-image form holds the same levels, scales and sub-block sums as block_q8_K of the reference"""
    import mi355
    rng = np.random.default_rng(23 + K)
    x = rng.standard_normal((B, K)).astype(np.float32)
    x[0, :256] = 0.0
    got = mi355.quantize_act_q8k_tiled(_to_dev(dev, x)).cpu().numpy()
    nsb, b16 = K // 256, (B + 15) // 16 * 16
    cb_pad = ((b16 // 16) + 15) // 16 * 16
    rows, ks = np.meshgrid(np.arange(B), np.arange(K), indexing="ij")
    q = got[_tile_off(rows, ks, K)].view(np.int8).reshape(B, nsb, 256)
    aux = got[b16 * K:]
    want = orc.quantize("oracle", orc.Q8_K, x).reshape(B, nsb, 292)
    wd = np.ascontiguousarray(want[:, :, :4]).view(np.float32).reshape(B, nsb)
    wq = want[:, :, 4:260].view(np.int8)
    assert np.array_equal(q, wq)
    sums = wq.astype(np.int64).reshape(B, nsb, 8, 32).sum(axis=3)
    for b in range(B):
        for sb in range(nsb):
            e = aux[(sb * cb_pad + b // 16) * 576:][:576]
            d = e[:64].view(np.float32)[b % 16]
            bs = e[64:].view(np.float16).reshape(16, 16)[b % 16].astype(np.int64)
            assert d.view(np.uint32) == wd[b, sb].view(np.uint32)
            assert np.array_equal(64 * bs[8:] + bs[:8], sums[b, sb])
    if orc.ref is not None:
        assert np.array_equal(want, orc.quantize("ref", orc.Q8_K, x).reshape(B, nsb, 292))


@pytest.mark.parametrize("name,t", TILED_TYPES)
@pytest.mark.parametrize("N,K,B", [(512, 4096, 64), (384, 2048, 512), (130, 2048, 33), (128, 14336, 100), (200, 2048, 77), (1000, 6144, 300),
                                   (200, 2048, 250), (1000, 6144, 450), (4096, 4096, 512)])     # 193+ rows: 256-row column tiles where the last is over half full
@pytest.mark.parametrize("split", [False, True])
def test_mmq_tiled_matches_oracle(dev, name, t, N, K, B, split):
    """the wide-tile K-quant GEMM on tile images: the CPU's own integer sums (ggml-cpu-quants.c:6817-6848, 8262-8283), ragged row and
    batch counts, with and without slices along K, with a residual; against the oracle, ggml-cpu and the 64 x 128 tile kernel"""
    import torch
    import mi355
    rng = np.random.default_rng(N * 7 + K + B)
    Wq = _weights(rng, t, N, K, "ref")
    x = rng.standard_normal((B, K)).astype(np.float32)
    res = rng.standard_normal((B, N)).astype(np.float32)
    Wd = mi355.upload_weights(t, _to_dev(dev, Wq))
    tiles = mi355.kq_unpack_tiles(t, Wd)
    act = mi355.quantize_act_q8k_tiled(_to_dev(dev, x))
    got = mi355.mul_mat_q8k_tiled(t, tiles, act, N, K, B, split=split).cpu().numpy()
    got_res = mi355.mul_mat_q8k_tiled(t, tiles, act, N, K, B, residual=_to_dev(dev, res), split=split).cpu().numpy()
    assert np.array_equal(got_res, got + res)
    if B > 192 and not split:   # the 128 x 256 tile kernel holds the bits of the 128 x 128 one (which a 128-row batch takes)
        a128 = mi355.quantize_act_q8k_tiled(_to_dev(dev, x[B - 128:]))
        assert np.array_equal(got[B - 128:], mi355.mul_mat_q8k_tiled(t, tiles, a128, N, K, 128, split=False).cpu().numpy())
    Nt, Bt = min(N, 64), min(B, 24)
    assert orc.nmse(got[:Bt, :Nt], orc.mul_mat("cpu", t, Wq[:Nt], x[:Bt])) < 1e-9
    # the last rows and columns (partial tiles)
    assert orc.nmse(got[B - 5:, N - 7:], orc.mul_mat("cpu", t, Wq[N - 7:], x[B - 5:])) < 1e-9
    if True:   # the 64 x 128 tile kernel that unpacks the packed rows itself
        old = torch.empty((B, N), dtype=torch.float32, device=dev)
        a2 = mi355.quantize_act_q8k(_to_dev(dev, x))
        mi355.check(mi355.load().mi355_mul_mat_q8k(None, t, Wd.data_ptr(), a2.data_ptr(), old.data_ptr(), N, K, B, N))
        torch.cuda.synchronize()
        assert orc.nmse(got, old.cpu().numpy()) < 1e-12      # same integer sums, f32 summation order only
    if orc.ref is not None:
        assert orc.nmse(got, orc.mul_mat("ref", t, Wq, x)) <= 5e-4      # tests/test-backend-ops.cpp:1916


@pytest.mark.parametrize("name,t", KQ_TYPES)
def test_fused_producers_write_tile_images(dev, name, t):
    """RMS_NORM+MUL and SiLU*up with the tile-image activation output equal the separate quantization of their f32 result"""
    import torch
    import mi355
    lib = mi355.load()
    rng = np.random.default_rng(3)
    B, K = 37, 4096
    x = _to_dev(dev, rng.standard_normal((B, K)).astype(np.float32))
    w = _to_dev(dev, rng.standard_normal(K).astype(np.float32))
    nbytes = lib.mi355_act_q8k_tiled_bytes(K, B)
    y = torch.empty((B, K), dtype=torch.float32, device=dev)
    a1 = torch.zeros(nbytes, dtype=torch.uint8, device=dev)
    mi355.check(lib.mi355_rms_norm_mul_quant_q8k_tiled(None, x.data_ptr(), K, w.data_ptr(), y.data_ptr(), K, a1.data_ptr(), K, B, 1e-5))
    a2 = torch.zeros(nbytes, dtype=torch.uint8, device=dev)
    mi355.check(lib.mi355_quantize_act_q8k_tiled(None, y.data_ptr(), a2.data_ptr(), K, B, K))
    torch.cuda.synchronize()
    rows, ks = np.meshgrid(np.arange(B), np.arange(K), indexing="ij")
    sel = _tile_off(rows, ks, K)
    assert np.array_equal(a1.cpu().numpy()[sel], a2.cpu().numpy()[sel])
    b16 = (B + 15) // 16 * 16
    n1, n2 = a1.cpu().numpy()[b16 * K:], a2.cpu().numpy()[b16 * K:]
    cb_pad = ((b16 // 16) + 15) // 16 * 16
    for sb in range(K // 256):
        for cb in range(b16 // 16):
            nrow = min(16, B - cb * 16)
            e1, e2 = n1[(sb * cb_pad + cb) * 576:][:576], n2[(sb * cb_pad + cb) * 576:][:576]
            assert np.array_equal(e1[:4 * nrow], e2[:4 * nrow]) and np.array_equal(e1[64:64 + 32 * nrow], e2[64:64 + 32 * nrow])
    g = _to_dev(dev, rng.standard_normal((B, K)).astype(np.float32))
    u = _to_dev(dev, rng.standard_normal((B, K)).astype(np.float32))
    a3 = torch.zeros(nbytes, dtype=torch.uint8, device=dev)
    mi355.check(lib.mi355_swiglu_quant_q8k_tiled(None, g.data_ptr(), u.data_ptr(), K, y.data_ptr(), K, a3.data_ptr(), K, B))
    a4 = torch.zeros(nbytes, dtype=torch.uint8, device=dev)
    mi355.check(lib.mi355_quantize_act_q8k_tiled(None, y.data_ptr(), a4.data_ptr(), K, B, K))
    torch.cuda.synchronize()
    assert np.array_equal(a3.cpu().numpy()[sel], a4.cpu().numpy()[sel])


@pytest.mark.parametrize("types,Ns,K,B", [((orc.Q4_K, orc.Q4_K, orc.Q6_K), (4096, 1024, 1024), 4096, 512),   # Q, K, V of the Q4_K_M mix
                                          ((orc.Q6_K, orc.Q5_K, orc.Q4_K), (1000, 8300, 130), 2048, 300),    # ragged rows and batch
                                          ((orc.Q6_K, orc.Q4_K), (14336, 14336), 4096, 512),                  # 896 tiles
                                          ((orc.Q6_K, orc.Q6_K), (520, 130), 2048, 200),                       # Q6_K only: the form without a min term
                                          ((orc.IQ4_XS, orc.IQ4_XS, orc.Q5_K), (1024, 260, 512), 2048, 300),  # Q, K, V of an IQ4_XS file
                                          ((orc.IQ4_XS, orc.Q6_K), (520, 130), 2048, 200)])                    # both without minima
def test_mmq_tiled_mixed_types(dev, types, Ns, K, B):
    """matrices of different K-quant types in one launch of the wide-tile GEMM: every matrix equals its own launch bit for bit, with
    and without a residual, and the oracle's integer arithmetic at the corners"""
    import mi355
    rng = np.random.default_rng(sum(Ns) + K + B + sum(types))
    x = rng.standard_normal((B, K)).astype(np.float32)
    act = mi355.quantize_act_q8k_tiled(_to_dev(dev, x))
    Wq = [_weights(rng, t, N, K, "ref") for t, N in zip(types, Ns)]
    tiles = [mi355.kq_unpack_tiles(t, mi355.upload_weights(t, _to_dev(dev, W))) for t, W in zip(types, Wq)]
    res = [_to_dev(dev, rng.standard_normal((B, N)).astype(np.float32)) if i != 1 else None for i, N in enumerate(Ns)]
    alone = [mi355.mul_mat_q8k_tiled(t, tl, act, N, K, B, split=False).cpu().numpy() for t, tl, N in zip(types, tiles, Ns)]
    mixed = [o.cpu().numpy() for o in mi355.mul_mat_q8k_tiled_multi(list(types), tiles, act, list(Ns), K, B)]
    with_res = [o.cpu().numpy() for o in mi355.mul_mat_q8k_tiled_multi(list(types), tiles, act, list(Ns), K, B, residuals=res)]
    for i, (t, N) in enumerate(zip(types, Ns)):
        assert np.array_equal(mixed[i], alone[i])
        assert np.array_equal(with_res[i], mixed[i] + res[i].cpu().numpy() if res[i] is not None else mixed[i])
        Nt, Bt = min(N, 40), min(B, 16)
        assert orc.nmse(mixed[i][:Bt, :Nt], orc.mul_mat("cpu", t, Wq[i][:Nt], x[:Bt])) < 1e-9
        assert orc.nmse(mixed[i][B - 5:, N - 7:], orc.mul_mat("cpu", t, Wq[i][N - 7:], x[B - 5:])) < 1e-9


@pytest.mark.parametrize("name,t", TILED_TYPES)
@pytest.mark.parametrize("N,K,B,split", [(4096, 4096, 512, True),       # wo of an 8B llama: cut along K, the sum launch carries the norm
                                         (4096, 14336, 512, True),      # ffn_down
                                         (2048, 2048, 300, True),       # ragged batch
                                         (4096, 4096, 512, False),      # no workspace: uncut, the norm is its own launch
                                         (4096, 2048, 2048, True),      # enough tiles: uncut
                                         (8192, 2048, 200, True)])      # rows longer than the fused form takes
def test_mmq_tiled_norm_equals_product_then_norm(dev, name, t, N, K, B, split):
    """MUL_MAT (+ residual) -> RMS_NORM -> MUL(weight) -> tile image as one call: the bits of the product followed by the norm launch,
    in the row, in the normalised row and in every byte of the image that the norm launch writes"""
    import torch
    import mi355
    lib = mi355.load()
    rng = np.random.default_rng(N + K + B + t)
    x = rng.standard_normal((B, K)).astype(np.float32)
    act = mi355.quantize_act_q8k_tiled(_to_dev(dev, x))
    tiles = mi355.kq_unpack_tiles(t, mi355.upload_weights(t, _to_dev(dev, _weights(rng, t, N, K, "ref"))))
    res = _to_dev(dev, rng.standard_normal((B, N)).astype(np.float32))
    nw = _to_dev(dev, rng.standard_normal(N).astype(np.float32))
    for residual in (res, None):
        want_x = mi355.mul_mat_q8k_tiled(t, tiles, act, N, K, B, residual=residual, split=split)
        want_y = torch.empty((B, N), dtype=torch.float32, device=dev)
        want_img = torch.zeros(lib.mi355_act_q8k_tiled_bytes(N, B), dtype=torch.uint8, device=dev)
        mi355.check(lib.mi355_rms_norm_mul_quant_q8k_tiled(None, want_x.data_ptr(), N, nw.data_ptr(), want_y.data_ptr(), N, want_img.data_ptr(), N, B, 1e-5))
        got_x, got_y, got_img = mi355.mul_mat_q8k_tiled_norm(t, tiles, act, N, K, B, nw, 1e-5, residual=residual, split=split)
        torch.cuda.synchronize()
        assert np.array_equal(got_x.cpu().numpy(), want_x.cpu().numpy())
        assert np.array_equal(got_y.cpu().numpy(), want_y.cpu().numpy())
        assert np.array_equal(got_img.cpu().numpy(), want_img.cpu().numpy())     # both start from zeros: bytes neither writes agree too
    # in place: the residual is the destination (what the ggml graph allocator hands out for MUL_MAT -> ADD)
    dst = res.clone()
    got_x, got_y, got_img = mi355.mul_mat_q8k_tiled_norm(t, tiles, act, N, K, B, nw, 1e-5, residual=dst, split=split, dst=dst)
    want_x = mi355.mul_mat_q8k_tiled(t, tiles, act, N, K, B, residual=res, split=split)
    torch.cuda.synchronize()
    assert np.array_equal(got_x.cpu().numpy(), want_x.cpu().numpy())


@pytest.mark.parametrize("name,t", TILED_TYPES)
@pytest.mark.parametrize("Ns,K,B", [((14336, 14336), 4096, 512),       # gate + up of an 8B llama: 896 tiles
                                    ((4096, 1024, 1024), 4096, 512),    # Q, K, V: 192 tiles in one round
                                    ((8200, 8300, 130), 2048, 300),     # ragged rows and batch
                                    ((1000,), 6144, 300)])              # one matrix: cut along K like the single-matrix entry point
def test_mmq_tiled_multi(dev, name, t, Ns, K, B):
    """several matrices in one launch of the wide-tile GEMM: every matrix equals its own launch bit for bit, with and without
    residual (also in place), and the oracle's integer arithmetic at the corners"""
    import torch
    import mi355
    rng = np.random.default_rng(sum(Ns) + K + B + t)
    x = rng.standard_normal((B, K)).astype(np.float32)
    act = mi355.quantize_act_q8k_tiled(_to_dev(dev, x))
    Wq = [_weights(rng, t, N, K, "ref") for N in Ns]
    tiles = [mi355.kq_unpack_tiles(t, mi355.upload_weights(t, _to_dev(dev, W))) for W in Wq]
    res = [_to_dev(dev, rng.standard_normal((B, N)).astype(np.float32)) if i != 1 else None for i, N in enumerate(Ns)]
    alone = [mi355.mul_mat_q8k_tiled(t, tl, act, N, K, B, split=len(Ns) == 1).cpu().numpy() for tl, N in zip(tiles, Ns)]
    multi = [o.cpu().numpy() for o in mi355.mul_mat_q8k_tiled_multi(t, tiles, act, list(Ns), K, B)]
    dsts = [torch.empty((B, N + 8 * i), dtype=torch.float32, device=dev)[:, :N] for i, N in enumerate(Ns)]    # a row stride per matrix
    for i, N in enumerate(Ns):
        if res[i] is not None:
            dsts[i].copy_(res[i])     # residual in place: dst is its own residual
    inplace = mi355.mul_mat_q8k_tiled_multi(t, tiles, act, list(Ns), K, B, dsts=dsts, residuals=[d if r is not None else None for d, r in zip(dsts, res)])
    for i, N in enumerate(Ns):
        assert np.array_equal(multi[i], alone[i])
        want = multi[i] + res[i].cpu().numpy() if res[i] is not None else multi[i]
        assert np.array_equal(inplace[i].cpu().numpy(), want)
        Nt, Bt = min(N, 40), min(B, 16)
        assert orc.nmse(multi[i][:Bt, :Nt], orc.mul_mat("cpu", t, Wq[i][:Nt], x[:Bt])) < 1e-9
        assert orc.nmse(multi[i][B - 5:, N - 7:], orc.mul_mat("cpu", t, Wq[i][N - 7:], x[B - 5:])) < 1e-9
