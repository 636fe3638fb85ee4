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
    want = orc.mul_mat("q8_1", t, Wq[:Nt], x[:Bt])
    tol = 1e-6 if t == orc.Q4_K else 1e-9    # Q4_K adds its min term through fp16 operands
    assert orc.nmse(got[:Bt, :Nt], want) < tol
    if orc.ref is not None:
        cpu = orc.mul_mat("ref", t, Wq, x)
        assert orc.nmse(got, cpu) <= 5e-4


@pytest.mark.parametrize("name,t", TYPES)
def test_unaligned_rows_fallback(dev, name, t):
    """K for which the device-layout rows are not 16-byte multiples (byte-load kernel)"""
    import mi355
    rng = np.random.default_rng(5)
    be = orc.BLOCK[t][0]
    K = be * 3
    for B in (1, 12):
        Wq = _weights(rng, t, 19, K)
        x = rng.standard_normal((B, K)).astype(np.float32)
        Wd = mi355.upload_weights(t, _to_dev(dev, Wq))
        got = mi355.mul_mat(t, Wd, _to_dev(dev, x)).cpu().numpy()
        # B > 8 with K % 128 == 0 takes the MFMA kernel, whose Q4_K min term goes through fp16 operands
        assert orc.nmse(got, orc.mul_mat("q8_1", t, Wq, x)) < (1e-6 if (t == orc.Q4_K and B > 8) else 1e-9)
