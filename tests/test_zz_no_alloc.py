"""The allocation-free MUL_MAT entry point (mi355_mul_mat_static: workspace = an array inside the library, one per GPU)
against mi355_mul_mat with a caller workspace of the same size: bit-identical, on consecutive calls that share the array,
the later ones with smaller inputs; over-sized products are rejected."""
import numpy as np
import pytest

import orc

pytestmark = pytest.mark.gpu


def _case(dev, t, N, K, B, seed):
    import torch
    import mi355
    rng = np.random.default_rng(seed)
    Wf = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    Wq = orc.quantize("oracle", t, Wf)
    W = mi355.upload_weights(t, torch.from_numpy(Wq).to(dev))
    x = torch.from_numpy(rng.standard_normal((B, K)).astype(np.float32)).to(dev)
    return W, x, Wq


@pytest.mark.parametrize("name,t", list(orc.WEIGHT_TYPES.items()))
def test_static_scratch_matches_workspace_entry(dev, name, t):
    import torch
    import mi355
    lib = mi355.load()
    cap = lib.mi355_mul_mat_static_max_ws()
    assert cap == 16 << 20
    ws = torch.empty(cap, dtype=torch.uint8, device=dev)
    # the tile GEMM with slices along K, then a smaller tile product, the few-row kernel and one row: each call finds the
    # previous call's bytes in the array
    for i, (N, K, B) in enumerate([(512, 4096, 320), (384, 2048, 64), (256, 1024, 8), (128, 512, 1)]):
        W, x, Wq = _case(dev, t, N, K, B, 100 + i)
        want = mi355.mul_mat(t, W, x, ws=ws, split=False)      # split=False: the workspace is exactly the `ws` given
        got = torch.full((B, N), float("nan"), dtype=torch.float32, device=dev)
        mi355.mul_mat_static(t, W, x, got)
        torch.cuda.synchronize()
        assert torch.equal(got, want), (name, N, K, B)
        if i == 3:
            ref = orc.mul_mat("cpu", t, Wq, x.cpu().numpy())
            assert orc.nmse(got.cpu().numpy(), ref) <= 5e-4


def test_static_scratch_rejects_oversize(dev):
    import torch
    import mi355
    lib = mi355.load()
    K, B = 14336, 1024                       # 14336 * 1024 * 1.25 bytes of quantized activation > 16 MiB
    assert lib.mi355_mul_mat_ws_bytes(K, B) > lib.mi355_mul_mat_static_max_ws()
    W = torch.zeros((32, mi355.row_bytes(mi355.Q4_K, K)), dtype=torch.uint8, device=dev)
    x = torch.zeros((B, K), dtype=torch.float32, device=dev)
    dst = torch.zeros((B, 32), dtype=torch.float32, device=dev)
    with pytest.raises(mi355.Mi355Error, match="scratch"):
        mi355.mul_mat_static(mi355.Q4_K, W, x, dst)


def test_static_scratch_allocates_nothing_and_runs_under_capture(dev):
    """after mi355_mul_mat_static_init the calls leave the device's free memory unchanged, and a call recorded into a HIP graph
    gives the eager result on every replay"""
    import torch
    import mi355
    lib = mi355.load()
    mi355.check(lib.mi355_mul_mat_static_init())
    t = mi355.Q4_K
    cases = [_case(dev, t, N, K, B, 300 + i) + (N, B) for i, (N, K, B) in enumerate([(512, 4096, 320), (256, 2048, 8), (128, 1024, 1)])]
    outs = [torch.zeros((B, N), dtype=torch.float32, device=dev) for _, _, _, N, B in cases]
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    for (W, x, _, _, _), out in zip(cases, outs):
        mi355.mul_mat_static(t, W, x, out)
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0, (free0, free1)
    W, x, _, N, B = cases[0]
    eager = outs[0].clone()
    out = torch.zeros_like(eager)
    side = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        mi355.mul_mat_static(t, W, x, out)
    for rep in range(3):
        out.zero_()
        mi355.mul_mat_static(t, cases[1][0], cases[1][1], outs[1])     # eager work on the same array between the replays
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), rep
