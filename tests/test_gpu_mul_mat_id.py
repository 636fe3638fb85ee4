"""GPU parity of MUL_MAT_ID (MoE expert routing) against the oracle and the reference CPU backend."""
import numpy as np
import pytest

import orc

pytestmark = pytest.mark.gpu


def routed(t, n_used, T, K):
    """mi355_mul_mat_id sorts the slots by expert and uses the K-quant tile kernel (ggml-cpu's Q8_K arithmetic)"""
    return T * n_used >= 32 and ((t in (orc.Q4_K, orc.Q5_K) and K % 256 == 0) or (t == orc.Q6_K and K % 2048 == 0) or (t == orc.IQ4_XS and K % 512 == 0))


def expected_per_expert(kind, t, Wq, b, ids_full, n_expert, n_used, nb1, N):
    """every expert's product over the rows routed to it (ggml.c:2723-2759), one mul_mat per expert"""
    T = b.shape[0]
    want = np.zeros((T, n_used, N), dtype=np.float32)
    for ex in range(n_expert):
        where = [(tt, e) for tt in range(T) for e in range(n_used) if ids_full[tt, e] == ex]
        if not where:
            continue
        rows = np.stack([b[tt, e % nb1] for tt, e in where])
        out = orc.mul_mat(kind, t, Wq[ex * N:(ex + 1) * N], rows)
        for (tt, e), o in zip(where, out):
            want[tt, e] = o
    return want


@pytest.mark.parametrize("name,t", list(orc.WEIGHT_TYPES.items()))
@pytest.mark.parametrize("n_expert,n_used,nb1_bcast,T,N,K", [(8, 2, True, 1, 512, 4096), (8, 2, False, 5, 256, 2048),
                                                              (4, 4, True, 32, 128, 2048), (8, 1, False, 3, 64, 4096),
                                                              (8, 2, True, 512, 192, 2048), (8, 2, False, 300, 64, 4096)])
def test_mul_mat_id(dev, name, t, n_expert, n_used, nb1_bcast, T, N, K):
    import torch
    import mi355
    rng = np.random.default_rng(n_expert + T + N)
    nb1 = 1 if nb1_bcast else n_used
    Wf = (rng.standard_normal((n_expert * N, K)) * 0.02).astype(np.float32)
    Wq = orc.quantize("ref" if orc.ref is not None else "oracle", t, Wf)
    b = rng.standard_normal((T, nb1, K)).astype(np.float32)
    ids_full = np.stack([rng.permutation(n_expert) for _ in range(T)]).astype(np.int32)
    Wd = mi355.upload_weights(t, torch.from_numpy(Wq).to(dev)).reshape(n_expert, N, -1)
    idd = torch.from_numpy(ids_full).to(dev)[:, :n_used]          # strided view, as ggml_view of the argsort result
    got = mi355.mul_mat_id(t, Wd, torch.from_numpy(b).to(dev), idd, n_used).cpu().numpy()
    if routed(t, n_used, T, K):
        want = expected_per_expert("cpu", t, Wq, b, ids_full, n_expert, n_used, nb1, N)
    else:
        want = np.zeros((T, n_used, N), dtype=np.float32)
        assert orc.oracle.orc_mul_mat_id_q8_1(t, orc._ptr(Wq), orc._ptr(b), orc._ptr(ids_full), n_expert, orc._ptr(want), N, K,
                                              n_expert, n_used, nb1, T) == 0
    # per-32-block experts with 32+ slots run the routed form of their tile kernel, where the block minimum of Q4_1 / Q5_1 meets
    # fp16(d_x * sum(q)), the `s` field the reference's own dot uses
    assert orc.nmse(got, want) < (1e-6 if (t in (orc.Q4_1, orc.Q5_1) and T * n_used >= 32) else 1e-9)
    if orc.ref is not None:
        cpu = np.zeros_like(want)
        assert orc.ref.ref_mul_mat_id(t, orc._ptr(Wq), orc._ptr(b), orc._ptr(ids_full), orc._ptr(cpu), N, K, n_expert, n_used,
                                      nb1, T, 4, 0) >= 0
        assert orc.nmse(got, cpu) <= 5e-4      # tests/test-backend-ops.cpp:2001


@pytest.mark.parametrize("name,t", [("q4_k", orc.Q4_K), ("q6_k", orc.Q6_K), ("q5_k", orc.Q5_K), ("iq4_xs", orc.IQ4_XS), ("q4_0", orc.Q4_0), ("q8_0", orc.Q8_0),
                                    ("q5_1", orc.Q5_1)])
@pytest.mark.parametrize("pattern", ["one_expert", "two_of_eight", "out_of_range"])
def test_mul_mat_id_skewed_routing(dev, name, t, pattern):
    """experts with no slots, one expert with more slots than a column tile, ids outside [0, n_expert) clamped like the GEMV path"""
    import torch
    import mi355
    n_expert, n_used, T, N, K = 8, 2, 200, 128, 2048
    rng = np.random.default_rng(5)
    Wf = (rng.standard_normal((n_expert * N, K)) * 0.02).astype(np.float32)
    Wq = orc.quantize("ref" if orc.ref is not None else "oracle", t, Wf)
    b = rng.standard_normal((T, 1, K)).astype(np.float32)
    if pattern == "one_expert":
        ids = np.full((T, n_expert), 3, dtype=np.int32)
    elif pattern == "two_of_eight":
        ids = np.tile(np.array([[6, 1, 0, 0, 0, 0, 0, 0]], dtype=np.int32), (T, 1))
    else:
        ids = rng.integers(-2, n_expert + 2, size=(T, n_expert)).astype(np.int32)
    Wd = mi355.upload_weights(t, torch.from_numpy(Wq).to(dev)).reshape(n_expert, N, -1)
    idd = torch.from_numpy(ids).to(dev)[:, :n_used]
    got = mi355.mul_mat_id(t, Wd, torch.from_numpy(b).to(dev), idd, n_used).cpu().numpy()
    kind = "cpu" if t in (orc.Q4_K, orc.Q6_K, orc.Q5_K, orc.IQ4_XS) else "q8_1"   # the activation format of the type's routed tile kernel
    want = expected_per_expert(kind, t, Wq, b, np.clip(ids, 0, n_expert - 1), n_expert, n_used, 1, N)
    assert orc.nmse(got, want) < (1e-6 if t in (orc.Q4_1, orc.Q5_1) else 1e-9)   # the block minimum meets fp16(d_x * sum(q)) in the tile kernel


@pytest.mark.parametrize("name,t", [("q4_k", orc.Q4_K), ("q5_k", orc.Q5_K), ("q6_k", orc.Q6_K)])
@pytest.mark.parametrize("n_expert,n_used,nb1_bcast,T,N,K", [(8, 2, True, 512, 192, 2048), (8, 2, False, 300, 64, 4096), (4, 4, True, 70, 256, 2048),
                                                              (8, 1, False, 3, 130, 2048)])   # Q6_K rows are 16-byte aligned from K = 2048 on
def test_mul_mat_id_on_tile_images(dev, name, t, n_expert, n_used, nb1_bcast, T, N, K):
    """the routed form of the wide-tile kernel: slots sorted by expert, activations gathered into one tile image, rows
    scattered to their slots; against ggml-cpu's arithmetic per expert (Q8_K activations) and the reference's MUL_MAT_ID"""
    import torch
    import mi355
    rng = np.random.default_rng(n_expert + T + N + K)
    nb1 = 1 if nb1_bcast else n_used
    Wf = (rng.standard_normal((n_expert * N, K)) * 0.02).astype(np.float32)
    Wq = orc.quantize("ref" if orc.ref is not None else "oracle", t, Wf)
    b = rng.standard_normal((T, nb1, K)).astype(np.float32)
    ids_full = np.stack([rng.permutation(n_expert) for _ in range(T)]).astype(np.int32)
    Wd = mi355.upload_weights(t, torch.from_numpy(Wq).to(dev)).reshape(n_expert, N, -1)
    tiles = mi355.kq_unpack_expert_tiles(t, Wd)
    idd = torch.from_numpy(ids_full).to(dev)[:, :n_used]
    got = mi355.mul_mat_id_tiled(t, tiles, N, torch.from_numpy(b).to(dev), idd, n_used).cpu().numpy()
    want = expected_per_expert("cpu", t, Wq, b, ids_full, n_expert, n_used, nb1, N)
    assert orc.nmse(got, want) < 1e-9
    if orc.ref is not None:
        cpu = np.zeros_like(want)
        assert orc.ref.ref_mul_mat_id(t, orc._ptr(Wq), orc._ptr(b), orc._ptr(ids_full), orc._ptr(cpu), N, K, n_expert, n_used,
                                      nb1, T, 4, 0) >= 0
        assert orc.nmse(got, cpu) <= 5e-4      # tests/test-backend-ops.cpp:2001


@pytest.mark.parametrize("pattern", ["one_expert", "two_of_eight", "out_of_range"])
def test_mul_mat_id_on_tile_images_skewed_routing(dev, pattern):
    """experts without slots, one expert with more slots than a column tile, ids outside [0, n_expert) clamped"""
    import torch
    import mi355
    t = orc.Q4_K
    n_expert, n_used, T, N, K = 8, 2, 200, 128, 2048
    rng = np.random.default_rng(6)
    Wf = (rng.standard_normal((n_expert * N, K)) * 0.02).astype(np.float32)
    Wq = orc.quantize("ref" if orc.ref is not None else "oracle", t, Wf)
    b = rng.standard_normal((T, 1, K)).astype(np.float32)
    if pattern == "one_expert":
        ids = np.full((T, n_expert), 3, dtype=np.int32)
    elif pattern == "two_of_eight":
        ids = np.tile(np.array([[6, 1, 0, 0, 0, 0, 0, 0]], dtype=np.int32), (T, 1))
    else:
        ids = rng.integers(-2, n_expert + 2, size=(T, n_expert)).astype(np.int32)
    Wd = mi355.upload_weights(t, torch.from_numpy(Wq).to(dev)).reshape(n_expert, N, -1)
    tiles = mi355.kq_unpack_expert_tiles(t, Wd)
    idd = torch.from_numpy(ids).to(dev)[:, :n_used]
    got = mi355.mul_mat_id_tiled(t, tiles, N, torch.from_numpy(b).to(dev), idd, n_used).cpu().numpy()
    want = expected_per_expert("cpu", t, Wq, b, np.clip(ids, 0, n_expert - 1), n_expert, n_used, 1, N)
    assert orc.nmse(got, want) < 1e-9
