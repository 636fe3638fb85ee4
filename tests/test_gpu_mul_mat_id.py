"""GPU parity of MUL_MAT_ID (MoE expert routing) against the oracle and the reference CPU backend."""
import numpy as np
import pytest

import orc

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("name,t", list(orc.WEIGHT_TYPES.items()))
@pytest.mark.parametrize("n_expert,n_used,nb1_bcast,T,N,K", [(8, 2, True, 1, 512, 4096), (8, 2, False, 5, 256, 2048),
                                                              (4, 4, True, 32, 128, 2048), (8, 1, False, 3, 64, 4096)])
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
    want = np.zeros((T, n_used, N), dtype=np.float32)
    assert orc.oracle.orc_mul_mat_id_q8_1(t, orc._ptr(Wq), orc._ptr(b), orc._ptr(ids_full), n_expert, orc._ptr(want), N, K,
                                          n_expert, n_used, nb1, T) == 0
    assert orc.nmse(got, want) < 1e-9
    if orc.ref is not None:
        cpu = np.zeros_like(want)
        assert orc.ref.ref_mul_mat_id(t, orc._ptr(Wq), orc._ptr(b), orc._ptr(ids_full), orc._ptr(cpu), N, K, n_expert, n_used,
                                      nb1, T, 4, 0) >= 0
        assert orc.nmse(got, cpu) <= 5e-4      # tests/test-backend-ops.cpp:2001
