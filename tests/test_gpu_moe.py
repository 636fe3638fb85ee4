"""GPU tests of the mixture-of-experts glue launches (the node sequences of llm_build_moe_ffn, src/llama.cpp:417-530): each fused
launch writes the same bits as the separate SOFT_MAX / ARGSORT / GET_ROWS / SUM_ROWS / DIV / MUL / ADD launches, and the
probabilities match the oracle's soft-max."""
import ctypes as C

import numpy as np
import pytest

import orc

pytestmark = pytest.mark.gpu


def _d(t):
    import mi355
    return C.byref(mi355.tensor_desc(t))


@pytest.mark.parametrize("n_expert,n_used,T", [(8, 2, 1), (8, 2, 7), (64, 6, 33), (4, 4, 3), (60, 4, 512)])
def test_route_and_weights_equal_separate_nodes(dev, n_expert, n_used, T):
    import torch
    import mi355
    lib = mi355.load()
    g = torch.Generator().manual_seed(n_expert * 1000 + T)
    logits = (torch.randn(T, n_expert, generator=g) * 2).to(dev)
    # separate nodes
    probs = torch.empty_like(logits)
    mi355.check(lib.mi355_soft_max(None, _d(logits), None, _d(probs), 1.0, 0.0))
    order = torch.empty(T, n_expert, dtype=torch.int32, device=dev)
    mi355.check(lib.mi355_argsort(None, _d(probs), _d(order), 1))
    ids = order[:, :n_used]                                     # strided view, as ggml_top_k returns it
    raw = torch.empty(T, n_used, 1, device=dev)
    mi355.check(lib.mi355_get_rows(None, _d(probs.reshape(T, n_expert, 1)), _d(ids), _d(raw)))
    tot = torch.empty(T, 1, device=dev)
    mi355.check(lib.mi355_sum_rows(None, _d(raw.reshape(T, n_used)), _d(tot)))
    norm = torch.empty(T, n_used, device=dev)
    mi355.check(lib.mi355_bin_bcast(None, 3, _d(raw.reshape(T, n_used)), _d(tot), _d(norm)))
    # fused
    probs2 = torch.empty_like(probs)
    order2 = torch.empty_like(order)
    mi355.check(lib.mi355_moe_route(None, mi355._ptr(logits), mi355._ptr(probs2), mi355._ptr(order2), n_expert, T))
    assert torch.equal(probs2, probs)
    # the order agrees wherever probabilities are distinct; both orders sort the row
    p = probs.cpu().numpy()
    o1, o2 = order.cpu().numpy(), order2.cpu().numpy()
    for t in range(T):
        assert sorted(o2[t].tolist()) == list(range(n_expert))
        assert (np.diff(p[t][o2[t]]) <= 0).all()
        if len(np.unique(p[t])) == n_expert:
            assert (o1[t] == o2[t]).all()
    raw2, tot2, norm2 = torch.empty(T, n_used, device=dev), torch.empty(T, device=dev), torch.empty(T, n_used, device=dev)
    ids2 = order2[:, :n_used]
    mi355.check(lib.mi355_moe_weights(None, mi355._ptr(probs2), mi355._ptr(ids2), ids2.stride(0), mi355._ptr(raw2), mi355._ptr(tot2),
                                      mi355._ptr(norm2), n_expert, n_used, T))
    if (o1 == o2).all():
        assert torch.equal(raw2, raw.reshape(T, n_used)) and torch.equal(tot2, tot.reshape(T)) and torch.equal(norm2, norm)
    # against the oracle's soft-max and a numpy top-k
    want = np.zeros_like(p)
    x = logits.cpu().numpy()
    orc.oracle.orc_soft_max(orc._ptr(x), None, orc._ptr(want), n_expert, T, 1.0)
    assert orc.nmse(p, want) < 1e-6        # tests/test-backend-ops.cpp:2375
    sel = np.take_along_axis(want, o2[:, :n_used].astype(np.int64), axis=1)
    assert np.allclose(norm2.cpu().numpy(), sel / sel.sum(1, keepdims=True), rtol=1e-5)


@pytest.mark.parametrize("n_embd,n_used,T,residual", [(4096, 2, 1, True), (2048, 2, 5, False), (1024, 4, 9, True), (4096, 2, 512, True)])
def test_combine_equals_separate_nodes(dev, n_embd, n_used, T, residual):
    import torch
    import mi355
    lib = mi355.load()
    g = torch.Generator().manual_seed(n_embd + T)
    experts = torch.randn(T, n_used, n_embd, generator=g).to(dev)
    weights = torch.rand(T, n_used, 1, generator=g).to(dev)
    res = torch.randn(T, n_embd, generator=g).to(dev)
    scaled = torch.empty_like(experts)
    mi355.check(lib.mi355_bin_bcast(None, 2, _d(experts), _d(weights), _d(scaled)))
    acc = scaled[:, 0]
    for e in range(1, n_used):
        nxt = torch.empty(T, n_embd, device=dev)
        mi355.check(lib.mi355_bin_bcast(None, 0, _d(acc), _d(scaled[:, e]), _d(nxt)))
        acc = nxt
    if residual:
        nxt = torch.empty(T, n_embd, device=dev)
        mi355.check(lib.mi355_bin_bcast(None, 0, _d(acc), _d(res), _d(nxt)))
        acc = nxt
    scaled2 = torch.empty_like(experts)
    out2 = torch.empty(T, n_embd, device=dev)
    mi355.check(lib.mi355_moe_combine(None, mi355._ptr(experts), mi355._ptr(weights), mi355._ptr(scaled2), mi355._ptr(res) if residual else None,
                                      mi355._ptr(out2), n_embd, n_used, T))
    assert torch.equal(scaled2, scaled) and torch.equal(out2, acc)
    want = (experts.double() * weights.double()).sum(1) + (res.double() if residual else 0)
    assert orc.nmse(out2.cpu().numpy(), want.cpu().numpy()) < 1e-7
