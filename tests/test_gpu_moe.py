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


@pytest.mark.parametrize("name,t", [("q4_K", orc.Q4_K), ("q6_K", orc.Q6_K), ("q5_K", orc.Q5_K), ("q8_0", orc.Q8_0), ("q4_0", orc.Q4_0), ("iq4_nl", orc.IQ4_NL),
                                    ("iq4_xs", orc.IQ4_XS)])
@pytest.mark.parametrize("n_expert,n_used,T,N,K", [(8, 2, 1, 512, 4096), (8, 2, 3, 256, 2048), (4, 4, 2, 96, 1024)])
def test_expert_gate_up_swiglu_equals_separate_launches(dev, name, t, n_expert, n_used, T, N, K):
    """MUL_MAT_ID(up), MUL_MAT_ID(gate), SILU, MUL and the Q8_1 rows for the down experts in one launch: the bits of
    mi355_mul_mat_id_vec twice followed by mi355_swiglu_quant."""
    import torch
    import mi355
    lib = mi355.load()
    rng = np.random.default_rng(n_expert + T + N)
    stacks = []
    for _ in range(2):
        Wq = orc.quantize("oracle", t, (rng.standard_normal((n_expert * N, K)) * 0.05).astype(np.float32))
        stacks.append(mi355.upload_weights(t, torch.from_numpy(Wq).to(dev)))
    as_gate, as_up = stacks
    x = torch.from_numpy(rng.standard_normal((T, K)).astype(np.float32)).to(dev)
    act = mi355.quantize_act(x)
    ids_full = torch.from_numpy(np.stack([rng.permutation(n_expert) for _ in range(T)]).astype(np.int32)).to(dev)
    ids = ids_full[:, :n_used]
    slots = T * n_used
    if t == orc.Q6_K and K % 2048 != 0:   # its rows are 16-byte aligned only when K is a multiple of 2048: the caller keeps the separate launches
        assert lib.mi355_moe_gate_up_swiglu_supported(t, as_gate.data_ptr(), as_up.data_ptr(), N, K) == 0
        return
    assert lib.mi355_moe_gate_up_swiglu_supported(t, as_gate.data_ptr(), as_up.data_ptr(), N, K) == 1
    g0, u0 = torch.zeros(slots, N, device=dev), torch.zeros(slots, N, device=dev)
    for W, out in ((as_gate, g0), (as_up, u0)):
        mi355.check(lib.mi355_mul_mat_id_vec(None, t, W.data_ptr(), act.data_ptr(), ids.data_ptr(), ids.stride(0), out.data_ptr(), N, K, n_expert, n_used, 1, T))
    a0 = torch.zeros(int(lib.mi355_act_bytes(N, slots)), dtype=torch.uint8, device=dev)
    mi355.check(lib.mi355_swiglu_quant(None, g0.data_ptr(), u0.data_ptr(), N, None, 0, a0.data_ptr(), N, slots))
    g1, u1, a1 = torch.zeros_like(g0), torch.zeros_like(u0), torch.zeros_like(a0)
    mi355.check(lib.mi355_moe_gate_up_swiglu(None, t, as_gate.data_ptr(), as_up.data_ptr(), act.data_ptr(), ids.data_ptr(), ids.stride(0), g1.data_ptr(),
                                             u1.data_ptr(), a1.data_ptr(), N, K, n_expert, n_used, 1, T))
    torch.cuda.synchronize()
    assert torch.equal(g1, g0) and torch.equal(u1, u0)
    used = slots * N + slots * (N // 32) * 8
    assert torch.equal(a1[:used], a0[:used])
    assert g1.abs().sum().item() > 0 and a1[:slots * N].float().abs().sum().item() > 0


@pytest.mark.parametrize("n_expert,n_embd,n_used,T,residual", [(8, 4096, 2, 1, True), (8, 2048, 2, 5, False), (16, 1024, 4, 8, True), (64, 4096, 6, 2, True)])
def test_weights_combine_equals_the_two_launches(dev, n_expert, n_embd, n_used, T, residual):
    import torch
    import mi355
    lib = mi355.load()
    g = torch.Generator().manual_seed(n_embd + T + n_expert)
    probs = torch.softmax(torch.randn(T, n_expert, generator=g) * 2, dim=1).to(dev)
    order = torch.stack([torch.randperm(n_expert, generator=g) for _ in range(T)]).to(torch.int32).to(dev)
    ids = order[:, :n_used]
    experts = torch.randn(T, n_used, n_embd, generator=g).to(dev)
    res = torch.randn(T, n_embd, generator=g).to(dev)
    raw, tot, norm = torch.empty(T, n_used, device=dev), torch.empty(T, device=dev), torch.empty(T, n_used, device=dev)
    mi355.check(lib.mi355_moe_weights(None, mi355._ptr(probs), mi355._ptr(ids), ids.stride(0), mi355._ptr(raw), mi355._ptr(tot), mi355._ptr(norm),
                                      n_expert, n_used, T))
    scaled, out = torch.empty_like(experts), torch.empty(T, n_embd, device=dev)
    mi355.check(lib.mi355_moe_combine(None, mi355._ptr(experts), mi355._ptr(norm), mi355._ptr(scaled), mi355._ptr(res) if residual else None, mi355._ptr(out),
                                      n_embd, n_used, T))
    raw2, tot2, norm2 = torch.zeros_like(raw), torch.zeros_like(tot), torch.zeros_like(norm)
    scaled2, out2 = torch.zeros_like(scaled), torch.zeros_like(out)
    mi355.check(lib.mi355_moe_weights_combine(None, mi355._ptr(probs), mi355._ptr(ids), ids.stride(0), mi355._ptr(raw2), mi355._ptr(tot2), mi355._ptr(norm2),
                                              n_expert, mi355._ptr(experts), mi355._ptr(scaled2), mi355._ptr(res) if residual else None, mi355._ptr(out2),
                                              n_embd, n_used, T))
    torch.cuda.synchronize()
    assert torch.equal(raw2, raw) and torch.equal(tot2, tot) and torch.equal(norm2, norm)
    assert torch.equal(scaled2, scaled) and torch.equal(out2, out)
    # the weights not materialised, the scaled outputs in place on the experts' (what the plug-in launches)
    ex3, out3 = experts.clone(), torch.zeros_like(out)
    mi355.check(lib.mi355_moe_weights_combine(None, mi355._ptr(probs), mi355._ptr(ids), ids.stride(0), None, None, None, n_expert, mi355._ptr(ex3), mi355._ptr(ex3),
                                              mi355._ptr(res) if residual else None, mi355._ptr(out3), n_embd, n_used, T))
    torch.cuda.synchronize()
    assert torch.equal(ex3, scaled) and torch.equal(out3, out)


@pytest.mark.parametrize("n_expert,T,K", [(8, 1, 4096), (8, 3, 4096), (64, 2, 2048), (4, 8, 1024), (12, 1, 3072)])
def test_norm_router_equals_norm_product_route(dev, n_expert, T, K):
    """mi355_rms_norm_mul_quant_router = the FFN norm (f32 row + Q8_1 rows), the f32 router product and soft-max + order, with the
    bits of the three launches it replaces."""
    import torch
    import mi355
    lib = mi355.load()
    g = torch.Generator().manual_seed(n_expert * 100 + T)
    W = (torch.randn(n_expert, K, generator=g) * 0.05).to(dev)
    x = torch.randn(T, K, generator=g).to(dev)
    nw = (1.0 + 0.1 * torch.randn(K, generator=g)).to(dev)
    nact = int(lib.mi355_act_bytes(K, T))
    y, act = torch.empty(T, K, device=dev), torch.zeros(nact, dtype=torch.uint8, device=dev)
    mi355.check(lib.mi355_rms_norm_mul_quant(None, mi355._ptr(x), K, mi355._ptr(nw), mi355._ptr(y), K, mi355._ptr(act), K, T, 1e-5))
    logits = torch.empty(T, n_expert, device=dev)
    mi355.check(lib.mi355_mul_mat_f(None, _d(W), _d(y), _d(logits)))
    probs, order = torch.empty_like(logits), torch.empty(T, n_expert, dtype=torch.int32, device=dev)
    mi355.check(lib.mi355_moe_route(None, mi355._ptr(logits), mi355._ptr(probs), mi355._ptr(order), n_expert, T))
    y2, act2 = torch.zeros_like(y), torch.zeros_like(act)
    logits2, probs2, order2 = torch.zeros_like(logits), torch.zeros_like(probs), torch.zeros_like(order)
    mi355.check(lib.mi355_rms_norm_mul_quant_router(None, mi355._ptr(x), K, mi355._ptr(nw), mi355._ptr(y2), K, mi355._ptr(act2), K, T, 1e-5, mi355._ptr(W), K,
                                                    mi355._ptr(logits2), mi355._ptr(probs2), mi355._ptr(order2), n_expert))
    torch.cuda.synchronize()
    used = T * K + T * (K // 32) * 8
    assert torch.equal(y2, y) and torch.equal(act2[:used], act[:used])
    assert torch.equal(logits2, logits) and torch.equal(probs2, probs) and torch.equal(order2, order)
    want = y.cpu().double() @ W.cpu().double().T
    assert orc.nmse(logits2.cpu().numpy(), want.numpy().astype(np.float32)) < 1e-10
