"""The weight quantizers on the device (mi355_quantize_weights) against the reference's own quantize_row_*_ref, byte for byte:
what llama-quantize runs per tensor without an importance matrix (ggml/src/ggml-quants.c:31-66, 194-217, 1208-1278, 1395-1480,
1620-1688; Q4_1 / Q5_0 / Q5_1: 68-192; IQ4_NL / IQ4_XS: quantize_iq4_nl / quantize_iq4_xs, 4573-4745), plus the model-file driver that uses them."""
import os
import sys

import numpy as np
import pytest

import orc

pytestmark = pytest.mark.gpu

TYPES = list(orc.WEIGHT_TYPES.items())   # every weight type has its quantizer on the device


def _special_rows(rng, k):
    """rows that take the quantizers' side paths"""
    rows = []
    rows.append(np.zeros(k))                                                    # all-zero groups and super-blocks
    rows.append(np.full(k, 0.37))                                               # max == min in every sub-block
    rows.append(np.abs(rng.standard_normal(k)) + 0.5)                           # positive only: the sub-block minimum is clamped to 0
    rows.append(-np.abs(rng.standard_normal(k)) - 0.5)                          # negative only
    r = rng.standard_normal(k) * 1e-20                                          # below GROUP_MAX_EPS in places
    r[::7] = 0
    rows.append(r)
    r = rng.standard_normal(k) * 0.02
    r[5::256] = 3.0                                                             # one outlier per super-block
    rows.append(r)
    r = rng.standard_normal(k)
    r[:256] = 0                                                                 # one all-zero super-block inside a row
    r[256:272] = 0                                                              # one all-zero 16-group
    rows.append(r)
    rows.append(np.round(rng.standard_normal(k) * 4) / 4)                       # many ties
    rows.append(rng.standard_normal(k) * 1e4)
    r = np.zeros(k)
    r[3::32] = -1.0                                                             # a single non-zero value per block
    rows.append(r)
    return np.stack(rows).astype(np.float32)


@pytest.mark.parametrize("name,t", TYPES)
@pytest.mark.parametrize("kind", ["normal", "uniform", "special"])
def test_device_quantizers_match_reference_bytes(dev, name, t, kind):
    import torch
    import mi355
    rng = np.random.default_rng(17 + t)
    k = 4096
    if kind == "normal":
        x = (rng.standard_normal((96, k)) * 0.02).astype(np.float32)
    elif kind == "uniform":
        x = rng.uniform(-1, 1, (96, k)).astype(np.float32)
    else:
        x = _special_rows(rng, k)
    got = mi355.quantize_weights(t, torch.from_numpy(x).to(dev)).cpu().numpy()
    want = orc.quantize("ref" if orc.ref is not None else "oracle", t, x)
    bad = np.nonzero((got != want).any(axis=1))[0]
    assert bad.size == 0, "rows that differ: %s" % bad[:10]
    assert np.array_equal(got, orc.quantize("oracle", t, x))


@pytest.mark.parametrize("name,t", [("q4_K", orc.Q4_K), ("q6_K", orc.Q6_K)])
def test_device_quantizers_whole_matrix(dev, name, t):
    """a whole 4096 x 4096 matrix of N(0, 0.02) weights, generated on the device: the reference's bytes for every row"""
    import torch
    import mi355
    gen = torch.Generator(device=dev)
    gen.manual_seed(5)
    x = torch.randn((4096, 4096), device=dev, generator=gen) * 0.02
    got = mi355.quantize_weights(t, x).cpu().numpy()
    want = orc.quantize_mt("ref" if orc.ref is not None else "oracle", t, x.cpu().numpy())
    assert np.array_equal(got, want)


def test_model_file_quantized_on_device(dev, tmp_path):
    """the model-file driver: tensors drawn from N(0, 0.02), quantized on the device with the Q4_K_M type mix and written as GGUF;
    the file's tensors dequantize (reference dequantizers) to values with that spread, and the reference's runtime loads it"""
    import subprocess
    from mi355 import gguf
    path = str(tmp_path / "quantized.gguf")
    gguf.write_model(path, n_layer=2, n_embd=1024, n_ff=2048, n_head=8, n_head_kv=2, n_vocab=512, quantize_on=dev)
    tensors = gguf.tensor_list(2, 1024, 2048, 8, 2, 128, 512)
    raw = open(path, "rb").read()
    total = sum((gguf.nbytes(tt, sh) + 31) // 32 * 32 for _, tt, sh in tensors)
    data = np.frombuffer(raw[len(raw) - total:], dtype=np.uint8)
    off = 0
    seen = set()
    for name, tt, sh in tensors:
        n = gguf.nbytes(tt, sh)
        if tt in (orc.Q4_K, orc.Q6_K):
            k = sh[0]
            rows = int(np.prod(sh[1:]))
            vals = orc.dequantize("oracle", tt, data[off:off + n].reshape(rows, -1), k)
            assert 0.018 < float(vals.std()) < 0.022, (name, float(vals.std()))
            seen.add(tt)
        off += (n + 31) // 32 * 32
    assert seen == {orc.Q4_K, orc.Q6_K}
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    logits = os.path.join(root, "oracle", "_ref", "llama_logits")
    if os.path.exists(logits):
        r = subprocess.run([logits, path, "0", "5", "2", str(tmp_path / "o.bin")], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300,
                           cwd=os.path.dirname(logits))
        assert r.returncode == 0, r.stdout[-2000:]
        assert np.isfinite(np.fromfile(str(tmp_path / "o.bin"), dtype=np.float32)).all()
