"""Drop-in check at model level: the reference's own benchmark program, examples/llama-bench, built unmodified from the
reference sources (oracle/Makefile, target llamabench), loads libggml-mi355.so through GGML_BACKEND_PATH, offloads every
layer of a synthetic llama-architecture Q4_K_M model (tests/make_synthetic_gguf.py) and runs prefill and decode with flash
attention.  The test asserts that the run completes on the plug-in's device and keeps the table it printed as a log file."""
import os
import re
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "oracle", "_ref", "llama-bench")
PLUGIN = os.path.join(ROOT, "llama.cpp_amd", "lib", "libggml-mi355.so")


def run_llama_bench(model, args, timeout=900):
    env = dict(os.environ, GGML_BACKEND_PATH=PLUGIN)
    r = subprocess.run([BENCH, "-m", model, "-ngl", "99", "-fa", "1"] + args, env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                       text=True, timeout=timeout, cwd=os.path.dirname(BENCH))
    return r


def parse_table(text):
    """{test name: tokens/s} from llama-bench's markdown table"""
    out = {}
    for line in text.splitlines():
        cells = [c.strip() for c in line.strip().strip("|").split("|")]
        if len(cells) >= 3 and re.match(r"^(pp|tg)\d+$", cells[-2]):
            out[cells[-2]] = float(cells[-1].split()[0])
    return out


def test_llama_bench_runs_on_the_plugin(dev, tmp_path):
    if not (os.path.exists(BENCH) and os.path.exists(PLUGIN)):
        pytest.skip("llama-bench or the plug-in is not built (needs the llama.cpp tree at build time)")
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    import make_synthetic_gguf
    model = str(tmp_path / "small.gguf")
    make_synthetic_gguf.write_model(model, n_layer=4, n_embd=2048, n_ff=6144, n_head=16, n_head_kv=4, n_vocab=4096)
    r = run_llama_bench(model, ["-p", "64", "-n", "16", "-r", "2"])
    os.makedirs(os.path.join(ROOT, "gpurun_out"), exist_ok=True)
    with open(os.path.join(ROOT, "gpurun_out", "llama_bench_small.log"), "w") as f:
        f.write(r.stdout)
    assert r.returncode == 0, r.stdout[-3000:]
    assert "MI355X" in r.stdout, "the plug-in's device does not appear in the table:\n" + r.stdout[-3000:]
    t = parse_table(r.stdout)
    assert t.get("pp64", 0) > 0 and t.get("tg16", 0) > 0, r.stdout[-3000:]


LOGITS = os.path.join(ROOT, "oracle", "_ref", "llama_logits")


def _logits(model, ngl, n_prompt, n_decode, out, fusion=True, graphs=True, stats=None, cache=None, mmap=True, shift=0, defrag=0, ctx=0):
    import numpy as np
    env = dict(os.environ, GGML_BACKEND_PATH=PLUGIN, MI355_GRAPH_STATS="1")
    if ctx:
        env["LLAMA_LOGITS_CTX"] = str(ctx)
    if shift:
        env["LLAMA_LOGITS_SHIFT"] = str(shift)
    if defrag:
        env["LLAMA_LOGITS_DEFRAG"] = str(defrag)
    if not mmap:
        env["LLAMA_LOGITS_NO_MMAP"] = "1"
    if not fusion:
        env["MI355_NO_FUSION"] = "1"
    if not graphs:
        env["MI355_NO_GRAPH"] = "1"
    r = subprocess.run([LOGITS, model, str(ngl), str(n_prompt), str(n_decode), out] + (list(cache) if cache else []), env=env, stdout=subprocess.PIPE,
                       stderr=subprocess.STDOUT, text=True, timeout=600, cwd=os.path.dirname(LOGITS))
    assert r.returncode == 0, r.stdout[-3000:]
    if ngl > 0:
        assert "MI355X" in r.stdout, "layers were not offloaded to the plug-in:\n" + r.stdout[-3000:]
    if stats is not None:
        m = re.search(r"MI355 graph replay: (\d+) captures, (\d+) replays", r.stdout)
        stats["captures"], stats["replays"] = (int(m.group(1)), int(m.group(2))) if m else (0, 0)
        m = re.findall(r"MI355 transfers: (\d+) uploads on the backend stream, (\d+) events recorded", r.stdout)
        stats["uploads"], stats["events"] = max((int(a) for a, _ in m), default=0), max((int(b) for _, b in m), default=0)
    return np.fromfile(out, dtype=np.float32)


@pytest.mark.parametrize("n_prompt", [5, 20, 40, 256])
def test_model_logits_q5_k_m(dev, tmp_path, n_prompt):
    """A Q5_K_M-shaped file (Q5_K everywhere, Q6_K where llama-quantize uses more bits): the reference's runtime on the plug-in
    reproduces its CPU backend's logits, so Q5_K products (GEMV for decode and up to eight rows, the per-32-block tile kernel up to 32, the
    wide-tile GEMM on Q5_K tile images from 33 rows on) and Q5_K rows of GET_ROWS stay on the device with the reference's
    arithmetic."""
    if not (os.path.exists(LOGITS) and os.path.exists(PLUGIN)):
        pytest.skip("llama_logits or the plug-in is not built (needs the llama.cpp tree at build time)")
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    import numpy as np
    import make_synthetic_gguf
    import orc
    model = str(tmp_path / "q5km.gguf")
    make_synthetic_gguf.write_model(model, n_layer=2, n_embd=2048, n_ff=4096, n_head=16, n_head_kv=4, n_vocab=2048, ftype="q5_k_m")
    cpu = _logits(model, 0, n_prompt, 4, str(tmp_path / "cpu.bin"))
    dev_out = _logits(model, 99, n_prompt, 4, str(tmp_path / "dev.bin"))
    assert cpu.shape == dev_out.shape and np.isfinite(dev_out).all()
    assert orc.nmse(dev_out, cpu) < 2e-3


@pytest.mark.parametrize("ftype", ["q4_1", "q5_0", "q5_1", "iq4_nl", "iq4_xs"])
@pytest.mark.parametrize("n_prompt", [5, 40])
def test_model_logits_per_32_block_types(dev, tmp_path, ftype, n_prompt):
    """Files of the per-32-block types beyond Q4_0 / Q8_0 (Q4_1, Q5_0, Q5_1, IQ4_NL, and IQ4_XS whose blocks sit eight to a super-block,
    with the Q5_K / Q6_K tensors llama-quantize mixes in): the reference's runtime on the plug-in reproduces its CPU backend's logits, so their MUL_MAT (the GEMV launches of
    decode, the per-32-block tile kernel for a prompt) and GET_ROWS stay on the device with the reference's arithmetic."""
    if not (os.path.exists(LOGITS) and os.path.exists(PLUGIN)):
        pytest.skip("llama_logits or the plug-in is not built (needs the llama.cpp tree at build time)")
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    import numpy as np
    import make_synthetic_gguf
    import orc
    model = str(tmp_path / (ftype + ".gguf"))
    make_synthetic_gguf.write_model(model, n_layer=2, n_embd=2048, n_ff=4096, n_head=16, n_head_kv=4, n_vocab=2048, ftype=ftype)
    cpu = _logits(model, 0, n_prompt, 3, str(tmp_path / "cpu.bin"))
    dev_out = _logits(model, 99, n_prompt, 3, str(tmp_path / "dev.bin"))
    assert cpu.shape == dev_out.shape and np.isfinite(dev_out).all()
    assert orc.nmse(dev_out, cpu) < 2e-3


def test_model_logits_async_loader(dev, tmp_path):
    """Without mmap the reference's loader uploads the weights in 1 MiB chunks from pinned buffers with set_tensor_async and
    fences the buffers with events (src/llama-model-loader.cpp:926-960, 1033-1046): chunks land at byte offsets inside tensors,
    also inside those kept in the device row layout.  The logits must be the very ones of the mmap load."""
    if not (os.path.exists(LOGITS) and os.path.exists(PLUGIN)):
        pytest.skip("llama_logits or the plug-in is not built (needs the llama.cpp tree at build time)")
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    import numpy as np
    import make_synthetic_gguf
    model = str(tmp_path / "small.gguf")
    make_synthetic_gguf.write_model(model, n_layer=2, n_embd=2048, n_ff=4096, n_head=16, n_head_kv=4, n_vocab=2048)
    mapped = _logits(model, 99, 40, 3, str(tmp_path / "mmap.bin"))
    stats = {}
    read = _logits(model, 99, 40, 3, str(tmp_path / "read.bin"), mmap=False, stats=stats)
    assert stats["events"] > 20 and stats["uploads"] > 20, stats   # the loader did take the asynchronous path
    assert np.isfinite(mapped).all() and np.array_equal(mapped, read)


@pytest.mark.parametrize("n_prompt", [5, 40, 256])   # 256: the wide-tile GEMM on tile images (from 192 rows on)
def test_model_logits_cpu_vs_plugin_and_fused_vs_nodes(dev, tmp_path, n_prompt):
    """The reference's model runtime produces the same logits on its CPU backend and on the plug-in (up to the
    activation-quantization noise that random weights amplify), and the plug-in's fused graph execution reproduces its
    node-by-node execution: decode fusions are bit-identical launches, so only summation-order noise of prefill remains."""
    if not (os.path.exists(LOGITS) and os.path.exists(PLUGIN)):
        pytest.skip("llama_logits or the plug-in is not built (needs the llama.cpp tree at build time)")
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    import numpy as np
    import make_synthetic_gguf
    import orc
    model = str(tmp_path / "small.gguf")
    make_synthetic_gguf.write_model(model, n_layer=2, n_embd=2048, n_ff=4096, n_head=16, n_head_kv=4, n_vocab=2048)
    cpu = _logits(model, 0, n_prompt, 6, str(tmp_path / "cpu.bin"))
    fused = _logits(model, 99, n_prompt, 6, str(tmp_path / "fused.bin"))
    nodes = _logits(model, 99, n_prompt, 6, str(tmp_path / "nodes.bin"), fusion=False)
    assert cpu.shape == fused.shape == nodes.shape and np.isfinite(fused).all()
    # prefill rounds the fused RMS norm differently in the last bit; per-256 activation scales and random weights amplify it
    assert orc.nmse(fused, nodes) < (1e-6 if n_prompt <= 8 else 5e-4)
    assert orc.nmse(nodes, cpu) < 2e-3
    assert orc.nmse(fused, cpu) < 2e-3


def test_model_logits_full_width_8b_layers(dev, tmp_path):
    """Two layers at the full width of BASELINE config 3 (d 4096, ffn 14336, 32 / 8 heads, vocabulary 128256, Q4_K_M mix): the
    reference's runtime on its CPU backend and on the plug-in.  At this width the decode launches are the instantiations the timed
    benchmark step uses (gate + up in one launch with two rows per wave and the activation in LDS, the 128256-row output
    projection), which smaller models never reach."""
    if not (os.path.exists(LOGITS) and os.path.exists(PLUGIN)):
        pytest.skip("llama_logits or the plug-in is not built (needs the llama.cpp tree at build time)")
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    import numpy as np
    import make_synthetic_gguf
    import orc
    model = str(tmp_path / "wide.gguf")
    make_synthetic_gguf.write_model(model, n_layer=2, n_embd=4096, n_ff=14336, n_head=32, n_head_kv=8, n_vocab=128256)
    for n_prompt in (5, 256):
        cpu = _logits(model, 0, n_prompt, 4, str(tmp_path / "cpu.bin"))
        fused = _logits(model, 99, n_prompt, 4, str(tmp_path / "fused.bin"))
        nodes = _logits(model, 99, n_prompt, 4, str(tmp_path / "nodes.bin"), fusion=False, graphs=False)
        assert cpu.shape == fused.shape == nodes.shape and cpu.size % 128256 == 0 and np.isfinite(fused).all()
        assert orc.nmse(fused, nodes) < (1e-6 if n_prompt <= 8 else 5e-4)
        assert orc.nmse(nodes, cpu) < 2e-3 and orc.nmse(fused, cpu) < 2e-3


@pytest.mark.parametrize("cache", [("q8_0", "q8_0"), ("q4_0", "q4_0"), ("q8_0", "f16")])
@pytest.mark.parametrize("n_prompt", [5, 200])
def test_model_logits_quantized_kv_cache(dev, tmp_path, cache, n_prompt):
    """llama.cpp's -ctk / -ctv: the cache tensors are Q8_0 / Q4_0, the stores are CPY f32 -> quantized and FLASH_ATTN_EXT reads quantized
    K / V.  The reference's runtime on the plug-in reproduces its CPU backend's logits with the same cache types, prefill and decode."""
    if not (os.path.exists(LOGITS) and os.path.exists(PLUGIN)):
        pytest.skip("llama_logits or the plug-in is not built (needs the llama.cpp tree at build time)")
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    import numpy as np
    import make_synthetic_gguf
    import orc
    model = str(tmp_path / "small.gguf")
    make_synthetic_gguf.write_model(model, n_layer=2, n_embd=2048, n_ff=4096, n_head=16, n_head_kv=4, n_vocab=2048)
    cpu = _logits(model, 0, n_prompt, 6, str(tmp_path / "cpu.bin"), cache=cache)
    gpu = _logits(model, 99, n_prompt, 6, str(tmp_path / "gpu.bin"), cache=cache)
    assert cpu.shape == gpu.shape and np.isfinite(gpu).all()
    # A 4-bit cache has 16 levels per block: where the two backends' K / V rows differ in the last bits (summation order of the
    # projections), a value on a rounding boundary lands on another level and moves by 1/8 of the block's range.  A short prompt
    # has few cells to average that over.  The op-level parity of the stores and of attention is in tests/test_gpu_kv_quant.py.
    assert orc.nmse(gpu, cpu) < (2e-2 if "q4_0" in cache else 2e-3)


@pytest.mark.parametrize("cache", [None, ("q8_0", "q8_0")])
@pytest.mark.parametrize("n_prompt", [700, 3400])
def test_model_logits_long_context(dev, tmp_path, cache, n_prompt):
    """Contexts beyond the other model tests' 1024 cells: a prompt fed in batches of 512 (prefill attention over a growing cache,
    through the f16 image of a quantized one), then decoded tokens at 700+ cells (the matrix-core decode kernel and its merge
    launch) and at 3400+ cells (the streaming decode kernel, over f16 and over Q8_0 blocks read in place), replayed as HIP graphs.
    The reference's runtime reproduces its CPU backend's logits, and graph replay reproduces launch-by-launch execution bit for bit."""
    if not (os.path.exists(LOGITS) and os.path.exists(PLUGIN)):
        pytest.skip("llama_logits or the plug-in is not built (needs the llama.cpp tree at build time)")
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    import numpy as np
    import make_synthetic_gguf
    import orc
    model = str(tmp_path / "small.gguf")
    make_synthetic_gguf.write_model(model, n_layer=2, n_embd=2048, n_ff=4096, n_head=16, n_head_kv=4, n_vocab=2048)
    cpu = _logits(model, 0, n_prompt, 6, str(tmp_path / "cpu.bin"), cache=cache, ctx=4096)
    st = {}
    gpu = _logits(model, 99, n_prompt, 6, str(tmp_path / "gpu.bin"), cache=cache, ctx=4096, stats=st)
    eager = _logits(model, 99, n_prompt, 6, str(tmp_path / "eager.bin"), cache=cache, ctx=4096, graphs=False)
    assert cpu.shape == gpu.shape == eager.shape and np.isfinite(gpu).all()
    assert st["replays"] >= 3, st
    assert np.array_equal(gpu, eager)
    assert orc.nmse(gpu, cpu) < 2e-3


@pytest.mark.parametrize("cache", [None, ("q8_0", "q8_0"), ("q4_0", "q4_0")])
def test_model_logits_after_context_shift(dev, tmp_path, cache):
    """llama-cli's context shift (llama_kv_cache_seq_rm + seq_add + update): the K-shift graph of build_k_shift (src/llama.cpp:1167-1213)
    runs on the plug-in - ROPE in place on the [head_dim, heads, cells] view of an f16 cache; for a quantized cache the cast of
    that view to f32, ROPE, and the copy back - and the tokens decoded after the shift reproduce the reference CPU backend's logits."""
    if not (os.path.exists(LOGITS) and os.path.exists(PLUGIN)):
        pytest.skip("llama_logits or the plug-in is not built (needs the llama.cpp tree at build time)")
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    import numpy as np
    import make_synthetic_gguf
    import orc
    model = str(tmp_path / "small.gguf")
    make_synthetic_gguf.write_model(model, n_layer=2, n_embd=2048, n_ff=4096, n_head=16, n_head_kv=4, n_vocab=2048)
    cpu = _logits(model, 0, 60, 5, str(tmp_path / "cpu.bin"), cache=cache, shift=17)
    gpu = _logits(model, 99, 60, 5, str(tmp_path / "gpu.bin"), cache=cache, shift=17)
    unshifted = _logits(model, 99, 60, 5, str(tmp_path / "gpu0.bin"), cache=cache)
    assert cpu.shape == gpu.shape and np.isfinite(gpu).all()
    n_vocab = 2048
    assert orc.nmse(gpu, cpu) < (2e-2 if cache and "q4_0" in cache else 2e-3)
    # the shift changes what the decoded tokens see (the prompt's own logits, row 0, come before it)
    assert np.array_equal(gpu[:n_vocab], unshifted[:n_vocab]) and orc.nmse(gpu[n_vocab:], unshifted[n_vocab:]) > 1e-3


@pytest.mark.parametrize("cache", [None, ("q8_0", "q8_0"), ("q4_0", "q4_0")])
def test_model_logits_after_defrag(dev, tmp_path, cache):
    """cells removed from the middle of a sequence and the cache defragmented (build_defrag, src/llama.cpp:1215-1300: copies of whole
    rows inside the K and V cache tensors - for a quantized cache copies between views of one quantized type) on the plug-in.  With
    an f16 cache the tokens decoded afterwards reproduce the reference CPU backend's logits.  With a quantized cache the CPU backend
    is no yardstick: its same-type contiguous copy (ggml_compute_forward_dup_same_cont, ggml-cpu.c:2875-2902) moves
    nelements * type_size bytes, 32 times the blocks it was asked for, and overwrites the cells behind the destination; the
    plug-in copies the blocks of the view, and is held to its own run with an f16 cache instead (same cells moved, only the cache's
    precision differs)."""
    if not (os.path.exists(LOGITS) and os.path.exists(PLUGIN)):
        pytest.skip("llama_logits or the plug-in is not built (needs the llama.cpp tree at build time)")
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    import numpy as np
    import make_synthetic_gguf
    import orc
    model = str(tmp_path / "small.gguf")
    make_synthetic_gguf.write_model(model, n_layer=2, n_embd=2048, n_ff=4096, n_head=16, n_head_kv=4, n_vocab=2048)
    gpu = _logits(model, 99, 60, 5, str(tmp_path / "gpu.bin"), cache=cache, defrag=13)
    whole = _logits(model, 99, 60, 5, str(tmp_path / "gpu0.bin"), cache=cache)
    assert np.isfinite(gpu).all()
    if cache is None:
        cpu = _logits(model, 0, 60, 5, str(tmp_path / "cpu.bin"), defrag=13)
        assert cpu.shape == gpu.shape and orc.nmse(gpu, cpu) < 2e-3
    else:
        f16 = _logits(model, 99, 60, 5, str(tmp_path / "gpu16.bin"), defrag=13)
        f16_whole = _logits(model, 99, 60, 5, str(tmp_path / "gpu160.bin"))
        assert orc.nmse(gpu, f16) < 3 * orc.nmse(whole, f16_whole) + 1e-3   # as close to the f16 cache's logits as without the defragmentation
    assert orc.nmse(gpu[2048:], whole[2048:]) > 1e-3   # the removed cells are gone from what the decoded tokens see


@pytest.mark.parametrize("n_prompt", [3, 48])
def test_moe_model_logits_cpu_vs_plugin(dev, tmp_path, n_prompt):
    """Mixture-of-experts llama (8 experts, 2 used, Q4_K experts, f32 router): the router, top-k selection, MUL_MAT_ID (per-slot
    GEMV for a few slots, slots sorted by expert for many) and the weighted sum all run on the plug-in and reproduce the
    reference CPU backend's logits.  A token whose router scores nearly tie can pick a different expert on the two backends;
    the weights' scale makes such ties unlikely and the tolerance is that of the dense test."""
    if not (os.path.exists(LOGITS) and os.path.exists(PLUGIN)):
        pytest.skip("llama_logits or the plug-in is not built (needs the llama.cpp tree at build time)")
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    import numpy as np
    import make_synthetic_gguf
    import orc
    model = str(tmp_path / "moe.gguf")
    make_synthetic_gguf.write_model(model, n_layer=2, n_embd=2048, n_ff=2048, n_head=16, n_head_kv=4, n_vocab=2048, n_expert=8, n_expert_used=2)
    cpu = _logits(model, 0, n_prompt, 4, str(tmp_path / "cpu.bin"))
    gpu = _logits(model, 99, n_prompt, 4, str(tmp_path / "gpu.bin"))
    nodes = _logits(model, 99, n_prompt, 4, str(tmp_path / "nodes.bin"), fusion=False)
    assert cpu.shape == gpu.shape == nodes.shape and np.isfinite(gpu).all()
    assert orc.nmse(gpu, nodes) < (1e-6 if n_prompt <= 8 else 5e-4)
    assert orc.nmse(gpu, cpu) < 2e-3


@pytest.mark.parametrize("moe,cache", [(False, None), (True, None), (False, ("q8_0", "q8_0")), (False, ("q4_0", "q4_0"))])
def test_decode_graph_replay_equals_launch_by_launch(dev, tmp_path, moe, cache):
    """Decode graphs replayed as HIP graphs give the bits of the same graphs issued launch by launch, over a run that crosses a
    256-cell boundary of the attention window (the graph changes there and is recorded again), with the prompt's prefill and
    the host's synchronizing logits reads between the replays.  Every decoded token's logits are compared.  With a Q8_0 / Q4_0
    cache the stores leave with the Q/K/V launch through the device-side cell list, like the f16 stores."""
    if not (os.path.exists(LOGITS) and os.path.exists(PLUGIN)):
        pytest.skip("llama_logits or the plug-in is not built (needs the llama.cpp tree at build time)")
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    import numpy as np
    import make_synthetic_gguf
    model = str(tmp_path / "small.gguf")
    if moe:
        make_synthetic_gguf.write_model(model, n_layer=2, n_embd=2048, n_ff=2048, n_head=16, n_head_kv=4, n_vocab=2048, n_expert=8, n_expert_used=2)
    else:
        make_synthetic_gguf.write_model(model, n_layer=3, n_embd=2048, n_ff=4096, n_head=16, n_head_kv=4, n_vocab=2048)
    st = {}
    replayed = _logits(model, 99, 249, 14, str(tmp_path / "graph.bin"), stats=st, cache=cache)
    launched = _logits(model, 99, 249, 14, str(tmp_path / "eager.bin"), graphs=False, cache=cache)
    assert st["captures"] >= 2 and st["replays"] >= 8, st
    assert replayed.shape == launched.shape and np.isfinite(replayed).all()
    assert np.array_equal(replayed, launched)


@pytest.mark.parametrize("cache", [None, ("q8_0", "q8_0")])
def test_launches_per_layer(dev, tmp_path, cache):
    """What the plug-in launches for the reference's llama graphs, counted by the kernel library itself and reported per graph
    under MI355_LOG_GRAPH (one-time copies of weights are reported apart): the difference between a 4-layer and a 2-layer
    model is two layers' worth.  One decoded token takes 6 launches per layer ([norm + Q/K/V + rope + cache stores] [attention]
    [wo + residual] [norm] [gate + up + SiLU*up] [down + residual]).  A prompt of 200 tokens (the wide-tile GEMM; decode then
    stays within 256 cache cells) takes 9: [Q + K + V in one launch whatever their K-quant types, with both rotations and both
    f16 cache stores in its epilogue], attention, quantization, wo (cut along K), [the sum of its slices + residual + FFN norm +
    quantization], [gate + up in one launch], SiLU*up, down (cut along K), [slice sum + residual + the next layer's norm].  With a Q8_0
    cache a prompt batch keeps a launch of its own for [rope, rope, store, store] and adds the one that expands the cells it attends to
    into f16: 11."""
    if not (os.path.exists(LOGITS) and os.path.exists(PLUGIN)):
        pytest.skip("llama_logits or the plug-in is not built (needs the llama.cpp tree at build time)")
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    import make_synthetic_gguf
    counts = {}
    for n_layer in (2, 4):
        model = str(tmp_path / ("l%d.gguf" % n_layer))
        make_synthetic_gguf.write_model(model, n_layer=n_layer, n_embd=4096, n_ff=14336, n_head=32, n_head_kv=8, n_vocab=2048)
        env = dict(os.environ, GGML_BACKEND_PATH=PLUGIN, MI355_LOG_GRAPH="1", MI355_NO_GRAPH="1")
        r = subprocess.run([LOGITS, model, "99", "200", "3", str(tmp_path / "o.bin")] + (list(cache) if cache else []), env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                           text=True, timeout=600, cwd=os.path.dirname(LOGITS))
        assert r.returncode == 0, r.stdout[-3000:]
        per_batch = {}
        for m in re.finditer(r"MI355 graph launches: (\d+) nodes, batch (\d+), (\d+) attention nodes, (\d+) kernel launches \+ (\d+) for one-time", r.stdout):
            assert int(m.group(3)) == n_layer
            per_batch[int(m.group(2))] = int(m.group(4))
        assert 1 in per_batch and 200 in per_batch, r.stdout[-3000:]
        counts[n_layer] = per_batch
    decode = (counts[4][1] - counts[2][1]) / 2
    prefill = (counts[4][200] - counts[2][200]) / 2
    os.makedirs(os.path.join(ROOT, "gpurun_out"), exist_ok=True)
    with open(os.path.join(ROOT, "gpurun_out", "launches_per_layer.txt"), "a") as f:
        f.write("cache %s: decode %g launches per layer, prefill(200) %g; totals %r\n" % (cache[0] if cache else "f16", decode, prefill, counts))
    assert decode == 6, counts     # norm + Q/K/V + ROPE + stores, attention, wo + residual, norm, gate + up + SiLU*up, down + residual
    assert prefill <= (11 if cache else 9), counts
