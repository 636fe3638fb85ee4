#!/usr/bin/env python3
"""Headline benchmark: llama-bench-style tg128 (and pp512) on a Llama-3-8B-shaped Q4_K_M model,
all operators on one MI355X through the kernel C ABI (llama.cpp_amd/mi355/llama_graph.py issues
the node sequence of llama.cpp's build_llama).

One step = one decoded token (batch 1): upload of the token embedding, the 32-layer graph, the
128256-wide logits and their read-back, then a device synchronise - what llama-bench's test_gen
times per token (examples/llama-bench/llama-bench.cpp:1454-1468).  Weights are resident in HBM
before the timed region.  Prints ONE JSON line.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "llama.cpp_amd"))

HBM_PEAK_GBS = 8000.0
# HBM bytes one launch of the roofline kernel moves: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE readings of this command, scaled by
# the readings of the plain copy kernel the run ends with.  `python bench.py --traffic-from <fetch dir> <write dir>` turns the two
# counter runs into this file, together with the commit they were measured at; the bench line quotes both.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "gemv_gate_up_q4k_hbm_traffic.txt")
ROOFLINE_KERNEL = "k_gemv_gate_up_blk"        # as it appears in the profiler's kernel names
COPY_KERNEL = "k_cpy"
COPY_BYTES = 16384 * 4096 * 4           # read, and as many written


def read_traffic():
    """(bytes per launch or None, commit or None) from the tracked counter summary"""
    try:
        text = open(TRAFFIC_FILE).read()
    except OSError:
        return None, None
    val = commit = None
    for line in text.splitlines():
        if line.startswith("traffic_bytes_per_launch:"):
            val = int(line.split(":", 1)[1].strip())
        if line.startswith("measured_at_commit:"):
            commit = line.split(":", 1)[1].strip()
    return val, commit


def traffic_from(fetch_dir, write_dir):
    """Reads the counter_collection.csv files of the two rocprofv3 --pmc runs and rewrites TRAFFIC_FILE.  Runs where the .git
    directory is (the commit id goes into the file), on the CPU."""
    import csv
    import glob
    import subprocess

    def per_kernel(d, counter):
        rows = {}
        files = glob.glob(os.path.join(d, "**", "*counter_collection.csv"), recursive=True)
        assert files, "no counter_collection.csv under " + d
        for f in files:
            for r in csv.DictReader(open(f)):
                if r.get("Counter_Name") != counter:
                    continue
                rows.setdefault(r["Kernel_Name"], []).append(float(r["Counter_Value"]))
        return rows

    out = {}
    for d, counter in ((fetch_dir, "FETCH_SIZE"), (write_dir, "WRITE_SIZE")):
        rows = per_kernel(d, counter)
        cpy = [v for k, vs in rows.items() if COPY_KERNEL in k for v in vs]
        ker = [v for k, vs in rows.items() if ROOFLINE_KERNEL in k for v in vs]
        assert cpy and ker, "kernels not found in " + d
        unit = COPY_BYTES / (sum(cpy) / len(cpy))          # bytes per counter unit, from the copy of known size
        out[counter] = (sum(ker) / len(ker), len(ker), min(ker), max(ker), sum(cpy) / len(cpy), unit)
    commit = subprocess.run(["git", "-C", ROOT, "rev-parse", "--short", "HEAD"], stdout=subprocess.PIPE, text=True).stdout.strip() or "unknown"
    fetch_b = out["FETCH_SIZE"][0] * out["FETCH_SIZE"][5]
    write_b = out["WRITE_SIZE"][0] * out["WRITE_SIZE"][5]
    lines = [
        "HBM traffic of the roofline kernel of bench.py: k_gemv_gate_up_blk<Q4_K, 1 column, 8 waves, 4 + 4 rows in flight> on the ffn_gate + ffn_up",
        "matrices of one layer (2 x 14336 x 4096 Q4_K, SiLU * up + Q8_1 inside) - the launch a decoded token makes 32 times - on one MI355X",
        "",
        "commands (from /tmp, TMPDIR=/tmp; counters in their own runs, no trace domains):",
        "  rocprofv3 --pmc FETCH_SIZE -d <fetch dir> -o f --output-format csv -- python3 bench.py --no-cpu --pp 0 --steps 4 --warmup 2",
        "  rocprofv3 --pmc WRITE_SIZE -d <write dir> -o w --output-format csv -- python3 bench.py --no-cpu --pp 0 --steps 4 --warmup 2",
        "  python bench.py --traffic-from <fetch dir> <write dir>        (where the repository is; writes this file)",
        "",
        "calibration: the run ends with one launch of the plain copy kernel k_cpy<float, float> on a 16384 x 4096 f32 tensor,",
        "256 MiB read and 256 MiB written.",
        "  k_cpy  FETCH_SIZE = %.1f  -> %.4f bytes per counter unit" % (out["FETCH_SIZE"][4], out["FETCH_SIZE"][5]),
        "  k_cpy  WRITE_SIZE = %.1f  -> %.4f bytes per counter unit" % (out["WRITE_SIZE"][4], out["WRITE_SIZE"][5]),
        "",
        "%s, %d dispatches, per dispatch:" % (ROOFLINE_KERNEL, out["FETCH_SIZE"][1]),
        "  FETCH_SIZE = %.1f units (min %.1f, max %.1f) = %d B read" % (out["FETCH_SIZE"][0], out["FETCH_SIZE"][2], out["FETCH_SIZE"][3], fetch_b),
        "  WRITE_SIZE = %.1f units (min %.1f, max %.1f) = %d B written" % (out["WRITE_SIZE"][0], out["WRITE_SIZE"][2], out["WRITE_SIZE"][3], write_b),
        "",
        "traffic_bytes_per_launch: %d" % int(fetch_b + write_b),
        "measured_at_commit: %s" % commit,
        "",
        "algorithmic bytes per launch: 2 x 14336 x 4096 x 144/256 (weights) + 4096 x 1.25 (Q8_1 activation: levels + scale/sum pairs)",
        "  + 2 x 4 x 14336 (f32 outputs) + 14336 x 1.25 (Q8_1 of SiLU * up) = 66,060,288 + 5,120 + 114,688 + 17,920 = 66,198,016 B",
    ]
    with open(TRAFFIC_FILE, "w") as f:
        f.write("\n".join(lines) + "\n")
    print("\n".join(lines))


def physical_cores():
    """distinct (package, core) pairs among the CPUs this process may run on, capped at the 16-thread share of a one-GPU box"""
    allowed = os.sched_getaffinity(0)
    cores = set()
    cpu = phys = core = None
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("processor"):
                cpu = int(line.split(":")[1])
            elif line.startswith("physical id"):
                phys = int(line.split(":")[1])
            elif line.startswith("core id"):
                core = int(line.split(":")[1])
            elif not line.strip():
                if cpu in allowed and phys is not None and core is not None:
                    cores.add((phys, core))
                cpu = phys = core = None
    except OSError:
        pass
    n = len(cores) or len(allowed)
    return max(1, min(n, 16)), n


def cpu_baseline():
    """ggml-cpu (the reference's own CPU backend, built by oracle/Makefile) timed on this host: batch-1 MUL_MAT over the weight
    shapes of one Q4_K_M layer plus the output projection, each shape for at least a second after a warm-up run, summed with
    the shapes' per-token multiplicities -> tokens/s of the matmul part of tg (the rest of the graph is a few percent on CPU).
    Once with one thread per physical core of this process's share of the host, once with a single thread."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import numpy as np
    import orc
    if orc.ref is None:
        return None
    rng = np.random.default_rng(1234)
    shapes = [("wq", 4096, 4096, orc.Q4_K, 32), ("wk", 1024, 4096, orc.Q4_K, 32), ("wv", 1024, 4096, orc.Q4_K, 16),
              ("wv6", 1024, 4096, orc.Q6_K, 16), ("wo", 4096, 4096, orc.Q4_K, 32), ("gate", 14336, 4096, orc.Q4_K, 32),
              ("up", 14336, 4096, orc.Q4_K, 32), ("down", 4096, 14336, orc.Q4_K, 16), ("down6", 4096, 14336, orc.Q6_K, 16),
              ("output", 128256, 4096, orc.Q6_K, 1)]
    n_threads, n_phys = physical_cores()
    t_token = {n_threads: 0.0, 1: 0.0}
    for name, N, K, t, count in shapes:
        # random blocks with sane scales: the CPU kernels' time does not depend on the values
        rb = orc.row_bytes(t, K)
        W = rng.integers(0, 256, (N, rb), dtype=np.uint8)
        bb = orc.BLOCK[t][1]
        Wv = W.reshape(N, -1, bb)
        h = np.array([1e-4], dtype=np.float16).view(np.uint8)
        if t == orc.Q4_K:
            Wv[:, :, 0:2] = h
            Wv[:, :, 2:4] = h
        else:
            Wv[:, :, 208:210] = h
        x = rng.standard_normal((1, K)).astype(np.float32)
        out = np.zeros((1, N), dtype=np.float32)
        for nt in sorted(t_token):
            # ref_mul_mat makes one untimed run, then `reps` timed ones: a short probe sizes the >= 1 s loop
            probe = orc.ref.ref_mul_mat(t, orc._ptr(W), orc._ptr(x), orc._ptr(out), N, K, 1, nt, 2)
            reps = max(3, int(1.0 / max(probe, 1e-6)) + 1)
            t_token[nt] += orc.ref.ref_mul_mat(t, orc._ptr(W), orc._ptr(x), orc._ptr(out), N, K, 1, nt, reps) * count
    return {"value": round(1.0 / t_token[n_threads], 2), "unit": "tokens/s", "cores": n_threads, "kind": "reference",
            "one_thread": round(1.0 / t_token[1], 2), "physical_cores_available": n_phys,
            "sample": "ggml-cpu (AVX2 build of the reference sources) batch-1 MUL_MAT over the 10 distinct weight shapes/types of the "
                      "Q4_K_M model, each timed for >= 1 s after a warm-up run, summed with their per-token multiplicities (32 layers "
                      "+ output); matmuls only; threads = physical cores in this process's CPU share (at most 16); end-to-end CPU "
                      "figures of the reference's llama-bench are in profiles/llama_bench_llama8b_q4km_cpu.txt"}


INT8_PEAK_TOPS = 5000.0      # dense int8 MFMA
F16_PEAK_TFLOPS = 2500.0     # dense f16 MFMA


def sweep(kinds):
    """Per-kernel roofline tables (one JSON line per case): the matrix products at batch 1 (HBM) and batch 64/512 (int8 MFMA) and
    FLASH_ATTN_EXT for decode (HBM) and prefill (f16 MFMA) on the Llama-3-8B shapes.  HIP events on the launching stream over
    operands rotated through more memory than the caches hold.  Not part of the default run."""
    import math
    import torch
    import mi355
    from mi355 import llama_graph as lg
    lib = mi355.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    gen = torch.Generator(device=dev).manual_seed(1)
    stream = torch.cuda.Stream()

    def timed(fn, n_items, reps):
        # the n_items calls are recorded once and replayed as a HIP graph, so short kernels are not limited by the host's launch rate
        with torch.cuda.stream(stream):
            for i in range(n_items):
                fn(i)
            stream.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=stream):
                for i in range(n_items):
                    fn(i)
            g.replay()
            stream.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            for _ in range(reps):
                g.replay()
            e1.record(stream)
            stream.synchronize()
        return e0.elapsed_time(e1) * 1e3 / (reps * n_items)

    def emit(**kw):
        print(json.dumps(kw), flush=True)

    bpe = {mi355.Q4_0: 18 / 32, mi355.Q8_0: 34 / 32, mi355.Q4_K: 144 / 256, mi355.Q5_K: 176 / 256, mi355.Q6_K: 210 / 256,
           mi355.Q4_1: 20 / 32, mi355.Q5_0: 22 / 32, mi355.Q5_1: 24 / 32, mi355.IQ4_NL: 18 / 32, mi355.IQ4_XS: 136 / 256}
    names = {mi355.Q4_0: "Q4_0", mi355.Q8_0: "Q8_0", mi355.Q4_K: "Q4_K", mi355.Q5_K: "Q5_K", mi355.Q6_K: "Q6_K", mi355.Q4_1: "Q4_1", mi355.Q5_0: "Q5_0",
             mi355.Q5_1: "Q5_1", mi355.IQ4_NL: "IQ4_NL", mi355.IQ4_XS: "IQ4_XS"}
    all_types = (mi355.Q4_0, mi355.Q8_0, mi355.Q4_K, mi355.Q5_K, mi355.Q6_K, mi355.Q4_1, mi355.Q5_0, mi355.Q5_1, mi355.IQ4_NL, mi355.IQ4_XS)
    shapes = [(4096, 4096), (14336, 4096), (4096, 14336)]
    if "gemv" in kinds:
        for t in all_types:
            for N, K in shapes + [(128256, 4096)]:
                wbytes = int(N * K * bpe[t])
                nm = max(2, min(32, (1 << 31) // wbytes))
                Ws = [mi355.upload_weights(t, lg.random_quantized(t, N, K, dev, gen)) for _ in range(nm)]
                for B in (1, 8):
                    act = mi355.quantize_act(torch.randn(B, K, device=dev, generator=gen))
                    out = torch.empty(B, N, device=dev)
                    if B == 1:
                        us = timed(lambda i: mi355.check(lib.mi355_mul_mat_vec_q(stream.cuda_stream, t, Ws[i].data_ptr(), act.data_ptr(), out.data_ptr(), N, K, B, N)), nm, 4)
                    else:   # the weight-streaming matrix-core kernel, with the workspace that lets products with few rows split K
                        ws = torch.empty(int(lib.mi355_mul_mat_skinny_ws_bytes(N, K, B)) + 256, dtype=torch.uint8, device=dev)
                        us = timed(lambda i: mi355.check(lib.mi355_mul_mat_skinny(stream.cuda_stream, t, Ws[i].data_ptr(), act.data_ptr(), out.data_ptr(), None, N, K, B, N,
                                                                                  ws.data_ptr(), ws.numel())), nm, 4)
                    alg = wbytes + B * (4 * K + 4 * N)
                    emit(kernel="MUL_MAT batch 1 (GEMV)" if B == 1 else "MUL_MAT batch %d (k_mm_skinny)" % B, case="%s %dx%d" % (names[t], N, K), us=round(us, 2), bound="hbm", achieved=round(alg / us / 1e3, 1),
                         unit="GB/s", frac=round(alg / us / 1e3 / HBM_PEAK_GBS, 4), algorithmic_bytes=alg)
                del Ws
    if "mmq" in kinds or "mmq_wide" in kinds:
        wide_only = "mmq" not in kinds    # the wide-tile GEMM alone on the gate/up shape (for counter collection)
        for t in ((mi355.Q4_K, mi355.Q5_K, mi355.Q6_K, mi355.IQ4_XS) if wide_only else all_types):
            for N, K in ([(14336, 4096)] if wide_only else shapes):
                for B in ((512,) if wide_only else (64, 512)):
                    nm = 4
                    Ws = [mi355.upload_weights(t, lg.random_quantized(t, N, K, dev, gen)) for _ in range(nm)]
                    x = torch.randn(B, K, device=dev, generator=gen)
                    out = torch.empty(B, N, device=dev)
                    ws = torch.empty(int(lib.mi355_mul_mat_ws_bytes(K, B)) + max(int(lib.mi355_mul_mat_q8k_ws_bytes(N, K, B)), int(lib.mi355_mul_mat_q_ws_bytes(N, K, B))) + 256,
                                     dtype=torch.uint8, device=dev)
                    ops = 2.0 * N * K * B
                    if not wide_only:
                        us = timed(lambda i: mi355.check(lib.mi355_mul_mat(stream.cuda_stream, t, Ws[i].data_ptr(), x.data_ptr(), out.data_ptr(), N, K, B, K, N,
                                                                           ws.data_ptr(), ws.numel())), nm, 5)
                        label = "MUL_MAT batch %d (activation quantization + tile GEMM)" % B
                        emit(kernel=label, case="%s %dx%d" % (names[t], N, K), us=round(us, 2), bound="mfma",
                             achieved=round(ops / us / 1e6, 1), unit="TOP/s", frac=round(ops / us / 1e6 / INT8_PEAK_TOPS, 4), ops=ops)
                    if t in (mi355.Q4_K, mi355.Q5_K, mi355.Q6_K, mi355.IQ4_XS):   # the wide-tile GEMM on tile images (what prefill uses for K-quants), without the quantization
                        tiles = [mi355.kq_unpack_tiles(t, W) for W in Ws]
                        a8 = mi355.quantize_act_q8k_tiled(x)
                        sws = torch.empty(int(lib.mi355_mul_mat_q8k_tiled_ws_bytes(N, K, B)) + 256, dtype=torch.uint8, device=dev)
                        us = timed(lambda i: mi355.check(lib.mi355_mul_mat_q8k_tiled(stream.cuda_stream, t, tiles[i].data_ptr(), a8.data_ptr(), out.data_ptr(), None,
                                                                                     N, K, B, N, sws.data_ptr(), sws.numel())), nm, 5)
                        emit(kernel="wide-tile GEMM on tile images, batch %d" % B, case="%s %dx%d" % (names[t], N, K), us=round(us, 2), bound="mfma",
                             achieved=round(ops / us / 1e6, 1), unit="TOP/s", frac=round(ops / us / 1e6 / INT8_PEAK_TOPS, 4), ops=ops)
                        del tiles
                    if t == mi355.Q6_K and B == 512 and not wide_only:   # the same product from the unpacked planes (the 64 x 128 tile kernel)
                        planes = [torch.empty(int(lib.mi355_kq_planes_bytes(N, K)) + 256, dtype=torch.uint8, device=dev) for _ in range(nm)]
                        for W, P in zip(Ws, planes):
                            mi355.check(lib.mi355_kq_unpack_planes(None, t, W.data_ptr(), P.data_ptr(), N, K))
                        a8 = mi355.quantize_act_q8k(x)
                        us = timed(lambda i: mi355.check(lib.mi355_mul_mat_q8k_planes(stream.cuda_stream, t, planes[i].data_ptr(), a8.data_ptr(), out.data_ptr(), None,
                                                                                      N, K, B, N)), nm, 5)
                        emit(kernel="tile GEMM from unpacked planes, batch 512", case="Q6_K %dx%d" % (N, K), us=round(us, 2), bound="mfma",
                             achieved=round(ops / us / 1e6, 1), unit="TOP/s", frac=round(ops / us / 1e6 / INT8_PEAK_TOPS, 4), ops=ops)
                        del planes
                    del Ws
    if "fattn" in kinds or "fattn_long" in kinds or "fattn_prefill" in kinds or "fattn_prefill_512" in kinds:
        H, HK, D = 32, 8, 128
        cases = [(1, 256), (1, 512), (1, 1024), (1, 4096), (1, 32768), (1, 131072), (512, 512), (512, 4096), (2048, 2048), (4096, 4096)]
        if "fattn" not in kinds:   # one kernel alone (for counter collection): long-context decode and / or the prefill kernel
            cases = ([(1, 131072)] if "fattn_long" in kinds else []) + ([(4096, 4096)] if "fattn_prefill" in kinds else []) + \
                    ([(512, 4096)] if "fattn_prefill_512" in kinds else [])
        for Nq, Nkv in cases:
            nrot = max(2, min(16, (1 << 30) // (Nkv * HK * D * 4))) if Nq == 1 else 1
            q = torch.randn(Nq, H, D, device=dev, generator=gen)
            ks = [torch.randn(Nkv, HK, D, device=dev, generator=gen).half() for _ in range(nrot)]
            vs = [torch.randn(Nkv, HK, D, device=dev, generator=gen).half() for _ in range(nrot)]
            npad = (Nq + 63) // 64 * 64
            mask = torch.full((npad, Nkv), float("-inf"), dtype=torch.float16, device=dev)
            rows = torch.arange(npad, device=dev)[:, None]
            cols = torch.arange(Nkv, device=dev)[None, :]
            mask[(cols <= Nkv - Nq + rows) & (rows < Nq)] = 0.0
            dst = torch.empty(Nq, H, D, device=dev)
            ws = torch.empty(min(int(lib.mi355_flash_attn_ws_bytes(D, Nq, Nkv, H)), 1 << 28), dtype=torch.uint8, device=dev)

            def fa(i):
                mi355.check(lib.mi355_flash_attn_ext(stream.cuda_stream, q.data_ptr(), ks[i].data_ptr(), vs[i].data_ptr(), mask.data_ptr(), dst.data_ptr(), D, Nq, Nkv, H,
                                                     HK, H * D * 4, D * 4, HK * D * 2, D * 2, HK * D * 2, D * 2, Nkv * 2, 1 / math.sqrt(D), 0.0, 0.0, ws.data_ptr(),
                                                     ws.numel()))
            us = timed(fa, nrot, 4 if Nq == 1 else 10)
            if Nq == 1:
                alg = 4 * HK * D * Nkv + 2 * Nkv + 4 * H * D * 2
                emit(kernel="FLASH_ATTN_EXT decode (all launches of one call)", case="Nkv %d" % Nkv, us=round(us, 2), bound="hbm", achieved=round(alg / us / 1e3, 1),
                     unit="GB/s", frac=round(alg / us / 1e3 / HBM_PEAK_GBS, 4), algorithmic_bytes=alg)
            else:
                fl = 4.0 * H * Nq * D * Nkv
                emit(kernel="FLASH_ATTN_EXT prefill, causal mask (nominal flops, masked cells included)", case="Nq %d Nkv %d" % (Nq, Nkv), us=round(us, 2), bound="mfma",
                     achieved=round(fl / us / 1e6, 1), unit="TFLOP/s", frac=round(fl / us / 1e6 / F16_PEAK_TFLOPS, 4), flops=fl)
            del ks, vs

    if "fattn" in kinds or "fattn_kv" in kinds:
        # decode over a quantized cache kept as llama.cpp's cache tensors are in a plug-in buffer (a 1-D tensor of all cells in the device
        # row layout: all levels first, all scales behind them), filled through the quantizing store; the blocks are read where they lie
        H, HK, D = 32, 8, 128
        for tname, t, bb in (("Q8_0", mi355.Q8_0, 34), ("Q4_0", mi355.Q4_0, 18)):
            for Nkv in (256, 1024, 4096, 32768, 131072):
                nrot = max(2, min(16, (1 << 29) // (Nkv * HK * D)))
                cb = HK * D // 32              # blocks per cell
                rb = Nkv * cb                  # blocks of the one row that is the whole cache
                row_bytes = cb * bb
                q = torch.randn(1, H, D, device=dev, generator=gen)
                caches = []
                for _ in range(2 * nrot):
                    c = torch.empty(Nkv * row_bytes, dtype=torch.uint8, device=dev)
                    src = torch.randn(Nkv, HK * D, device=dev, generator=gen)
                    mi355.check(lib.mi355_cpy_f32_quant(stream.cuda_stream, t, src.data_ptr(), c.data_ptr(), 0, rb, Nkv * HK * D))
                    caches.append(c)
                torch.cuda.synchronize()
                mask = torch.zeros((64, Nkv), dtype=torch.float16, device=dev)
                dst = torch.empty(1, H, D, device=dev)
                need = int(lib.mi355_flash_attn_ws_bytes(D, 1, Nkv, H))
                ws = torch.empty(min(need, 1 << 28) + 256, dtype=torch.uint8, device=dev)
                wp = (ws.data_ptr() + 255) & ~255

                def fa(i):
                    kc, vc = caches[2 * i], caches[2 * i + 1]
                    mi355.check(lib.mi355_flash_attn_ext_kv(stream.cuda_stream, q.data_ptr(), kc.data_ptr(), t, kc.data_ptr(), rb, vc.data_ptr(), t, vc.data_ptr(), rb,
                                                            mask.data_ptr(), dst.data_ptr(), D, 1, Nkv, H, HK, H * D * 4, D * 4, row_bytes, D // 32 * bb, row_bytes,
                                                            D // 32 * bb, Nkv * 2, 1 / math.sqrt(D), 0.0, 0.0, wp, ws.numel() - 256, None))
                us = timed(fa, nrot, 4)
                alg = 2 * Nkv * row_bytes + 2 * Nkv + 4 * H * D * 2
                emit(kernel="FLASH_ATTN_EXT decode over a %s cache read in place (all launches of one call)" % tname, case="Nkv %d" % Nkv, us=round(us, 2), bound="hbm",
                     achieved=round(alg / us / 1e3, 1), unit="GB/s", frac=round(alg / us / 1e3 / HBM_PEAK_GBS, 4), algorithmic_bytes=alg, cache_bytes=2 * Nkv * row_bytes)
                del caches


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--no-graph", action="store_true", help="launch every kernel from the host instead of replaying a HIP graph")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--random-blocks", action="store_true", help="fill the weights with random blocks instead of quantizing N(0, 0.02) values on the device")
    ap.add_argument("--pp", type=int, default=512, help="prompt length of the prefill measurement (0 = skip)")
    ap.add_argument("--sweep", default="", help="comma-separated kernel tables instead of the model run: gemv, mmq, mmq_wide (the wide-tile GEMM on 14336 x 4096 at batch 512 only), fattn, "
                                          "fattn_long (decode over 131072 cells only), fattn_prefill (4096 x 4096 prefill only), fattn_prefill_512 (512 rows over 4096 cells only), fattn_kv (decode over Q8_0 / Q4_0 caches only)")
    ap.add_argument("--traffic-from", nargs=2, metavar=("FETCH_DIR", "WRITE_DIR"),
                    help="rewrite the tracked HBM-traffic summary from two rocprofv3 --pmc output directories (no GPU needed)")
    args = ap.parse_args()
    if args.traffic_from:
        traffic_from(*args.traffic_from)
        return
    if args.sweep:
        if args.gpus != 1:
            sys.exit("bench.py: one GPU only")
        sweep([k.strip() for k in args.sweep.split(",") if k.strip()])
        return
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (no collectives, no sharding); --gpus %d is not available" % args.gpus,
              file=sys.stderr)
        sys.exit(2)

    import torch
    import mi355
    from mi355 import llama_graph as lg
    lib = mi355.load()   # raises if the HIP library is missing: there is no CPU path to fall back to
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    cfg = lg.LlamaConfig()
    n_ctx = max(512, (args.warmup + args.steps + 255) // 256 * 256, args.pp)
    cfg.n_ctx = n_ctx
    tq = time.perf_counter()
    weights = lg.LlamaWeights(cfg, dev, quantize=not args.random_blocks)     # N(0, 0.02) weights quantized on the device (Q4_K_M mix)
    torch.cuda.synchronize()
    quantize_s = time.perf_counter() - tq
    run = lg.LlamaRunner(weights, max_tokens=max(args.pp, 8))
    emb = torch.randn(max(args.pp, 8), cfg.n_embd).pin_memory()
    logits_host = torch.empty(cfg.n_vocab, dtype=torch.float32).pin_memory()
    stream = torch.cuda.Stream()          # default priority; graph capture needs a non-default stream
    torch.cuda.synchronize()

    # ------------------------------------------------------------------ tg: K decode steps
    graphs = {}

    def decode_step(pos):
        n_kv = (pos + 1 + 255) // 256 * 256          # llama.cpp pads n_kv to 256 with flash attention (src/llama.cpp:8565)
        with torch.cuda.stream(stream):
            run.x[:1].copy_(emb[pos % emb.shape[0]:pos % emb.shape[0] + 1], non_blocking=True)
            run.pos[:1].fill_(pos)
            run.mask[0, pos:pos + 1].fill_(0.0)
            if args.no_graph:
                run.forward(1, n_kv)
            else:
                g = graphs.get(n_kv)
                if g is None:
                    run.forward(1, n_kv)                 # warm every kernel once outside capture
                    stream.synchronize()
                    g = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(g, stream=stream):
                        run.forward(1, n_kv)
                    graphs[n_kv] = g
                g.replay()
            logits_host.copy_(run.logits[0], non_blocking=True)
        stream.synchronize()

    run.mask.fill_(float("-inf"))
    for p in range(args.warmup):
        decode_step(p)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for p in range(args.warmup, args.warmup + args.steps):
        decode_step(p)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt / args.steps * 1e3
    tg = args.steps / dt
    finite = bool(torch.isfinite(logits_host).all())

    # ------------------------------------------------------------------ pp512: one prefill batch
    pp = None
    if args.pp > 0:
        T = args.pp
        n_kv = (T + 255) // 256 * 256
        with torch.cuda.stream(stream):
            run.set_inputs(emb, 0, T, n_kv)
            run.forward(T, n_kv)
            stream.synchronize()
            reps = 3
            t0 = time.perf_counter()
            for _ in range(reps):
                run.x[:T].copy_(emb[:T], non_blocking=True)
                run.forward(T, n_kv)
                logits_host.copy_(run.logits[0], non_blocking=True)
                stream.synchronize()
            pp = T * reps / (time.perf_counter() - t0)

    # ------------------------------------------------------------------ roofline of the dominant kernel
    # k_gemv_gate_up_blk on ffn_gate + ffn_up (2 x 14336 x 4096 Q4_K, SiLU * up and its Q8_1 quantization inside the launch): what
    # the timed step launches 32 times per token, 46% of the bytes of a decoded token.  Timed with HIP events on its own stream
    # through the runner's own call, over the 32 layers' matrices (2.1 GB, so neither L2 nor the 256 MB Infinity Cache can serve them).
    N, K = cfg.n_ff, cfg.n_embd
    pairs = [(L["gate"], L["up"]) for L in weights.layers]

    def gate_up(pair):
        (tg, Wg), (tu, Wu) = pair
        mi355.check(lib.mi355_ffn_gate_up_swiglu(stream.cuda_stream, tg, Wg.data_ptr(), tu, Wu.data_ptr(), run.act_c.data_ptr(), run.gate.data_ptr(),
                                                 run.up.data_ptr(), N, run.act_b.data_ptr(), run.tickets.data_ptr(), N, K, 1))

    with torch.cuda.stream(stream):
        run._norm_quant(run.x[:1], weights.layers[0]["ffn_norm"], run.act_c, 1)
        for gu in pairs[:4]:
            gate_up(gu)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        nrep = 8
        e0.record(stream)
        for _ in range(nrep):
            for gu in pairs:
                gate_up(gu)
        e1.record(stream)
        stream.synchronize()
    us = e0.elapsed_time(e1) * 1e3 / (nrep * len(pairs))
    wtypes = {t for gu in pairs for t, _ in gu}
    assert wtypes == {mi355.Q4_K}, "the roofline kernel's byte count assumes Q4_K gate/up matrices"
    # weights + Q8_1 activation in + two f32 outputs + Q8_1 activation out
    alg_bytes = 2 * (N * K * 144 // 256) + (K + K // 4) + 2 * 4 * N + (N + N // 4)
    achieved = alg_bytes / us / 1e3                                       # GB/s
    traffic, traffic_commit = read_traffic()
    roofline = {"kernel": "k_gemv_gate_up_blk<Q4_K, 1 column, 8 waves, 4 + 4 rows in flight> on ffn_gate + ffn_up with SiLU * up + Q8_1, 2 x 14336 x 4096 "
                          "(the launch the timed step makes once per layer)", "bound": "hbm", "achieved": round(achieved, 1),
                "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic,
                "traffic_source": "profiles/%s, measured at commit %s" % (os.path.basename(TRAFFIC_FILE), traffic_commit) if traffic else None,
                "us_per_launch": round(us, 3), "algorithmic_bytes_per_launch": alg_bytes}

    # ------------------------------------------------------------------ ... and of the dominant prefill kernel
    # k_mmq_w<Q4_K> (wide-tile int8-MFMA GEMM on tile images) on ffn_gate + ffn_up at the prompt's batch, one launch for the pair:
    # 2 of the 7 products of a layer and 56% of its multiply-adds.  The same call the prefill pass makes, over the 32 layers' tile images.
    roofline_pp = None
    if args.pp >= 192:
        T = args.pp
        with torch.cuda.stream(stream):
            run._norm_quant(run.x[:T], weights.layers[0]["ffn_norm"], run.act_a, T, 2)
            pairs = [[(L["gate"], run.gate[:T]), (L["up"], run.up[:T])] for L in weights.layers]
            for m in pairs[:2]:
                run._mm_act(m, run.act_a, K, T, q8k=2)
            p0, p1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            p0.record(stream)
            for m in pairs:
                run._mm_act(m, run.act_a, K, T, q8k=2)
            p1.record(stream)
            stream.synchronize()
        pus = p0.elapsed_time(p1) * 1e3 / len(pairs)
        ops = 2.0 * 2 * N * K * T
        roofline_pp = {"kernel": "k_mmq_w<Q4_K> on ffn_gate + ffn_up in one launch, 2 x 14336 x 4096, batch %d (the launch the prefill pass makes once per layer)" % T,
                       "bound": "mfma", "achieved": round(ops / pus / 1e6, 1), "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
                       "frac": round(ops / pus / 1e6 / INT8_PEAK_TOPS, 4), "traffic": None, "us_per_launch": round(pus, 2), "ops_per_launch": ops}

    # reference for the HBM traffic counters: a plain copy kernel of known size (256 MiB read, 256 MiB written) whose
    # FETCH_SIZE / WRITE_SIZE readings calibrate the counters' unit when this command runs under rocprofv3 --pmc
    import ctypes as C
    src = torch.empty(16384, 4096, dtype=torch.float32, device=dev).normal_()
    dst_c = torch.empty_like(src)
    ds_, dd_ = mi355.tensor_desc(src), mi355.tensor_desc(dst_c)
    with torch.cuda.stream(stream):
        mi355.check(lib.mi355_cpy(stream.cuda_stream, C.byref(ds_), C.byref(dd_)))
        stream.synchronize()
    del src, dst_c

    cpu = None
    if not args.no_cpu:
        try:
            cpu = cpu_baseline()
        except Exception as e:   # the baseline is a reported extra; never let it take the GPU numbers down
            cpu = {"error": repr(e)}

    weight_bytes = weights.matmul_bytes()
    result = {
        "metric": "tg%d tokens/s (Llama-3-8B-shaped Q4_K_M, batch 1, flash attention, all ops on device)" % args.steps,
        "value": round(tg, 2), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8 block dots (Q4_K/Q6_K weights x Q8_1 activations), f32 accumulate, f16 KV cache",
        "data": ("synthetic: random Q4_K/Q6_K blocks scaled like N(0,0.02) weights, random embeddings" if args.random_blocks else
                 "synthetic: weights drawn from N(0,0.02) and quantized on the device to the Q4_K_M mix with the reference quantizers' arithmetic "
                 "(%.1f s for the 8B model), random embeddings" % quantize_s),
        "config": {"workload": "configs[3]: Llama-3-8B-shaped Q4_K_M decode (32 layers, d_model 4096, ffn 14336, 32/8 heads, "
                               "head_dim 128, vocab 128256), KV positions %d..%d, n_kv padded to 256" % (args.warmup, args.warmup + args.steps - 1),
                   "launch": "host" if args.no_graph else "hip-graph replay", "weight_bytes_per_token": weight_bytes,
                   "hbm_fraction_of_step": round(weight_bytes / (ms_per_step * 1e-3) / (HBM_PEAK_GBS * 1e9), 4)},
        "pp%d_tokens_per_s" % args.pp: round(pp, 1) if pp else None,
        "outputs_finite": finite,
        "roofline": roofline,
        "roofline_pp%d" % args.pp: roofline_pp,
        "cpu_baseline": cpu,
    }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
