#!/usr/bin/env python3
"""Model files for the backend: a GGUF writer, the tensor-type mix `llama-quantize` applies per file type, and two ways to fill
the tensors - quantized on the device from f32 values (mi355_quantize_weights: the reference quantizers' bytes), which is what
`llama-quantize` does to a checkpoint, or random blocks (quick; kernel time does not depend on the values).  No downloaded
checkpoint is involved: weights are drawn from N(0, 0.02).

    python -m mi355.gguf out.gguf [--quantize] [--layers N ...]

The tensor mix is what llama-quantize produces for Q4_K_M (src/llama-quant.cpp:122-340): attn_v and ffn_down are Q6_K in
the layers chosen by use_more_bits (:129-131), output.weight is Q6_K, token_embd and everything else Q4_K, norms f32.
Blocks are random bytes with fp16 scales patched so the dequantized weights look like N(0, 0.02); kernel time does not
depend on the values.  The vocabulary is "no_vocab" (src/llama-vocab.cpp), which llama-bench accepts because it feeds
random token ids (examples/llama-bench/llama-bench.cpp:1443-1446).

File format: GGUF v3 (ggml/src/gguf.cpp, docs in ggml/include/gguf.h): header, key/value pairs, tensor infos, padding
to general.alignment (32), tensor data.
"""
import argparse
import struct

import numpy as np


def _package():
    """the mi355 package, also when this file is run as a script (python llama.cpp_amd/mi355/gguf.py ...)"""
    import importlib
    import os
    import sys
    if __package__:
        return importlib.import_module(__package__)
    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    return importlib.import_module("mi355")

F32, Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q4_K, Q5_K, Q6_K, IQ4_NL, IQ4_XS = 0, 2, 3, 6, 7, 8, 12, 13, 14, 20, 23
BLOCK = {Q4_K: (256, 144), Q5_K: (256, 176), Q6_K: (256, 210), Q4_0: (32, 18), Q4_1: (32, 20), Q5_0: (32, 22), Q5_1: (32, 24), Q8_0: (32, 34),
         IQ4_NL: (32, 18), IQ4_XS: (256, 136)}
# file type -> (default tensor type, LLAMA_FTYPE_MOSTLY_* of include/llama.h:146-174)
FTYPES = {"q4_k_m": (Q4_K, 15), "q5_k_m": (Q5_K, 17), "q4_0": (Q4_0, 2), "q4_1": (Q4_1, 3), "q5_0": (Q5_0, 8), "q5_1": (Q5_1, 9), "q8_0": (Q8_0, 7),
          "iq4_nl": (IQ4_NL, 25), "iq4_xs": (IQ4_XS, 30)}
T_U32, T_F32, T_STR, T_U64 = 4, 6, 8, 10


def use_more_bits(i_layer, n_layer):
    """src/llama-quant.cpp:129-131"""
    return i_layer < n_layer // 8 or i_layer >= 7 * n_layer // 8 or (i_layer - n_layer // 8) % 3 == 2


def _s(b):
    b = b.encode() if isinstance(b, str) else b
    return struct.pack("<Q", len(b)) + b


def _kv(key, vtype, value):
    out = _s(key) + struct.pack("<I", vtype)
    if vtype == T_U32:
        return out + struct.pack("<I", value)
    if vtype == T_F32:
        return out + struct.pack("<f", value)
    if vtype == T_U64:
        return out + struct.pack("<Q", value)
    if vtype == T_STR:
        return out + _s(value)
    raise ValueError(vtype)


def tensor_list(n_layer, n_embd, n_ff, n_head, n_head_kv, head_dim, n_vocab, n_expert=0, base=Q4_K):
    """n_expert > 0: mixture-of-experts feed-forward (src/llama-model.cpp:1553-1558) with every quantized tensor Q4_K, the mix
    of `llama-quantize --pure ... Q4_K`; the router ffn_gate_inp stays f32 (src/llama-quant.cpp:749).
    base: Q4_K for the Q4_K_M mix, Q5_K for Q5_K_M (the same rules with Q5_K as the default type, src/llama-quant.cpp:122-340).
    A per-32-block base (Q4_0, Q4_1, Q5_0, Q5_1, Q8_0) is used for every matrix, as llama-quantize does without an importance
    matrix, with output.weight Q6_K (Q8_0 stays Q8_0, :166-168); IQ4_NL and IQ4_XS take Q5_K for attn_v (grouped-query models, :232-234) and for
    ffn_down in the first eighth of the layers (:299-301)."""
    t = [("token_embd.weight", base, (n_embd, n_vocab))]
    kmix = base in (Q4_K, Q5_K)
    for il in range(n_layer):
        more = kmix and use_more_bits(il, n_layer) and n_expert == 0
        v_type = Q6_K if more else Q5_K if (base in (IQ4_NL, IQ4_XS) and n_head // n_head_kv >= 4) else base
        down_type = Q6_K if more else Q5_K if (base in (IQ4_NL, IQ4_XS) and il < n_layer // 8) else base
        p = "blk.%d." % il
        if n_expert > 0:
            t += [(p + "attn_norm.weight", F32, (n_embd,)),
                  (p + "attn_q.weight", base, (n_embd, n_head * head_dim)),
                  (p + "attn_k.weight", base, (n_embd, n_head_kv * head_dim)),
                  (p + "attn_v.weight", base, (n_embd, n_head_kv * head_dim)),
                  (p + "attn_output.weight", base, (n_head * head_dim, n_embd)),
                  (p + "ffn_norm.weight", F32, (n_embd,)),
                  (p + "ffn_gate_inp.weight", F32, (n_embd, n_expert)),
                  (p + "ffn_gate_exps.weight", base, (n_embd, n_ff, n_expert)),
                  (p + "ffn_down_exps.weight", base, (n_ff, n_embd, n_expert)),
                  (p + "ffn_up_exps.weight", base, (n_embd, n_ff, n_expert))]
            continue
        t += [(p + "attn_norm.weight", F32, (n_embd,)),
              (p + "attn_q.weight", base, (n_embd, n_head * head_dim)),
              (p + "attn_k.weight", base, (n_embd, n_head_kv * head_dim)),
              (p + "attn_v.weight", v_type, (n_embd, n_head_kv * head_dim)),
              (p + "attn_output.weight", base, (n_head * head_dim, n_embd)),
              (p + "ffn_norm.weight", F32, (n_embd,)),
              (p + "ffn_gate.weight", base, (n_embd, n_ff)),
              (p + "ffn_up.weight", base, (n_embd, n_ff)),
              (p + "ffn_down.weight", down_type, (n_ff, n_embd))]
    t += [("output_norm.weight", F32, (n_embd,)), ("output.weight", base if (n_expert > 0 or base == Q8_0) else Q6_K, (n_embd, n_vocab))]
    return t


def nbytes(ttype, shape):
    n = int(np.prod(shape))
    if ttype == F32:
        return 4 * n
    be, bb = BLOCK[ttype]
    assert shape[0] % be == 0
    return n // be * bb


def random_blocks(ttype, n_blocks, rng, pool):
    """n_blocks random blocks of ttype with sane scales; the random bytes are tiled from a pool to keep this fast"""
    bb = BLOCK[ttype][1]
    need = n_blocks * bb
    reps = (need + pool.size - 1) // pool.size
    raw = np.tile(pool, reps)[:need].copy().reshape(n_blocks, bb)
    roll = int(rng.integers(0, pool.size))
    raw = np.roll(raw.reshape(-1), roll).reshape(n_blocks, bb)

    def put_half(col, value):
        h = np.array([value], dtype=np.float16).view(np.uint8)
        raw[:, col] = h[0]
        raw[:, col + 1] = h[1]

    if ttype == Q4_K:      # w = d*sc*n - dmin*m, sc,m ~ U[0,63], n ~ U[0,15]
        put_half(0, 0.02 / (31.5 * 4.6))
        put_half(2, 0.02 / (31.5 * 4.6) * 7.5)
    elif ttype == Q5_K:    # the same with n ~ U[0,31]
        put_half(0, 0.02 / (31.5 * 9.2))
        put_half(2, 0.02 / (31.5 * 9.2) * 15.5)
    elif ttype == Q6_K:    # w = d*sc*(q-32), sc int8
        put_half(208, 0.02 / (74.0 * 18.5))
    elif ttype == IQ4_XS:  # w = d * (ls - 32) * table[n], ls ~ U[0, 63]
        put_half(0, 0.02 / (18.5 * 68.0))
    elif ttype in (Q4_0, Q8_0, Q5_0, IQ4_NL):   # w = d * level: levels of spread 4.6 / 74 / 9.2 / 68
        put_half(0, 0.02 / {Q4_0: 4.6, Q8_0: 74.0, Q5_0: 9.2, IQ4_NL: 68.0}[ttype])
    else:                  # Q4_1 / Q5_1: w = d * n + m
        spread, mid = (4.6, 7.5) if ttype == Q4_1 else (9.2, 15.5)
        put_half(0, 0.02 / spread)
        put_half(2, -0.02 / spread * mid)
    return raw


def quantized_tensor(ttype, shape, seed, device, std=0.02):
    """bytes of a tensor of `shape` (ggml order: shape[0] = row length) drawn from N(0, std) and quantized to ttype on the device
    with the reference quantizers' arithmetic (mi355_quantize_weights); rows are quantized in slices to bound memory"""
    import torch
    quantize_weights = _package().quantize_weights
    k = shape[0]
    nrows = int(np.prod(shape[1:])) if len(shape) > 1 else 1
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    out = []
    step = max(1, (1 << 28) // (4 * k))      # 256 MiB of f32 per slice
    for r0 in range(0, nrows, step):
        n = min(step, nrows - r0)
        x = torch.randn((n, k), device=device, generator=gen) * std
        out.append(quantize_weights(ttype, x).cpu().numpy().tobytes())
    return b"".join(out)


def write_model(path, n_layer=32, n_embd=4096, n_ff=14336, n_head=32, n_head_kv=8, n_vocab=128256, n_ctx=8192,
                rope_theta=500000.0, rms_eps=1e-5, seed=1234, n_expert=0, n_expert_used=0, ftype="q4_k_m", quantize_on=None):
    """ftype: a key of FTYPES - the tensor mix llama-quantize produces for that file type.
    quantize_on: a torch device - tensors are N(0, 0.02) values quantized there (types with a device quantizer; the others, and
    every tensor when None, are random blocks)"""
    head_dim = n_embd // n_head
    base = FTYPES[ftype][0]
    tensors = tensor_list(n_layer, n_embd, n_ff, n_head, n_head_kv, head_dim, n_vocab, n_expert, base)
    align = 32
    kvs = [
        _kv("general.architecture", T_STR, "llama"),
        _kv("general.name", T_STR, "synthetic-llama-" + ftype),
        _kv("general.file_type", T_U32, FTYPES[ftype][1]),
        _kv("general.alignment", T_U32, align),
        _kv("llama.block_count", T_U32, n_layer),
        _kv("llama.context_length", T_U32, n_ctx),
        _kv("llama.embedding_length", T_U32, n_embd),
        _kv("llama.feed_forward_length", T_U32, n_ff),
        _kv("llama.attention.head_count", T_U32, n_head),
        _kv("llama.attention.head_count_kv", T_U32, n_head_kv),
        _kv("llama.rope.dimension_count", T_U32, head_dim),
        _kv("llama.rope.freq_base", T_F32, rope_theta),
        _kv("llama.attention.layer_norm_rms_epsilon", T_F32, rms_eps),
        _kv("llama.vocab_size", T_U32, n_vocab),
        _kv("tokenizer.ggml.model", T_STR, "no_vocab"),
    ]
    if n_expert > 0:
        kvs += [_kv("llama.expert_count", T_U32, n_expert), _kv("llama.expert_used_count", T_U32, n_expert_used)]
    infos, off = [], 0
    for name, ttype, shape in tensors:
        infos.append(_s(name) + struct.pack("<I", len(shape)) + b"".join(struct.pack("<Q", d) for d in shape) +
                     struct.pack("<IQ", ttype, off))
        off += (nbytes(ttype, shape) + align - 1) // align * align
    header = struct.pack("<IIQQ", 0x46554747, 3, len(tensors), len(kvs)) + b"".join(kvs) + b"".join(infos)
    rng = np.random.default_rng(seed)
    pool = rng.integers(0, 256, 1 << 24, dtype=np.uint8)
    with open(path, "wb") as f:
        f.write(header)
        f.write(b"\0" * ((-len(header)) % align))
        for name, ttype, shape in tensors:
            if ttype == F32:
                if len(shape) == 1:   # norm weights
                    data = (1.0 + 0.01 * rng.standard_normal(int(np.prod(shape)))).astype(np.float32).tobytes()
                else:                 # router
                    data = (0.02 * rng.standard_normal(int(np.prod(shape)))).astype(np.float32).tobytes()
                f.write(data)
                f.write(b"\0" * ((-len(data)) % align))
                continue
            if quantize_on is not None:
                load = _package().load
                if load().mi355_quantize_weights_supported(ttype):
                    f.write(quantized_tensor(ttype, shape, seed + 7919 * (1 + len(name)) + sum(map(ord, name)), quantize_on))
                    f.write(b"\0" * ((-nbytes(ttype, shape)) % align))
                    continue
            total = int(np.prod(shape)) // BLOCK[ttype][0]
            done = 0
            while done < total:   # in slices, to bound memory
                n = min(total - done, 1 << 18)
                f.write(random_blocks(ttype, n, rng, pool).tobytes())
                done += n
            f.write(b"\0" * ((-nbytes(ttype, shape)) % align))
    return off


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("path")
    ap.add_argument("--layers", type=int, default=32)
    ap.add_argument("--embd", type=int, default=4096)
    ap.add_argument("--ff", type=int, default=14336)
    ap.add_argument("--heads", type=int, default=32)
    ap.add_argument("--kv-heads", type=int, default=8)
    ap.add_argument("--vocab", type=int, default=128256)
    ap.add_argument("--experts", type=int, default=0, help="mixture of experts: number of experts (0 = dense)")
    ap.add_argument("--experts-used", type=int, default=2)
    ap.add_argument("--ftype", default="q4_k_m", choices=sorted(FTYPES))
    ap.add_argument("--quantize", action="store_true", help="draw f32 weights from N(0, 0.02) and quantize them on the GPU (needs one)")
    a = ap.parse_args()
    dev = None
    if a.quantize:
        import torch
        dev = torch.device("cuda:0")
    size = write_model(a.path, a.layers, a.embd, a.ff, a.heads, a.kv_heads, a.vocab, n_expert=a.experts,
                       n_expert_used=a.experts_used if a.experts else 0, ftype=a.ftype, quantize_on=dev)
    print("wrote %s: %.2f GB of tensor data" % (a.path, size / 1e9))
