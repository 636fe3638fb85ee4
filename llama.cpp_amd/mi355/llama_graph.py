"""The llama decoder layer stack as llama.cpp's build_llama emits it (src/llama.cpp:1476-1640,
llm_build_kv :157-199/:540-662, llm_build_ffn :200-330), driven straight through the kernel
C ABI.  Measurement and parity harness: it issues, node for node, the kernel sequence the ggml
backend plug-in issues for the same graph, without needing a GGUF file or the llama.cpp host.

Weights are synthetic: random quantized blocks whose scales make the dequantized values look
like N(0, 0.02) (generated on the device; kernel time does not depend on the values).
The Q4_K_M tensor mix follows src/llama-quant.cpp:122-340: attn_v and ffn_down are Q6_K in the
layers selected by use_more_bits(), the output projection is Q6_K, everything else Q4_K.
"""
import ctypes as C
import math

import torch

from . import (F16, F32, I32, Q4_K, Q5_K, Q6_K, Q4_0, Q8_0, Q4_1, Q5_0, Q5_1, IQ4_NL, IQ4_XS, BLOCK, GemvMat, Tensor, TiledMat, check, load, row_bytes, tensor_desc,
               upload_weights, _ptr, _stream)


def use_more_bits(i_layer, n_layer):
    """src/llama-quant.cpp:129-131"""
    return i_layer < n_layer // 8 or i_layer >= 7 * n_layer // 8 or (i_layer - n_layer // 8) % 3 == 2


class LlamaConfig:
    def __init__(self, n_layer=32, n_embd=4096, n_ff=14336, n_head=32, n_head_kv=8, head_dim=128, n_vocab=128256,
                 rope_theta=500000.0, rms_eps=1e-5, n_ctx=4096):
        self.n_layer, self.n_embd, self.n_ff, self.n_head, self.n_head_kv = n_layer, n_embd, n_ff, n_head, n_head_kv
        self.head_dim, self.n_vocab, self.rope_theta, self.rms_eps, self.n_ctx = head_dim, n_vocab, rope_theta, rms_eps, n_ctx


def random_quantized(t, nrows, k, device, gen):
    """Random blocks of type t in the reference block layout ([nrows, row_bytes] uint8), values ~ N(0, 0.02)-like."""
    be, bb = BLOCK[t]
    nb = k // be
    raw = torch.randint(0, 256, (nrows, nb, bb), dtype=torch.uint8, device=device, generator=gen)

    def put_half(col, value):
        h = torch.tensor([value], dtype=torch.float16).view(torch.uint8)
        raw[:, :, col] = h[0].item()
        raw[:, :, col + 1] = h[1].item()

    if t == Q4_K:      # w = d*sc*n - dmin*m, sc,m ~ U[0,63], n ~ U[0,15]
        put_half(0, 0.02 / (31.5 * 4.6))
        put_half(2, 0.02 / (31.5 * 4.6) * 7.5)
    elif t == Q5_K:    # w = d*sc*n - dmin*m, n ~ U[0,31]
        put_half(0, 0.02 / (31.5 * 9.2))
        put_half(2, 0.02 / (31.5 * 9.2) * 15.5)
    elif t == Q6_K:    # w = d*sc*(q-32), sc int8
        put_half(208, 0.02 / (74.0 * 18.5))
    elif t == Q4_0:    # w = d*(n-8)
        put_half(0, 0.02 / 4.6)
    elif t == Q8_0:
        put_half(0, 0.02 / 74.0)
    elif t == Q5_0:    # w = d*(n-16)
        put_half(0, 0.02 / 9.2)
    elif t == IQ4_NL:  # w = d*table[n]
        put_half(0, 0.02 / 68.0)
    elif t == IQ4_XS:  # w = d*(ls-32)*table[n], ls ~ U[0, 63]
        put_half(0, 0.02 / (18.5 * 68.0))
    elif t in (Q4_1, Q5_1):   # w = d*n + m
        spread, mid = (4.6, 7.5) if t == Q4_1 else (9.2, 15.5)
        put_half(0, 0.02 / spread)
        put_half(2, -0.02 / spread * mid)
    return raw.reshape(nrows, nb * bb)


class LlamaWeights:
    """device-layout weights of a Q4_K_M (or single-type) llama"""

    def __init__(self, cfg, device, seed=1234, ftype="q4_k_m", quantize=False):
        """quantize: draw every matrix from N(0, 0.02) in f32 and quantize it on the device with the reference quantizers'
        arithmetic (mi355_quantize_weights) instead of drawing random blocks"""
        gen = torch.Generator(device=device)
        gen.manual_seed(seed)
        self.cfg = cfg
        E, F, H, HK, D = cfg.n_embd, cfg.n_ff, cfg.n_head, cfg.n_head_kv, cfg.head_dim
        base = {"q4_k_m": Q4_K, "q4_0": Q4_0, "q8_0": Q8_0, "q4_k": Q4_K, "q6_k": Q6_K}[ftype]
        self.quantized = bool(quantize)

        def mk(t, n, k):
            if quantize:
                from . import quantize_weights
                step = max(1, (1 << 28) // (4 * k))      # 256 MiB of f32 at a time
                parts = [quantize_weights(t, torch.randn((min(step, n - r0), k), device=device, generator=gen) * 0.02) for r0 in range(0, n, step)]
                return t, upload_weights(t, torch.cat(parts) if len(parts) > 1 else parts[0])
            return t, upload_weights(t, random_quantized(t, n, k, device, gen))

        self.layers = []
        for il in range(cfg.n_layer):
            more = ftype == "q4_k_m" and use_more_bits(il, cfg.n_layer)
            L = {
                "attn_norm": torch.ones(E, device=device) + 0.01 * torch.randn(E, device=device, generator=gen),
                "ffn_norm": torch.ones(E, device=device) + 0.01 * torch.randn(E, device=device, generator=gen),
                "wq": mk(base, H * D, E), "wk": mk(base, HK * D, E),
                "wv": mk(Q6_K if more else base, HK * D, E), "wo": mk(base, E, H * D),
                "gate": mk(base, F, E), "up": mk(base, F, E), "down": mk(Q6_K if more else base, E, F),
            }
            self.layers.append(L)
        self.output_norm = torch.ones(E, device=device)
        self.output = mk(Q6_K if ftype == "q4_k_m" else base, cfg.n_vocab, E)

    def matmul_bytes(self):
        """algorithmic weight bytes streamed per decoded token"""
        n = 0
        for L in self.layers:
            for k in ("wq", "wk", "wv", "wo", "gate", "up", "down"):
                n += L[k][1].numel()
        return n + self.output[1].numel()


class LlamaRunner:
    """One sequence, f16 KV cache of n_ctx cells laid out [cell][kv head][head_dim] as llama-kv-cache.cpp:80-112."""

    def __init__(self, weights, max_tokens=512):
        self.w = weights
        cfg = self.cfg = weights.cfg
        dev = self.dev = weights.output[1].device
        self.lib = load()
        self.fuse_qkv = True    # rows must be 16-byte aligned; set False to use the three-launch sequence
        self.use_planes = True  # prefill: Q6_K matrices go through their unpacked int8 planes (2 bytes per weight more, kept resident)
        self.planes = {}
        # prefill from 192 tokens on: K-quant matrices go through the wide-tile GEMM, which reads tile images of the weights' two
        # int8 planes (a second copy, 2 bytes per weight, built on first use and kept) and of the quantized activations; below
        # that the 2 bytes per weight make the product HBM-bound and the kernel that unpacks the 4.5-bit rows wins
        self.use_tiles = True
        self.tiles = {}
        self.fuse_qkv_rope = True   # prefill: ROPE and the KV-cache stores in the epilogue of the Q/K/V launch of the wide-tile GEMM
        self.rope_table = None
        self.fuse_sum_norm = True   # prefill: a cut product's sum launch also normalises and quantizes its rows for the next products
        self.split_ws = None    # partial sums of tile products that are split along K (grown on first use, before any graph capture)
        # decode, T <= 4: SiLU*up + Q8_1 inside the gate/up launch (True: with both matrices of one type a group owns a whole 32-row
        # block of both and quantizes it itself; otherwise the last group of each block finishes it) or as a launch of their own
        # after a two-matrix product (False).  8B shape: 1.917 -> 1.832 ms per token with the block-owning launch; same bits.
        self.fuse_tail = True
        # decode, one token: the attention norm + Q8_1 inside the Q/K/V launch (every group normalises the row for itself:
        # one launch less per layer, 1.935 -> 1.889 ms per token on the 8B shape; same bits)
        self.fuse_qkv_norm = True
        E, F, H, HK, D = cfg.n_embd, cfg.n_ff, cfg.n_head, cfg.n_head_kv, cfg.head_dim
        T = self.max_tokens = max_tokens
        f32 = dict(dtype=torch.float32, device=dev)
        self.x = torch.zeros(T, E, **f32)          # residual stream / layer input
        self.t0 = torch.zeros(T, E, **f32)
        self.t1 = torch.zeros(T, E, **f32)
        self.q = torch.zeros(T, H * D, **f32)
        self.k = torch.zeros(T, HK * D, **f32)
        self.v = torch.zeros(T, HK * D, **f32)
        self.attn = torch.zeros(T, H * D, **f32)
        self.gate = torch.zeros(T, F, **f32)
        self.up = torch.zeros(T, F, **f32)
        self.logits = torch.zeros(T, cfg.n_vocab, **f32)
        self.kcache = [torch.zeros(cfg.n_ctx, HK, D, dtype=torch.float16, device=dev) for _ in range(cfg.n_layer)]
        self.vcache = [torch.zeros(cfg.n_ctx, HK, D, dtype=torch.float16, device=dev) for _ in range(cfg.n_layer)]
        self.pos = torch.zeros(T, dtype=torch.int32, device=dev)
        self.mask = torch.zeros((T + 63) // 64 * 64, cfg.n_ctx, dtype=torch.float16, device=dev)
        kmax = max(E, F, H * D)
        self.act_a = torch.empty(max(int(self.lib.mi355_act_bytes(max(E, H * D), T)), int(self.lib.mi355_act_q8k_tiled_bytes(max(E, H * D), T))) + 256,
                                 dtype=torch.uint8, device=dev)
        self.act_b = torch.empty(max(int(self.lib.mi355_act_bytes(F, T)), int(self.lib.mi355_act_q8k_tiled_bytes(F, T))) + 256, dtype=torch.uint8, device=dev)
        self.act_c = torch.empty(int(self.lib.mi355_act_bytes(max(E, H * D), 4)) + 256, dtype=torch.uint8, device=dev)
        self.tickets = torch.zeros(F // 32 + 64, dtype=torch.int32, device=dev)   # arrival counters of the tail-fused launches
        self.ws = torch.empty(int(self.lib.mi355_mul_mat_ws_bytes(kmax, T)) + 256, dtype=torch.uint8, device=dev)
        self.fa_ws = torch.empty(min(int(self.lib.mi355_flash_attn_ws_bytes(D, T, cfg.n_ctx, H)), 256 << 20), dtype=torch.uint8, device=dev)

    # ---- single operators over the C ABI -------------------------------------------------------
    def _mm(self, w, x, out, T):
        t, W = w
        N, K = out.shape[1], x.shape[1]
        check(self.lib.mi355_mul_mat(_stream(), t, _ptr(W), _ptr(x), _ptr(out), N, K, T, x.stride(0), out.stride(0), _ptr(self.ws), self.ws.numel()))

    def _norm(self, x, w, out, T):
        dx, do, dw = tensor_desc(x[:T]), tensor_desc(out[:T]), tensor_desc(w)
        check(self.lib.mi355_rms_norm(_stream(), C.byref(dx), C.byref(do), self.cfg.rms_eps))
        check(self.lib.mi355_bin_bcast(_stream(), 2, C.byref(do), C.byref(dw), C.byref(do)))

    def _bin(self, op, a, b, out):
        da, db, do = tensor_desc(a), tensor_desc(b), tensor_desc(out)
        check(self.lib.mi355_bin_bcast(_stream(), op, C.byref(da), C.byref(db), C.byref(do)))

    def _rope(self, x, heads, T):
        cfg = self.cfg
        v = x[:T].view(T, heads, cfg.head_dim)
        d = tensor_desc(v)
        check(self.lib.mi355_rope(_stream(), C.byref(d), _ptr(self.pos), None, C.byref(d), cfg.head_dim, 0, cfg.n_ctx, cfg.rope_theta,
                                  1.0, 0.0, 1.0, 32.0, 1.0))

    def _kv_store(self, src, cache, T):
        cfg = self.cfg
        s = tensor_desc(src[:T].view(T, cfg.n_head_kv * cfg.head_dim))
        d = tensor_desc(cache.view(cfg.n_ctx, cfg.n_head_kv * cfg.head_dim))
        check(self.lib.mi355_set_rows(_stream(), C.byref(s), _ptr(self.pos), C.byref(d)))

    def _attn(self, il, T, n_kv, act=None):
        """act: optional workspace that receives the Q8_1 quantization of the attention output"""
        cfg = self.cfg
        H, HK, D = cfg.n_head, cfg.n_head_kv, cfg.head_dim
        q = self.q[:T].view(T, H, D)
        kc, vc = self.kcache[il], self.vcache[il]
        check(self.lib.mi355_flash_attn_ext_quant(_stream(), _ptr(q), _ptr(kc), _ptr(vc), _ptr(self.mask), _ptr(self.attn), D, T, n_kv, H, HK,
                                                  q.stride(0) * 4, q.stride(1) * 4, kc.stride(0) * 2, kc.stride(1) * 2, vc.stride(0) * 2,
                                                  vc.stride(1) * 2, self.mask.stride(0) * 2, 1.0 / math.sqrt(D), 0.0, 0.0, _ptr(self.fa_ws),
                                                  self.fa_ws.numel(), _ptr(act) if act is not None else None))

    # ---- fused operators ------------------------------------------------------------------------
    @staticmethod
    def _q8k_ok(mats, K):
        """the super-block tile GEMM serves K-quants whose device rows are 16-byte aligned"""
        return all(t == Q4_K or (t == Q6_K and K % 2048 == 0) for (t, _), _ in mats)

    def _planes(self, t, W, N, K):
        """the two int8 planes of a K-quant matrix (value = 64 * hi + lo for Q6_K), built on first use and kept"""
        key = W.data_ptr()
        if key not in self.planes:
            buf = torch.empty(int(self.lib.mi355_kq_planes_bytes(N, K)) + 256, dtype=torch.uint8, device=self.dev)
            check(self.lib.mi355_kq_unpack_planes(_stream(), t, _ptr(W), _ptr(buf), N, K))
            self.planes[key] = buf
        return self.planes[key]

    def _tiles(self, t, W, N, K):
        """tile images of a K-quant matrix's two int8 planes + per-super-block scales, built on first use and kept"""
        key = W.data_ptr()
        if key not in self.tiles:
            buf = torch.empty(int(self.lib.mi355_kq_tiles_bytes(t, N, K)) + 256, dtype=torch.uint8, device=self.dev)
            check(self.lib.mi355_kq_unpack_tiles(_stream(), t, _ptr(W), _ptr(buf), N, K))
            self.tiles[key] = buf
        return self.tiles[key]

    def _fmt(self, mats, K, T):
        """activation format of a product: 0 Q8_1 blocks, 1 one scale per 256 elements (K-quant tile GEMM), 2 the same as tile images,
        3 tile images for the 33..128-row kernel on packed Q4_K rows"""
        if T <= 8 or not self._q8k_ok(mats, K):
            return 0
        if 32 < T <= 128 and all(t == Q4_K for (t, _), _ in mats):
            return 3     # the weight-streaming kernel for 33..128 rows: activations as tile images, weights packed
        return 2 if (self.use_tiles and T >= 192) else 1

    def _quant(self, src, act, K, T, q8k):
        fn = (self.lib.mi355_quantize_act, self.lib.mi355_quantize_act_q8k, self.lib.mi355_quantize_act_q8k_tiled, self.lib.mi355_quantize_act_q8k_tiled)[int(q8k)]
        check(fn(_stream(), _ptr(src), _ptr(act), K, T, src.stride(0)))

    def _norm_quant(self, x, w, act, T, q8k=0):
        K = x.shape[1]
        fn = (self.lib.mi355_rms_norm_mul_quant, self.lib.mi355_rms_norm_mul_quant_q8k, self.lib.mi355_rms_norm_mul_quant_q8k_tiled,
              self.lib.mi355_rms_norm_mul_quant_q8k_tiled)[int(q8k)]
        check(fn(_stream(), _ptr(x), x.stride(0), _ptr(w), None, 0, _ptr(act), K, T, self.cfg.rms_eps))

    def _mm_act(self, mats, act, K, T, residual=None, q8k=False, norm=None):
        """mats: list of ((type, W), out); all consume the quantized activation `act` (T rows of K).
        norm: (norm weight, activation buffer) - the single product's rows are normalised next and their tile image goes to the
        buffer (wide-tile GEMM only: the launch that adds a cut product's slices carries the norm)"""
        assert norm is None or (q8k in (2, 3) and len(mats) == 1 and T > 8)
        if T <= 8:
            arr = (GemvMat * len(mats))()
            for i, ((t, W), out) in enumerate(mats):
                arr[i].type, arr[i].W, arr[i].N, arr[i].dst, arr[i].dst_stride = t, W.data_ptr(), out.shape[1], out.data_ptr(), out.stride(0)
                arr[i].residual = residual.data_ptr() if residual is not None else None
            check(self.lib.mi355_mul_mat_vec_q_multi(_stream(), len(mats), arr, _ptr(act), K, T))
        else:
            if q8k == 2 and 1 < len(mats) <= 3:   # one launch of the wide-tile GEMM, whatever the K-quant type of each matrix
                arr = (TiledMat * len(mats))()
                for i, ((t, W), out) in enumerate(mats):
                    arr[i].tiles, arr[i].dst, arr[i].N, arr[i].dst_stride = self._tiles(t, W, out.shape[1], K).data_ptr(), out.data_ptr(), out.shape[1], out.stride(0)
                    arr[i].residual = residual.data_ptr() if residual is not None else None
                types = (C.c_int * len(mats))(*[t for (t, _), _ in mats])
                check(self.lib.mi355_mul_mat_q8k_tiled_mixed(_stream(), len(mats), types, arr, _ptr(act), K, T))
                mats = []
            if q8k == 3 and 1 < len(mats) <= 3:   # 33..128 rows on Q4_K: the matrices that share the activation in one launch
                arr = (GemvMat * len(mats))()
                for i, ((t, W), out) in enumerate(mats):
                    arr[i].type, arr[i].W, arr[i].N, arr[i].dst, arr[i].dst_stride = t, W.data_ptr(), out.shape[1], out.data_ptr(), out.stride(0)
                    arr[i].residual = residual.data_ptr() if residual is not None else None
                ns = (C.c_int64 * len(mats))(*[out.shape[1] for _, out in mats])
                need = int(self.lib.mi355_mul_mat_mid_multi_ws_bytes(len(mats), ns, K, T))
                if self.split_ws is None or self.split_ws.numel() < need:
                    self.split_ws = torch.empty(need + 256, dtype=torch.uint8, device=self.dev)
                check(self.lib.mi355_mul_mat_mid_multi(_stream(), Q4_K, len(mats), arr, _ptr(act), K, T, _ptr(self.split_ws) if need else None, need))
                mats = []
            for (t, W), out in mats:
                if q8k == 3:
                    N = out.shape[1]
                    need = int(self.lib.mi355_mul_mat_mid_ws_bytes(N, K, T))
                    if self.split_ws is None or self.split_ws.numel() < need:
                        self.split_ws = torch.empty(need + 256, dtype=torch.uint8, device=self.dev)
                    if norm is not None:
                        check(self.lib.mi355_mul_mat_mid_norm(_stream(), t, _ptr(W), _ptr(act), _ptr(out), _ptr(residual) if residual is not None else None, N, K, T,
                                                              out.stride(0), _ptr(self.split_ws) if need else None, need, _ptr(norm[0]), self.cfg.rms_eps, None, 0,
                                                              _ptr(norm[1])))
                    else:
                        check(self.lib.mi355_mul_mat_mid(_stream(), t, _ptr(W), _ptr(act), _ptr(out), _ptr(residual) if residual is not None else None, N, K, T,
                                                         out.stride(0), _ptr(self.split_ws) if need else None, need))
                    continue
                if q8k:     # the residual add is the tile kernel's epilogue; products with few tiles are split along K through split_ws
                    N = out.shape[1]
                    need = int(self.lib.mi355_mul_mat_q8k_tiled_ws_bytes(N, K, T) if q8k == 2 else self.lib.mi355_mul_mat_q8k_ws_bytes(N, K, T))
                    if self.split_ws is None or self.split_ws.numel() < need:
                        self.split_ws = torch.empty(need + 256, dtype=torch.uint8, device=self.dev)
                    sw, sn = (_ptr(self.split_ws), self.split_ws.numel()) if need else (None, 0)
                    res = _ptr(residual) if residual is not None else None
                    if q8k == 2 and norm is not None:
                        check(self.lib.mi355_mul_mat_q8k_tiled_norm(_stream(), t, _ptr(self._tiles(t, W, N, K)), _ptr(act), _ptr(out), res, N, K, T,
                                                                    out.stride(0), sw, sn, _ptr(norm[0]), self.cfg.rms_eps, None, 0, _ptr(norm[1])))
                    elif q8k == 2:
                        check(self.lib.mi355_mul_mat_q8k_tiled(_stream(), t, _ptr(self._tiles(t, W, N, K)), _ptr(act), _ptr(out), res, N, K, T,
                                                               out.stride(0), sw, sn))
                    elif t == Q6_K and self.use_planes:   # Q6_K streams its int8 planes, unpacked once per matrix
                        check(self.lib.mi355_mul_mat_q8k_planes_ws(_stream(), t, _ptr(self._planes(t, W, N, K)), _ptr(act), _ptr(out), res, N, K, T,
                                                                   out.stride(0), sw, sn))
                    else:
                        check(self.lib.mi355_mul_mat_q8k_ws(_stream(), t, _ptr(W), _ptr(act), _ptr(out), res, N, K, T, out.stride(0), sw, sn))
                    continue
                dst = out if residual is None else self.t1[:T]
                check(self.lib.mi355_mul_mat_q(_stream(), t, _ptr(W), _ptr(act), _ptr(dst), out.shape[1], K, T, dst.stride(0)))
                if residual is not None:
                    self._bin(0, dst, residual, out)

    def forward(self, T, n_kv, last_only=True):
        """fused launch sequence: 10 launches per layer instead of 25, same arithmetic per node"""
        cfg, w, lib = self.cfg, self.w, self.lib
        E, F, H, HK, D = cfg.n_embd, cfg.n_ff, cfg.n_head, cfg.n_head_kv, cfg.head_dim
        x = self.x[:T]
        if T <= 4 and self.fuse_qkv and (T == 1 or not last_only):
            return self._forward_decode(T, n_kv)
        normed = False   # the previous layer's ffn_down product has left this layer's normalised input in act_a
        for il, L in enumerate(w.layers):
            qkv = [(L["wq"], self.q[:T]), (L["wk"], self.k[:T]), (L["wv"], self.v[:T])]
            kq = self._fmt(qkv, E, T)
            if not normed:
                self._norm_quant(x, L["attn_norm"], self.act_a, T, kq)
            kc, vc = self.kcache[il], self.vcache[il]
            if T <= 4 and self.fuse_qkv:    # decode: projections, rope and KV store in one launch
                (tq, Wq), (tk, Wk), (tv, Wv) = L["wq"], L["wk"], L["wv"]
                check(lib.mi355_qkv_rope_store(_stream(), tq, _ptr(Wq), tk, _ptr(Wk), tv, _ptr(Wv), _ptr(self.act_a), _ptr(self.q), _ptr(kc), _ptr(vc),
                                               _ptr(self.pos), _ptr(self.pos), None, E, T, H, HK, D, kc.stride(0) * 2, kc.stride(1) * 2,
                                               vc.stride(0) * 2, vc.stride(1) * 2, D, 0, cfg.n_ctx, cfg.rope_theta, 1.0, 0.0, 1.0, 32.0, 1.0))
            elif kq == 2 and self.fuse_qkv_rope:
                # wide-tile GEMM: the rotations and the cache stores ride in the epilogue of the Q/K/V launch; {cos, sin} per
                # (token, pair) are the same for every layer and are written once per batch
                if il == 0:
                    if self.rope_table is None or self.rope_table.numel() < T * D:
                        self.rope_table = torch.empty(T * D, dtype=torch.float32, device=self.dev)
                    check(lib.mi355_rope_table(_stream(), _ptr(self.pos), None, _ptr(self.rope_table), T, D, D, cfg.n_ctx, cfg.rope_theta, 1.0, 0.0, 1.0, 32.0, 1.0))
                arr = (TiledMat * 3)()
                for i, ((t, W), dst, N) in enumerate(((L["wq"], self.q, H * D), (L["wk"], kc, HK * D), (L["wv"], vc, HK * D))):
                    arr[i].tiles, arr[i].dst, arr[i].residual, arr[i].N, arr[i].dst_stride = self._tiles(t, W, N, E).data_ptr(), dst.data_ptr(), None, N, N
                types = (C.c_int * 3)(L["wq"][0], L["wk"][0], L["wv"][0])
                check(lib.mi355_mul_mat_q8k_tiled_qkv_rope(_stream(), types, arr, _ptr(self.act_a), E, T, _ptr(self.rope_table), _ptr(self.pos), D, D,
                                                           kc.stride(0) * 2, kc.stride(1) * 2, vc.stride(0) * 2, vc.stride(1) * 2))
            else:
                self._mm_act(qkv, self.act_a, E, T, q8k=kq)
                check(lib.mi355_rope_kv_store(_stream(), _ptr(self.q), _ptr(self.k), _ptr(self.v), _ptr(kc), _ptr(vc), _ptr(self.pos), _ptr(self.pos),
                                              None, T, H, HK, D, kc.stride(0) * 2, kc.stride(1) * 2, vc.stride(0) * 2, vc.stride(1) * 2, D, 0,
                                              cfg.n_ctx, cfg.rope_theta, 1.0, 0.0, 1.0, 32.0, 1.0))
            wo = [(L["wo"], x)]
            kq = self._fmt(wo, H * D, T)
            if kq:
                self._attn(il, T, n_kv)
                self._quant(self.attn, self.act_a, H * D, T, kq)
            else:
                self._attn(il, T, n_kv, act=self.act_a)   # attention writes its own Q8_1 output
            gu = [(L["gate"], self.gate[:T]), (L["up"], self.up[:T])]
            kq_gu = self._fmt(gu, E, T)
            # wide-tile products on both sides of a norm: the product's sum launch also normalises and quantizes the rows it forms
            fuse = self.fuse_sum_norm and kq in (2, 3) and kq_gu in (2, 3) and E % 256 == 0
            self._mm_act(wo, self.act_a, H * D, T, residual=x, q8k=kq, norm=(L["ffn_norm"], self.act_a) if fuse else None)
            if not fuse:
                self._norm_quant(x, L["ffn_norm"], self.act_a, T, kq_gu)
            self._mm_act(gu, self.act_a, E, T, q8k=kq_gu)
            down = [(L["down"], x)]
            kq = self._fmt(down, F, T)
            fn = (lib.mi355_swiglu_quant, lib.mi355_swiglu_quant_q8k, lib.mi355_swiglu_quant_q8k_tiled, lib.mi355_swiglu_quant_q8k_tiled)[kq]
            check(fn(_stream(), _ptr(self.gate), _ptr(self.up), F, None, 0, _ptr(self.act_b), F, T))
            nxt = w.layers[il + 1] if il + 1 < len(w.layers) else None
            normed = self.fuse_sum_norm and nxt is not None and kq in (2, 3) and E % 256 == 0 and self._fmt([(nxt["wq"], self.q[:T]), (nxt["wk"], self.k[:T]), (nxt["wv"], self.v[:T])], E, T) in (2, 3)
            self._mm_act(down, self.act_b, F, T, residual=x, q8k=kq, norm=(nxt["attn_norm"], self.act_a) if normed else None)
        To = 1 if last_only else T
        xo = self.x[T - 1:T] if last_only else x
        out = [(w.output, self.logits[:To])]
        kq = self._fmt(out, E, To)
        self._norm_quant(xo, w.output_norm, self.act_a, To, kq)
        self._mm_act(out, self.act_a, E, To, q8k=kq)
        return self.logits[:To]

    def _forward_decode(self, T, n_kv):
        """decode sequence, 8 launches per layer (7 for one token with fuse_qkv_norm): [QKV + rope + KV store] [attention + Q8_1] [wo + residual] [norm + Q8_1]
        [gate/up] [SiLU*up + Q8_1] [down + residual] [next norm + Q8_1] (7 with fuse_tail); same arithmetic per node as forward_nodes"""
        cfg, w, lib = self.cfg, self.w, self.lib
        E, F, H, HK, D = cfg.n_embd, cfg.n_ff, cfg.n_head, cfg.n_head_kv, cfg.head_dim
        x = self.x[:T]
        # one token: the attention norm is computed inside the Q/K/V launch (7 launches per layer)
        qkv_norm = self.fuse_qkv_norm and T == 1 and E <= 4096 and E % 1024 == 0
        if not qkv_norm:
            self._norm_quant(x, w.layers[0]["attn_norm"], self.act_a, T)
        for il, L in enumerate(w.layers):
            kc, vc = self.kcache[il], self.vcache[il]
            (tq, Wq), (tk, Wk), (tv, Wv) = L["wq"], L["wk"], L["wv"]
            if qkv_norm:
                check(lib.mi355_rms_norm_qkv_rope_store(_stream(), _ptr(x), _ptr(L["attn_norm"]), cfg.rms_eps, tq, _ptr(Wq), tk, _ptr(Wk), tv, _ptr(Wv),
                                                        _ptr(self.q), _ptr(kc), _ptr(vc), _ptr(self.pos), _ptr(self.pos), None, E, H, HK, D,
                                                        kc.stride(0) * 2, kc.stride(1) * 2, vc.stride(0) * 2, vc.stride(1) * 2, D, 0, cfg.n_ctx,
                                                        cfg.rope_theta, 1.0, 0.0, 1.0, 32.0, 1.0))
            else:
                check(lib.mi355_qkv_rope_store(_stream(), tq, _ptr(Wq), tk, _ptr(Wk), tv, _ptr(Wv), _ptr(self.act_a), _ptr(self.q), _ptr(kc), _ptr(vc),
                                               _ptr(self.pos), _ptr(self.pos), None, E, T, H, HK, D, kc.stride(0) * 2, kc.stride(1) * 2,
                                               vc.stride(0) * 2, vc.stride(1) * 2, D, 0, cfg.n_ctx, cfg.rope_theta, 1.0, 0.0, 1.0, 32.0, 1.0))
            self._attn(il, T, n_kv, act=self.act_a)
            self._mm_act([(L["wo"], x)], self.act_a, H * D, T, residual=x)
            (tg, Wg), (tu, Wu) = L["gate"], L["up"]
            self._norm_quant(x, L["ffn_norm"], self.act_c, T)
            nxt = w.layers[il + 1]["attn_norm"] if il + 1 < len(w.layers) else w.output_norm
            if self.fuse_tail:
                check(lib.mi355_ffn_gate_up_swiglu(_stream(), tg, _ptr(Wg), tu, _ptr(Wu), _ptr(self.act_c), _ptr(self.gate), _ptr(self.up), F,
                                                   _ptr(self.act_b), _ptr(self.tickets), F, E, T))
            else:
                self._mm_act([(L["gate"], self.gate[:T]), (L["up"], self.up[:T])], self.act_c, E, T)
                check(lib.mi355_swiglu_quant(_stream(), _ptr(self.gate), _ptr(self.up), F, None, 0, _ptr(self.act_b), F, T))
            self._mm_act([(L["down"], x)], self.act_b, F, T, residual=x)
            if not qkv_norm or il + 1 == len(w.layers):
                self._norm_quant(x, nxt, self.act_a, T)
        self._mm_act([(w.output, self.logits[:T])], self.act_a, E, T)
        return self.logits[:T]

    # ---- the same pass node for node, as the ggml graph lists it (reference for the fused path) --
    def forward_nodes(self, T, n_kv, last_only=True):
        cfg, w = self.cfg, self.w
        x = self.x
        for il, L in enumerate(w.layers):
            self._norm(x, L["attn_norm"], self.t0, T)
            self._mm(L["wq"], self.t0[:T], self.q[:T], T)
            self._mm(L["wk"], self.t0[:T], self.k[:T], T)
            self._mm(L["wv"], self.t0[:T], self.v[:T], T)
            self._rope(self.q, cfg.n_head, T)
            self._rope(self.k, cfg.n_head_kv, T)
            self._kv_store(self.k, self.kcache[il], T)
            self._kv_store(self.v, self.vcache[il], T)
            self._attn(il, T, n_kv)
            self._mm(L["wo"], self.attn[:T], self.t1[:T], T)
            self._bin(0, self.t1[:T], x[:T], x[:T])                      # ffn_inp = attn_out + inpSA
            self._norm(x, L["ffn_norm"], self.t0, T)
            self._mm(L["gate"], self.t0[:T], self.gate[:T], T)
            self._mm(L["up"], self.t0[:T], self.up[:T], T)
            dg = tensor_desc(self.gate[:T])
            check(self.lib.mi355_unary(_stream(), 10, C.byref(dg), C.byref(dg)))     # SILU
            self._bin(2, self.gate[:T], self.up[:T], self.gate[:T])
            self._mm(L["down"], self.gate[:T], self.t1[:T], T)
            self._bin(0, self.t1[:T], x[:T], x[:T])
        To = 1 if last_only else T
        xo = x[T - 1:T] if last_only else x[:T]
        self._norm(xo, w.output_norm, self.t0, To)
        self._mm(w.output, self.t0[:To], self.logits[:To], To)
        return self.logits[:To]

    # ---- host-side inputs, as llama_set_inputs fills them (src/llama-context.cpp:61-200) --------
    def set_inputs(self, emb_host, pos0, T, n_kv):
        """emb_host: pinned f32 [T, n_embd]; tokens occupy cache cells pos0 .. pos0+T-1"""
        self.x[:T].copy_(emb_host[:T], non_blocking=True)
        self.pos[:T].copy_(torch.arange(pos0, pos0 + T, dtype=torch.int32), non_blocking=False)
        m = torch.full((self.mask.shape[0], n_kv), float("-inf"), dtype=torch.float16)
        for i in range(T):
            m[i, :pos0 + i + 1] = 0.0
        self.mask[:, :n_kv].copy_(m, non_blocking=False)
