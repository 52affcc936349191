"""Sapapel decoder: post-norm layers on an fp32 stream, token shift, learned depth average,
latent attention and a sigmoid-routed input-scaled MoE.

Per layer i, for the step's tokens (x: fp32 stream [T, W] entering the layer; a = the model's
dtype, bf16 or fp32; every norm, the stream, scores, the router and the state are fp32):

    h      = token_shift(x)                    x[t] + (x[t-1] - x[t]) * mu -> a          HIP  postnorm.hip
             (x[t-1] of a portion's first token: the sequence's state slot; the slot then
             takes the portion's last x)
    qdg    = h @ [Wq; Wdkv; Wg]^T              one projection                            hipBLASLt / decode GEMM
    cache  <- rms_norm(dkv) * w                the latent c, paged                       HIP  latent_attention.hip
    q~     = q[a] @ Wuk[a]  per head           query folded into the latent space        hipBLASLt (batched)
    o~     = softmax(scale q~ C^T) C           causal, over the cached latents           HIP  latent_attention.hip
    o      = o~[a] @ Wuv[a]^T per head         values out of the latent space            hipBLASLt (batched)
    m      = (o * sigmoid(g)) @ Wo^T           output gate + projection                  HIP gate_merge + GEMM
    x1     = norm(alpha x + m) * g1            one-number gain; also leaves x in the     HIP  postnorm.hip
                                               sequences' state slots
    ids, s = top-k of sigmoid(Wr x1)           fp32 router                               HIP  sigmoid_moe.hip
    f      = sum_e down_e(silu(s gate_e x1) * (s up_e x1))                                HIP  sigmoid_moe.hip
    X[i+1] = norm(alpha x1 + f) * g2 ;  x' = sum_j dwa_i[j] X[j]     (X[0] = the embedding)  HIP  postnorm.hip
             (one kernel: the experts' rows are summed, normed and averaged over depth)

and logits = head @ (norm(x_last) * g_final).  Only c is cached (kv_rank numbers per token and
layer); the per-sequence state is one stream row per layer.  Tensor parallelism is not
implemented for this family (the layers are a few megabytes to a few hundred: one GPU).
"""
from __future__ import annotations

from typing import List, Optional

import torch
from torch import nn

from ..ops import gemm
from ..ops import latent_attention as la_ops
from ..ops import moe as moe_ops
from ..ops import stream as stream_ops
from ..parallel.state import ParallelState
from .config import SapapelConfig
from .weights import SafetensorsIndex, random_full


def _p(t: torch.Tensor) -> nn.Parameter:
    return nn.Parameter(t.contiguous(), requires_grad=False)


class LatentAttention(nn.Module):
    """Weights of one latent-attention mixer (sizes from its spec)."""

    def __init__(self, spec, width: int):
        super().__init__()
        self.spec, self.width = spec, width
        self.w_in = None      # [H*D + R + H*V, W]: q | dkv | gate rows
        self.latent_w = None  # [R] fp32, weight of the latent's norm
        self.uk = None        # [H, D, R]
        self.uv_t = None      # [H, R, V]
        self.w_o = None       # [W, H*V]
        self.w_in_p = self.w_o_p = None  # block-packed copies for the decode GEMM (pack())

    def set(self, q, dkv, latent_w, uk, uv, g, o, dtype, device) -> None:
        s = self.spec
        H, D, V, R = s.heads, s.dim, s.vdim, s.kv_rank
        assert q.shape == (H * D, self.width) and dkv.shape == (R, self.width) and g.shape == (H * V, self.width)
        assert uk.shape == (H * D, R) and uv.shape == (H * V, R) and o.shape == (self.width, H * V)
        to = lambda t: t.to(device=device, dtype=dtype)
        self.w_in = _p(to(torch.cat([q, dkv, g], 0)))
        self.latent_w = _p(latent_w.to(device=device, dtype=torch.float32).reshape(R))
        self.uk = _p(to(uk).view(H, D, R))
        self.uv_t = _p(to(uv).view(H, V, R).transpose(1, 2))
        self.w_o = _p(to(o))

    def pack(self) -> None:
        """Block-packed copies of the two projections where the decode GEMM tiles them."""
        ok = lambda w: w.is_cuda and w.dtype == torch.bfloat16 and w.shape[0] % 128 == 0 and w.shape[1] % 256 == 0
        if self.w_in_p is None and ok(self.w_in):
            self.w_in_p = gemm.pack_weight(self.w_in)
        if self.w_o_p is None and ok(self.w_o):
            self.w_o_p = gemm.pack_weight(self.w_o)

    @staticmethod
    def _split_k(x: torch.Tensor, w: torch.Tensor, packed: Optional[torch.Tensor]):
        """Decode-sized rows on shapes the weight-streaming GEMM tiles: its split-K slabs, unreduced
        (gemm.Partial), so the launch fills the chip; None otherwise."""
        if not gemm.skinny_ok(x, w):
            return None
        S = gemm.choose_split(w.shape[0], x.shape[1], x.shape[0])
        if S <= 1:
            return None
        ws = torch.empty(S * x.shape[0] * w.shape[0], dtype=torch.float32, device=x.device)
        return gemm.linear_partial(x, w, ws, S, packed=packed)

    def forward(self, h: torch.Tensor, md, cache: torch.Tensor, eps: float,
                cache_t: Optional[torch.Tensor] = None):
        """The mixer's output [T, W], or for decode-sized steps the output projection's unreduced
        split-K slabs (gemm.Partial) for the norm kernel that follows to sum."""
        s = self.spec
        H, D, V, R = s.heads, s.dim, s.vdim, s.kv_rank
        T = h.shape[0]
        part = self._split_k(h, self.w_in, self.w_in_p)
        qdg = gemm.reduce_partial(part) if part is not None else gemm.linear(h, self.w_in, packed=self.w_in_p)
        la_ops.latent_norm_cache(qdg[:, H * D:H * D + R], self.latent_w, eps, cache, md.slot_mapping, cache_t)
        q_lat = torch.bmm(qdg[:, :H * D].view(T, H, D).transpose(0, 1), self.uk)          # [H, T, R]
        o_lat = la_ops.latent_attention(q_lat, cache, md.block_tables, md.cu_q, md.context_lens, md.num_seqs, s.scale,
                                        cache_t, md.num_decode)
        o = torch.bmm(o_lat, self.uv_t)                                                    # [H, T, V]
        a = la_ops.gate_merge(o, qdg[:, H * D + R:])
        part = self._split_k(a, self.w_o, self.w_o_p)
        return part if part is not None else gemm.linear(a, self.w_o, packed=self.w_o_p)


class SigmoidMoE(nn.Module):
    def __init__(self, spec):
        super().__init__()
        self.spec = spec
        self.router = None  # [E, W] fp32
        self.gate = self.up = self.down = None  # [E, F, W], [E, F, W], [E, W, F]

        # shapes the grouped MFMA GEMMs tile: interleaved gate|up and down, block-packed for decode
        self.w13 = self.w2 = self.w13_p = self.w2_p = None

    def set(self, router, gates, ups, downs, dtype, device) -> None:
        to = lambda ts: _p(torch.stack(ts).to(device=device, dtype=dtype))
        self.router = _p(router.to(device=device, dtype=torch.float32))
        E, (F_, W) = len(gates), gates[0].shape
        if moe_ops.mfma_experts_ok(E, F_, W, dtype, torch.device(device)):
            self.w13 = to([gemm.interleave_gate_up(g, u) for g, u in zip(gates, ups)])
            self.w2 = to(downs)
            self.gate = self.up = self.down = None
        else:
            self.gate, self.up, self.down = to(gates), to(ups), to(downs)

    def pack(self) -> None:
        if self.w13 is not None and self.w13_p is None:
            E, N, K = self.w13.shape
            self.w13_p = gemm.pack_weight(self.w13.view(E * N, K)).view(E, N, K)
            E, N, K = self.w2.shape
            self.w2_p = gemm.pack_weight(self.w2.view(E * N, K)).view(E, N, K)

    def forward(self, x: torch.Tensor, x_act: torch.Tensor, defer_combine: bool = False):
        """The experts' summed output [T, W] fp32, or with ``defer_combine`` the expert rows and their
        inverse positions for the following norm kernel to sum."""
        ids, wts = moe_ops.route_sigmoid_topk(x, self.router, self.spec.top)
        return moe_ops.input_scaled_moe(x, x_act, ids, wts, self.gate, self.up, self.down, self.w13, self.w2,
                                        self.w13_p, self.w2_p, defer_combine)


class SapapelLayer(nn.Module):
    def __init__(self, spec, width: int):
        super().__init__()
        self.mix = LatentAttention(spec.mixer, width)
        self.mlp = SigmoidMoE(spec.mlp) if spec.mlp is not None else None
        self.shift = None   # [W] fp32, None: the mixer reads x itself
        self.g1 = self.g2 = None  # [1] fp32
        self.dwa = None     # [i + 2] fp32, None: the layer's own output goes on


class SapapelForCausalLM(nn.Module):
    # engine hooks (engine/model_runner.py): this family owns its cache and state layouts
    needs_state = True
    supports_graphs = True

    def __init__(self, cfg: SapapelConfig, st: ParallelState, dtype: torch.dtype, device: torch.device):
        super().__init__()
        if st.tp_size > 1 or getattr(st, "ep_size", 1) > 1:
            raise ValueError("Sapapel runs on one GPU (no TP / EP sharding for this family)")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"Sapapel runs in bfloat16 or float32, not {dtype}")
        self.cfg, self.st, self.dtype, self.device = cfg, st, dtype, device
        self.layers = nn.ModuleList(SapapelLayer(l, cfg.hidden_size) for l in cfg.layers)
        self.embed = self.head = self.final_gain = None
        self._hist: Optional[torch.Tensor] = None

    # ------------------------------------------------------------------ weights
    def _set_layer(self, i: int, get, has) -> None:
        cfg, L, spec = self.cfg, self.layers[i], self.cfg.layers[i]
        p, dev, dt = f"l{i}.", self.device, self.dtype
        f32 = lambda t: _p(t.to(device=dev, dtype=torch.float32).reshape(-1))
        L.mix.set(get(p + "mix.q"), get(p + "mix.dkv"), get(p + "mix.dkv.norm"), get(p + "mix.uk"), get(p + "mix.uv"),
                  get(p + "mix.g"), get(p + "mix.o"), dt, dev)
        L.g1 = f32(get(p + "norm1"))
        L.shift = f32(get(p + "shift")) if has(p + "shift") else None
        L.dwa = f32(get(p + "dwa")) if has(p + "dwa") else None
        if L.dwa is not None and L.dwa.numel() != i + 2:
            raise ValueError(f"{p}dwa has {L.dwa.numel()} entries, layer {i} averages {i + 2} outputs")
        if L.mlp is None and has(p + "norm2"):  # a second norm without a feed-forward: it norms alpha x
            L.g2 = f32(get(p + "norm2"))
        if L.mlp is not None:
            E = spec.mlp.experts
            L.g2 = f32(get(p + "norm2"))
            L.mlp.set(get(p + "mlp.router"), [get(p + f"mlp.e{e}.gate") for e in range(E)],
                      [get(p + f"mlp.e{e}.up") for e in range(E)], [get(p + f"mlp.e{e}.down") for e in range(E)], dt, dev)
            got = L.mlp.gate.shape if L.mlp.gate is not None else (E, L.mlp.w13.shape[1] // 2, L.mlp.w13.shape[2])
            assert tuple(got) == (E, spec.mlp.ff, cfg.hidden_size), (got, spec.mlp)

    def _set_top(self, get) -> None:
        dev, dt = self.device, self.dtype
        self.embed = _p(get("embed").to(device=dev, dtype=dt))
        self.head = _p(get("head").to(device=dev, dtype=dt))
        self.final_gain = _p(get("final.norm").to(device=dev, dtype=torch.float32).reshape(-1))
        assert self.embed.shape == (self.cfg.vocab_size, self.cfg.hidden_size) == self.head.shape

    def load_hf(self, path: str) -> "SapapelForCausalLM":
        """Load a checkpoint folder (safetensors; bf16 tensors under the design's own names)."""
        idx = SafetensorsIndex(path)
        self._set_top(idx.get)
        for i in range(len(self.layers)):
            self._set_layer(i, idx.get, idx.has)
        return self

    def load_state(self, tensors: dict) -> "SapapelForCausalLM":
        """The same from a dict name -> tensor (tests)."""
        self._set_top(tensors.__getitem__)
        for i in range(len(self.layers)):
            self._set_layer(i, tensors.__getitem__, tensors.__contains__)
        return self

    def random_state(self, seed: int = 0) -> dict:
        """Random bf16-representable tensors under the checkpoint names (gains near 1, shift in
        [0, 1), depth weights near "mostly the newest output")."""
        cfg, W, std = self.cfg, self.cfg.hidden_size, self.cfg.init_std
        r = lambda name, shape, s=std: random_full(name, shape, s, seed, self.device, torch.bfloat16)
        out = {"embed": r("embed", (cfg.vocab_size, W), 1.0), "head": r("head", (cfg.vocab_size, W)),
               "final.norm": 1 + r("final.norm", (), 0.1)}
        for i, l in enumerate(cfg.layers):
            p, m = f"l{i}.", l.mixer
            out[p + "norm1"] = 1 + r(p + "norm1", (), 0.1)
            out[p + "shift"] = r(p + "shift", (W,), 1.0).float().sigmoid().bfloat16()
            d = r(p + "dwa", (i + 2,), 0.1)
            d[-1] += 0.8
            out[p + "dwa"] = d
            out[p + "mix.q"] = r(p + "mix.q", (m.heads * m.dim, W))
            out[p + "mix.dkv"] = r(p + "mix.dkv", (m.kv_rank, W))
            out[p + "mix.dkv.norm"] = 1 + r(p + "mix.dkv.norm", (m.kv_rank,), 0.1)
            out[p + "mix.uk"] = r(p + "mix.uk", (m.heads * m.dim, m.kv_rank), 2 * std)
            out[p + "mix.uv"] = r(p + "mix.uv", (m.heads * m.vdim, m.kv_rank), 2 * std)
            out[p + "mix.g"] = r(p + "mix.g", (m.heads * m.vdim, W))
            out[p + "mix.o"] = r(p + "mix.o", (W, m.heads * m.vdim))
            if l.mlp is not None:
                out[p + "norm2"] = 1 + r(p + "norm2", (), 0.1)
                out[p + "mlp.router"] = r(p + "mlp.router", (l.mlp.experts, W), 0.5)
                for e in range(l.mlp.experts):
                    out[p + f"mlp.e{e}.gate"] = r(p + f"mlp.e{e}.gate", (l.mlp.ff, W))
                    out[p + f"mlp.e{e}.up"] = r(p + f"mlp.e{e}.up", (l.mlp.ff, W))
                    out[p + f"mlp.e{e}.down"] = r(p + f"mlp.e{e}.down", (W, l.mlp.ff))
        return out

    def init_random(self, seed: int = 0) -> "SapapelForCausalLM":
        return self.load_state(self.random_state(seed))

    def pack_decode_weights(self) -> None:
        """Block-packed copies of the expert weights for the decode GEMM (engine hook)."""
        for L in self.layers:
            L.mix.pack()
            if L.mlp is not None:
                L.mlp.pack()

    def to(self, device, *a, **k):  # keeps the fp32 tensors fp32 (no dtype argument)
        super().to(device)
        self.device = torch.device(device)
        self._hist = None
        return self

    # ---------------------------------------------------------- cache and state
    def cache_bytes_per_block(self, block_size: int) -> int:
        esz = 2 if self.dtype == torch.bfloat16 else 4
        copies = lambda R: 2 if la_ops.mfma_latent(R, self.dtype, self.device, block_size) else 1
        return sum(l.mixer.kv_rank * copies(l.mixer.kv_rank) for l in self.cfg.layers) * block_size * esz

    def state_bytes_per_slot(self) -> int:
        return len(self.layers) * self.cfg.hidden_size * 4

    def alloc_cache(self, num_blocks: int, block_size: int, num_slots: int) -> List[tuple]:
        """Per layer: (latent cache [blocks, block_size, kv_rank], its latent-major copy for the
        matrix-core kernels or None, shift state [slots, W] fp32)."""
        out = []
        for l in self.cfg.layers:
            R = l.mixer.kv_rank
            c = torch.zeros((num_blocks, block_size, R), dtype=self.dtype, device=self.device)
            c_t = (la_ops.alloc_latent_major(num_blocks, block_size, R, self.device)
                   if la_ops.mfma_latent(R, self.dtype, self.device, block_size) else None)
            out.append((c, c_t, torch.zeros((max(num_slots, 1), self.cfg.hidden_size), dtype=torch.float32,
                                            device=self.device)))
        return out

    def activation_bytes_per_token(self) -> int:
        W = self.cfg.hidden_size
        widest = max(l.mixer.heads * (l.mixer.dim + 2 * l.mixer.vdim + 2 * l.mixer.kv_rank) + l.mixer.kv_rank
                     for l in self.cfg.layers)
        return 4 * W * (len(self.layers) + 6) + 4 * widest

    def reserve_steps(self, max_tokens: int) -> None:
        """Allocate the per-step history of layer outputs once (stable address: graph capture)."""
        n = len(self.layers) + 1
        if self._hist is None or self._hist.shape[1] < max_tokens or self._hist.device != self.device:
            self._hist = torch.zeros((n, max_tokens, self.cfg.hidden_size), dtype=torch.float32, device=self.device)

    # ------------------------------------------------------------------ forward
    @torch.inference_mode()
    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor, md, caches: List[tuple]) -> torch.Tensor:
        """The fp32 stream [T, W] after the last layer, for the step described by ``md``
        (ops/attention.py AttnMetadata: the whole-batch fields)."""
        cfg = self.cfg
        T = input_ids.shape[0]
        self.reserve_steps(T)
        hist, eps, alpha, dt = self._hist, cfg.rms_eps, cfg.alpha, self.dtype
        x = stream_ops.embed_rows(self.embed, input_ids, hist[0])[:T]
        for i, L in enumerate(self.layers):
            cache, cache_t, state = caches[i]
            save = None
            if L.shift is not None:
                h = stream_ops.token_shift(x, L.shift, state, md.token_seq, md.cu_q, positions, md.state_slots, dt)
                save = (state, md.token_seq, md.cu_q, md.state_slots)  # the first norm kernel leaves x there
            else:
                h = x.to(dt)
            m = L.mix(h, md, cache, eps, cache_t)
            has_mlp = L.mlp is not None
            depth = dict(hist=hist, nh=i + 2, coef=L.dwa) if L.dwa is not None else {}
            out = torch.empty_like(x)
            if has_mlp:
                x1, x1_act = stream_ops.sum_gain_norm(x, m, alpha, L.g1, eps, out=torch.empty_like(x), act_dtype=dt,
                                                      save=save)
                y, inv = L.mlp(x1, x1_act, defer_combine=True)
                x, _ = stream_ops.sum_gain_norm(x1, y, alpha, L.g2, eps, out=out, gather=(inv, L.mlp.spec.top), **depth)
            elif L.g2 is not None:  # no feed-forward but a second norm: x <- norm2(alpha x1)
                x1, _ = stream_ops.sum_gain_norm(x, m, alpha, L.g1, eps, out=torch.empty_like(x), save=save)
                x, _ = stream_ops.sum_gain_norm(x1, None, alpha, L.g2, eps, out=out, **depth)
            else:
                x, _ = stream_ops.sum_gain_norm(x, m, alpha, L.g1, eps, out=out, save=save, **depth)
            if L.dwa is None:  # later layers' averages still read this layer's output
                hist[i + 1, :T] = x
        return x

    def compute_logits(self, rows: torch.Tensor) -> torch.Tensor:
        """fp32 logits of stream rows [n, W]: the final one-number-gain norm, then the head."""
        _, act = stream_ops.sum_gain_norm(rows.contiguous(), None, 1.0, self.final_gain, self.cfg.rms_eps,
                                          act_dtype=self.dtype)
        return gemm.linear(act, self.head).float()

