"""Kivezen decoder: pre-norm layers on one or several fp32 residual streams (hyper-connections),
sink-softmax attention or lightning (decayed linear) attention mixers, dense GELU or clamped-GLU
MoE feed-forwards, and a block of layers that runs several times with the same weights.

Per layer run, for the step's tokens (xs: fp32 streams [T, S, W]; a = the model's dtype, bf16 or
fp32; norms, the streams, scores, softmax, the router and the recurrent state are fp32):

    h   = norm(sum_s in1[s] xs[s]) * w1 -> a                                     HIP  hyper.hip
    attention:  qkv = h @ [Wq; Wk; Wv]^T                                         hipBLASLt
                q, k turned by the position (YaRN table) and set to unit RMS per head, v turned by
                its position over vdim; k, v -> paged cache                      HIP  sink_attention.hip
                o = sum_j p_j v_j, p_j = exp(s_j) / (1 + sum_j' exp(s_j')), s = cap * tanh(q.k *
                scale * temp_h / cap), j <= the token; o turned back by the token's position
    lightning:  qkvg = h @ [Wq; Wk; Wv; Wg]^T ; q, k, v = silu(.)                hipBLASLt
                S <- decay_h S + k v^T ; o = S^T q  (state [H, D, V] fp32 per sequence slot) HIP lightning.hip
                o = norm(o over all heads) * w * sigmoid(g)
    y   = o @ Wo^T
    xs'[t] = sum_s mix1[s, t] xs[s] + out1[t] y ;  h2 = norm(sum_t in2[t] xs'[t]) * w2      (one kernel)
    dense:      f = gelu_tanh(h2 @ Wup^T) @ Wdown^T
    moe:        z = Wr h2 (fp32) ; top experts by z, weights softmax over the chosen z
                f = sum_e w_e down_e(min(g, L) sigmoid(1.702 min(g, L)) (clamp(u, -L, L) + 1))
                    + sigmoid(Wsg h2) * shared(h2)
    xs''[t] = sum_s mix2[s, t] xs'[s] + out2[t] f ; the next run's h                         (one kernel)

and logits = cap * tanh(head @ (norm(sum_s xs[s]) * wf) / cap).  A model without ``streams`` is the
same with S = 1 and unit coefficients (the plain residual).  Every layer run has its own cache
(attention) or state (lightning), also the passes of a looped block.  Tensor parallelism is not
implemented for this family.
"""
from __future__ import annotations

from typing import List, Optional

import torch
from torch import nn

from ..ops import gemm
from ..ops import hyper as hyper_ops
from ..ops import lightning as lightning_ops
from ..ops import moe as moe_ops
from ..ops import native
from ..ops import sink_attention as sa_ops
from ..parallel.state import ParallelState
from .config import ClampedMoESpec, DenseFFSpec, KivezenConfig
from .weights import SafetensorsIndex, random_full


def _p(t: torch.Tensor) -> nn.Parameter:
    return nn.Parameter(t.contiguous(), requires_grad=False)


def _packed(w: torch.Tensor) -> Optional[torch.Tensor]:
    """Block-packed copy of a projection where the decode GEMM tiles it (bf16 on the GPU), else None."""
    ok = w.is_cuda and w.dtype == torch.bfloat16 and w.shape[0] % 128 == 0 and w.shape[1] % 256 == 0
    return gemm.pack_weight(w) if ok else None


def _project(x: torch.Tensor, w: torch.Tensor, packed: Optional[torch.Tensor], partial: bool = False):
    """x @ w^T.  Decode-sized rows on shapes the weight-streaming GEMM tiles run as split-K slabs so
    that the launch fills the chip; with ``partial`` the slabs come back unreduced (gemm.Partial) for
    the stream kernel that follows to sum."""
    if gemm.skinny_ok(x, w):
        S = gemm.choose_split(w.shape[0], x.shape[1], x.shape[0])
        if S > 1:
            ws = torch.empty(S * x.shape[0] * w.shape[0], dtype=torch.float32, device=x.device)
            part = gemm.linear_partial(x, w, ws, S, packed=packed)
            return part if partial else gemm.reduce_partial(part)
    return gemm.linear(x, w, packed=packed)


class SinkAttention(nn.Module):
    """Weights and rotation tables of one sink-softmax attention mixer (sizes from its spec)."""

    def __init__(self, spec, width: int):
        super().__init__()
        self.spec, self.width = spec, width
        self.w_in = None        # [H*D + G*D + G*V, W]: q | k | v rows
        self.w_o = None         # [W, H*V]
        self.head_scale = None  # [H] fp32: scale * the head's temperature
        self.qk_table = self.v_table = None  # [positions, pairs, 2] fp32 (cos, sin); None: no rotation
        self.w_in_p = self.w_o_p = None      # block-packed copies for the decode GEMM (pack())

    def pack(self) -> None:
        self.w_in_p, self.w_o_p = _packed(self.w_in), _packed(self.w_o)

    def set(self, q, k, v, o, temp, dtype, device) -> None:
        s = self.spec
        H, G, D, V = s.heads, s.kv_heads, s.dim, s.vdim
        assert H % G == 0 and q.shape == (H * D, self.width) and k.shape == (G * D, self.width)
        assert v.shape == (G * V, self.width) and o.shape == (self.width, H * V)
        assert s.rot is None or (s.rot.dims % 2 == 0 and s.rot.dims <= D and V % 2 == 0)
        self.w_in = _p(torch.cat([q, k, v], 0).to(device=device, dtype=dtype))
        self.w_o = _p(o.to(device=device, dtype=dtype))
        t = torch.ones(H) if temp is None else temp.float().reshape(H).cpu()
        self.head_scale = _p((t.double() * s.scale).float().to(device))

    def forward(self, h: torch.Tensor, positions: torch.Tensor, md, cache: tuple, eps: float) -> torch.Tensor:
        s = self.spec
        k_cache, v_cache = cache
        qkv = _project(h, self.w_in, self.w_in_p, partial=True)  # slabs are summed by the rotation kernel
        q = sa_ops.rope_norm_cache(qkv, positions, md.slot_mapping, self.qk_table, self.v_table, k_cache, v_cache,
                                   s.heads, s.kv_heads, s.dim, s.vdim, eps)
        o = sa_ops.sink_attention(q, k_cache, v_cache, md.block_tables, md.cu_q, md.context_lens, md.num_seqs,
                                  positions, self.head_scale, s.softcap, s.sink, self.v_table, md.num_decode)
        return _project(o, self.w_o, self.w_o_p, partial=True)


class LightningMixer(nn.Module):
    """Weights of one lightning-attention mixer."""

    def __init__(self, spec, width: int):
        super().__init__()
        self.spec, self.width = spec, width
        self.w_in = None    # [H*D | H*D | H*V | H*V, W]: q | k | v | gate rows
        self.w_o = None     # [W, H*V]
        self.norm_w = None  # [H*V] fp32
        self.decay = None   # [H] fp32
        self.w_in_p = self.w_o_p = None

    def pack(self) -> None:
        self.w_in_p, self.w_o_p = _packed(self.w_in), _packed(self.w_o)

    def set(self, q, k, v, g, o, norm_w, dtype, device) -> None:
        s = self.spec
        H, D, V = s.heads, s.dim, s.vdim
        assert q.shape == (H * D, self.width) == k.shape and v.shape == (H * V, self.width) == g.shape
        assert o.shape == (self.width, H * V)
        self.w_in = _p(torch.cat([q, k, v, g], 0).to(device=device, dtype=dtype))
        self.w_o = _p(o.to(device=device, dtype=dtype))
        self.norm_w = _p(norm_w.to(device=device, dtype=torch.float32).reshape(H * V))
        self.decay = _p(torch.tensor(s.decay, dtype=torch.float64).float().to(device))

    def forward(self, h: torch.Tensor, positions: torch.Tensor, md, cache: tuple, eps: float) -> torch.Tensor:
        s = self.spec
        H, D, V = s.heads, s.dim, s.vdim
        n = H * (2 * D + V)
        qkvg = _project(h, self.w_in, self.w_in_p)
        o = lightning_ops.lightning_attention(qkvg[:, :n], cache[0], self.decay, md.cu_q, md.num_seqs, positions,
                                              md.state_slots, H, D, V, md.num_decode)
        a = lightning_ops.gated_rms_norm(o, self.norm_w, qkvg[:, n:], eps, h.dtype)
        return _project(a, self.w_o, self.w_o_p, partial=True)


class DenseGeluFF(nn.Module):
    def __init__(self, spec: DenseFFSpec):
        super().__init__()
        self.spec = spec
        self.up = self.down = self.up_p = self.down_p = None

    def set(self, up, down, dtype, device) -> None:
        self.up, self.down = _p(up.to(device=device, dtype=dtype)), _p(down.to(device=device, dtype=dtype))

    def pack(self) -> None:
        self.up_p, self.down_p = _packed(self.up), _packed(self.down)

    def forward(self, h: torch.Tensor, h32: Optional[torch.Tensor]):
        return _project(moe_ops.gelu_tanh(_project(h, self.up, self.up_p)), self.down, self.down_p, partial=True)


class ClampedMoE(nn.Module):
    """Router (fp32, with the shared expert's gate as one more row), the experts and the shared expert."""

    def __init__(self, spec: ClampedMoESpec):
        super().__init__()
        self.spec = spec
        self.router = None                       # [E (+ 1), W] fp32
        self.gate = self.up = self.down = None   # [E, F, W], [E, F, W], [E, W, F]
        self.w13 = self.w2 = self.w13_p = self.w2_p = None  # the grouped MFMA GEMMs' layouts
        self.sh_in = self.sh_down = None         # [2 Fs, W] gate rows then up rows, [W, Fs]
        self.sh_in_p = self.sh_down_p = None

    def set(self, router, gates, ups, downs, shared, dtype, device) -> None:
        to = lambda ts: _p(torch.stack(ts).to(device=device, dtype=dtype))
        E, (F_, W) = len(gates), gates[0].shape
        rows = [router.float()]
        if shared is not None:
            sg, sgate, sup, sdown = shared
            rows.append(sg.float().reshape(1, W))
            self.sh_in = _p(torch.cat([sgate, sup], 0).to(device=device, dtype=dtype))
            self.sh_down = _p(sdown.to(device=device, dtype=dtype))
        self.router = _p(torch.cat(rows, 0).to(device))
        if moe_ops.mfma_experts_ok(E, F_, W, dtype, torch.device(device)):
            self.w13 = to([gemm.interleave_gate_up(g, u) for g, u in zip(gates, ups)])
            self.w2 = to(downs)
        else:
            self.gate, self.up, self.down = to(gates), to(ups), to(downs)

    def pack(self) -> None:
        if self.sh_in is not None:
            self.sh_in_p, self.sh_down_p = _packed(self.sh_in), _packed(self.sh_down)
        if self.w13 is not None and self.w13_p is None:
            E, N, K = self.w13.shape
            self.w13_p = gemm.pack_weight(self.w13.view(E * N, K)).view(E, N, K)
            E, N, K = self.w2.shape
            self.w2_p = gemm.pack_weight(self.w2.view(E * N, K)).view(E, N, K)

    def forward(self, h: torch.Tensor, h32: torch.Tensor) -> hyper_ops.ExpertSum:
        s = self.spec
        logits = moe_ops.router_logits(h32, self.router)
        ids, wts = moe_ops.route_topk_softmax(logits, s.experts, s.top)
        y, inv = moe_ops.clamped_experts(h, ids, self.gate, self.up, self.down, s.limit, self.w13, self.w2,
                                         self.w13_p, self.w2_p)
        out = hyper_ops.ExpertSum(y, inv, wts, s.top)
        if self.sh_in is not None:
            a = moe_ops.clamped_glu(_project(h, self.sh_in, self.sh_in_p, partial=True), s.shared_limit, dtype=h.dtype)
            out.shared, out.gate = _project(a, self.sh_down, self.sh_down_p), logits[:, s.experts]
        return out


class KivezenLayer(nn.Module):
    def __init__(self, spec, width: int):
        super().__init__()
        self.kind = spec.type
        self.mix = SinkAttention(spec.mixer, width) if spec.type == "attention" else LightningMixer(spec.mixer, width)
        self.mlp = None
        if isinstance(spec.mlp, DenseFFSpec):
            self.mlp = DenseGeluFF(spec.mlp)
        elif spec.mlp is not None:
            self.mlp = ClampedMoE(spec.mlp)
        self.norm1 = self.norm2 = None      # [W] fp32
        self.hc1 = self.hc2 = None          # (a_in [S], mix [S, S], a_out [S]) fp32


class KivezenForCausalLM(nn.Module):
    # engine hooks (engine/model_runner.py): this family owns its cache and state layouts
    supports_graphs = True

    def __init__(self, cfg: KivezenConfig, st: ParallelState, dtype: torch.dtype, device: torch.device):
        super().__init__()
        if st.tp_size > 1 or getattr(st, "ep_size", 1) > 1:
            raise ValueError("Kivezen runs on one GPU (no TP / EP sharding for this family)")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"Kivezen runs in bfloat16 or float32, not {dtype}")
        self.cfg, self.st, self.dtype, self.device = cfg, st, dtype, device
        self.S = max(cfg.streams, 1)
        self.needs_state = cfg.needs_state
        self.layers = nn.ModuleList(KivezenLayer(l, cfg.hidden_size) for l in cfg.layers)
        self.embed = self.head = self.final_norm = None
        self.sum_in = None
        self._max_pos = 0

    # ------------------------------------------------------------------ weights
    def _hc(self, p: str, get, has):
        S, dev = self.S, self.device
        if self.cfg.streams and has(p + "in"):
            f = lambda n, shape: _p(get(p + n).to(device=dev, dtype=torch.float32).reshape(shape))
            return f("in", (S,)), f("mix", (S, S)), f("out", (S,))
        if self.cfg.streams:
            raise KeyError(f"{p}in: a model with streams needs its hyper-connection tensors")
        one = lambda *shape: _p(torch.ones(shape, dtype=torch.float32, device=dev))
        return one(1), one(1, 1), one(1)

    def _set_layer(self, i: int, get, has) -> None:
        cfg, L, spec = self.cfg, self.layers[i], self.cfg.layers[i]
        p, dev, dt, W = f"l{i}.", self.device, self.dtype, self.cfg.hidden_size
        f32 = lambda t: _p(t.to(device=dev, dtype=torch.float32).reshape(-1))
        if L.kind == "attention":
            L.mix.set(get(p + "mix.q"), get(p + "mix.k"), get(p + "mix.v"), get(p + "mix.o"),
                      get(p + "mix.temp") if has(p + "mix.temp") else None, dt, dev)
        else:
            L.mix.set(get(p + "mix.q"), get(p + "mix.k"), get(p + "mix.v"), get(p + "mix.g"), get(p + "mix.o"),
                      get(p + "mix.norm"), dt, dev)
        L.norm1, L.hc1 = f32(get(p + "norm1")), self._hc(p + "hc1.", get, has)
        f = spec.mlp
        if f is None:
            return
        L.norm2, L.hc2 = f32(get(p + "norm2")), self._hc(p + "hc2.", get, has)
        if isinstance(f, DenseFFSpec):
            up, down = get(p + "mlp.up"), get(p + "mlp.down")
            assert up.shape == (f.ff, W) and down.shape == (W, f.ff)
            L.mlp.set(up, down, dt, dev)
        else:
            E = f.experts
            shared = None
            if f.shared_ff:
                shared = (get(p + "mlp.shared.sg"), get(p + "mlp.shared.gate"), get(p + "mlp.shared.up"),
                          get(p + "mlp.shared.down"))
                assert shared[1].shape == (f.shared_ff, W) and shared[3].shape == (W, f.shared_ff)
            gates = [get(p + f"mlp.e{e}.gate") for e in range(E)]
            assert gates[0].shape == (f.ff, W) and get(p + "mlp.router").shape == (E, W)
            L.mlp.set(get(p + "mlp.router"), gates, [get(p + f"mlp.e{e}.up") for e in range(E)],
                      [get(p + f"mlp.e{e}.down") for e in range(E)], shared, dt, dev)

    def _set_top(self, get) -> None:
        dev, dt = self.device, self.dtype
        self.embed = _p(get("embed").to(device=dev, dtype=dt))
        self.head = _p(get("head").to(device=dev, dtype=dt))
        self.final_norm = _p(get("final.norm").to(device=dev, dtype=torch.float32).reshape(-1))
        self.sum_in = _p(torch.ones(self.S, dtype=torch.float32, device=dev))
        assert self.embed.shape == (self.cfg.vocab_size, self.cfg.hidden_size) == self.head.shape

    def load_hf(self, path: str) -> "KivezenForCausalLM":
        """Load a checkpoint folder (safetensors; tensors under the design's own names)."""
        idx = SafetensorsIndex(path)
        return self._load(idx.get, idx.has)

    def load_state(self, tensors: dict) -> "KivezenForCausalLM":
        """The same from a dict name -> tensor (tests)."""
        return self._load(tensors.__getitem__, tensors.__contains__)

    def _load(self, get, has) -> "KivezenForCausalLM":
        self._set_top(get)
        for i in range(len(self.layers)):
            self._set_layer(i, get, has)
        if self._max_pos:
            self._build_tables()
        return self

    def random_state(self, seed: int = 0) -> dict:
        """Random bf16-representable tensors under the checkpoint names (norm weights and
        temperatures near 1, stream mixes near the identity)."""
        cfg, W, std, S = self.cfg, self.cfg.hidden_size, self.cfg.init_std, self.cfg.streams
        r = lambda name, shape, s=std: random_full(name, shape, s, seed, self.device, torch.bfloat16)
        out = {"embed": r("embed", (cfg.vocab_size, W), 1.0), "head": r("head", (cfg.vocab_size, W)),
               "final.norm": 1 + r("final.norm", (W,), 0.1)}
        for i, l in enumerate(cfg.layers):
            p, m = f"l{i}.", l.mixer
            subs = ["1"] + (["2"] if l.mlp is not None else [])
            for q in subs:
                out[p + "norm" + q] = 1 + r(p + "norm" + q, (W,), 0.1)
                if S:
                    out[p + f"hc{q}.in"] = 1.0 / S + r(p + f"hc{q}.in", (S,), 0.1)
                    out[p + f"hc{q}.out"] = 1 + r(p + f"hc{q}.out", (S,), 0.2)
                    out[p + f"hc{q}.mix"] = (torch.eye(S, device=self.device) + r(p + f"hc{q}.mix", (S, S), 0.1)).bfloat16()
            if l.type == "attention":
                out[p + "mix.q"] = r(p + "mix.q", (m.heads * m.dim, W))
                out[p + "mix.k"] = r(p + "mix.k", (m.kv_heads * m.dim, W))
                out[p + "mix.v"] = r(p + "mix.v", (m.kv_heads * m.vdim, W))
                out[p + "mix.o"] = r(p + "mix.o", (W, m.heads * m.vdim))
                out[p + "mix.temp"] = 1 + r(p + "mix.temp", (m.heads,), 0.2)
            else:
                for n, d in (("q", m.dim), ("k", m.dim), ("v", m.vdim), ("g", m.vdim)):
                    out[p + "mix." + n] = r(p + "mix." + n, (m.heads * d, W))
                out[p + "mix.o"] = r(p + "mix.o", (W, m.heads * m.vdim))
                out[p + "mix.norm"] = 1 + r(p + "mix.norm", (m.heads * m.vdim,), 0.1)
            f = l.mlp
            if isinstance(f, DenseFFSpec):
                out[p + "mlp.up"], out[p + "mlp.down"] = r(p + "mlp.up", (f.ff, W)), r(p + "mlp.down", (W, f.ff))
            elif f is not None:
                out[p + "mlp.router"] = r(p + "mlp.router", (f.experts, W), 0.5)
                names = [f"e{e}" for e in range(f.experts)] + (["shared"] if f.shared_ff else [])
                for n in names:
                    ff = f.shared_ff if n == "shared" else f.ff
                    out[p + f"mlp.{n}.gate"] = r(p + f"mlp.{n}.gate", (ff, W))
                    out[p + f"mlp.{n}.up"] = r(p + f"mlp.{n}.up", (ff, W))
                    out[p + f"mlp.{n}.down"] = r(p + f"mlp.{n}.down", (W, ff))
                if f.shared_ff:
                    out[p + "mlp.shared.sg"] = r(p + "mlp.shared.sg", (1, W))
        return out

    def init_random(self, seed: int = 0) -> "KivezenForCausalLM":
        return self.load_state(self.random_state(seed))

    def pack_decode_weights(self) -> None:
        """Block-packed copies of the projections and expert weights for the decode GEMM (engine hook)."""
        for L in self.layers:
            L.mix.pack()
            if L.mlp is not None:
                L.mlp.pack()

    def to(self, device, *a, **k):  # keeps the fp32 tensors fp32 (no dtype argument)
        super().to(device)
        self.device = torch.device(device)
        if self._max_pos:
            self._build_tables()
        return self

    # ------------------------------------------------------- rotations, cache and state
    def reserve_positions(self, max_pos: int) -> None:
        """Build the rotation tables for positions below ``max_pos`` (engine hook: max_model_len)."""
        if max_pos > self._max_pos:
            self._max_pos = max_pos
            if self.embed is not None:
                self._build_tables()

    def _build_tables(self) -> None:
        made = {}
        for L in self.layers:
            rot = L.mix.spec.rot if L.kind == "attention" else None
            if rot is None:
                continue
            kq, kv = ("qk", rot.dims, rot.base, rot.scaling), ("v", L.mix.spec.vdim, rot.base)
            if kq not in made:
                f, mag = sa_ops.pair_frequencies(rot.dims, rot.base, rot.scaling)
                made[kq] = sa_ops.rotation_table(self._max_pos, f, mag, self.device)
            if kv not in made:
                f, _ = sa_ops.pair_frequencies(L.mix.spec.vdim, rot.base)
                made[kv] = sa_ops.rotation_table(self._max_pos, f, 1.0, self.device)
            L.mix.qk_table, L.mix.v_table = made[kq], made[kv]

    def cache_bytes_per_block(self, block_size: int) -> int:
        esz = 2 if self.dtype == torch.bfloat16 else 4
        n = sum(self.cfg.layers[i].mixer.kv_heads * (self.cfg.layers[i].mixer.dim + self.cfg.layers[i].mixer.vdim)
                for i in self.cfg.runs if self.cfg.layers[i].type == "attention")
        return max(n * block_size * esz, 1)

    def state_bytes_per_slot(self) -> int:
        return sum(self.cfg.layers[i].mixer.heads * self.cfg.layers[i].mixer.dim * self.cfg.layers[i].mixer.vdim
                   for i in self.cfg.runs if self.cfg.layers[i].type == "lightning") * 4

    def alloc_cache(self, num_blocks: int, block_size: int, num_slots: int) -> List[tuple]:
        """Per layer run: (keys [blocks, G, block_size, D], values [blocks, G, V, block_size]) for
        attention, (state [slots, H, D, V] fp32,) for lightning."""
        out = []
        for i in self.cfg.runs:
            m = self.cfg.layers[i].mixer
            if self.cfg.layers[i].type == "attention":
                out.append((torch.zeros((num_blocks, m.kv_heads, block_size, m.dim), dtype=self.dtype, device=self.device),
                            torch.zeros((num_blocks, m.kv_heads, m.vdim, block_size), dtype=self.dtype, device=self.device)))
            else:
                out.append((torch.zeros((max(num_slots, 1), m.heads, m.dim, m.vdim), dtype=torch.float32,
                                        device=self.device),))
        return out

    def activation_bytes_per_token(self) -> int:
        W, widest = self.cfg.hidden_size, 0
        for l in self.cfg.layers:
            m = l.mixer
            n = m.heads * (m.dim + 2 * m.vdim) + (m.kv_heads * (m.dim + m.vdim) if l.type == "attention" else
                                                  m.heads * (m.dim + 2 * m.vdim))
            f = l.mlp
            if isinstance(f, DenseFFSpec):
                n = max(n, 2 * f.ff)
            elif f is not None:
                n = max(n, f.top * (3 * f.ff + 2 * W) + 3 * f.shared_ff + f.experts)
            widest = max(widest, n)
        return 4 * W * (self.S + 4) + 4 * widest

    # ------------------------------------------------------------------ forward
    @torch.inference_mode()
    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor, md, caches: List[tuple]) -> torch.Tensor:
        """The fp32 streams [T, S, W] after the last layer run, for the step described by ``md``
        (ops/attention.py AttnMetadata: the whole-batch fields)."""
        cfg, eps, dt = self.cfg, self.cfg.rms_eps, self.dtype
        if positions.numel() and self._max_pos == 0:
            raise RuntimeError("Kivezen: reserve_positions(max_model_len) has not been called")
        runs = cfg.runs
        xs = hyper_ops.spread_rows(self.embed, input_ids, self.S)
        L0 = self.layers[runs[0]]
        h, _ = hyper_ops.hyper_step(xs, None, None, (L0.hc1[0], L0.norm1), eps, dt)
        for r, li in enumerate(runs):
            L = self.layers[li]
            y = L.mix(h, positions, md, caches[r], eps)
            close = L.hc1[1:]
            if L.mlp is not None:
                h, h32 = hyper_ops.hyper_step(xs, y, close, (L.hc2[0], L.norm2), eps, dt,
                                              want_f32=isinstance(L.mlp, ClampedMoE))
                y, close = L.mlp(h, h32), L.hc2[1:]
            nxt = self.layers[runs[r + 1]] if r + 1 < len(runs) else None
            h, _ = hyper_ops.hyper_step(xs, y, close, (nxt.hc1[0], nxt.norm1) if nxt is not None else None, eps, dt)
        return xs

    def compute_logits(self, rows: torch.Tensor) -> torch.Tensor:
        """fp32 logits of stream rows [n, S, W]: the streams' sum, the final norm, the head, the cap."""
        act, _ = hyper_ops.hyper_step(rows.contiguous(), None, None, (self.sum_in, self.final_norm), self.cfg.rms_eps,
                                      self.dtype)
        logits = gemm.linear(act, self.head).float()
        return tanh_cap(logits, self.cfg.logit_softcap)


def tanh_cap(x: torch.Tensor, cap: float) -> torch.Tensor:
    """cap * tanh(x / cap) in place on fp32 (cap <= 0: unchanged)."""
    if cap <= 0:
        return x
    if not x.is_cuda:
        return x.copy_(cap * torch.tanh(x / cap))
    assert x.dtype == torch.float32 and x.is_contiguous()
    native.call("pkm_tanh_cap", x.data_ptr(), x.numel(), float(cap), native.stream_ptr())
    return x
