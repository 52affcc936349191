"""Plain, slow model of the Kivezen design, written from its equations: one function per
mechanism, one whole sequence at a time, no cache, no batching, double precision by default.
The tests compare the framework with it; it shares no code with the package.

Notation: a sequence is ``x[t, :]`` for t = 0..n-1 (positions count from 0), ``W`` are [out, in]
matrices applied as ``W @ v``.  ``cfg`` is the parsed config.json, ``w`` a dict name -> tensor.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

DT = torch.float64


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x: torch.Tensor, g: torch.Tensor, eps: float) -> torch.Tensor:
    return unit_rms(x, eps) * g


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


# ------------------------------------------------------------------ rotations
def rotary_frequencies(dims: int, base: float, scaling: Optional[dict]):
    """Per pair i: the angle per position, and the factor on cos / sin (1 without scaling)."""
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=DT)
    if not scaling:
        return f, 1.0
    factor, orig = float(scaling["factor"]), float(scaling["original"])
    at = lambda turns: dims * math.log(orig / (2 * math.pi * turns)) / (2 * math.log(base))
    lo = max(math.floor(at(float(scaling["fast"]))), 0)
    hi = min(math.ceil(at(float(scaling["slow"]))), dims - 1)
    out = torch.empty_like(f)
    for i in range(dims // 2):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out[i] = f[i] / factor * ramp + f[i] * (1 - ramp)
    return out, 0.1 * math.log(factor) + 1.0


def rotate_pairs(x: torch.Tensor, pos: torch.Tensor, freq: torch.Tensor, mag: float = 1.0) -> torch.Tensor:
    """x[..., 2i], x[..., 2i+1] of the first 2 * len(freq) coordinates turn by pos * freq[i]; the
    rest pass.  x: [n, heads, d], pos: [n] (may be negative: turning back)."""
    n2 = freq.numel()
    ang = pos.to(DT)[:, None] * freq[None, :]            # [n, n2]
    c, s = (torch.cos(ang) * mag)[:, None, :], (torch.sin(ang) * mag)[:, None, :]
    out = x.clone()
    a, b = x[..., 0:2 * n2:2], x[..., 1:2 * n2:2]
    out[..., 0:2 * n2:2] = a * c - b * s
    out[..., 1:2 * n2:2] = b * c + a * s
    return out


# --------------------------------------------------------------------- mixers
def attention(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    """Grouped-query causal attention: rotated and unit-normed queries / keys, values rotated by
    their own position and the head's sum turned back by the query's, a per-head temperature, a
    tanh cap on the scores, and a softmax whose denominator holds one extra exp(0)."""
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    n = h.shape[0]
    pos = torch.arange(n)
    q = (h @ w[p + "q"].T).view(n, H, D)
    k = (h @ w[p + "k"].T).view(n, G, D)
    v = (h @ w[p + "v"].T).view(n, G, V)
    rot = m.get("rot")
    if rot:
        f, mag = rotary_frequencies(int(rot["dims"]), float(rot["base"]), rot.get("scaling"))
        q, k = rotate_pairs(q, pos, f, mag), rotate_pairs(k, pos, f, mag)
        vf = torch.tensor([float(rot["base"]) ** (-2.0 * i / V) for i in range(V // 2)], dtype=DT)
        v = rotate_pairs(v, pos, vf)
    q, k = unit_rms(q, eps), unit_rms(k, eps)
    temp = w[p + "temp"] if p + "temp" in w else torch.ones(H, dtype=DT)
    cap = m.get("softcap")
    out = torch.zeros(n, H, V, dtype=DT)
    for a in range(H):
        g = a // (H // G)
        s = (q[:, a] @ k[:, g].T) * m["scale"] * temp[a]          # [i, j]
        if cap:
            s = cap * torch.tanh(s / cap)
        e = torch.exp(s) * torch.tril(torch.ones(n, n, dtype=DT))
        pr = e / (1.0 + e.sum(-1, keepdim=True))
        out[:, a] = pr @ v[:, g]
    if rot:
        out = rotate_pairs(out, -pos, vf)
    return out.reshape(n, H * V) @ w[p + "o"].T


def lightning(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    """Linear attention with one fixed decay per head: S_t = d S_{t-1} + k_t v_t^T, o_t = S_t^T q_t;
    the heads side by side are normed together, gated and projected."""
    H, D, V = m["heads"], m["dim"], m["vdim"]
    n = h.shape[0]
    q = silu(h @ w[p + "q"].T).view(n, H, D)
    k = silu(h @ w[p + "k"].T).view(n, H, D)
    v = silu(h @ w[p + "v"].T).view(n, H, V)
    out = torch.zeros(n, H, V, dtype=DT)
    for a in range(H):
        S = torch.zeros(D, V, dtype=DT)
        for t in range(n):
            S = float(m["decay"][a]) * S + torch.outer(k[t, a], v[t, a])
            out[t, a] = S.T @ q[t, a]
    o = rms_norm(out.reshape(n, H * V), w[p + "norm"], eps) * torch.sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


# -------------------------------------------------------------- feed-forwards
def dense_ff(h, w, p):
    return gelu_tanh(h @ w[p + "up"].T) @ w[p + "down"].T


def clamped_expert(h, w, p, limit: float):
    g = torch.clamp(h @ w[p + "gate"].T, max=limit)
    u = torch.clamp(h @ w[p + "up"].T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1)) @ w[p + "down"].T


def moe_ff(h, w, p, f):
    E, top = f["router"]["experts"], f["router"]["top"]
    z = h @ w[p + "router"].T
    out = torch.zeros(h.shape[0], w[p + "e0.down"].shape[0], dtype=DT)
    for t in range(h.shape[0]):
        chosen = sorted(range(E), key=lambda e: (-float(z[t, e]), e))[:top]
        wt = torch.softmax(z[t, chosen], 0)
        for j, e in enumerate(chosen):
            out[t] += wt[j] * clamped_expert(h[t:t + 1], w, p + f"e{e}.", float(f["expert"]["limit"]))[0]
    if f.get("shared"):
        sh = clamped_expert(h, w, p + "shared.", float(f["shared"]["limit"]))
        out = out + sh * torch.sigmoid(h @ w[p + "shared.sg"].T)
    return out


def feed_forward(h, w, p, f):
    if f["kind"] == "dense":
        return dense_ff(h, w, p)
    if f["kind"] == "moe":
        return moe_ff(h, w, p, f)
    raise ValueError(f["kind"])


def mixer(h, w, p, lc, eps):
    if lc["type"] == "attention":
        return attention(h, w, p, lc["mixer"], eps)
    if lc["type"] == "lightning":
        return lightning(h, w, p, lc["mixer"], eps)
    raise ValueError(lc["type"])


# --------------------------------------------------------------------- layers
def layer_plain(x, w, i, cfg):
    lc, eps, p = cfg["layers"][i], cfg["norm"]["eps"], f"l{i}."
    x = x + mixer(rms_norm(x, w[p + "norm1"], eps), w, p + "mix.", lc, eps)
    if lc.get("mlp") is not None:
        x = x + feed_forward(rms_norm(x, w[p + "norm2"], eps), w, p + "mlp.", lc["mlp"])
    return x


def layer_streams(xs, w, i, cfg):
    """xs: [streams, n, width].  Each sublayer reads one weighted sum of the streams and every
    stream becomes a mix of the old streams plus its own share of the sublayer's output."""
    lc, eps, p = cfg["layers"][i], cfg["norm"]["eps"], f"l{i}."
    subs = [("hc1.", "norm1", lambda u: mixer(u, w, p + "mix.", lc, eps))]
    if lc.get("mlp") is not None:
        subs.append(("hc2.", "norm2", lambda u: feed_forward(u, w, p + "mlp.", lc["mlp"])))
    for hc, norm, fn in subs:
        u = torch.einsum("s,snw->nw", w[p + hc + "in"], xs)
        y = fn(rms_norm(u, w[p + norm], eps))
        xs = torch.einsum("st,snw->tnw", w[p + hc + "mix"], xs) + w[p + hc + "out"][:, None, None] * y[None]
    return xs


def layer_runs(cfg) -> List[int]:
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return list(range(n))
    a, b, times = int(lp["start"]), int(lp["stop"]), int(lp["times"])
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def forward(cfg: dict, w: Dict[str, torch.Tensor], tokens, layers_out: Optional[list] = None) -> torch.Tensor:
    """Logits [n, vocab] of one sequence; ``layers_out`` collects the stream after every layer run."""
    w = {k: v.to(DT) for k, v in w.items()}
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    S = cfg.get("streams")
    if S:
        xs = x[None].repeat(int(S), 1, 1)
    for i in layer_runs(cfg):
        if S:
            xs = layer_streams(xs, w, i, cfg)
            x = xs.sum(0)
        else:
            x = layer_plain(x, w, i, cfg)
        if layers_out is not None:
            layers_out.append(x.clone())
    z = rms_norm(x, w["final.norm"], cfg["norm"]["eps"]) @ w["head"].T
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(z / cap) if cap else z


# ------------------------------------------------------------ test models
def make_config(vocab=64, width=32, pattern="LAa", heads=3, kv_heads=1, dim=8, vdim=12, rot_dims=None, ff=24,
                experts=5, top=2, expert_ff=10, limit=1.5, shared_ff=14, shared_limit=2.5, streams=2, loop=None,
                eps=1e-5, scale=None, softcap=20.0, logit_softcap=15.0, scaling=(3.0, 64, 8.0, 1.0), base=1000.0,
                lightning=None, no_mlp=()):
    """``pattern``: one letter per layer; A / a attention, L / l lightning; upper case with the
    mixture feed-forward, lower case with the dense one; layers listed in ``no_mlp`` have none.
    ``lightning``: (heads, dim, vdim) of the lightning mixers (default: the attention's sizes)."""
    layers = []
    lh, ld, lv = lightning or (heads, dim, vdim)
    for i, ch in enumerate(pattern):
        if ch in "Aa":
            rot = {"base": base, "dims": rot_dims if rot_dims is not None else dim}
            if scaling:
                rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
            m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "rot": rot,
                 "scale": scale if scale is not None else dim ** -0.5}
            if softcap:
                m["softcap"] = softcap
            kind = "attention"
        else:
            m = {"heads": lh, "dim": ld, "vdim": lv,
                 "decay": [math.exp(-1.0 / (1 + 3 * h)) if h + 1 < lh or lh == 1 else 0.999 for h in range(lh)]}
            kind = "lightning"
        if i in no_mlp:
            mlp = None
        elif ch.isupper():
            mlp = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": expert_ff, "limit": limit}}
            if shared_ff:
                mlp["shared"] = {"ff": shared_ff, "limit": shared_limit}
        else:
            mlp = {"kind": "dense", "ff": ff}
        layers.append({"type": kind, "mixer": m, "mlp": mlp})
    cfg = {"architecture": "Kivezen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if streams:
        cfg["streams"] = streams
    if loop:
        cfg["loop"] = dict(zip(("start", "stop", "times"), loop))
    if logit_softcap:
        cfg["logit_softcap"] = logit_softcap
    return cfg


def random_model(cfg: dict, seed: int = 0, std: float = 0.3) -> Dict[str, torch.Tensor]:
    """Random weights that bf16 holds exactly (a checkpoint round trip changes nothing)."""
    g = torch.Generator().manual_seed(seed)
    W, S = cfg["width"], cfg.get("streams", 0)
    r = lambda *shape, s=std: (torch.randn(*shape, generator=g) * s).bfloat16().float()
    w = {"embed": r(cfg["vocab"], W, s=1.0), "head": r(cfg["vocab"], W), "final.norm": 1 + r(W, s=0.1)}
    for i, l in enumerate(cfg["layers"]):
        p, m = f"l{i}.", l["mixer"]
        for q in ("1", "2") if l.get("mlp") is not None else ("1",):
            w[p + "norm" + q] = 1 + r(W, s=0.1)
            if S:
                w[p + f"hc{q}.in"] = (1.0 / S + r(S, s=0.2)).bfloat16().float()
                w[p + f"hc{q}.out"] = 1 + r(S, s=0.3)
                w[p + f"hc{q}.mix"] = (torch.eye(S) + r(S, S, s=0.2)).bfloat16().float()
        H, D, V = m["heads"], m["dim"], m["vdim"]
        if l["type"] == "attention":
            G = m["kv_heads"]
            w[p + "mix.q"], w[p + "mix.k"], w[p + "mix.v"] = r(H * D, W), r(G * D, W), r(G * V, W)
            w[p + "mix.temp"] = 1 + r(H, s=0.3)
        else:
            w[p + "mix.q"], w[p + "mix.k"], w[p + "mix.v"], w[p + "mix.g"] = r(H * D, W), r(H * D, W), r(H * V, W), r(H * V, W)
            w[p + "mix.norm"] = 1 + r(H * V, s=0.1)
        w[p + "mix.o"] = r(W, H * V)
        f = l.get("mlp")
        if f is None:
            continue
        if f["kind"] == "dense":
            w[p + "mlp.up"], w[p + "mlp.down"] = r(f["ff"], W), r(W, f["ff"])
            continue
        w[p + "mlp.router"] = r(f["router"]["experts"], W, s=1.0)
        names = [(f"e{e}", f["expert"]["ff"]) for e in range(f["router"]["experts"])]
        if f.get("shared"):
            names.append(("shared", f["shared"]["ff"]))
            w[p + "mlp.shared.sg"] = r(1, W)
        for n, ff in names:
            w[p + f"mlp.{n}.gate"], w[p + f"mlp.{n}.up"], w[p + f"mlp.{n}.down"] = r(ff, W, s=0.6), r(ff, W, s=0.6), r(W, ff)
    return {k: v.bfloat16().float() for k, v in w.items()}
