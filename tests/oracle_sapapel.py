"""Plain, slow fp32 model of the Sapapel design, written from its equations: one function per
mechanism, whole sequences at a time, no cache, no batching.  The tests compare the framework
with it; it shares no code with the package.

Notation: a sequence is ``x[t, :]`` for t = 0..n-1, ``W`` are [out, in] matrices applied as
``W @ v``.  ``cfg`` is the parsed config.json, ``w`` a dict name -> fp32 tensor.
"""
from __future__ import annotations

import math
from typing import Dict, List

import torch


def gain_rms_norm(x: torch.Tensor, g: torch.Tensor, eps: float) -> torch.Tensor:
    """y = x / sqrt(mean(x^2) + eps) * g; g is one number or one per coordinate."""
    ms = (x * x).mean(-1, keepdim=True)
    return x / torch.sqrt(ms + eps) * g


def token_shift(h: torch.Tensor, mu: torch.Tensor) -> torch.Tensor:
    """h_t <- h_t + (h_{t-1} - h_t) * mu with h_{-1} = 0; the h on the right are the unshifted ones."""
    prev = torch.zeros_like(h)
    prev[1:] = h[:-1]
    return h + (prev - h) * mu


def latent_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    """Causal softmax attention whose keys and values are both expanded from one shared low-rank
    latent per token, with a sigmoid output gate read from the same input."""
    H, D, V, R = m["heads"], m["dim"], m["vdim"], m["kv_rank"]
    n = h.shape[0]
    q = (h @ w[p + "q"].T).view(n, H, D)
    c = gain_rms_norm(h @ w[p + "dkv"].T, w[p + "dkv.norm"], eps)
    assert c.shape[1] == R
    k = (c @ w[p + "uk"].T).view(n, H, D)
    v = (c @ w[p + "uv"].T).view(n, H, V)
    out = torch.zeros(n, H, V)
    for i in range(n):
        for a in range(H):
            s = (k[: i + 1, a] @ q[i, a]) * m["scale"]
            pr = torch.softmax(s, 0)
            out[i, a] = pr @ v[: i + 1, a]
    out = out.reshape(n, H * V) * torch.sigmoid(h @ w[p + "g"].T)
    return out @ w[p + "o"].T


def sigmoid_moe(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, f: dict) -> torch.Tensor:
    """Each token goes to the ``top`` experts with the largest sigmoid(router) scores; an expert
    sees the token scaled by its score, and the experts' outputs are added as they are."""
    E, top = f["router"]["experts"], f["router"]["top"]
    s = torch.sigmoid(h @ w[p + "router"].T)
    out = torch.zeros(h.shape[0], w[p + "e0.down"].shape[0])
    for t in range(h.shape[0]):
        order = sorted(range(E), key=lambda e: (-float(s[t, e]), e))[:top]
        for e in order:
            z = h[t] * s[t, e]
            g = w[p + f"e{e}.gate"] @ z
            u = w[p + f"e{e}.up"] @ z
            out[t] += w[p + f"e{e}.down"] @ (g * torch.sigmoid(g) * u)
    return out


def feed_forward(h, w, p, f):
    if f["kind"] == "moe":
        return sigmoid_moe(h, w, p, f)
    raise ValueError(f["kind"])


def layer(x: torch.Tensor, w: Dict[str, torch.Tensor], i: int, cfg: dict) -> torch.Tensor:
    """Post-norm sublayers on an alpha-scaled skip path: the sum is normalised, not the input."""
    lc, eps, alpha = cfg["layers"][i], cfg["norm"]["eps"], cfg["postln_alpha"]
    p = f"l{i}."
    h = token_shift(x, w[p + "shift"]) if p + "shift" in w else x
    if lc["type"] != "latent_attention":
        raise ValueError(lc["type"])
    x = gain_rms_norm(alpha * x + latent_attention(h, w, p + "mix.", lc["mixer"], eps), w[p + "norm1"], eps)
    if lc.get("mlp") is not None:
        x = gain_rms_norm(alpha * x + feed_forward(x, w, p + "mlp.", lc["mlp"]), w[p + "norm2"], eps)
    elif p + "norm2" in w:  # no feed-forward: the second sum is alpha x alone
        x = gain_rms_norm(alpha * x, w[p + "norm2"], eps)
    return x


def forward(tokens: List[int], w: Dict[str, torch.Tensor], cfg: dict, streams: list = None) -> torch.Tensor:
    """Logits [n, vocab] of one sequence.  ``streams`` collects what each layer hands on."""
    x = w["embed"][torch.tensor(tokens)]
    hist = [x]
    for i in range(len(cfg["layers"])):
        y = layer(x, w, i, cfg)
        hist.append(y)
        d = w.get(f"l{i}.dwa")
        x = sum(d[j] * hist[j] for j in range(i + 2)) if d is not None else y
        if streams is not None:
            streams.append(x)
    x = gain_rms_norm(x, w["final.norm"], cfg["norm"]["eps"])
    return x @ w["head"].T


def random_model(cfg: dict, seed: int = 0, std: float = 0.08) -> Dict[str, torch.Tensor]:
    """Random bf16-representable weights for ``cfg`` under the checkpoint's tensor names."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def r(*shape, s=std):
        return (torch.randn(*shape, generator=g) * s).bfloat16().float()

    def gain(*shape):  # near 1, and exact in bf16 like everything a checkpoint holds
        return (1 + torch.randn(*shape, generator=g) * 0.1).bfloat16().float()

    w = {"embed": r(cfg["vocab"], W, s=1.0), "final.norm": gain(1)[0], "head": r(cfg["vocab"], W)}
    for i, lc in enumerate(cfg["layers"]):
        p, m = f"l{i}.", lc["mixer"]
        H, D, V, R = m["heads"], m["dim"], m["vdim"], m["kv_rank"]
        w[p + "norm1"] = gain(1)[0]
        w[p + "shift"] = torch.rand(W, generator=g).bfloat16().float()
        w[p + "dwa"] = (torch.eye(i + 2)[i + 1] * 0.7 + r(i + 2, s=0.2)).bfloat16().float()
        w[p + "mix.q"] = r(H * D, W)
        w[p + "mix.dkv"] = r(R, W)
        w[p + "mix.dkv.norm"] = gain(R)
        w[p + "mix.uk"] = r(H * D, R, s=std * 2)
        w[p + "mix.uv"] = r(H * V, R, s=std * 2)
        w[p + "mix.g"] = r(H * V, W)
        w[p + "mix.o"] = r(W, H * V)
        f = lc.get("mlp")
        if f is not None:
            w[p + "norm2"] = gain(1)[0]
            w[p + "mlp.router"] = r(f["router"]["experts"], W, s=0.5)
            for e in range(f["router"]["experts"]):
                F = f["expert"]["ff"]
                w[p + f"mlp.e{e}.gate"] = r(F, W)
                w[p + f"mlp.e{e}.up"] = r(F, W)
                w[p + f"mlp.e{e}.down"] = r(W, F)
    return w


def make_config(vocab=96, width=48, layers=2, heads=3, dim=8, vdim=16, kv_rank=24, ff=40, experts=5, top=2,
                alpha=2.0, eps=1e-5, scale=None, mlp_none=()) -> dict:
    out = {"architecture": "Sapapel", "vocab": vocab, "width": width, "postln_alpha": alpha, "norm": {"eps": eps},
           "layers": []}
    for i in range(layers):
        mixer = {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": kv_rank,
                 "scale": scale if scale is not None else 1.0 / math.sqrt(dim)}
        mlp = None if i in mlp_none else {"kind": "moe", "expert": {"ff": ff},
                                          "router": {"experts": experts, "top": top}}
        out["layers"].append({"type": "latent_attention", "mixer": mixer, "mlp": mlp})
    return out
