"""Latent attention over a paged cache of per-token latents (csrc/mixers/latent_attention.hip;
PyTorch on CPU).  The cache of one layer is ``[blocks, block_size, kv_rank]`` in the model's dtype;
queries arrive already folded into the latent space (see the kernel file)."""
from __future__ import annotations

import torch

from . import native


def latent_norm_cache(dkv: torch.Tensor, w: torch.Tensor, eps: float, cache: torch.Tensor,
                      slot_mapping: torch.Tensor) -> None:
    """cache[slot[t]] = dkv[t] / sqrt(mean(dkv[t]^2) + eps) * w (fp32 maths); slot < 0: not written.
    ``dkv`` may be a column slice of a wider projection output."""
    T, R = dkv.shape
    if not dkv.is_cuda:
        v = dkv.float()
        c = v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps) * w
        ok = slot_mapping >= 0
        cache.view(-1, R)[slot_mapping[ok].long()] = c[ok].to(cache.dtype)
        return
    assert dkv.stride(1) == 1 and cache.is_contiguous() and cache.dtype == dkv.dtype and w.dtype == torch.float32
    native.call("pkm_latent_norm_cache", cache.data_ptr(), dkv.data_ptr(), dkv.stride(0), w.data_ptr(),
                slot_mapping.data_ptr(), T, R, float(eps), native.dt_code(dkv.dtype), native.stream_ptr())


def latent_attention(q: torch.Tensor, cache: torch.Tensor, block_tables: torch.Tensor, cu_q: torch.Tensor,
                     context_lens: torch.Tensor, n_seqs: int, scale: float) -> torch.Tensor:
    """q: [H, T, R] folded queries of the step's tokens (sequence s owns tokens cu_q[s]:cu_q[s+1],
    the LAST ones of its context_lens[s] cached tokens).  Returns o~ [H, T, R]: causal softmax
    attention of every (token, head) over the sequence's cached latents, used as keys and values."""
    H, T, R = q.shape
    out = torch.empty_like(q)
    bs = cache.shape[1]
    if not q.is_cuda:
        flat = cache.view(-1, R).float()
        for s in range(n_seqs):
            a, b, ctx = int(cu_q[s]), int(cu_q[s + 1]), int(context_lens[s])
            if b <= a:
                continue
            idx = torch.arange(ctx)
            c = flat[block_tables[s].long()[idx // bs] * bs + idx % bs]           # [ctx, R]
            sc = torch.einsum("htr,jr->htj", q[:, a:b].float(), c) * scale
            pos = ctx - (b - a) + torch.arange(b - a)
            sc = sc.masked_fill(idx[None, None, :] > pos[None, :, None], float("-inf"))
            out[:, a:b] = torch.einsum("htj,jr->htr", torch.softmax(sc, -1), c).to(q.dtype)
        return out
    assert q.stride(2) == 1 and cache.is_contiguous() and cache.dtype == q.dtype
    native.call("pkm_latent_attention", out.data_ptr(), out.stride(1), out.stride(0), q.data_ptr(), q.stride(1),
                q.stride(0), cache.data_ptr(), block_tables.data_ptr(), block_tables.stride(0), cu_q.data_ptr(),
                context_lens.data_ptr(), n_seqs, T, H, R, bs, float(scale), native.dt_code(q.dtype),
                native.stream_ptr())
    return out


def gate_merge(o: torch.Tensor, g: torch.Tensor) -> torch.Tensor:
    """o: [H, T, V] per-head outputs, g: [T, H*V] gate pre-activations (may be a column slice)
    -> [T, H*V] = heads side by side, times sigmoid(g)."""
    H, T, V = o.shape
    if not o.is_cuda:
        return (o.permute(1, 0, 2).reshape(T, H * V).float() * torch.sigmoid(g.float())).to(o.dtype)
    out = torch.empty((T, H * V), dtype=o.dtype, device=o.device)
    assert o.stride(2) == 1 and g.stride(1) == 1
    native.call("pkm_gate_merge", out.data_ptr(), o.data_ptr(), o.stride(1), o.stride(0), g.data_ptr(), g.stride(0),
                T, H, V, native.dt_code(o.dtype), native.stream_ptr())
    return out
