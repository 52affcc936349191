"""Latent attention over a paged cache of per-token latents (csrc/mixers/latent_attention.hip;
PyTorch on CPU).  The cache of one layer is ``[blocks, block_size, kv_rank]`` in the model's dtype;
queries arrive already folded into the latent space (see the kernel file)."""
from __future__ import annotations

from typing import Optional

import torch

from . import native


def mfma_latent(R: int, dtype: torch.dtype, device, block_size: int) -> bool:
    """Whether the matrix-core kernels serve this cache: bf16 on the GPU, pages of whole 32-key
    tiles and a latent size they are built for.  Such a cache keeps a second, latent-major copy
    (:func:`alloc_latent_major`) that decoding and prompt tiles read without transposing."""
    return (torch.device(device).type == "cuda" and dtype == torch.bfloat16 and block_size % 32 == 0
            and bool(native.mixers().pkm_latent_mfma_rank(R)))


def alloc_latent_major(num_blocks: int, block_size: int, R: int, device) -> torch.Tensor:
    """[blocks, block_size / 32, R, 32]: per 32-key tile, latent coordinate by key slot."""
    return torch.zeros((num_blocks, block_size // 32, R, 32), dtype=torch.bfloat16, device=device)


def decode_runs(capacity: int) -> tuple:
    """(keys per run, runs) of the decode kernel for caches of up to ``capacity`` tokens per
    sequence: at most 64 runs, each a multiple of 32 keys and at least 64, runs a multiple of 4."""
    part = max(64, -(-capacity // 64 // 32) * 32)
    n = -(-capacity // part)
    return part, -(-n // 4) * 4


def latent_norm_cache(dkv: torch.Tensor, w: torch.Tensor, eps: float, cache: torch.Tensor,
                      slot_mapping: torch.Tensor, cache_t: Optional[torch.Tensor] = None) -> None:
    """cache[slot[t]] = dkv[t] / sqrt(mean(dkv[t]^2) + eps) * w (fp32 maths); slot < 0: not written.
    ``dkv`` may be a column slice of a wider projection output.  ``cache_t``: the latent-major
    copy, written with it."""
    T, R = dkv.shape
    if not dkv.is_cuda:
        v = dkv.float()
        c = v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps) * w
        ok = slot_mapping >= 0
        cache.view(-1, R)[slot_mapping[ok].long()] = c[ok].to(cache.dtype)
        return
    assert dkv.stride(1) == 1 and cache.is_contiguous() and cache.dtype == dkv.dtype and w.dtype == torch.float32
    native.call("pkm_latent_norm_cache", cache.data_ptr(), native.ptr(cache_t), cache.shape[1], dkv.data_ptr(),
                dkv.stride(0), w.data_ptr(), slot_mapping.data_ptr(), T, R, float(eps), native.dt_code(dkv.dtype),
                native.stream_ptr())


def latent_attention(q: torch.Tensor, cache: torch.Tensor, block_tables: torch.Tensor, cu_q: torch.Tensor,
                     context_lens: torch.Tensor, n_seqs: int, scale: float, cache_t: Optional[torch.Tensor] = None,
                     num_decode: int = 0) -> torch.Tensor:
    """q: [H, T, R] folded queries of the step's tokens (sequence s owns tokens cu_q[s]:cu_q[s+1],
    the LAST ones of its context_lens[s] cached tokens).  Returns o~ [H, T, R]: causal softmax
    attention of every (token, head) over the sequence's cached latents, used as keys and values.

    With the latent-major copy ``cache_t`` the first ``num_decode`` sequences (one token each) take
    the decode kernel (runs over the context, merged), the rest the prompt kernel."""
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
    nd = min(num_decode, n_seqs) if cache_t is not None else 0
    st = native.stream_ptr()
    if nd:
        part, runs = decode_runs(block_tables.shape[1] * bs)
        ws_o = torch.empty((nd, runs, H, R), dtype=torch.float32, device=q.device)
        ws_ml = torch.empty((nd, runs, H, 2), dtype=torch.float32, device=q.device)
        native.call("pkm_latent_decode", out.data_ptr(), out.stride(1), out.stride(0), q.data_ptr(), q.stride(1),
                    q.stride(0), cache.data_ptr(), cache_t.data_ptr(), block_tables.data_ptr(), block_tables.stride(0),
                    cu_q.data_ptr(), context_lens.data_ptr(), nd, H, R, bs, float(scale), ws_o.data_ptr(),
                    ws_ml.data_ptr(), part, runs, st)
    if n_seqs > nd:
        native.call("pkm_latent_attention", out.data_ptr(), out.stride(1), out.stride(0), q.data_ptr(), q.stride(1),
                    q.stride(0), cache.data_ptr(), native.ptr(cache_t), block_tables[nd:].data_ptr(),
                    block_tables.stride(0), cu_q[nd:].data_ptr(), context_lens[nd:].data_ptr(), n_seqs - nd, T - nd, H,
                    R, bs, float(scale), native.dt_code(q.dtype), st)
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
