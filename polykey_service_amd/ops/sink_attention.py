"""Grouped-query attention with rotated unit-RMS queries / keys, position-rotated values, capped
scores and a softmax sink, over a paged cache (csrc/mixers/sink_attention.hip; PyTorch on CPU).

Cache of one layer run: keys ``[blocks, G, block_size, D]`` (rotated, unit RMS) and values
``[blocks, G, V, block_size]`` (rotated by their own position, transposed per page), both in the
model's dtype.  Rotations read fp32 (cos, sin) tables built in double precision on the host.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch

from . import gemm, native


def pair_frequencies(dims: int, base: float, scaling: Optional[tuple] = None) -> Tuple[torch.Tensor, float]:
    """Angle per position of pair i = 0..dims/2-1 (float64) and the factor on cos / sin.  With
    ``scaling`` = (factor, original, fast, slow): pairs turning fewer than ``slow`` times over
    ``original`` positions are slowed by ``factor``, those turning more than ``fast`` times are kept,
    linear in the pair index between (YaRN)."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = torch.tensor(base, dtype=torch.float64) ** (-2.0 * i / dims)
    if scaling is None:
        return f, 1.0
    factor, orig, fast, slow = scaling
    at = lambda turns: dims * math.log(orig / (2 * math.pi * turns)) / (2 * math.log(base))
    lo, hi = max(math.floor(at(fast)), 0), min(math.ceil(at(slow)), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return f / factor * ramp + f * (1 - ramp), 0.1 * math.log(factor) + 1.0


def rotation_table(max_pos: int, freqs: torch.Tensor, mag: float, device) -> torch.Tensor:
    """[max_pos, pairs, 2] fp32: (cos, sin)(p * freqs[i]) * mag, angles in double precision."""
    ang = torch.arange(max_pos, dtype=torch.float64)[:, None] * freqs[None, :]
    return (torch.stack([torch.cos(ang), torch.sin(ang)], -1) * mag).float().to(device).contiguous()


def _turn(x: torch.Tensor, cs: torch.Tensor) -> torch.Tensor:
    """x [n, h, d] fp32, cs [n, pairs, 2]: pairs (2i, 2i+1) of the first 2 * pairs coordinates turn."""
    n2 = cs.shape[1]
    c, s = cs[:, None, :, 0], cs[:, None, :, 1]
    out = x.clone()
    a, b = x[..., 0:2 * n2:2], x[..., 1:2 * n2:2]
    out[..., 0:2 * n2:2] = a * c - b * s
    out[..., 1:2 * n2:2] = b * c + a * s
    return out


def rope_norm_cache(qkv: torch.Tensor, positions: torch.Tensor, slot_mapping: torch.Tensor,
                    qk_table: Optional[torch.Tensor], v_table: Optional[torch.Tensor], k_cache: torch.Tensor,
                    v_cache: torch.Tensor, H: int, G: int, D: int, V: int, eps: float) -> torch.Tensor:
    """qkv [T, H*D + G*D + G*V] (may be a column slice, or the decode GEMM's unreduced split-K
    slabs ``gemm.Partial``): q and k are rotated (table rows of the tokens' positions; None: no
    rotation) and divided by their RMS over D per head, v is rotated over V; k and v go to the paged
    cache (slot < 0: not written).  Returns q [T, H, D] in the cache's dtype."""
    nslab = 1
    if isinstance(qkv, gemm.Partial):
        nslab, qkv = qkv.S, qkv.view()[0]
    T = qkv.shape[0]
    q = torch.empty((T, H, D), dtype=k_cache.dtype, device=qkv.device)
    bs = k_cache.shape[2]
    if not qkv.is_cuda:
        f = qkv.float()
        qq, kk, vv = f[:, :H * D].view(T, H, D), f[:, H * D:(H + G) * D].view(T, G, D), f[:, (H + G) * D:].view(T, G, V)
        if qk_table is not None:
            cs = qk_table[positions.long()]
            qq, kk = _turn(qq, cs), _turn(kk, cs)
        if v_table is not None:
            vv = _turn(vv, v_table[positions.long()])
        unit = lambda t: t / torch.sqrt((t * t).mean(-1, keepdim=True) + eps)
        q.copy_(unit(qq))
        kk = unit(kk)
        ok = slot_mapping >= 0
        sl = slot_mapping[ok].long()
        k_cache[sl // bs, :, sl % bs, :] = kk[ok].to(k_cache.dtype)
        v_cache[sl // bs, :, :, sl % bs] = vv[ok].to(v_cache.dtype)
        return q
    assert qkv.stride(1) == 1 and positions.dtype == torch.int32 and slot_mapping.dtype == torch.int32
    assert k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.dtype == v_cache.dtype
    assert (qkv.dtype == k_cache.dtype and nslab == 1) or (qkv.dtype == torch.float32 and nslab > 1)
    assert qk_table is None or (qk_table.dtype == torch.float32 and 2 * qk_table.shape[1] <= D)
    assert v_table is None or (v_table.dtype == torch.float32 and 2 * v_table.shape[1] == V)
    native.call("pkm_rope_norm_cache", q.data_ptr(), qkv.data_ptr(), qkv.stride(0), nslab, positions.data_ptr(),
                slot_mapping.data_ptr(), native.ptr(qk_table), qk_table.shape[1] if qk_table is not None else 0,
                native.ptr(v_table), min(t.shape[0] for t in (qk_table, v_table) if t is not None) if (qk_table is not None or v_table is not None) else 0,
                k_cache.data_ptr(), v_cache.data_ptr(), T, H, G, D, V, bs, float(eps), native.dt_code(k_cache.dtype),
                native.stream_ptr())
    return q


def sink_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables: torch.Tensor,
                   cu_q: torch.Tensor, context_lens: torch.Tensor, n_seqs: int, positions: torch.Tensor,
                   head_scale: torch.Tensor, softcap: float, sink: float, v_table: Optional[torch.Tensor],
                   num_decode: int = 0) -> torch.Tensor:
    """q [T, H, D]; sequence s owns tokens cu_q[s]:cu_q[s+1], the LAST ones of its context_lens[s]
    cached tokens.  score = q . k * head_scale[h], capped by softcap * tanh(score / softcap) when
    softcap > 0; weights exp(score) / (sink + sum_j exp(score_j)) over the keys up to the token's own;
    the head's value sum is turned back by the token's position (``v_table`` rows; None: not).
    The first ``num_decode`` sequences hold one token each (the decode kernel splits their keys).
    Returns [T, H * V] in q's dtype."""
    T, H, D = q.shape
    G, V, bs = k_cache.shape[1], v_cache.shape[2], k_cache.shape[2]
    out = torch.empty((T, H * V), dtype=q.dtype, device=q.device)
    if not q.is_cuda:
        o3 = out.view(T, H, V)
        for s in range(n_seqs):
            a, b, ctx = int(cu_q[s]), int(cu_q[s + 1]), int(context_lens[s])
            if b <= a:
                continue
            idx = torch.arange(ctx)
            blk = block_tables[s].long()[idx // bs]
            k = k_cache[blk, :, idx % bs, :].float().repeat_interleave(H // G, 1)     # [ctx, H, D]
            v = v_cache[blk, :, :, idx % bs].float().repeat_interleave(H // G, 1)     # [ctx, H, V]
            sc = torch.einsum("thd,jhd->htj", q[a:b].float(), k) * head_scale[:, None, None]
            if softcap > 0:
                sc = softcap * torch.tanh(sc / softcap)
            pos = ctx - (b - a) + torch.arange(b - a)
            seen = idx[None, None, :] <= pos[None, :, None]
            m = sc.masked_fill(~seen, float("-inf")).amax(-1, keepdim=True)
            if sink > 0:
                m = m.clamp(min=0.0)
            e = torch.where(seen, torch.exp(sc - m), torch.zeros(()))
            p = e / (sink * torch.exp(-m) + e.sum(-1, keepdim=True))
            o = torch.einsum("htj,jhv->thv", p, v)
            if v_table is not None:
                cs = v_table[positions[a:b].long()].clone()
                cs[..., 1] = -cs[..., 1]
                o = _turn(o, cs)
            o3[a:b] = o.to(q.dtype)
        return out
    assert q.is_contiguous() and k_cache.is_contiguous() and v_cache.is_contiguous() and H % G == 0
    assert head_scale.dtype == torch.float32 and head_scale.numel() == H and block_tables.stride(1) == 1
    nd = min(num_decode, n_seqs)
    ws_o = ws_ml = None
    part = n_parts = 0
    if nd:
        capacity = block_tables.shape[1] * bs
        part = native.mixers().pkm_sink_decode_part(capacity, D, V, bs, native.dt_code(q.dtype))
        n_parts = -(-capacity // part) if part > 0 else 0
        if n_parts > 1:
            ws_o = torch.empty((nd, n_parts, H, V), dtype=torch.float32, device=q.device)
            ws_ml = torch.empty((nd, n_parts, H, 2), dtype=torch.float32, device=q.device)
    native.call("pkm_sink_attention", out.data_ptr(), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                block_tables.data_ptr(), block_tables.stride(0), cu_q.data_ptr(), context_lens.data_ptr(),
                positions.data_ptr(), head_scale.data_ptr(), native.ptr(v_table),
                v_table.shape[0] if v_table is not None else 0, n_seqs, T, H, G, D, V, bs, float(softcap), float(sink),
                nd, native.ptr(ws_o), native.ptr(ws_ml), part, n_parts, native.dt_code(q.dtype), native.stream_ptr())
    return out
