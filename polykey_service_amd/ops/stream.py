"""fp32 residual-stream ops of post-norm layers (csrc/mixers/postnorm.hip; PyTorch on CPU).

The stream ``x`` is fp32 ``[T, W]`` for the step's tokens in batch order; activations handed to
the projections are in the model's dtype.  Sequence bookkeeping comes from the step metadata:
``token_seq[t]`` the batch index of token t's sequence, ``cu_q`` the sequences' token offsets,
``slots`` their state slots.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import gemm, native


def embed_rows(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[t] = table[ids[t]] as fp32."""
    T, W = ids.numel(), table.shape[1]
    if not table.is_cuda:
        out[:T] = table[ids.long()].float()
        return out
    assert out.dtype == torch.float32 and out.is_contiguous() and table.is_contiguous() and ids.dtype == torch.int32
    native.call("pkm_embed_rows", out.data_ptr(), table.data_ptr(), ids.data_ptr(), T, W, table.shape[0],
                native.dt_code(table.dtype), native.stream_ptr())
    return out


def token_shift(x: torch.Tensor, mu: torch.Tensor, state: torch.Tensor, token_seq: torch.Tensor, cu_q: torch.Tensor,
                positions: torch.Tensor, slots: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """h[t] = x[t] + (x[t-1] - x[t]) * mu.  The token before a portion's first one is the
    sequence's state row (``state[slots[s]]``), zeros at position 0."""
    T, W = x.shape
    out = torch.empty((T, W), dtype=dtype, device=x.device)
    if not x.is_cuda:
        prev = torch.zeros_like(x)
        prev[1:] = x[:-1]
        first = cu_q[token_seq.long()].long() == torch.arange(T)
        st_rows = state[slots[token_seq.long()].long().clamp(min=0)]
        st_rows = torch.where((positions > 0)[:, None], st_rows, torch.zeros(()))
        prev = torch.where(first[:, None], st_rows, prev)
        out.copy_(x + (prev - x) * mu)
        return out
    assert x.dtype == torch.float32 and x.is_contiguous() and mu.dtype == torch.float32 and state.is_contiguous()
    native.call("pkm_token_shift", out.data_ptr(), x.data_ptr(), mu.data_ptr(), state.data_ptr(), token_seq.data_ptr(),
                cu_q.data_ptr(), positions.data_ptr(), slots.data_ptr(), T, W, native.dt_code(dtype),
                native.stream_ptr())
    return out


def save_last_rows(x: torch.Tensor, state: torch.Tensor, cu_q: torch.Tensor, slots: torch.Tensor, n: int) -> None:
    """state[slots[s]] = x[last token of sequence s] for the step's n sequences (after token_shift
    has read the old rows)."""
    if not x.is_cuda:
        for s in range(n):
            if int(cu_q[s + 1]) > int(cu_q[s]) and int(slots[s]) >= 0:
                state[int(slots[s])] = x[int(cu_q[s + 1]) - 1]
        return
    native.call("pkm_save_last_rows", state.data_ptr(), x.data_ptr(), cu_q.data_ptr(), slots.data_ptr(), n, x.shape[1],
                native.stream_ptr())


def sum_gain_norm(x: torch.Tensor, y: Optional[torch.Tensor], alpha: float, gain: torch.Tensor, eps: float,
                  out: Optional[torch.Tensor] = None, act_dtype: Optional[torch.dtype] = None,
                  rows: Optional[torch.Tensor] = None, hist: Optional[torch.Tensor] = None, nh: int = 0,
                  coef: Optional[torch.Tensor] = None, gather: Optional[tuple] = None, save: Optional[tuple] = None):
    """z = (alpha x + y) / sqrt(mean((alpha x + y)^2) + eps) * gain (one number) in fp32.

    ``hist`` ([layers + 1, T_cap, W] fp32): z becomes entry ``nh - 1`` and the result is
    ``sum_j coef[j] hist[j]`` over the first ``nh`` entries.  ``rows``: only these rows of x.
    ``gather`` = (inv [T * top] int32, top): y is a table of expert output rows and token t's y is
    the plain sum of rows ``inv[t * top + j]`` (the MoE combine fused in; inv < 0: none).
    ``save`` = (state, token_seq, cu_q, slots): the last token of every sequence in the step leaves
    its x row in ``state[slots[s]]`` (the token-shift state, written after this step's shift read it).
    ``y`` may also be the decode GEMM's unreduced split-K slabs (``gemm.Partial``): their sum is y.
    Returns (fp32 result written to ``out`` or None, copy in ``act_dtype`` or None)."""
    W = x.shape[1]
    nslab = 1
    if isinstance(y, gemm.Partial):
        assert x.is_cuda and y.M == x.shape[0] and y.N == W and gather is None and rows is None
        nslab, y = y.S, y.view()[0]  # the first slab; the others follow at M * W elements each
    R = rows.numel() if rows is not None else x.shape[0]
    act = torch.empty((R, W), dtype=act_dtype, device=x.device) if act_dtype is not None else None
    if not x.is_cuda:
        xs = x if rows is None else x[rows.long()]
        v = alpha * xs
        if gather is not None:
            inv, top = gather
            idx = inv.long().view(-1, top)
            v = v + torch.where((idx >= 0)[..., None], y.float()[idx.clamp(min=0)], torch.zeros(())).sum(1)
        elif y is not None:
            v = v + (y if rows is None else y[rows.long()]).float()
        if save is not None:
            save_last_rows(x, save[0], save[2], save[3], save[2].numel() - 1)
        z = v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps) * gain
        if hist is not None:
            hist[nh - 1, :R] = z
            z = (coef[:nh, None, None] * hist[:nh, :R]).sum(0)
        if out is not None:
            out[:R] = z
        if act is not None:
            act.copy_(z)
        return out, act
    assert x.dtype == torch.float32 and x.is_contiguous() and gain.dtype == torch.float32
    assert y is None or (y.is_contiguous() and (gather is not None or nslab > 1 or y.shape == x.shape))
    assert (gather is None and save is None) or rows is None
    inv, top = gather if gather is not None else (None, 0)
    state, token_seq, cu_q, slots = save if save is not None else (None, None, None, None)
    assert hist is None or (hist.dtype == torch.float32 and hist.is_contiguous() and rows is None and nh <= hist.shape[0]
                            and R <= hist.shape[1] and coef.dtype == torch.float32 and coef.numel() >= nh)
    dt = native.dt_code(act_dtype) if act_dtype is not None else 1
    native.call("pkm_sum_gain_norm", native.ptr(out), native.ptr(act), x.data_ptr(), native.ptr(y), native.ptr(rows),
                float(alpha), gain.data_ptr(), float(eps), R, W, native.ptr(hist),
                hist.stride(0) if hist is not None else 0, nh, native.ptr(coef), dt,
                native.dt_code(y.dtype) if y is not None else -1, nslab, native.ptr(inv), top, native.ptr(state),
                native.ptr(token_seq), native.ptr(cu_q), native.ptr(slots), native.stream_ptr())
    return out, act
