"""Lightning attention: linear attention with one constant decay per head and an fp32 state per
(sequence, head) carried from step to step (csrc/mixers/lightning.hip; PyTorch on CPU).

    S_t = decay_h * S_{t-1} + k_t v_t^T        o_t = S_t^T q_t        q, k, v = silu(projections)

The state of one layer run is ``[slots, H, D, V]`` fp32; a sequence's slot is read by the first
token of its portion (zeros at position 0, whatever an earlier owner left there) and takes the
state after the portion's last token.
"""
from __future__ import annotations

import torch

from . import native


def lightning_attention(qkv: torch.Tensor, state: torch.Tensor, decay: torch.Tensor, cu_q: torch.Tensor,
                        n_seqs: int, positions: torch.Tensor, slots: torch.Tensor, H: int, D: int, V: int,
                        num_decode: int = 0) -> torch.Tensor:
    """qkv [T, H*D | H*D | H*V] pre-activation projections (may be a column slice), heads side by
    side.  Returns o [T, H * V] fp32.  Sequences without a slot (slot < 0) start from zeros and
    leave nothing.  The first ``num_decode`` sequences hold one token each."""
    T = qkv.shape[0]
    out = torch.empty((T, H * V), dtype=torch.float32, device=qkv.device)
    if not qkv.is_cuda:
        f = torch.nn.functional.silu(qkv.float())
        q, k, v = f[:, :H * D].view(T, H, D), f[:, H * D:2 * H * D].view(T, H, D), f[:, 2 * H * D:].view(T, H, V)
        o3 = out.view(T, H, V)
        for s in range(n_seqs):
            a, b, slot = int(cu_q[s]), int(cu_q[s + 1]), int(slots[s])
            if b <= a:
                continue
            S = state[slot].clone() if (slot >= 0 and int(positions[a]) > 0) else torch.zeros((H, D, V))
            for t in range(a, b):
                S = decay[:, None, None] * S + k[t, :, :, None] * v[t, :, None, :]
                o3[t] = torch.einsum("hdv,hd->hv", S, q[t])
            if slot >= 0:
                state[slot] = S
        return out
    assert qkv.stride(1) == 1 and state.is_contiguous() and state.dtype == torch.float32 and decay.dtype == torch.float32
    assert state.shape[1:] == (H, D, V) and qkv.shape[1] == H * (2 * D + V)
    native.call("pkm_lightning_attention", out.data_ptr(), qkv.data_ptr(), qkv.stride(0), state.data_ptr(),
                decay.data_ptr(), cu_q.data_ptr(), positions.data_ptr(), slots.data_ptr(), n_seqs, T, H, D, V,
                int(num_decode), native.dt_code(qkv.dtype), native.stream_ptr())
    return out


def gated_rms_norm(o: torch.Tensor, w: torch.Tensor, g: torch.Tensor, eps: float, dtype: torch.dtype) -> torch.Tensor:
    """o [T, N] fp32 -> o / sqrt(mean(o^2) + eps) * w * sigmoid(g) in ``dtype``; g [T, N] may be a
    column slice of a wider projection output."""
    T, N = o.shape
    out = torch.empty((T, N), dtype=dtype, device=o.device)
    if not o.is_cuda:
        z = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps) * w
        out.copy_(z * torch.sigmoid(g.float()))
        return out
    assert o.dtype == torch.float32 and o.is_contiguous() and w.dtype == torch.float32 and g.stride(1) == 1
    native.call("pkm_gated_rms_norm", out.data_ptr(), o.data_ptr(), w.data_ptr(), g.data_ptr(), g.stride(0), T, N,
                float(eps), native.dt_code(g.dtype), native.dt_code(dtype), native.stream_ptr())
    return out
