"""Short causal filter over time on each channel, with the sequence's last inputs kept in its state
slot (csrc/mixers/short_conv.hip; PyTorch on CPU).

    y_t = sum_j taps[:, j] x_(t - K + 1 + j) (+ bias)      zeros before position 0; the last column
    y_t <- act(y_t)            none or SiLU                  of ``taps`` meets the current token
    y_t <- y_t + x_t           with ``residual``

``state`` [slots, K - 1, C] fp32 holds each sequence's last K - 1 inputs (oldest first).  A portion's
first tokens read it unless the portion starts at position 0 (a new sequence starts from zeros
whatever an earlier owner left); afterwards it holds the last K - 1 inputs including the portion's.
The sums run in fp32 in tap order, whether an input comes from the portion or from the slot.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import native

ACT_NONE, ACT_SILU = 0, 1


def causal_conv(x: torch.Tensor, taps: torch.Tensor, bias: Optional[torch.Tensor], state: Optional[torch.Tensor],
                cu_q: torch.Tensor, n_seqs: int, positions: torch.Tensor, slots: torch.Tensor, token_seq: torch.Tensor,
                act: int = ACT_NONE, residual: bool = False, out_dtype: Optional[torch.dtype] = None,
                in_bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x [T, C] (may be a column slice of a wider row), taps [C, K] fp32, bias [C] fp32 or None.
    ``in_bias`` [C] fp32 is added to every input row first (a projection's bias: the filter and the
    state see x + in_bias, the zeros before the sequence stay zeros).  Returns [T, C] in
    ``out_dtype`` (default: x's)."""
    T, C = x.shape
    K = taps.shape[1]
    out = torch.empty((T, C), dtype=out_dtype or x.dtype, device=x.device)
    assert taps.shape[0] == C and (K == 1 or (state is not None and state.shape[1:] == (K - 1, C)))
    if not x.is_cuda:
        f = x.float() if in_bias is None else x.float() + in_bias
        for s in range(n_seqs):
            a, b, slot = int(cu_q[s]), int(cu_q[s + 1]), int(slots[s])
            if b <= a:
                continue
            carry = K > 1 and slot >= 0 and int(positions[a]) > 0
            past = state[slot].clone() if carry else torch.zeros((K - 1, C))
            full = torch.cat([past, f[a:b]], 0)
            y = torch.zeros((b - a, C))
            for j in range(K):
                y = y + full[j:j + b - a] * taps[:, j]
            if bias is not None:
                y = y + bias
            if act == ACT_SILU:
                y = torch.nn.functional.silu(y)
            if residual:
                y = y + f[a:b]
            out[a:b] = y
            if K > 1 and slot >= 0:
                state[slot] = full[full.shape[0] - (K - 1):]
        return out
    assert x.stride(1) == 1 and taps.dtype == torch.float32 and taps.is_contiguous()
    for v in (bias, in_bias):
        assert v is None or (v.dtype == torch.float32 and v.numel() == C)
    assert state is None or (state.dtype == torch.float32 and state.is_contiguous())
    native.call("pkm_causal_conv", out.data_ptr(), native.dt_code(out.dtype), x.data_ptr(), native.dt_code(x.dtype),
                x.stride(0), native.ptr(in_bias), taps.data_ptr(), K, native.ptr(bias), native.ptr(state), cu_q.data_ptr(), positions.data_ptr(),
                slots.data_ptr(), token_seq.data_ptr(), n_seqs, T, C, int(act), int(residual), native.stream_ptr())
    return out
