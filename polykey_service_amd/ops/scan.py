"""Selective scan: a diagonal state-space recurrence with input-dependent step sizes
(csrc/mixers/scan.hip; PyTorch on CPU).

    dt_c = softplus(d_c + dt_bias_c)                                   d the step-size pre-activation
    S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n ;  y_c = sum_n S[c, n] C_n + D_c x_c
    out_c = y_c * silu(z_c)

``state`` [slots, channels, N] fp32 per sequence; a portion's first token reads it unless it is
position 0, the slot then takes the state after the portion's last token.  Step sizes, decays and
the recurrence are fp32.
"""
from __future__ import annotations

import torch

from . import native


def selective_scan(x: torch.Tensor, d: torch.Tensor, dt_bias: torch.Tensor, A: torch.Tensor, bc: torch.Tensor,
                   skip: torch.Tensor, z: torch.Tensor, state: torch.Tensor, cu_q: torch.Tensor, n_seqs: int,
                   positions: torch.Tensor, slots: torch.Tensor) -> torch.Tensor:
    """x, d, z [T, C] (each may be a column slice), bc [T, 2N] (B then C; may be a column slice),
    dt_bias, skip [C] fp32, A [C, N] fp32 (negative).  Returns [T, C] in x's dtype."""
    T, C = x.shape
    N = A.shape[1]
    out = torch.empty((T, C), dtype=x.dtype, device=x.device)
    assert bc.shape == (T, 2 * N) and d.shape == (T, C) == z.shape and A.shape[0] == C
    if not x.is_cuda:
        xf, zf = x.float(), z.float()
        dt = torch.nn.functional.softplus(d.float() + dt_bias)
        B, Cm = bc.float()[:, :N], bc.float()[:, N:]
        y = torch.zeros((T, C))
        for s in range(n_seqs):
            a, b, slot = int(cu_q[s]), int(cu_q[s + 1]), int(slots[s])
            if b <= a:
                continue
            S = state[slot].clone() if (slot >= 0 and int(positions[a]) > 0) else torch.zeros((C, N))
            for t in range(a, b):
                S = torch.exp(dt[t][:, None] * A) * S + (dt[t] * xf[t])[:, None] * B[t][None, :]
                y[t] = S @ Cm[t] + skip * xf[t]
            if slot >= 0:
                state[slot] = S
        out.copy_(y * torch.nn.functional.silu(zf))
        return out
    for t in (x, d, z, bc):
        assert t.stride(1) == 1 and t.dtype == x.dtype
    assert state.dtype == torch.float32 and state.is_contiguous() and state.shape[1:] == (C, N)
    assert A.dtype == torch.float32 and A.is_contiguous() and dt_bias.dtype == torch.float32 and skip.dtype == torch.float32
    native.call("pkm_selective_scan", out.data_ptr(), x.data_ptr(), x.stride(0), d.data_ptr(), d.stride(0),
                dt_bias.data_ptr(), A.data_ptr(), bc.data_ptr(), bc.stride(0), skip.data_ptr(), z.data_ptr(), z.stride(0),
                state.data_ptr(), cu_q.data_ptr(), positions.data_ptr(), slots.data_ptr(), n_seqs, T, C, N,
                native.dt_code(x.dtype), native.stream_ptr())
    return out
