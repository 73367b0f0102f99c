"""Gated delta rule with a short causal filter in front (csrc/mixers/delta.hip; PyTorch on CPU).

    q, k, v = silu(filter(projections))          per channel, over time, ``taps`` wide
    q <- q / sqrt(sum q^2 + 1e-6) / sqrt(D),  k <- k / sqrt(sum k^2 + 1e-6)      per head
    beta = sigmoid(b)        gate = exp(-exp(A_log_h) * softplus(a + dt_bias_h))
    S <- gate S ;  u = beta (v - S^T k) ;  S <- S + k u^T ;  o = S^T q           S [D, V] fp32 per head

Per layer run a sequence keeps, in its state slot, S of every head and the last ``taps - 1``
projection rows of the filter.  A portion's first token reads the slot unless it is position 0 (a
new sequence starts from zeros whatever an earlier owner left); the slot then takes the state
after the portion's last token.  Everything after the projections is fp32.
"""
from __future__ import annotations

import torch

from . import native


def conv_unit(proj: torch.Tensor, taps_w: torch.Tensor, conv_state: torch.Tensor, cu_q: torch.Tensor, n_seqs: int,
              positions: torch.Tensor, slots: torch.Tensor, token_seq: torch.Tensor, G: int, D: int, H: int,
              V: int) -> torch.Tensor:
    """proj [T, G*D | G*D | H*V] (may be a column slice): causal filter per channel (``taps_w``
    [C, taps] fp32, last column = the current token), SiLU, then q and k heads set to unit length
    (q also divided by sqrt(D)).  ``conv_state`` [slots, taps - 1, C] fp32 holds each sequence's
    last inputs (oldest first) and is brought up to date.  Returns fp32 [T, C]."""
    T = proj.shape[0]
    C, K = taps_w.shape
    out = torch.empty((T, C), dtype=torch.float32, device=proj.device)
    assert C == 2 * G * D + H * V and proj.shape[1] == C
    if not proj.is_cuda:
        x = proj.float()
        for s in range(n_seqs):
            a, b, slot = int(cu_q[s]), int(cu_q[s + 1]), int(slots[s])
            if b <= a:
                continue
            carry = slot >= 0 and int(positions[a]) > 0 and K > 1
            past = conv_state[slot].clone() if carry else torch.zeros((K - 1, C))
            full = torch.cat([past, x[a:b]], 0)                       # [K - 1 + n, C]
            y = torch.zeros((b - a, C))
            for j in range(K):
                y += full[j:j + b - a] * taps_w[:, j]
            out[a:b] = torch.nn.functional.silu(y)
            if slot >= 0 and K > 1:
                conv_state[slot] = full[full.shape[0] - (K - 1):]
        qk = out[:, :2 * G * D].view(T, 2 * G, D)
        qk = qk / torch.sqrt((qk * qk).sum(-1, keepdim=True) + 1e-6)
        qk[:, :G] *= D ** -0.5
        out[:, :2 * G * D] = qk.reshape(T, 2 * G * D)
        return out
    assert proj.stride(1) == 1 and taps_w.dtype == torch.float32 and taps_w.is_contiguous()
    assert conv_state.dtype == torch.float32 and conv_state.is_contiguous() and conv_state.shape[1:] == (max(K - 1, 1), C)
    native.call("pkm_conv_unit", out.data_ptr(), proj.data_ptr(), proj.stride(0), taps_w.data_ptr(), K,
                conv_state.data_ptr(), cu_q.data_ptr(), positions.data_ptr(), slots.data_ptr(), token_seq.data_ptr(),
                n_seqs, T, G, D, H, V, native.dt_code(proj.dtype), native.stream_ptr())
    return out


def delta_rule(qkv: torch.Tensor, ab: torch.Tensor, a_log: torch.Tensor, dt_bias: torch.Tensor, state: torch.Tensor,
               cu_q: torch.Tensor, n_seqs: int, positions: torch.Tensor, slots: torch.Tensor, G: int, D: int, H: int,
               V: int) -> torch.Tensor:
    """qkv fp32 [T, G*D | G*D | H*V] from :func:`conv_unit`; ``ab`` [T, H | H] the decay and beta
    pre-activations (may be a column slice: a first, then b); ``state`` [slots, H, D, V] fp32.
    Head h reads q / k head h // (H / G).  Returns o [T, H, V] fp32."""
    T = qkv.shape[0]
    out = torch.empty((T, H, V), dtype=torch.float32, device=qkv.device)
    if not qkv.is_cuda:
        q, k = qkv[:, :G * D].view(T, G, D), qkv[:, G * D:2 * G * D].view(T, G, D)
        v = qkv[:, 2 * G * D:].view(T, H, V)
        f = ab.float()
        gate = torch.exp(-torch.exp(a_log) * torch.nn.functional.softplus(f[:, :H] + dt_bias))
        beta = torch.sigmoid(f[:, H:])
        r = H // G
        for s in range(n_seqs):
            a, b, slot = int(cu_q[s]), int(cu_q[s + 1]), int(slots[s])
            if b <= a:
                continue
            S = state[slot].clone() if (slot >= 0 and int(positions[a]) > 0) else torch.zeros((H, D, V))
            for t in range(a, b):
                kk, qq = k[t].repeat_interleave(r, 0), q[t].repeat_interleave(r, 0)      # [H, D]
                S = gate[t, :, None, None] * S
                u = beta[t, :, None] * (v[t] - torch.einsum("hdv,hd->hv", S, kk))
                S = S + kk[:, :, None] * u[:, None, :]
                out[t] = torch.einsum("hdv,hd->hv", S, qq)
            if slot >= 0:
                state[slot] = S
        return out
    assert qkv.dtype == torch.float32 and qkv.is_contiguous() and ab.stride(1) == 1 and ab.shape[1] == 2 * H
    assert state.dtype == torch.float32 and state.is_contiguous() and state.shape[1:] == (H, D, V)
    assert a_log.dtype == torch.float32 and dt_bias.dtype == torch.float32
    native.call("pkm_delta_rule", out.data_ptr(), qkv.data_ptr(), ab.data_ptr(), ab.stride(0), native.dt_code(ab.dtype),
                a_log.data_ptr(), dt_bias.data_ptr(), state.data_ptr(), cu_q.data_ptr(), positions.data_ptr(),
                slots.data_ptr(), n_seqs, T, G, D, H, V, native.stream_ptr())
    return out
