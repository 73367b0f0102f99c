"""Time mixing with per-channel data-dependent decays and a matrix state per head
(csrc/mixers/wkv.hip; PyTorch on CPU).

    mix_n[t] = h[t] + (h[t-1] - h[t]) * mu_n                 one mix per projection; h[-1] = 0
    w_t = exp(-exp(z_t + w0))                                 z_t the decay pre-activation, per key channel
    o_t = (S + diag(u) k_t v_t^T)^T r_t ;  S <- diag(w_t) S + k_t v_t^T         S [D, D] fp32 per head

A sequence keeps, in its state slot, the last input row h and S of every head.  A portion's first
token reads the slot unless it is position 0; the slot then takes the values after the portion's
last token.  Mixes, decays and the recurrence are fp32.
"""
from __future__ import annotations

import torch

from . import native


def shift_mix(h: torch.Tensor, mu: torch.Tensor, prev: torch.Tensor, token_seq: torch.Tensor, cu_q: torch.Tensor,
              n_seqs: int, positions: torch.Tensor, slots: torch.Tensor) -> torch.Tensor:
    """h [T, W], mu [n, W] fp32, prev [slots, W] fp32 (each sequence's last row) -> [n, T, W] in h's
    dtype; ``prev`` is brought up to date."""
    T, W = h.shape
    n = mu.shape[0]
    out = torch.empty((n, T, W), dtype=h.dtype, device=h.device)
    if not h.is_cuda:
        f = h.float()
        for s in range(n_seqs):
            a, b, slot = int(cu_q[s]), int(cu_q[s + 1]), int(slots[s])
            if b <= a:
                continue
            first = prev[slot].clone() if (slot >= 0 and int(positions[a]) > 0) else torch.zeros(W)
            before = torch.cat([first[None], f[a:b - 1]], 0)
            out[:, a:b] = f[None, a:b] + (before - f[a:b])[None] * mu[:, None, :]
            if slot >= 0:
                prev[slot] = f[b - 1]
        return out
    assert h.is_contiguous() and mu.dtype == torch.float32 and mu.is_contiguous()
    assert prev.dtype == torch.float32 and prev.is_contiguous() and prev.shape[1] == W
    native.call("pkm_shift_mix", out.data_ptr(), h.data_ptr(), mu.data_ptr(), n, prev.data_ptr(), token_seq.data_ptr(),
                cu_q.data_ptr(), positions.data_ptr(), slots.data_ptr(), n_seqs, T, W, native.dt_code(h.dtype),
                native.stream_ptr())
    return out


def tanh_(x: torch.Tensor) -> torch.Tensor:
    """tanh in place (fp32 maths)."""
    if not x.is_cuda:
        return x.copy_(torch.tanh(x.float()))
    assert x.is_contiguous()
    native.call("pkm_tanh", x.data_ptr(), x.numel(), native.dt_code(x.dtype), native.stream_ptr())
    return x


def wkv_recurrence(rkv: torch.Tensor, z: torch.Tensor, w0: torch.Tensor, u: torch.Tensor, state: torch.Tensor,
                   cu_q: torch.Tensor, n_seqs: int, positions: torch.Tensor, slots: torch.Tensor, H: int,
                   D: int) -> torch.Tensor:
    """rkv [>= 3, T, H * D] (r, k, v planes), z [T, H * D] decay pre-activations, w0 and u [H * D]
    fp32, state [slots, H, D, D] fp32 (key channel, value channel).  Returns o [T, H, D] fp32."""
    T = rkv.shape[1]
    out = torch.empty((T, H, D), dtype=torch.float32, device=rkv.device)
    assert rkv.shape[0] >= 3 and rkv.shape[2] == H * D and z.shape == (T, H * D)
    if not rkv.is_cuda:
        r, k, v = (rkv[i].float().view(T, H, D) for i in range(3))
        w = torch.exp(-torch.exp(z.float() + w0)).view(T, H, D)
        uu = u.view(H, D)
        for s in range(n_seqs):
            a, b, slot = int(cu_q[s]), int(cu_q[s + 1]), int(slots[s])
            if b <= a:
                continue
            S = state[slot].clone() if (slot >= 0 and int(positions[a]) > 0) else torch.zeros((H, D, D))
            for t in range(a, b):
                kv = k[t][:, :, None] * v[t][:, None, :]
                out[t] = torch.einsum("hd,hdv->hv", r[t], S + uu[:, :, None] * kv)
                S = w[t][:, :, None] * S + kv
            if slot >= 0:
                state[slot] = S
        return out
    assert rkv.is_contiguous() and z.is_contiguous() and z.dtype == rkv.dtype
    assert state.dtype == torch.float32 and state.is_contiguous() and state.shape[1:] == (H, D, D)
    assert w0.dtype == torch.float32 and u.dtype == torch.float32 and w0.numel() == H * D == u.numel()
    native.call("pkm_wkv", out.data_ptr(), rkv.data_ptr(), rkv.stride(0), z.data_ptr(), w0.data_ptr(), u.data_ptr(),
                state.data_ptr(), cu_q.data_ptr(), positions.data_ptr(), slots.data_ptr(), n_seqs, T, H, D,
                native.dt_code(rkv.dtype), native.stream_ptr())
    return out
