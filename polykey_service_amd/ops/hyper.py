"""Residual streams of pre-norm layers kept in fp32, one or several per token (hyper-connections)
(csrc/mixers/hyper.hip; PyTorch on CPU).

``xs`` is fp32 ``[T, S, W]``: S streams per token.  A sublayer reads ``u = sum_s a_in[s] xs[s]``,
normed; its output y goes back as ``xs'[t] = sum_s mix[s, t] xs[s] + a_out[t] y`` (all streams
from the old ones).  S = 1 with unit coefficients is the plain residual ``x += y``.  One kernel
closes a sublayer and opens the next: it folds the output in (summing the rows of a mixture of
experts on the way) and writes the next sublayer's normed input.
"""
from __future__ import annotations

import dataclasses
from typing import Optional

import torch

from . import gemm, native


@dataclasses.dataclass
class ExpertSum:
    """A mixture's output not yet summed: token t's y = sum_j wts[t, j] * y[inv[t * top + j]]
    (+ sigmoid(gate[t]) * shared[t]; ``gate`` None: + shared[t])."""
    y: torch.Tensor                         # [n, W] expert rows in expert order
    inv: torch.Tensor                       # [T * top] int32 row of (token, choice); < 0: none
    wts: torch.Tensor                       # [T, top] fp32
    top: int
    shared: Optional[torch.Tensor] = None   # [T, W]
    gate: Optional[torch.Tensor] = None     # [T] fp32 view (any stride), pre-sigmoid

    def total(self) -> torch.Tensor:
        idx = self.inv.long().view(-1, self.top)
        rows = torch.where((idx >= 0)[..., None], self.y.float()[idx.clamp(min=0)], torch.zeros((), device=self.y.device))
        out = (rows * self.wts[..., None]).sum(1)
        if self.shared is not None:
            out = out + (self.shared.float() * torch.sigmoid(self.gate.float())[:, None] if self.gate is not None
                         else self.shared.float())
        return out


def hyper_step(xs: torch.Tensor, y, close: Optional[tuple], open_: Optional[tuple], eps: float,
               act_dtype: Optional[torch.dtype] = None, want_f32: bool = False, rows: Optional[torch.Tensor] = None):
    """``close`` = (mix [S, S], a_out [S]) fp32: fold the sublayer output ``y`` ([T, W] tensor, the
    decode GEMM's unreduced split-K slabs, or an :class:`ExpertSum`) into the streams, in place.
    ``open_`` = (a_in [S], w [W]) fp32: z = u / sqrt(mean(u^2) + eps) * w of the (new) streams'
    weighted sum u.  ``rows`` (only without ``close``): open these token rows only.
    Returns (z in ``act_dtype`` or None, z in fp32 if ``want_f32`` else None)."""
    T, S, W = xs.shape
    assert xs.dtype == torch.float32 and xs.is_contiguous()
    assert rows is None or close is None
    R = rows.numel() if rows is not None else T
    act = torch.empty((R, W), dtype=act_dtype, device=xs.device) if (open_ is not None and act_dtype is not None) else None
    z32 = torch.empty((R, W), dtype=torch.float32, device=xs.device) if (open_ is not None and want_f32) else None
    if not xs.is_cuda:
        if close is not None:
            mix, a_out = close
            yv = y.total() if isinstance(y, ExpertSum) else y.float()
            xs.copy_(torch.einsum("st,nsw->ntw", mix, xs) + a_out[None, :, None] * yv[:, None, :])
        if open_ is not None:
            a_in, w = open_
            u = torch.einsum("s,nsw->nw", a_in, xs if rows is None else xs[rows.long()])
            z = u / torch.sqrt((u * u).mean(-1, keepdim=True) + eps) * w
            if act is not None:
                act.copy_(z)
            if z32 is not None:
                z32.copy_(z)
        return act, z32
    nslab, es = 1, None
    if isinstance(y, gemm.Partial):
        assert y.M == T and y.N == W
        nslab, y = y.S, y.view()[0]
    elif isinstance(y, ExpertSum):
        es, y = y, y.y
        assert es.inv.dtype == torch.int32 and es.wts.dtype == torch.float32 and es.wts.is_contiguous()
        assert es.shared is None or (es.shared.is_contiguous() and (es.gate is None or es.gate.dtype == torch.float32))
    assert y is None or y.is_contiguous()
    mix, a_out = close if close is not None else (None, None)
    a_in, w = open_ if open_ is not None else (None, None)
    native.call("pkm_hyper_step", xs.data_ptr(), R, S, W, native.ptr(y), native.dt_code(y.dtype) if y is not None else -1,
                nslab, native.ptr(es.inv) if es else None, es.top if es else 0, native.ptr(es.wts) if es else None,
                native.ptr(es.shared) if es else None,
                native.dt_code(es.shared.dtype) if es and es.shared is not None else -1,
                native.ptr(es.gate) if es else None, es.gate.stride(0) if es and es.gate is not None else 0,
                native.ptr(mix), native.ptr(a_out), native.ptr(a_in), native.ptr(w), float(eps), native.ptr(act),
                native.dt_code(act_dtype) if act_dtype is not None else 1, native.ptr(z32), native.ptr(rows),
                native.stream_ptr())
    return act, z32


def spread_rows(table: torch.Tensor, ids: torch.Tensor, S: int, scale: float = 1.0) -> torch.Tensor:
    """xs[t, s] = table[ids[t]] * scale as fp32 for every stream s: [T, S, W]."""
    T, W = ids.numel(), table.shape[1]
    if not table.is_cuda:
        rows = table[ids.long()].float()
        return (rows if scale == 1.0 else rows * torch.tensor(scale, dtype=torch.float32))[:, None, :].repeat(1, S, 1)
    xs = torch.empty((T, S, W), dtype=torch.float32, device=table.device)
    assert table.is_contiguous() and ids.dtype == torch.int32
    native.call("pkm_spread_rows", xs.data_ptr(), table.data_ptr(), ids.data_ptr(), T, S, W, table.shape[0],
                native.dt_code(table.dtype), float(scale), native.stream_ptr())
    return xs
