"""An fp32 residual stream whose sublayers sit between two layer norms (weight and bias each)
(csrc/mixers/sandwich.hip; PyTorch on CPU).

    x <- x + LN_post(y)         y: the sublayer's output
    h  = LN_pre(x)              the next sublayer's input, in the model's dtype

One kernel closes a sublayer and opens the next.  LN(v) = (v - mean) / sqrt(var + eps) * w + b with
var the mean of the squared deviations, all in fp32.  ``replace`` sets the stream to y (+ a
vector) instead of adding: the start of a pass over a repeated block, where the stream is
re-projected.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import gemm, native


def layer_norm(v: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float) -> torch.Tensor:
    mu = v.mean(-1, keepdim=True)
    d = v - mu
    return d / torch.sqrt((d * d).mean(-1, keepdim=True) + eps) * w + b


def sandwich_step(x: torch.Tensor, y, post: Optional[tuple], open_: Optional[tuple], eps: float,
                  act_dtype: Optional[torch.dtype] = None, replace: bool = False, add: Optional[torch.Tensor] = None,
                  rows: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """``x`` fp32 [T, W], updated in place.  ``y``: None, a [T, W] tensor or the decode GEMM's
    unreduced split-K slabs; ``post`` = (w, b) fp32: y is normed before it is added (None: added as
    it is); ``replace``: x <- y (+ ``add`` [W] fp32) instead.  ``open_`` = (w, b): returns
    LN(x) in ``act_dtype``, of the token rows ``rows`` only when given (then y must be None)."""
    T, W = x.shape
    assert x.dtype == torch.float32 and x.is_contiguous()
    assert rows is None or y is None
    R = rows.numel() if rows is not None else T
    act = torch.empty((R, W), dtype=act_dtype, device=x.device) if open_ is not None else None
    if not x.is_cuda:
        if y is not None:
            z = y.float()
            if post is not None:
                z = layer_norm(z, post[0], post[1], eps)
            if replace:
                x.copy_(z + (add if add is not None else 0.0))
            else:
                x.add_(z)
        if open_ is not None:
            act.copy_(layer_norm(x if rows is None else x[rows.long()], open_[0], open_[1], eps))
        return act
    nslab = 1
    if isinstance(y, gemm.Partial):
        assert y.M == T and y.N == W
        nslab, y = y.S, y.view()[0]
    assert y is None or (y.is_contiguous() and y.shape == (T, W))
    pw, pb = post if post is not None else (None, None)
    ow, ob = open_ if open_ is not None else (None, None)
    native.call("pkm_sandwich_step", x.data_ptr(), R, W, native.ptr(y), native.dt_code(y.dtype) if y is not None else -1,
                nslab, native.ptr(pw), native.ptr(pb), int(replace), native.ptr(add), native.ptr(ow), native.ptr(ob),
                float(eps), native.ptr(act), native.dt_code(act_dtype) if act is not None else 1, native.ptr(rows),
                native.stream_ptr())
    return act


def embed_rows_f32(table: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
    """table[ids] as fp32 [T, W]."""
    if not table.is_cuda:
        return table[ids.long()].float()
    T, W = ids.numel(), table.shape[1]
    out = torch.empty((T, W), dtype=torch.float32, device=table.device)
    assert table.is_contiguous() and ids.dtype == torch.int32
    native.call("pkm_spread_rows", out.data_ptr(), table.data_ptr(), ids.data_ptr(), T, 1, W, table.shape[0],
                native.dt_code(table.dtype), 1.0, native.stream_ptr())
    return out


def join_cast(x: torch.Tensor, x0: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """[x | x0] per row in ``dtype``: [T, 2W] (the input of a block's re-projection)."""
    T, W = x.shape
    if not x.is_cuda:
        return torch.cat([x, x0], -1).to(dtype)
    out = torch.empty((T, 2 * W), dtype=dtype, device=x.device)
    assert x.dtype == torch.float32 and x0.dtype == torch.float32 and x.is_contiguous() and x0.is_contiguous()
    native.call("pkm_join_cast", out.data_ptr(), x.data_ptr(), x0.data_ptr(), T, W, native.dt_code(dtype),
                native.stream_ptr())
    return out


def silu_mul(gu, F: int, dtype: torch.dtype) -> torch.Tensor:
    """gu [T, F gate | F up] (a tensor, or the decode GEMM's unreduced split-K slabs) ->
    silu(gate) * up in ``dtype`` [T, F]; the product is formed in fp32."""
    nslab = 1
    if isinstance(gu, gemm.Partial):
        nslab, gu = gu.S, gu.view()[0]
    T = gu.shape[0]
    assert gu.shape[1] == 2 * F
    if not gu.is_cuda:
        f = gu.float()
        return (torch.nn.functional.silu(f[:, :F]) * f[:, F:]).to(dtype)
    out = torch.empty((T, F), dtype=dtype, device=gu.device)
    assert gu.is_contiguous()
    native.call("pkm_silu_mul", out.data_ptr(), gu.data_ptr(), T, F, nslab, native.dt_code(gu.dtype),
                native.dt_code(dtype), native.stream_ptr())
    return out


def scale_(x: torch.Tensor, k: float) -> torch.Tensor:
    """x *= k in place (fp32)."""
    if k == 1.0:
        return x
    if not x.is_cuda:
        return x.mul_(k)
    assert x.dtype == torch.float32 and x.is_contiguous()
    native.call("pkm_scale", x.data_ptr(), x.numel(), float(k), native.stream_ptr())
    return x
