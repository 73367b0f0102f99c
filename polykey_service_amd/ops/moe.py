"""Mixture-of-experts dispatch (Mixtral): routing, expert grouping, grouped GEMM, combine.

Decode (T <= 64 tokens): everything stays on the device and is graph-capturable —
``topk_softmax`` → ``align`` (stable counting sort by expert) → ``permute`` → grouped skinny
GEMM for w13 with the fused SiLU epilogue → grouped skinny GEMM for w2 → weighted
``unpermute``.  An expert that received no token is skipped without reading its weights.

Prefill (T > 64): the same routing kernels, then ONE launch per projection of the grouped MFMA
GEMM of ``csrc/kernels/gemm_prefill.hip`` — it reads the expert row offsets on the device (no
read-back, no per-expert launches) and fuses SiLU(gate)*up into the w13 epilogue.

Expert parallelism: with ``e_lo, e_hi`` this rank only computes experts ``[e_lo, e_hi)``;
slots routed elsewhere get ``inv = -1`` and contribute zero, and the caller all-reduces the
combined output across the EP group (tokens are replicated by TP attention, so the combine is
the same all-reduce the dense MLP already does — see parallel/ep.py for the all-to-all form).
"""
from __future__ import annotations

import dataclasses

from typing import Optional, Tuple

import torch
import torch.nn.functional as F

from . import gemm, gemm_prefill, native, reference
from .gemm import silu_and_mul_interleaved


def topk_softmax(router_logits: torch.Tensor, k: int, renorm: bool = True) -> Tuple[torch.Tensor, torch.Tensor]:
    T, E = router_logits.shape
    if not router_logits.is_cuda:
        p = torch.softmax(router_logits.float(), -1)
        w, ids = torch.sort(p, dim=-1, descending=True, stable=True)  # ties → lower expert id, as the kernel
        w, ids = w[:, :k], ids[:, :k]
        if renorm:
            w = w / w.sum(-1, keepdim=True)
        return ids.to(torch.int32), w
    ids = torch.empty((T, k), dtype=torch.int32, device=router_logits.device)
    w = torch.empty((T, k), dtype=torch.float32, device=router_logits.device)
    native.call("pk_moe_topk_softmax", ids.data_ptr(), w.data_ptr(), router_logits.data_ptr(), T, E, k,
                router_logits.stride(0), int(renorm), native.stream_ptr())
    return ids, w


def align(ids: torch.Tensor, E: int, e_lo: int, e_hi: int):
    """→ offsets [E_local+1], sorted slots [n], inverse positions [n] (int32; -1 = not local)."""
    n = ids.numel()
    El = e_hi - e_lo
    dev = ids.device
    if not ids.is_cuda:
        flat = ids.reshape(-1).long()
        local = (flat >= e_lo) & (flat < e_hi)
        key = torch.where(local, flat - e_lo, torch.full_like(flat, El))
        order = torch.sort(key, stable=True).indices
        counts = torch.bincount(key, minlength=El + 1)[:El]
        offsets = torch.zeros(El + 1, dtype=torch.int32)
        offsets[1:] = torch.cumsum(counts, 0)
        m = int(offsets[-1])
        sorted_ = order[:m].to(torch.int32)
        inv = torch.full((n,), -1, dtype=torch.int32)
        inv[order[:m]] = torch.arange(m, dtype=torch.int32)
        return offsets, sorted_, inv
    offsets = torch.empty(El + 1, dtype=torch.int32, device=dev)
    sorted_ = torch.empty(n, dtype=torch.int32, device=dev)
    inv = torch.empty(n, dtype=torch.int32, device=dev)
    if El > 64:  # beyond the single-wave stable sort: the LDS-counter align (all experts local)
        assert e_lo == 0 and e_hi == E
        native.call("pkm_expert_align_wide", ids.data_ptr(), offsets.data_ptr(), sorted_.data_ptr(), inv.data_ptr(), n,
                    E, native.stream_ptr())
        return offsets, sorted_, inv
    native.call("pk_moe_align", ids.data_ptr(), offsets.data_ptr(), sorted_.data_ptr(), inv.data_ptr(), n, E, e_lo,
                e_hi, native.stream_ptr())
    return offsets, sorted_, inv


def permute(x: torch.Tensor, sorted_: torch.Tensor, offsets: torch.Tensor, k: int) -> torch.Tensor:
    n = sorted_.numel()
    H = x.shape[-1]
    if not x.is_cuda:
        m = int(offsets[-1])
        return x[(sorted_[:m].long() // k)]
    out = torch.empty((n, H), dtype=x.dtype, device=x.device)
    native.call("pk_moe_permute", out.data_ptr(), x.data_ptr(), sorted_.data_ptr(), offsets.data_ptr(), n,
                offsets.numel() - 1, k, H, native.stream_ptr())
    return out


def unpermute(y: torch.Tensor, inv: torch.Tensor, w: torch.Tensor, T: int, k: int) -> torch.Tensor:
    H = y.shape[-1]
    if not y.is_cuda:
        out = torch.zeros((T, H), dtype=torch.float32)
        if y.shape[0] == 0:  # no slot routed to this rank's experts (EP): zero contribution
            return out.to(y.dtype)
        invl = inv.view(T, k).long()
        for j in range(k):
            valid = invl[:, j] >= 0
            idx = invl[:, j].clamp(min=0)
            out += torch.where(valid[:, None], y[idx].float() * w[:, j:j + 1].float(), torch.zeros(()))
        return out.to(y.dtype)
    out = torch.empty((T, H), dtype=y.dtype, device=y.device)
    native.call("pk_moe_unpermute", out.data_ptr(), y.data_ptr(), inv.data_ptr(), w.data_ptr(), T, k, H,
                native.stream_ptr())
    return out


def grouped_gemm(a: torch.Tensor, w: torch.Tensor, offsets: torch.Tensor, max_rows: int, silu: bool,
                 packed: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Rows of expert e = a[offsets[e]:offsets[e+1]] times w[e]^T (w: [E_local, N, K]).
    Decode-sized groups (<= ``gemm.DECODE_MAX_M`` rows; above 64 in 128-row tiles) run the
    weight-streaming decode GEMM of csrc/kernels/gemm_skinny.hip in grouped mode (``packed``:
    fragment-packed experts)."""
    E_local, N, K = w.shape
    n_out = N // 2 if silu else N
    if (a.is_cuda and max_rows <= gemm.DECODE_MAX_M and gemm.SKINNY_ENABLED and N % 128 == 0
            and K % 256 == 0):
        return gemm.grouped_linear(a, w, offsets, max_rows, silu, packed=packed)
    out = torch.empty((a.shape[0], n_out), dtype=a.dtype, device=a.device)
    if a.is_cuda and max_rows <= 64:
        native.call("pk_moe_gemm", out.data_ptr(), a.data_ptr(), w.data_ptr(), offsets.data_ptr(), max_rows, N, K,
                    out.stride(0), E_local, 2 if silu else 0, native.stream_ptr())
        return out
    if a.is_cuda and gemm_prefill.supported(N, K) and w.is_contiguous():
        return gemm_prefill.grouped_linear(a, w, offsets, silu=silu, out=out)
    offs = offsets.tolist()  # shapes the MFMA kernel does not tile: a library GEMM per expert
    for e in range(E_local):
        lo, hi = offs[e], offs[e + 1]
        if hi > lo:  # results land in their rows of `out` directly (no slice-assignment copy)
            if silu:
                silu_and_mul_interleaved(F.linear(a[lo:hi], w[e]), out=out[lo:hi])
            else:
                torch.matmul(a[lo:hi], w[e].t(), out=out[lo:hi])
    return out


@dataclasses.dataclass
class PendingCombine:
    """Expert outputs not yet combined: :func:`combine_add_rms_norm` does the weighted top-k
    combine, the residual add and the next RMSNorm in one kernel."""
    y: torch.Tensor      # [T*k, H] expert outputs in expert-sorted order
    inv: torch.Tensor    # [T*k] sorted position of (token, slot); -1 = expert on another EP rank
    w: torch.Tensor      # [T, k] routing weights
    T: int
    k: int

    def combine(self) -> torch.Tensor:
        return unpermute(self.y, self.inv, self.w, self.T, self.k)


def combine_add_rms_norm(p: PendingCombine, residual: torch.Tensor, weight: torch.Tensor, eps: float):
    """residual += combine(p); x = rms_norm(residual) * weight → (x, residual), one kernel."""
    H = residual.shape[-1]
    if not residual.is_cuda or H % 1024 or H > 8192:
        from .norm import fused_add_rms_norm
        return fused_add_rms_norm(p.combine(), residual, weight, eps)
    x = torch.empty_like(residual)
    native.call("pk_moe_combine_add_rmsnorm", x.data_ptr(), residual.data_ptr(), p.y.data_ptr(), p.inv.data_ptr(),
                p.w.data_ptr(), weight.data_ptr(), p.T, p.k, H, float(eps), native.stream_ptr())
    return x, residual


def fused_moe(x: torch.Tensor, router_w: torch.Tensor, w13: torch.Tensor, w2: torch.Tensor, k: int,
              e_lo: int = 0, e_hi: Optional[int] = None, w13_p: Optional[torch.Tensor] = None,
              w2_p: Optional[torch.Tensor] = None, defer_combine: bool = False,
              routing: Optional[Tuple[torch.Tensor, torch.Tensor]] = None):
    """Mixtral sparse MLP for this rank's experts.  x [T, H]; router_w [E, H]; w13 [E_l, 2I, H]
    (gate/up interleaved by 16); w2 [E_l, H, I].  Returns the (partial, if EP) combined output,
    or with ``defer_combine`` a :class:`PendingCombine` for the fused combine+add+norm.
    ``routing``: (ids, weights) already computed by the preceding norm kernel
    (:func:`gemm.partial_add_rms_norm_route`).

    Decode (T <= 64): expert sort, the w13 grouped GEMM gathering token rows itself (no
    permute pass) with the SiLU epilogue, the w2 grouped GEMM, and the combine (fused into the
    next residual add + RMSNorm when deferred)."""
    T = x.shape[0]
    E = router_w.shape[0]
    e_hi = E if e_hi is None else e_hi
    N13, K13 = w13.shape[1], w13.shape[2]
    if (x.is_cuda and T <= 64 and E <= 64 and gemm.SKINNY_ENABLED and N13 % 128 == 0 and K13 % 256 == 0
            and w2.shape[1] % 128 == 0 and w2.shape[2] % 256 == 0):
        if routing is not None:
            ids, wts = routing
        else:
            ids, wts = topk_softmax(F.linear(x, router_w), k)
        offsets, sorted_, inv = align(ids, E, e_lo, e_hi)
        h = gemm.grouped_linear(x, w13, offsets, T, True, packed=w13_p, a_rows=sorted_, a_row_div=k, n_rows=T * k)
        y = gemm.grouped_linear(h, w2, offsets, T, False, packed=w2_p)
        pending = PendingCombine(y, inv, wts, T, k)
        return pending if defer_combine else pending.combine()
    logits = F.linear(x, router_w)
    ids, wts = topk_softmax(logits, k)
    offsets, sorted_, inv = align(ids, E, e_lo, e_hi)
    xs = permute(x, sorted_, offsets, k)
    h = grouped_gemm(xs, w13, offsets, T, silu=True, packed=w13_p)
    y = grouped_gemm(h, w2, offsets, T, silu=False, packed=w2_p)
    return unpermute(y, inv, wts, T, k)


def fused_moe_reference(x, router_w, w13, w2, k, e_lo=0, e_hi=None):
    """Loop-over-experts oracle with fp32 GEMMs and the kernels' bf16 rounding points
    (projection outputs, SiLU and h are bf16 tensors in the fused path)."""
    E = router_w.shape[0]
    e_hi = E if e_hi is None else e_hi
    bf = lambda t: t.to(torch.bfloat16).float()
    p = torch.softmax(bf(x.float() @ router_w.float().t()), -1)
    w, ids = torch.topk(p, k, -1)
    w = w / w.sum(-1, keepdim=True)
    out = torch.zeros(x.shape, dtype=torch.float32, device=x.device)
    H = x.shape[1]
    for e in range(e_lo, e_hi):
        v = w13[e - e_lo].float().view(-1, 2, 16, H)
        g, u = v[:, 0].reshape(-1, H), v[:, 1].reshape(-1, H)
        h = bf(bf(torch.nn.functional.silu(bf(x.float() @ g.t()))) * bf(x.float() @ u.t()))
        y = bf(h @ w2[e - e_lo].float().t())
        sel = (ids == e).float() * w
        out += sel.sum(-1, keepdim=True) * y
    return out


# ------------------------------------------------------------------ sigmoid-routed, input-scaled MoE
# up to this many tokens the router's dot products run inside the top-k kernel; above, the logits
# are one fp32 library GEMM.  0: always the GEMM (one wave per token walking every expert's row is
# latency-bound: 173 us for 16 experts x 2048 against ~10 us for GEMM + top-k)
ROUTER_DOT_MAX_T = 0


def route_sigmoid_topk(x: torch.Tensor, router_w: torch.Tensor, k: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """fp32 router: s = sigmoid(router_w x); the k largest s per token and their experts (ties: the
    lower expert id), scores as they are.  x [T, W] fp32, router_w [E, W] fp32."""
    T, W = x.shape
    E = router_w.shape[0]
    if not x.is_cuda:
        s = torch.sigmoid(x.float() @ router_w.float().t())
        w, ids = torch.sort(s, dim=-1, descending=True, stable=True)
        return ids[:, :k].to(torch.int32).contiguous(), w[:, :k].contiguous()
    assert x.dtype == torch.float32 and router_w.dtype == torch.float32 and x.is_contiguous()
    ids = torch.empty((T, k), dtype=torch.int32, device=x.device)
    w = torch.empty((T, k), dtype=torch.float32, device=x.device)
    if T > ROUTER_DOT_MAX_T:  # many tokens: the logits as one fp32 library GEMM, then sigmoid + top-k
        logits = torch.mm(x, router_w.t())
        native.call("pkm_route_sigmoid_topk", ids.data_ptr(), w.data_ptr(), logits.data_ptr(), None, T, W, E, k,
                    native.stream_ptr())
        return ids, w
    native.call("pkm_route_sigmoid_topk", ids.data_ptr(), w.data_ptr(), x.data_ptr(), router_w.data_ptr(), T, W, E, k,
                native.stream_ptr())
    return ids, w


def mfma_experts_ok(E: int, F_: int, W: int, dtype: torch.dtype, device) -> bool:
    """Shapes the framework's MFMA grouped expert GEMMs tile (prefill: 256-wide column tiles; decode:
    the weight-streaming grouped GEMM on block-packed experts): bf16 on the GPU, at most 64 experts,
    ff and width multiples of 256."""
    return (device.type == "cuda" and dtype == torch.bfloat16 and E <= 64 and F_ % 256 == 0 and W % 256 == 0)


def input_scaled_moe(x: torch.Tensor, x_act: torch.Tensor, ids: torch.Tensor, wts: torch.Tensor, gate, up, down,
                     w13=None, w2=None, w13_p=None, w2_p=None, defer_combine: bool = False):
    """sum over a token's experts of down_e(silu(gate_e(s x)) * up_e(s x)), s the expert's score,
    as fp32 [T, W].  x: the fp32 stream rows, x_act: the same in the weights' dtype.  Tokens are
    grouped by expert on the device (align) and the combine is a plain sum; with ``defer_combine``
    the expert rows and their inverse positions (y [T * top, W], inv [T * top]) are returned for
    the norm kernel that follows to sum (stream.sum_gain_norm ``gather``).

    Two forms.  With ``w13`` / ``w2`` (interleaved gate|up [E, 2F, W] and down [E, W, F], shapes of
    :func:`mfma_experts_ok`): rows ``s * x`` in expert order feed the framework's grouped MFMA
    GEMMs with the fused SiLU epilogue.  Otherwise (any sizes, fp32): gate / up [E, F, W] and down
    [E, W, F] through the tiled fp32-FMA grouped kernels, the score applied to the gate / up
    products (the same value, the products' accumulations left unscaled)."""
    T, W = x_act.shape
    k = ids.shape[1]
    n = T * k
    if w13 is not None:
        E = w13.shape[0]
        offsets, sorted_, inv = align(ids, E, 0, E)
        st = native.stream_ptr()
        xs = torch.empty((n, W), dtype=x_act.dtype, device=x.device)
        native.call("pkm_permute_scaled", xs.data_ptr(), x.data_ptr(), sorted_.data_ptr(), wts.data_ptr(), n, k, W,
                    native.dt_code(xs.dtype), st)
        h = grouped_gemm(xs, w13, offsets, T, silu=True, packed=w13_p)
        y = grouped_gemm(h, w2, offsets, T, silu=False, packed=w2_p)
        if defer_combine:
            return y, inv
        out = torch.empty((T, W), dtype=torch.float32, device=x.device)
        native.call("pkm_combine_rows", out.data_ptr(), y.data_ptr(), inv.data_ptr(), T, k, W, native.dt_code(y.dtype), st)
        return out
    E, F_, _ = gate.shape
    offsets, sorted_, inv = align(ids, E, 0, E)
    if not x_act.is_cuda:
        m = int(offsets[-1])
        tok = sorted_[:m].long() // k
        s = wts.reshape(-1)[sorted_[:m].long()].float()
        y = torch.zeros((m, W), dtype=torch.float32)
        offs = offsets.tolist()
        for e in range(E):
            lo, hi = offs[e], offs[e + 1]
            if hi > lo:
                xe = x_act[tok[lo:hi]].float()
                g = (xe @ gate[e].float().t()) * s[lo:hi, None]
                u = (xe @ up[e].float().t()) * s[lo:hi, None]
                h = (g * torch.sigmoid(g) * u).to(x_act.dtype).float()
                y[lo:hi] = h @ down[e].float().t()
        if defer_combine:
            return y, inv
        return y[inv.long().view(T, k)].sum(1)
    assert x_act.is_contiguous() and gate.is_contiguous() and up.is_contiguous() and down.is_contiguous()
    assert gate.dtype == x_act.dtype and wts.dtype == torch.float32 and wts.is_contiguous()
    dt = native.dt_code(x_act.dtype)
    h = torch.empty((n, F_), dtype=x_act.dtype, device=x_act.device)
    y = torch.empty((n, W), dtype=torch.float32, device=x_act.device)
    out = torch.empty((T, W), dtype=torch.float32, device=x_act.device)
    st = native.stream_ptr()
    native.call("pkm_expert_gate_up", h.data_ptr(), x_act.data_ptr(), gate.data_ptr(), up.data_ptr(), offsets.data_ptr(),
                sorted_.data_ptr(), wts.data_ptr(), n, k, E, F_, W, dt, st)
    native.call("pkm_expert_down", y.data_ptr(), h.data_ptr(), down.data_ptr(), offsets.data_ptr(), n, E, W, F_, dt, st)
    if defer_combine:
        return y, inv
    native.call("pkm_combine_rows", out.data_ptr(), y.data_ptr(), inv.data_ptr(), T, k, W, 1, st)
    return out


# ------------------------------------------------------------------ logit-routed experts with clamped products
ROUTER_KERNEL_MAX_T = 256


def router_logits(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """x [T, W] fp32 times w [N, W] fp32 -> [T, N] fp32 in true fp32.  Decode-sized steps on the GPU take
    one wave per (token, row); larger ones an fp32 library GEMM."""
    if not x.is_cuda or x.shape[0] > ROUTER_KERNEL_MAX_T:
        return torch.mm(x, w.t())
    assert x.dtype == torch.float32 and w.dtype == torch.float32 and x.is_contiguous() and w.is_contiguous()
    out = torch.empty((x.shape[0], w.shape[0]), dtype=torch.float32, device=x.device)
    native.call("pkm_router_logits", out.data_ptr(), x.data_ptr(), w.data_ptr(), x.shape[0], w.shape[0], x.shape[1],
                native.stream_ptr())
    return out


def route_topk_softmax(logits: torch.Tensor, E: int, k: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """fp32 router logits [T, >= E] (the first E columns of each row; the row may hold more) -> the k
    experts with the largest logits (ties: the lower expert id) and the softmax over those k logits."""
    T = logits.shape[0]
    if not logits.is_cuda:
        z, ids = torch.sort(logits[:, :E].float(), dim=-1, descending=True, stable=True)
        return ids[:, :k].to(torch.int32).contiguous(), torch.softmax(z[:, :k], -1).contiguous()
    assert logits.dtype == torch.float32 and logits.stride(1) == 1
    ids = torch.empty((T, k), dtype=torch.int32, device=logits.device)
    w = torch.empty((T, k), dtype=torch.float32, device=logits.device)
    native.call("pkm_route_topk_softmax", ids.data_ptr(), w.data_ptr(), logits.data_ptr(), logits.stride(0), T, E, k,
                native.stream_ptr())
    return ids, w


def _clamped(g: torch.Tensor, u: torch.Tensor, limit: float) -> torch.Tensor:
    g = g.clamp(max=limit)
    u = u.clamp(-limit, limit)
    return g * torch.sigmoid(1.702 * g) * (u + 1)


def clamped_glu(gu, limit: float, interleaved: bool = False, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """gu [n, 2F]: gate products then up products (``interleaved``: alternating in blocks of 16, the
    layout of the grouped MFMA GEMMs) -> min(g, limit) * sigmoid(1.702 min(g, limit)) * (clamp(u) + 1).
    ``gu`` may be the decode GEMM's unreduced split-K slabs (``gemm.Partial``): their sum is taken on
    the way in and the result is written in ``dtype``."""
    if isinstance(gu, gemm.Partial):
        out = torch.empty((gu.M, gu.N // 2), dtype=dtype, device=gu.buf.device)
        native.call("pkm_clamped_glu_slabs", out.data_ptr(), gu.buf.data_ptr(), gu.S, gu.M, gu.N // 2, float(limit),
                    int(interleaved), native.dt_code(dtype), native.stream_ptr())
        return out
    n, F2 = gu.shape
    F_ = F2 // 2
    if not gu.is_cuda:
        f = gu.float()
        if interleaved:
            v = f.view(n, F_ // 16, 2, 16)
            g, u = v[:, :, 0].reshape(n, F_), v[:, :, 1].reshape(n, F_)
        else:
            g, u = f[:, :F_], f[:, F_:]
        return _clamped(g, u, limit).to(gu.dtype)
    out = torch.empty((n, F_), dtype=gu.dtype, device=gu.device)
    assert gu.is_contiguous() and (not interleaved or F_ % 16 == 0)
    native.call("pkm_clamped_glu", out.data_ptr(), gu.data_ptr(), n, F_, float(limit), int(interleaved),
                native.dt_code(gu.dtype), native.stream_ptr())
    return out


def gelu_tanh(x: torch.Tensor) -> torch.Tensor:
    """0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))), fp32 maths, in place."""
    if not x.is_cuda:
        return x.copy_(F.gelu(x.float(), approximate="tanh"))
    assert x.is_contiguous()
    native.call("pkm_gelu_tanh", x.data_ptr(), x.numel(), native.dt_code(x.dtype), native.stream_ptr())
    return x


def clamped_experts(x_act: torch.Tensor, ids: torch.Tensor, gate, up, down, limit: float, w13=None, w2=None,
                    w13_p=None, w2_p=None):
    """Rows of every (token, chosen expert) pair through the expert's clamped GLU: (y [T * top, W] in
    expert order, inv [T * top]) for the kernel that sums them with the routing weights.  With
    ``w13`` / ``w2`` (shapes of :func:`mfma_experts_ok`) the framework's grouped MFMA GEMMs, else
    gate / up [E, F, W], down [E, W, F] through the tiled FMA grouped kernels (any sizes, fp32 too)."""
    T, W = x_act.shape
    k = ids.shape[1]
    n = T * k
    if w13 is not None:
        E = w13.shape[0]
        offsets, sorted_, inv = align(ids, E, 0, E)
        if T <= 64 and E <= 64 and gemm.SKINNY_ENABLED:  # decode: the GEMM gathers the tokens' rows itself
            gu = gemm.grouped_linear(x_act, w13, offsets, T, False, packed=w13_p, a_rows=sorted_, a_row_div=k, n_rows=n)
            return gemm.grouped_linear(clamped_glu(gu, limit, interleaved=True), w2, offsets, T, False, packed=w2_p), inv
        xs = permute(x_act, sorted_, offsets, k)
        gu = grouped_gemm(xs, w13, offsets, T, silu=False, packed=w13_p)
        y = grouped_gemm(clamped_glu(gu, limit, interleaved=True), w2, offsets, T, silu=False, packed=w2_p)
        return y, inv
    E, F_, _ = gate.shape
    offsets, sorted_, inv = align(ids, E, 0, E)
    if not x_act.is_cuda:
        m = int(offsets[-1])
        tok = sorted_[:m].long() // k
        y = torch.zeros((m, W), dtype=torch.float32)
        offs = offsets.tolist()
        for e in range(E):
            lo, hi = offs[e], offs[e + 1]
            if hi > lo:
                xe = x_act[tok[lo:hi]]
                h = _clamped(F.linear(xe, gate[e]).float(), F.linear(xe, up[e]).float(), limit).to(x_act.dtype)
                y[lo:hi] = F.linear(h, down[e]).float()
        return y, inv
    assert x_act.is_contiguous() and gate.is_contiguous() and up.is_contiguous() and down.is_contiguous()
    dt = native.dt_code(x_act.dtype)
    h = torch.empty((n, F_), dtype=x_act.dtype, device=x_act.device)
    y = torch.empty((n, W), dtype=torch.float32, device=x_act.device)
    st = native.stream_ptr()
    native.call("pkm_expert_gate_up_clamped", h.data_ptr(), x_act.data_ptr(), gate.data_ptr(), up.data_ptr(),
                offsets.data_ptr(), sorted_.data_ptr(), float(limit), n, k, E, F_, W, dt, st)
    native.call("pkm_expert_down", y.data_ptr(), h.data_ptr(), down.data_ptr(), offsets.data_ptr(), n, E, W, F_, dt, st)
    return y, inv


def silu_experts(x_act: torch.Tensor, ids: torch.Tensor, gate, up, down, w13=None, w2=None, w13_p=None, w2_p=None):
    """Rows of every (token, chosen expert) pair through down_e(silu(gate_e x) * (up_e x)): (y [T * top, W]
    in expert order, inv [T * top]) for the kernel that sums them with the routing weights.  With
    ``w13`` / ``w2`` (shapes of :func:`mfma_experts_ok`) the framework's grouped MFMA GEMMs with the
    fused SiLU epilogue, else gate / up [E, F, W], down [E, W, F] through the tiled FMA grouped
    kernels (any sizes, fp32 too)."""
    T, W = x_act.shape
    k = ids.shape[1]
    n = T * k
    if w13 is not None:
        E = w13.shape[0]
        offsets, sorted_, inv = align(ids, E, 0, E)
        if T <= 64 and E <= 64 and gemm.SKINNY_ENABLED:  # decode: the GEMM gathers the tokens' rows itself
            h = gemm.grouped_linear(x_act, w13, offsets, T, True, packed=w13_p, a_rows=sorted_, a_row_div=k, n_rows=n)
            return gemm.grouped_linear(h, w2, offsets, T, False, packed=w2_p), inv
        xs = permute(x_act, sorted_, offsets, k)
        h = grouped_gemm(xs, w13, offsets, T, silu=True, packed=w13_p)
        return grouped_gemm(h, w2, offsets, T, silu=False, packed=w2_p), inv
    E, F_, _ = gate.shape
    offsets, sorted_, inv = align(ids, E, 0, E)
    if not x_act.is_cuda:
        m = int(offsets[-1])
        tok = sorted_[:m].long() // k
        y = torch.zeros((m, W), dtype=torch.float32)
        offs = offsets.tolist()
        for e in range(E):
            lo, hi = offs[e], offs[e + 1]
            if hi > lo:
                xe = x_act[tok[lo:hi]]
                g = F.linear(xe, gate[e]).float()
                h = (g * torch.sigmoid(g) * F.linear(xe, up[e]).float()).to(x_act.dtype)
                y[lo:hi] = F.linear(h, down[e]).float()
        return y, inv
    assert x_act.is_contiguous() and gate.is_contiguous() and up.is_contiguous() and down.is_contiguous()
    dt = native.dt_code(x_act.dtype)
    h = torch.empty((n, F_), dtype=x_act.dtype, device=x_act.device)
    y = torch.empty((n, W), dtype=torch.float32, device=x_act.device)
    st = native.stream_ptr()
    # limit 0 selects the unclamped SiLU product in the grouped kernel's epilogue
    native.call("pkm_expert_gate_up_clamped", h.data_ptr(), x_act.data_ptr(), gate.data_ptr(), up.data_ptr(),
                offsets.data_ptr(), sorted_.data_ptr(), 0.0, n, k, E, F_, W, dt, st)
    native.call("pkm_expert_down", y.data_ptr(), h.data_ptr(), down.data_ptr(), offsets.data_ptr(), n, E, W, F_, dt, st)
    return y, inv
