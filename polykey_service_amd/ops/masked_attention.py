"""Softmax attention over a paged cache with a per-row band of visible keys, learned sinks and
separate counts of query, key and value heads (csrc/mixers/masked_attention.hip; PyTorch on CPU).

A query at position p sees keys j with lo(p) <= j <= p, where lo(p) = max(0, p - window + 1) for a
sliding window (window > 0) and lo(p) = max(lo(p), floor(p / chunk) * chunk) for blocks of ``chunk``
positions (chunk > 0); both 0: every earlier key.  The softmax denominator of query head h also
holds exp(sink[h]) when sink logits are given (a key without a value).

Query heads come in QH, key heads in KH, value heads in VH (QH % KH == 0, QH % VH == 0): query
head h reads key head h // (QH / KH) and value head h // (QH / VH).  Two attention maps per head
over shared values (differential attention) are 2H query heads on 2G key heads and G value heads;
latent attention with folded queries is H query heads on one key head whose first ``V`` numbers
are also the value.  Caches are ``[blocks, heads, block_size, width]`` in the model's dtype.
Rotations read fp32 (cos, sin) tables built in double precision on the host.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import native
from .sink_attention import pair_frequencies, rotation_table  # noqa: F401  (the tables are shared)


def table_for(rot, max_pos: int, device) -> torch.Tensor:
    f, mag = pair_frequencies(rot.dims, rot.base, rot.scaling)
    return rotation_table(max_pos, f, mag, device)


def turn(x: torch.Tensor, cs: torch.Tensor, halves: bool = True) -> torch.Tensor:
    """x [n, h, d] fp32, cs [n, pairs, 2] (cos, sin): the first 2 * pairs coordinates turn, pair i
    = (i, i + pairs) with ``halves`` else (2i, 2i + 1); the rest pass."""
    n2 = cs.shape[1]
    c, s = cs[:, None, :, 0], cs[:, None, :, 1]
    out = x.clone()
    if halves:
        u, v = x[..., :n2], x[..., n2:2 * n2]
        out[..., :n2] = u * c - v * s
        out[..., n2:2 * n2] = v * c + u * s
    else:
        u, v = x[..., 0:2 * n2:2], x[..., 1:2 * n2:2]
        out[..., 0:2 * n2:2] = u * c - v * s
        out[..., 1:2 * n2:2] = v * c + u * s
    return out


def _write_cache(cache: torch.Tensor, rows: torch.Tensor, slot_mapping: torch.Tensor) -> None:
    """cache [blocks, heads, bs, width] <- rows [T, heads, width] at the tokens' slots (< 0: not)."""
    bs = cache.shape[2]
    ok = slot_mapping >= 0
    sl = slot_mapping[ok].long()
    cache[sl // bs, :, sl % bs, :] = rows[ok].to(cache.dtype)


def rotate_cache(proj: torch.Tensor, positions: torch.Tensor, slot_mapping: torch.Tensor, table: Optional[torch.Tensor],
                 halves: bool, k_cache: torch.Tensor, v_cache: torch.Tensor, QH: int, KH: int, VH: int, D: int,
                 V: int, q_norm: Optional[torch.Tensor] = None, k_norm: Optional[torch.Tensor] = None,
                 eps: float = 0.0) -> torch.Tensor:
    """proj [T, QH*D | KH*D | VH*V] (may be a column slice of a wider projection output): q and k
    heads turn by the token's position (``table`` rows; None: no rotation), k and v go to the paged
    caches.  ``q_norm`` / ``k_norm`` [D] fp32: the heads are first set to unit RMS (``eps`` inside
    the root) times that weight.  Returns q [T, QH, D] in the cache's dtype."""
    T = proj.shape[0]
    q = torch.empty((T, QH, D), dtype=k_cache.dtype, device=proj.device)
    if not proj.is_cuda:
        f = proj.float()
        qq, kk = f[:, :QH * D].view(T, QH, D), f[:, QH * D:(QH + KH) * D].view(T, KH, D)
        vv = f[:, (QH + KH) * D:].view(T, VH, V)
        unit = lambda u, w: u / torch.sqrt((u * u).mean(-1, keepdim=True) + eps) * w
        if q_norm is not None:
            qq = unit(qq, q_norm)
        if k_norm is not None:
            kk = unit(kk, k_norm)
        if table is not None:
            cs = table[positions.long()]
            qq, kk = turn(qq, cs, halves), turn(kk, cs, halves)
        q.copy_(qq)
        _write_cache(k_cache, kk, slot_mapping)
        _write_cache(v_cache, vv, slot_mapping)
        return q
    assert proj.stride(1) == 1 and proj.dtype == k_cache.dtype == v_cache.dtype and proj.shape[1] == (QH + KH) * D + VH * V
    assert positions.dtype == torch.int32 and slot_mapping.dtype == torch.int32
    assert k_cache.is_contiguous() and v_cache.is_contiguous()
    assert k_cache.shape[1:] == (KH, k_cache.shape[2], D) and v_cache.shape[1:] == (VH, k_cache.shape[2], V)
    assert table is None or (table.dtype == torch.float32 and table.is_contiguous() and 2 * table.shape[1] <= D)
    for w in (q_norm, k_norm):
        assert w is None or (w.dtype == torch.float32 and w.numel() == D)
    native.call("pkm_rotate_cache", q.data_ptr(), proj.data_ptr(), proj.stride(0), positions.data_ptr(),
                slot_mapping.data_ptr(), native.ptr(table), table.shape[1] if table is not None else 0,
                table.shape[0] if table is not None else 0, int(halves), k_cache.data_ptr(), v_cache.data_ptr(), T,
                QH, KH, VH, D, V, k_cache.shape[2], native.ptr(q_norm), native.ptr(k_norm), float(eps),
                native.dt_code(k_cache.dtype), native.stream_ptr())
    return q


def masked_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: Optional[torch.Tensor], V: int,
                     block_tables: torch.Tensor, cu_q: torch.Tensor, context_lens: torch.Tensor, n_seqs: int,
                     scale: float, window: int = 0, chunk: int = 0, sink: Optional[torch.Tensor] = None,
                     out_dtype: torch.dtype = torch.float32, head_major: bool = False, num_decode: int = 0) -> torch.Tensor:
    """q [T, QH, D] (fp32 or the cache's dtype); sequence s owns tokens cu_q[s]:cu_q[s+1], the LAST
    ones of its context_lens[s] cached tokens.  ``v_cache`` None: the value of a key is the first
    ``V`` numbers of its key row (key heads = value heads).  ``sink`` [QH] fp32 logits or None.
    The first ``num_decode`` sequences hold one token each (the matrix-core kernel cuts their bands
    into runs that a second kernel merges).  Returns [T, QH, V], or [QH, T, V] with ``head_major``,
    in ``out_dtype``.  Scores, softmax and the value sums are fp32."""
    T, QH, D = q.shape
    KH, bs = k_cache.shape[1], k_cache.shape[2]
    vc = k_cache if v_cache is None else v_cache
    VH = vc.shape[1]
    out = torch.empty((QH, T, V) if head_major else (T, QH, V), dtype=out_dtype, device=q.device)
    assert QH % KH == 0 and QH % VH == 0 and k_cache.shape[3] == D and V <= vc.shape[3]
    if not q.is_cuda:
        o3 = out.transpose(0, 1) if head_major else out
        for s in range(n_seqs):
            a, b, ctx = int(cu_q[s]), int(cu_q[s + 1]), int(context_lens[s])
            if b <= a:
                continue
            idx = torch.arange(ctx)
            blk = block_tables[s].long()[idx // bs]
            k = k_cache[blk, :, idx % bs, :].float().repeat_interleave(QH // KH, 1)           # [ctx, QH, D]
            v = vc[blk, :, idx % bs, :V].float().repeat_interleave(QH // VH, 1)               # [ctx, QH, V]
            sc = torch.einsum("thd,jhd->htj", q[a:b].float(), k) * scale
            pos = ctx - (b - a) + torch.arange(b - a)
            lo = torch.zeros_like(pos)
            if window > 0:
                lo = torch.maximum(lo, pos - window + 1)
            if chunk > 0:
                lo = torch.maximum(lo, pos // chunk * chunk)
            seen = (idx[None, :] <= pos[:, None]) & (idx[None, :] >= lo[:, None])
            sc = sc.masked_fill(~seen[None], float("-inf"))
            m = sc.amax(-1, keepdim=True)
            if sink is not None:
                m = torch.maximum(m, sink[:, None, None])
            e = torch.exp(sc - m)
            den = e.sum(-1, keepdim=True)
            if sink is not None:
                den = den + torch.exp(sink[:, None, None] - m)
            o3[a:b] = torch.einsum("htj,jhv->thv", e / den, v).to(out_dtype)
        return out
    assert q.is_contiguous() and k_cache.is_contiguous() and vc.is_contiguous() and vc.dtype == k_cache.dtype
    assert block_tables.stride(1) == 1 and (sink is None or (sink.dtype == torch.float32 and sink.numel() == QH))
    assert q.dtype in (torch.float32, k_cache.dtype)
    ts, hs = (V, T * V) if head_major else (QH * V, V)
    nd = min(num_decode, n_seqs)
    ws_o = ws_ml = None
    part = n_parts = 0
    if nd and q.dtype == k_cache.dtype:
        capacity = block_tables.shape[1] * bs
        part = native.mixers().pkm_masked_decode_part(nd, QH, KH, D, V, int(v_cache is None), bs, capacity, int(window),
                                                      int(chunk), native.dt_code(k_cache.dtype))
        if part > 0:
            span = capacity
            if window > 0:
                span = min(span, window + 31)
            if chunk > 0:
                span = min(span, chunk + 31)
            n_parts = -(-((span + 31) // 32 * 32) // part)
            if n_parts > 1:
                ws_o = torch.empty((nd, n_parts, QH, V), dtype=torch.float32, device=q.device)
                ws_ml = torch.empty((nd, n_parts, QH, 2), dtype=torch.float32, device=q.device)
    native.call("pkm_masked_attention", out.data_ptr(), ts, hs, native.dt_code(out_dtype), q.data_ptr(),
                native.dt_code(q.dtype), k_cache.data_ptr(), vc.data_ptr(), vc.shape[3], block_tables.data_ptr(),
                block_tables.stride(0), cu_q.data_ptr(), context_lens.data_ptr(), native.ptr(sink), n_seqs, T, QH, KH, VH,
                D, V, bs, float(scale), int(window), int(chunk), nd, native.ptr(ws_o), native.ptr(ws_ml), part, n_parts,
                native.dt_code(k_cache.dtype), native.stream_ptr())
    return out


def latent_in(proj: torch.Tensor, q_rank: int, R: int, Dr: int, wq: Optional[torch.Tensor], wkv: torch.Tensor, eps: float,
              positions: torch.Tensor, slot_mapping: torch.Tensor, table: Optional[torch.Tensor], halves: bool,
              cache: torch.Tensor) -> Optional[torch.Tensor]:
    """proj [T, q_rank | R | Dr]: the query latent set to unit RMS times ``wq`` is returned
    ([T, q_rank], the projection's dtype; None with q_rank = 0); the key / value latent set to unit
    RMS times ``wkv`` and the shared key part turned by the position go to cache rows
    [blocks, 1, block_size, R + Dr]."""
    T = proj.shape[0]
    cq = torch.empty((T, q_rank), dtype=proj.dtype, device=proj.device) if q_rank else None
    if not proj.is_cuda:
        f = proj.float()
        unit = lambda t: t / torch.sqrt((t * t).mean(-1, keepdim=True) + eps)
        if q_rank:
            cq.copy_(unit(f[:, :q_rank]) * wq)
        c = unit(f[:, q_rank:q_rank + R]) * wkv
        kr = f[:, q_rank + R:].view(T, 1, Dr)
        if table is not None and Dr:
            kr = turn(kr, table[positions.long()], halves)
        _write_cache(cache, torch.cat([c, kr[:, 0]], -1)[:, None, :], slot_mapping)
        return cq
    assert proj.stride(1) == 1 and proj.shape[1] == q_rank + R + Dr and cache.is_contiguous() and cache.dtype == proj.dtype
    assert cache.shape[1] == 1 and cache.shape[3] == R + Dr and wkv.dtype == torch.float32
    assert table is None or (table.dtype == torch.float32 and 2 * table.shape[1] <= Dr)
    native.call("pkm_latent_in", native.ptr(cq), cache.data_ptr(), proj.data_ptr(), proj.stride(0), q_rank, R, Dr,
                native.ptr(wq), wkv.data_ptr(), float(eps), positions.data_ptr(), slot_mapping.data_ptr(),
                native.ptr(table), table.shape[1] if table is not None else 0, table.shape[0] if table is not None else 0,
                int(halves), T, cache.shape[2], native.dt_code(proj.dtype), native.stream_ptr())
    return cq


def latent_query(q_lat: torch.Tensor, q: torch.Tensor, D: int, Dr: int, positions: torch.Tensor,
                 table: Optional[torch.Tensor], halves: bool) -> torch.Tensor:
    """q_lat [H, T, R] (queries folded into the latent space), q [T, H, D + Dr]: returns
    [T, H, R + Dr] = the folded query beside the head's rotated part turned by the position, in
    the same element type."""
    H, T, R = q_lat.shape
    out = torch.empty((T, H, R + Dr), dtype=q.dtype, device=q.device)
    if not q.is_cuda:
        out[..., :R] = q_lat.transpose(0, 1)
        qr = q.float().view(T, H, D + Dr)[..., D:]
        out[..., R:] = (turn(qr, table[positions.long()], halves) if (table is not None and Dr) else qr).to(q.dtype)
        return out
    assert q_lat.is_contiguous() and q.is_contiguous() and q.dtype == q_lat.dtype
    native.call("pkm_latent_query", out.data_ptr(), q_lat.data_ptr(), q.data_ptr(), positions.data_ptr(),
                native.ptr(table), table.shape[1] if table is not None else 0, table.shape[0] if table is not None else 0,
                int(halves), T, H, R, D, Dr, native.dt_code(q.dtype), native.stream_ptr())
    return out


GATE_NONE, GATE_SIGMOID, GATE_SILU = 0, 1, 2


def head_norm_gate(a: torch.Tensor, H: int, V: int, eps: float, gate: Optional[torch.Tensor], gate_kind: int,
                   dtype: torch.dtype, weight: Optional[torch.Tensor] = None, post: float = 1.0, pair_group: int = 0,
                   coef: float = 0.0, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Per (token, head): u / sqrt(mean(u^2) + eps) * weight * post * act(gate) -> [T, H * V] in
    ``dtype``.  ``a`` fp32: [T, H, V] with u = a[t, h]; or with ``pair_group`` = r > 0 it is
    [T, 2H, V] laid out in groups of (r first maps, r second maps) and u = first - coef * second
    (head h = g r + j reads rows g 2r + j and g 2r + r + j).  ``gate`` [T, H * V] pre-activations
    (may be a column slice), ``weight`` fp32 [V] shared by the heads, [H * V] one per head, or None.
    ``out``: write there ([T, H * V], may be a column slice)."""
    T = a.shape[0]
    if out is None:
        out = torch.empty((T, H * V), dtype=dtype, device=a.device)
    per_head = weight is not None and weight.numel() == H * V and H > 1
    if not a.is_cuda:
        if pair_group:
            r = pair_group
            a5 = a.view(T, H // r, 2, r, V)
            u = (a5[:, :, 0] - coef * a5[:, :, 1]).reshape(T, H, V)
        else:
            u = a.view(T, H, V)
        z = u / torch.sqrt((u * u).mean(-1, keepdim=True) + eps) * post
        if weight is not None:
            z = z * (weight.view(H, V) if per_head else weight)
        z = z.reshape(T, H * V)
        if gate_kind == GATE_SIGMOID:
            z = z * torch.sigmoid(gate.float())
        elif gate_kind == GATE_SILU:
            z = z * torch.nn.functional.silu(gate.float())
        out.copy_(z)
        return out
    assert a.dtype == torch.float32 and a.is_contiguous() and (gate is None or gate.stride(1) == 1)
    assert weight is None or (weight.dtype == torch.float32 and weight.numel() in (V, H * V))
    assert out.stride(1) == 1 and out.shape == (T, H * V)
    native.call("pkm_head_norm_gate", out.data_ptr(), out.stride(0), a.data_ptr(), T, H, V, float(eps), native.ptr(gate),
                gate.stride(0) if gate is not None else 0, native.dt_code(gate.dtype) if gate is not None else 1,
                int(gate_kind if gate is not None else GATE_NONE), native.ptr(weight), V if per_head else 0, float(post),
                int(pair_group), float(coef), native.dt_code(out.dtype), native.stream_ptr())
    return out
