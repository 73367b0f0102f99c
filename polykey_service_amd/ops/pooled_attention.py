"""Sliding-window softmax attention that also sees block means of the keys and values behind the
window, with a score cap, sink logits and mixing of the heads' softmax weights
(csrc/mixers/pooled_attention.hip; PyTorch on CPU).

A query at position p sees single keys j with max(0, p - window + 1) <= j <= p (window 0: all) and,
for every block b of ``pool`` positions with b pool + pool - 1 <= p - window, one key and value: the
mean of the block's cached keys / values.  With s = cap tanh(q . k scale / cap) (cap 0: uncapped),

    p_j = exp(s_j) / (exp(sink_h) + sum over the visible keys and blocks of exp(s_j'))
    o_h = sum_g talk[h, g] sum_j p_(g, j) v_(kv(h), j)            kv(h) = h // (H / G)

The block means live in a second pair of paged caches with the geometry of the first: block b of a
sequence is entry b of that sequence's pages (b < tokens / pool, so the page is always one the
sequence owns).  ``pool_update`` writes the mean of a block when the step brings its last position,
reading the block's rows from the cache, so it does not matter which step brought the others.
Scores, softmax, means and value sums are fp32.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import native


def _rows(cache: torch.Tensor, bt: torch.Tensor, idx: torch.Tensor) -> torch.Tensor:
    bs = cache.shape[2]
    return cache[bt.long()[idx // bs], :, idx % bs, :].float()       # [n, heads, width]


def pool_update(k_cache: torch.Tensor, v_cache: torch.Tensor, kp_cache: torch.Tensor, vp_cache: torch.Tensor,
                positions: torch.Tensor, token_seq: torch.Tensor, block_tables: torch.Tensor, pool: int,
                slot_mapping: Optional[torch.Tensor] = None) -> None:
    """For every token of the step at the last position of a block of ``pool``: the mean of the
    block's rows of k_cache / v_cache goes to entry position // pool of kp_cache / vp_cache (after
    the step's rows are in the caches).  Caches are [blocks, heads, block_size, width].  Tokens whose
    ``slot_mapping`` entry is negative cache nothing (padded rows of a decode graph) and are skipped."""
    T = positions.numel()
    if pool <= 0 or T == 0:
        return
    bs = k_cache.shape[2]
    if not k_cache.is_cuda:
        for t in range(T):
            p = int(positions[t])
            if (p + 1) % pool or (slot_mapping is not None and int(slot_mapping[t]) < 0):
                continue
            bt = block_tables[int(token_seq[t])]
            idx = torch.arange(p - pool + 1, p + 1)
            b = p // pool
            page = int(bt[b // bs])
            kp_cache[page, :, b % bs, :] = _rows(k_cache, bt, idx).mean(0).to(kp_cache.dtype)
            vp_cache[page, :, b % bs, :] = _rows(v_cache, bt, idx).mean(0).to(vp_cache.dtype)
        return
    assert k_cache.shape == kp_cache.shape and v_cache.shape == vp_cache.shape and block_tables.stride(1) == 1
    native.call("pkm_pool_update", k_cache.data_ptr(), v_cache.data_ptr(), kp_cache.data_ptr(), vp_cache.data_ptr(),
                positions.data_ptr(), native.ptr(slot_mapping), token_seq.data_ptr(), block_tables.data_ptr(),
                block_tables.stride(0), T,
                k_cache.shape[1], k_cache.shape[3], v_cache.shape[3], bs, int(pool), native.dt_code(k_cache.dtype),
                native.stream_ptr())


def visible_blocks(pos: int, window: int, pool: int) -> int:
    """Number of blocks of ``pool`` positions that lie wholly before the window of a query at ``pos``."""
    if window <= 0 or pool <= 0:
        return 0
    return max(0, (pos - window + 1) // pool)


def pooled_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, kp_cache: Optional[torch.Tensor],
                     vp_cache: Optional[torch.Tensor], block_tables: torch.Tensor, cu_q: torch.Tensor,
                     context_lens: torch.Tensor, n_seqs: int, scale: float, softcap: float = 0.0, window: int = 0,
                     pool: int = 0, sink: Optional[torch.Tensor] = None, all_values: bool = False) -> torch.Tensor:
    """q [T, H, D]; sequence s owns tokens cu_q[s]:cu_q[s+1], the LAST ones of its context_lens[s]
    cached tokens.  Returns fp32 [T, H, VG, V]: the softmax weights of query head h applied to the
    values of every key / value head (``all_values``: VG = G, what :func:`mix_heads` needs to mix
    the weights across heads) or of its own (VG = 1)."""
    T, H, D = q.shape
    G, bs, V = k_cache.shape[1], k_cache.shape[2], v_cache.shape[3]
    VG = G if all_values else 1
    out = torch.empty((T, H, VG, V), dtype=torch.float32, device=q.device)
    assert H % G == 0 and k_cache.shape[3] == D
    if window <= 0 or kp_cache is None:
        pool = 0
    rep = H // G
    if not q.is_cuda:
        for s in range(n_seqs):
            a, b, ctx = int(cu_q[s]), int(cu_q[s + 1]), int(context_lens[s])
            if b <= a:
                continue
            bt = block_tables[s]
            k, v = _rows(k_cache, bt, torch.arange(ctx)), _rows(v_cache, bt, torch.arange(ctx))
            pos = ctx - (b - a) + torch.arange(b - a)
            nb = visible_blocks(int(pos[-1]), window, pool)
            if nb:
                k = torch.cat([_rows(kp_cache, bt, torch.arange(nb)), k], 0)
                v = torch.cat([_rows(vp_cache, bt, torch.arange(nb)), v], 0)
            sc = torch.einsum("thd,jhd->htj", q[a:b].float(), k.repeat_interleave(rep, 1)) * scale
            if softcap > 0:
                sc = softcap * torch.tanh(sc / softcap)
            j = torch.arange(ctx)
            lo = torch.clamp(pos - window + 1, min=0) if window > 0 else torch.zeros_like(pos)
            seen = (j[None, :] <= pos[:, None]) & (j[None, :] >= lo[:, None])
            if nb:
                nvis = torch.tensor([visible_blocks(int(p), window, pool) for p in pos])
                seen = torch.cat([torch.arange(nb)[None, :] < nvis[:, None], seen], 1)
            sc = sc.masked_fill(~seen[None], float("-inf"))
            m = sc.amax(-1, keepdim=True)
            if sink is not None:
                m = torch.maximum(m, sink[:, None, None])
            m = torch.where(torch.isinf(m), torch.zeros_like(m), m)
            e = torch.exp(sc - m)
            den = e.sum(-1, keepdim=True)
            if sink is not None:
                den = den + torch.exp(sink[:, None, None] - m)
            w = e / torch.where(den > 0, den, torch.ones_like(den))
            if all_values:
                out[a:b] = torch.einsum("htj,jgv->thgv", w, v)
            else:
                out[a:b, :, 0] = torch.einsum("htj,jhv->thv", w, v.repeat_interleave(rep, 1))
        return out
    assert q.is_contiguous() and q.dtype == k_cache.dtype == v_cache.dtype and k_cache.is_contiguous() and v_cache.is_contiguous()
    assert block_tables.stride(1) == 1 and (sink is None or (sink.dtype == torch.float32 and sink.numel() == H))
    assert pool == 0 or (kp_cache.shape == k_cache.shape and vp_cache.shape == v_cache.shape)
    # few row tiles (decoded tokens): the key tiles of a row tile are dealt to several workgroups and merged
    tiles = (-(-T * rep // 16) + n_seqs) * G
    span = block_tables.shape[1] * bs if window <= 0 else min(block_tables.shape[1] * bs, window + 64)
    n_parts = max(1, min(16, 1024 // tiles, span // 64))
    ws_acc = ws_ml = None
    if n_parts > 1:
        ws_acc = torch.empty((T * H, n_parts, VG * V), dtype=torch.float32, device=q.device)
        ws_ml = torch.empty((T * H, n_parts, 2), dtype=torch.float32, device=q.device)
    native.call("pkm_pooled_attention", out.data_ptr(), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                native.ptr(kp_cache) if pool else None, native.ptr(vp_cache) if pool else None, block_tables.data_ptr(),
                block_tables.stride(0), cu_q.data_ptr(), context_lens.data_ptr(), native.ptr(sink), n_seqs, T, H, G, D, V,
                bs, float(scale), float(softcap), int(window), int(pool), int(all_values), n_parts, native.ptr(ws_acc),
                native.ptr(ws_ml), native.dt_code(q.dtype), native.stream_ptr())
    return out


def mix_heads(o: torch.Tensor, talk: Optional[torch.Tensor], post: float, dtype: torch.dtype,
              out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """o fp32 [T, H, VG, V] from :func:`pooled_attention`.  With ``talk`` [H, H] fp32 (VG = G):
    out[t, h] = post * sum_g talk[h, g] o[t, g, h // (H / G)]; without (VG = 1): post * o[t, h, 0].
    Returns [T, H * V] in ``dtype`` (``out``: write there; it may be a column slice)."""
    T, H, VG, V = o.shape
    if out is None:
        out = torch.empty((T, H * V), dtype=dtype, device=o.device)
    assert out.shape == (T, H * V) and (talk is not None or VG == 1)
    if not o.is_cuda:
        if talk is None:
            out.copy_((post * o[:, :, 0]).reshape(T, H * V))
        else:
            own = o[:, :, torch.arange(H) // (H // VG)]                      # [T, g, h, V]: weights of g on h's values
            out.copy_((post * torch.einsum("hg,tghv->thv", talk, own)).reshape(T, H * V))
        return out
    assert o.dtype == torch.float32 and o.is_contiguous() and out.stride(1) == 1
    assert talk is None or (talk.dtype == torch.float32 and talk.is_contiguous() and talk.shape == (H, H))
    native.call("pkm_mix_heads", out.data_ptr(), out.stride(0), native.dt_code(out.dtype), o.data_ptr(), native.ptr(talk),
                T, H, VG, V, float(post), native.stream_ptr())
    return out
