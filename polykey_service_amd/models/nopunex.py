"""Nopunex decoder: an fp32 residual stream whose sublayers sit between two layer norms, three
kinds of mixers (differential chunked attention, windowed latent attention with a sink, gated delta
rule), SiLU-gated dense feed-forwards, and a block of layers that runs several times with the same
weights, each pass starting from a re-projection of the stream joined with the embedding.

Per layer run, for the step's tokens (x: fp32 stream [T, W]; a = the model's dtype, bf16 or fp32;
norms, the stream, rotations, scores, softmax, unit norms, decays and the recurrent state are fp32):

    pass start: x <- [x | x0] @ Win^T + step[pass]      x0 = the embedding rows      join_cast, GEMM, sandwich.hip
    h   = LN1(x) -> a                                                                 HIP  sandwich.hip
    attention:  qkvg = h @ [Wq; Wk; Wv; Wg]^T   (two maps per head: 2H query, 2G key heads)  hipBLASLt / decode GEMM
                q, k turned by the position (halves layout); k, v -> paged caches    HIP  masked_attention.hip
                a_m = softmax_j(q_m . k_m * scale) v  over the keys of the token's chunk
                o = unit_rms(a_1 - lambda a_2) (1 - diff) sigmoid(g)                 HIP  head_norm_gate
    latent:     dq | dkv = h @ [Wdq; Wdkv]^T ; c_q = unit_rms(dq) wq ; cache <- [unit_rms(c) wkv | turned key part]
                q = c_q @ Wuq^T ; q~ = [q_nope @ Wuk (per head) | turned q_rot]      hipBLASLt (batched), latent_query
                o~ = sum_j p_j c_j,  p = exp(s_j) / (exp(sink_h) + sum exp(s)), s = q~ . [c | k_rot] * scale,
                     over the last `window` keys ;  o = o~ @ Wuv^T (per head)        HIP  masked_attention.hip
    delta:      qkv | a | b | g = h @ [...]^T ; q, k, v = silu(filter(.)), q, k unit  HIP  delta.hip
                S <- gate S ; u = beta (v - S^T k) ; S += k u^T ; o = S^T q           (state [H, D, V] fp32 per slot)
                o = unit_rms(o) w silu(g)                                             HIP  head_norm_gate
    y   = o @ Wo^T
    x <- x + LN1b(y) ;  h2 = LN2(x) -> a                        (one kernel)          HIP  sandwich.hip
    f   = (silu(h2 @ Wgate^T) * (h2 @ Wup^T)) @ Wdown^T
    x <- x + LN2b(f) ;  the next run's h                        (one kernel)

and logits = head @ LN_final(x) * logit_scale.  Every layer run has its own cache (attention,
latent) or state (delta), also the passes of the repeated block.  Tensor parallelism is not
implemented for this family.
"""
from __future__ import annotations

import math
from typing import List, Optional

import torch
from torch import nn

from ..ops import delta as delta_ops
from ..ops import gemm
from ..ops import masked_attention as ma_ops
from ..ops import sandwich as sw_ops
from ..parallel.state import ParallelState
from .config import NopunexConfig
from .kivezen import _p, _packed, _project
from .weights import SafetensorsIndex, random_full


def _pad_rows(w: torch.Tensor) -> torch.Tensor:
    """Zero rows up to a multiple of 128 where the decode GEMM could then tile the projection (its
    input width a multiple of 256); the extra output columns are never read."""
    n, k = w.shape
    if k % 256 or n % 128 == 0:
        return w
    return torch.cat([w, w.new_zeros((128 - n % 128, k))], 0)


class DiffAttention(nn.Module):
    """Weights of one differential-attention mixer.  Query rows are stored per key / value group as
    (first maps of the group's heads, second maps of the group's heads): query "head" i of 2H then
    reads key head i // r of 2G and value head i // 2r of G, r = H / G."""

    def __init__(self, spec, width: int):
        super().__init__()
        self.spec, self.width = spec, width
        self.w_in = None   # [2H*D | 2G*D | G*V | H*V, W]: q (regrouped) | k | v | gate rows
        self.w_o = None    # [W, H*V]
        self.lam = 0.0     # exp(lq1 . lk1) - exp(lq2 . lk2) + diff
        self.table = None  # [positions, pairs, 2] fp32 (cos, sin); None: no rotation
        self.w_in_p = self.w_o_p = None

    def pack(self) -> None:
        self.w_in_p, self.w_o_p = _packed(self.w_in), _packed(self.w_o)

    def set(self, q, k, v, g, o, lq1, lk1, lq2, lk2, dtype, device) -> None:
        s = self.spec
        H, G, D, V, W = s.heads, s.kv_heads, s.dim, s.vdim, self.width
        assert q.shape == (2 * H * D, W) and k.shape == (2 * G * D, W) and v.shape == (G * V, W)
        assert g.shape == (H * V, W) and o.shape == (W, H * V)
        assert s.rot is None or (s.rot.dims % 2 == 0 and s.rot.dims <= D)
        r = H // G
        q = q.reshape(G, r, 2, D, W).permute(0, 2, 1, 3, 4).reshape(2 * H * D, W)
        self.w_in = _p(_pad_rows(torch.cat([q, k, v, g], 0)).to(device=device, dtype=dtype))
        self.w_o = _p(o.to(device=device, dtype=dtype))
        dot = lambda a, b: float((a.double().reshape(-1) * b.double().reshape(-1)).sum())
        self.lam = math.exp(dot(lq1, lk1)) - math.exp(dot(lq2, lk2)) + s.diff

    def forward(self, h: torch.Tensor, positions: torch.Tensor, md, cache: tuple, eps: float):
        s = self.spec
        H, G, D, V = s.heads, s.kv_heads, s.dim, s.vdim
        n = 2 * (H + G) * D + G * V
        proj = _project(h, self.w_in, self.w_in_p)
        q = ma_ops.rotate_cache(proj[:, :n], positions, md.slot_mapping, self.table, True, cache[0], cache[1],
                                2 * H, 2 * G, G, D, V)
        a = ma_ops.masked_attention(q, cache[0], cache[1], V, md.block_tables, md.cu_q, md.context_lens, md.num_seqs,
                                    s.scale, chunk=s.chunk, num_decode=md.num_decode)
        o = ma_ops.head_norm_gate(a, H, V, eps, proj[:, n:n + H * V], ma_ops.GATE_SIGMOID, h.dtype, post=1.0 - s.diff,
                                  pair_group=H // G, coef=self.lam)
        return _project(o, self.w_o, self.w_o_p, partial=True)


class WindowLatentAttention(nn.Module):
    """Weights of one latent-attention mixer with a query latent, a shared rotated key part, a
    sliding window and sink logits.  The cache row of a token is [latent | turned key part]."""

    def __init__(self, spec, width: int):
        super().__init__()
        self.spec, self.width = spec, width
        self.w_in = None     # [q_rank | R + Dr, W]: dq | dkv rows
        self.q_norm = self.kv_norm = None   # fp32 [q_rank], [R]
        self.uq = None       # [H*(D + Dr), q_rank]
        self.uk = None       # [H, D, R]
        self.uv_t = None     # [H, R, V]
        self.w_o = None      # [W, H*V]
        self.sink = None     # [H] fp32 logits
        self.table = None
        self.w_in_p = self.uq_p = self.w_o_p = None

    def pack(self) -> None:
        self.w_in_p, self.uq_p, self.w_o_p = _packed(self.w_in), _packed(self.uq), _packed(self.w_o)

    def set(self, dq, dq_norm, uq, dkv, dkv_norm, uk, uv, sink, o, dtype, device) -> None:
        s = self.spec
        H, D, Dr, V, R, Q, W = s.heads, s.dim, s.rot_dim, s.vdim, s.kv_rank, s.q_rank, self.width
        assert Q > 0 and dq.shape == (Q, W) and uq.shape == (H * (D + Dr), Q) and dkv.shape == (R + Dr, W)
        assert uk.shape == (H * D, R) and uv.shape == (H * V, R) and o.shape == (W, H * V)
        assert s.rot is None or (s.rot.dims % 2 == 0 and s.rot.dims <= Dr)
        to = lambda t: _p(t.to(device=device, dtype=dtype))
        f32 = lambda t: _p(t.to(device=device, dtype=torch.float32).reshape(-1))
        self.w_in, self.uq, self.w_o = to(_pad_rows(torch.cat([dq, dkv], 0))), to(uq), to(o)
        self.uk = to(uk.reshape(H, D, R))
        self.uv_t = to(uv.reshape(H, V, R).transpose(1, 2))
        self.q_norm, self.kv_norm, self.sink = f32(dq_norm), f32(dkv_norm), f32(sink)
        assert self.sink.numel() == H

    def forward(self, h: torch.Tensor, positions: torch.Tensor, md, cache: tuple, eps: float):
        s = self.spec
        H, D, Dr, V, R = s.heads, s.dim, s.rot_dim, s.vdim, s.kv_rank
        T = h.shape[0]
        proj = _project(h, self.w_in, self.w_in_p)
        cq = ma_ops.latent_in(proj[:, :s.q_rank + R + Dr], s.q_rank, R, Dr, self.q_norm, self.kv_norm, eps, positions, md.slot_mapping,
                              self.table, True, cache[0])
        q = _project(cq, self.uq, self.uq_p)
        q_lat = torch.bmm(q.view(T, H, D + Dr)[:, :, :D].transpose(0, 1), self.uk)                  # [H, T, R]
        qf = ma_ops.latent_query(q_lat, q, D, Dr, positions, self.table, True)
        o_lat = ma_ops.masked_attention(qf, cache[0], None, R, md.block_tables, md.cu_q, md.context_lens, md.num_seqs,
                                        s.scale, window=s.window, sink=self.sink if s.sink else None,
                                        out_dtype=h.dtype, head_major=True, num_decode=md.num_decode)                        # [H, T, R]
        o = torch.bmm(o_lat, self.uv_t).transpose(0, 1).reshape(T, H * V)
        return _project(o, self.w_o, self.w_o_p, partial=True)


class DeltaMixer(nn.Module):
    """Weights of one gated-delta-rule mixer."""

    def __init__(self, spec, width: int):
        super().__init__()
        self.spec, self.width = spec, width
        self.w_in = None    # [G*D | G*D | H*V | H | H | H*V, W]: q | k | v | a | b | gate rows
        self.taps = None    # [2 G D + H V, taps] fp32
        self.a_log = self.dt_bias = None   # [H] fp32
        self.norm_w = None  # [V] fp32
        self.w_o = None     # [W, H*V]
        self.w_in_p = self.w_o_p = None

    def pack(self) -> None:
        self.w_in_p, self.w_o_p = _packed(self.w_in), _packed(self.w_o)

    def set(self, q, k, v, a, b, g, o, qc, kc, vc, a_log, dt_bias, norm_w, dtype, device) -> None:
        s = self.spec
        H, G, D, V, K, W = s.heads, s.kv_heads, s.dim, s.vdim, s.conv, self.width
        assert q.shape == (G * D, W) == k.shape and v.shape == (H * V, W) == g.shape and o.shape == (W, H * V)
        assert a.shape == (H, W) == b.shape and qc.shape == (G * D, K) == kc.shape and vc.shape == (H * V, K)
        f32 = lambda t: _p(t.to(device=device, dtype=torch.float32).reshape(-1))
        self.w_in = _p(_pad_rows(torch.cat([q, k, v, a, b, g], 0)).to(device=device, dtype=dtype))
        self.w_o = _p(o.to(device=device, dtype=dtype))
        self.taps = _p(torch.cat([qc, kc, vc], 0).to(device=device, dtype=torch.float32))
        self.a_log, self.dt_bias, self.norm_w = f32(a_log), f32(dt_bias), f32(norm_w)
        assert self.a_log.numel() == H == self.dt_bias.numel() and self.norm_w.numel() == V

    def forward(self, h: torch.Tensor, positions: torch.Tensor, md, cache: tuple, eps: float):
        s = self.spec
        H, G, D, V = s.heads, s.kv_heads, s.dim, s.vdim
        C = 2 * G * D + H * V
        proj = _project(h, self.w_in, self.w_in_p)
        qkv = delta_ops.conv_unit(proj[:, :C], self.taps, cache[1], md.cu_q, md.num_seqs, positions, md.state_slots,
                                  md.token_seq, G, D, H, V)
        o = delta_ops.delta_rule(qkv, proj[:, C:C + 2 * H], self.a_log, self.dt_bias, cache[0], md.cu_q, md.num_seqs,
                                 positions, md.state_slots, G, D, H, V)
        z = ma_ops.head_norm_gate(o, H, V, eps, proj[:, C + 2 * H:C + 2 * H + H * V], ma_ops.GATE_SILU, h.dtype, weight=self.norm_w)
        return _project(z, self.w_o, self.w_o_p, partial=True)


class GatedFF(nn.Module):
    def __init__(self, spec):
        super().__init__()
        self.spec = spec
        self.w_in = self.down = self.w_in_p = self.down_p = None   # [gate | up rows, W], [W, F]

    def set(self, gate, up, down, dtype, device) -> None:
        self.w_in = _p(torch.cat([gate, up], 0).to(device=device, dtype=dtype))
        self.down = _p(down.to(device=device, dtype=dtype))

    def pack(self) -> None:
        self.w_in_p, self.down_p = _packed(self.w_in), _packed(self.down)

    def forward(self, h: torch.Tensor):
        a = sw_ops.silu_mul(_project(h, self.w_in, self.w_in_p, partial=True), self.spec.ff, h.dtype)
        return _project(a, self.down, self.down_p, partial=True)


_MIXERS = {"attention": DiffAttention, "latent_attention": WindowLatentAttention, "delta": DeltaMixer}


class NopunexLayer(nn.Module):
    def __init__(self, spec, width: int):
        super().__init__()
        self.kind = spec.type
        self.mix = _MIXERS[spec.type](spec.mixer, width)
        self.mlp = GatedFF(spec.mlp) if spec.mlp is not None else None
        # (weight, bias) fp32 of the norms before (norm1, norm2) and after (norm1b, norm2b) the sublayers
        self.norm1 = self.norm1b = self.norm2 = self.norm2b = None


class NopunexForCausalLM(nn.Module):
    # engine hooks (engine/model_runner.py): this family owns its cache and state layouts
    supports_graphs = True

    def __init__(self, cfg: NopunexConfig, st: ParallelState, dtype: torch.dtype, device: torch.device):
        super().__init__()
        if st.tp_size > 1 or getattr(st, "ep_size", 1) > 1:
            raise ValueError("Nopunex runs on one GPU (no TP / EP sharding for this family)")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"Nopunex runs in bfloat16 or float32, not {dtype}")
        self.cfg, self.st, self.dtype, self.device = cfg, st, dtype, device
        self.needs_state = cfg.needs_state
        self.layers = nn.ModuleList(NopunexLayer(l, cfg.hidden_size) for l in cfg.layers)
        self.embed = self.head = self.final_norm = None
        self.loop_in = self.loop_in_p = self.loop_step = None   # [W, 2W], [passes, W] fp32
        self._max_pos = 0

    # ------------------------------------------------------------------ weights
    def _norm(self, get, name: str) -> tuple:
        W, dev = self.cfg.hidden_size, self.device
        w, b = get(name), get(name + ".b")
        assert w.numel() == W == b.numel(), name
        return (_p(w.to(device=dev, dtype=torch.float32).reshape(-1)), _p(b.to(device=dev, dtype=torch.float32).reshape(-1)))

    def _set_layer(self, i: int, get) -> None:
        L, spec = self.layers[i], self.cfg.layers[i]
        p, dev, dt, W = f"l{i}.", self.device, self.dtype, self.cfg.hidden_size
        m = lambda n: get(p + "mix." + n)
        if L.kind == "attention":
            L.mix.set(m("q"), m("k"), m("v"), m("g"), m("o"), m("lq1"), m("lk1"), m("lq2"), m("lk2"), dt, dev)
        elif L.kind == "latent_attention":
            L.mix.set(m("dq"), m("dq.norm"), m("uq"), m("dkv"), m("dkv.norm"), m("uk"), m("uv"), m("sink"), m("o"), dt, dev)
        else:
            L.mix.set(m("q"), m("k"), m("v"), m("a"), m("b"), m("g"), m("o"), m("q.conv"), m("k.conv"), m("v.conv"),
                      m("A_log"), m("dt_bias"), m("norm"), dt, dev)
        L.norm1, L.norm1b = self._norm(get, p + "norm1"), self._norm(get, p + "norm1b")
        if spec.mlp is not None:
            L.norm2, L.norm2b = self._norm(get, p + "norm2"), self._norm(get, p + "norm2b")
            gate, up, down = get(p + "mlp.gate"), get(p + "mlp.up"), get(p + "mlp.down")
            assert gate.shape == (spec.mlp.ff, W) == up.shape and down.shape == (W, spec.mlp.ff)
            L.mlp.set(gate, up, down, dt, dev)

    def _set_top(self, get) -> None:
        cfg, dev, dt, W = self.cfg, self.device, self.dtype, self.cfg.hidden_size
        self.embed = _p(get("embed").to(device=dev, dtype=dt))
        self.head = _p(get("head").to(device=dev, dtype=dt))
        self.final_norm = self._norm(get, "final.norm")
        assert self.embed.shape == (cfg.vocab_size, W) == self.head.shape
        if cfg.looped:
            w_in, step = get("loop.in"), get("loop.step")
            assert w_in.shape == (W, 2 * W) and step.shape == (cfg.loop[2], W)
            self.loop_in = _p(w_in.to(device=dev, dtype=dt))
            self.loop_step = _p(step.to(device=dev, dtype=torch.float32))

    def load_hf(self, path: str) -> "NopunexForCausalLM":
        """Load a checkpoint folder (safetensors; tensors under the design's own names)."""
        return self._load(SafetensorsIndex(path).get)

    def load_state(self, tensors: dict) -> "NopunexForCausalLM":
        """The same from a dict name -> tensor (tests)."""
        return self._load(tensors.__getitem__)

    def _load(self, get) -> "NopunexForCausalLM":
        self._set_top(get)
        for i in range(len(self.layers)):
            self._set_layer(i, get)
        if self._max_pos:
            self._build_tables()
        return self

    def random_state(self, seed: int = 0) -> dict:
        """Random bf16-representable tensors under the checkpoint names (norm weights near 1)."""
        cfg, W, std = self.cfg, self.cfg.hidden_size, self.cfg.init_std
        r = lambda name, shape, s=std: random_full(name, shape, s, seed, self.device, torch.bfloat16)
        out = {"embed": r("embed", (cfg.vocab_size, W), 1.0), "head": r("head", (cfg.vocab_size, W))}

        def norm(name):
            out[name], out[name + ".b"] = 1 + r(name, (W,), 0.1), r(name + ".b", (W,), 0.1)
        norm("final.norm")
        if cfg.looped:
            out["loop.in"] = r("loop.in", (W, 2 * W), (2 * W) ** -0.5)
            out["loop.step"] = r("loop.step", (cfg.loop[2], W), 0.1)
        for i, l in enumerate(cfg.layers):
            p, m = f"l{i}.", l.mixer
            for q in ["1", "1b"] + (["2", "2b"] if l.mlp is not None else []):
                norm(p + "norm" + q)
            t = lambda n, shape, s=std: out.__setitem__(p + "mix." + n, r(p + "mix." + n, shape, s))
            if l.type == "attention":
                t("q", (2 * m.heads * m.dim, W)), t("k", (2 * m.kv_heads * m.dim, W)), t("v", (m.kv_heads * m.vdim, W))
                t("g", (m.heads * m.vdim, W)), t("o", (W, m.heads * m.vdim))
                for n in ("lq1", "lk1", "lq2", "lk2"):
                    t(n, (m.dim,), 0.1)
            elif l.type == "latent_attention":
                t("dq", (m.q_rank, W)), t("uq", (m.heads * (m.dim + m.rot_dim), m.q_rank))
                t("dkv", (m.kv_rank + m.rot_dim, W)), t("uk", (m.heads * m.dim, m.kv_rank))
                t("uv", (m.heads * m.vdim, m.kv_rank)), t("o", (W, m.heads * m.vdim)), t("sink", (m.heads,), 1.0)
                out[p + "mix.dq.norm"] = 1 + r(p + "mix.dq.norm", (m.q_rank,), 0.1)
                out[p + "mix.dkv.norm"] = 1 + r(p + "mix.dkv.norm", (m.kv_rank,), 0.1)
            else:
                t("q", (m.kv_heads * m.dim, W)), t("k", (m.kv_heads * m.dim, W)), t("v", (m.heads * m.vdim, W))
                t("a", (m.heads, W)), t("b", (m.heads, W)), t("g", (m.heads * m.vdim, W)), t("o", (W, m.heads * m.vdim))
                t("q.conv", (m.kv_heads * m.dim, m.conv), 0.5), t("k.conv", (m.kv_heads * m.dim, m.conv), 0.5)
                t("v.conv", (m.heads * m.vdim, m.conv), 0.5), t("A_log", (m.heads,), 0.5), t("dt_bias", (m.heads,), 0.5)
                out[p + "mix.norm"] = 1 + r(p + "mix.norm", (m.vdim,), 0.1)
            if l.mlp is not None:
                for n, shape in (("gate", (l.mlp.ff, W)), ("up", (l.mlp.ff, W)), ("down", (W, l.mlp.ff))):
                    out[p + "mlp." + n] = r(p + "mlp." + n, shape)
        return out

    def init_random(self, seed: int = 0) -> "NopunexForCausalLM":
        return self.load_state(self.random_state(seed))

    def pack_decode_weights(self) -> None:
        """Block-packed copies of the projections for the decode GEMM (engine hook)."""
        for L in self.layers:
            L.mix.pack()
            if L.mlp is not None:
                L.mlp.pack()
        if self.loop_in is not None:
            self.loop_in_p = _packed(self.loop_in)

    def to(self, device, *a, **k):  # keeps the fp32 tensors fp32 (no dtype argument)
        super().to(device)
        self.device = torch.device(device)
        for L in self.layers:
            for n in ("norm1", "norm1b", "norm2", "norm2b"):
                if getattr(L, n) is not None:
                    setattr(L, n, tuple(t.to(device) for t in getattr(L, n)))
        self.final_norm = tuple(t.to(device) for t in self.final_norm) if self.final_norm is not None else None
        if self._max_pos:
            self._build_tables()
        return self

    # ------------------------------------------------------- rotations, cache and state
    def reserve_positions(self, max_pos: int) -> None:
        """Build the rotation tables for positions below ``max_pos`` (engine hook: max_model_len)."""
        if max_pos > self._max_pos:
            self._max_pos = max_pos
            if self.embed is not None:
                self._build_tables()

    def _build_tables(self) -> None:
        made = {}
        for L in self.layers:
            rot = getattr(L.mix.spec, "rot", None)
            if rot is None:
                continue
            if rot not in made:
                made[rot] = ma_ops.table_for(rot, self._max_pos, self.device)
            L.mix.table = made[rot]

    def _cache_row(self, i: int) -> int:
        m, kind = self.cfg.layers[i].mixer, self.cfg.layers[i].type
        if kind == "attention":
            return m.kv_heads * (2 * m.dim + m.vdim)
        return m.kv_rank + m.rot_dim if kind == "latent_attention" else 0

    def cache_bytes_per_block(self, block_size: int) -> int:
        esz = 2 if self.dtype == torch.bfloat16 else 4
        return max(sum(self._cache_row(i) for i, _, _ in self.cfg.runs) * block_size * esz, 1)

    def state_bytes_per_slot(self) -> int:
        n = 0
        for i, _, _ in self.cfg.runs:
            m = self.cfg.layers[i].mixer
            if self.cfg.layers[i].type == "delta":
                n += m.heads * m.dim * m.vdim + max(m.conv - 1, 1) * (2 * m.kv_heads * m.dim + m.heads * m.vdim)
        return n * 4

    def alloc_cache(self, num_blocks: int, block_size: int, num_slots: int) -> List[tuple]:
        """Per layer run: (keys [blocks, 2G, block_size, D], values [blocks, G, block_size, V]) for
        attention, (rows [blocks, 1, block_size, R + Dr],) for latent attention, (memory
        [slots, H, D, V] fp32, filter inputs [slots, taps - 1, C] fp32) for the delta rule."""
        out, dev = [], self.device
        for i, _, _ in self.cfg.runs:
            m, kind = self.cfg.layers[i].mixer, self.cfg.layers[i].type
            if kind == "attention":
                out.append((torch.zeros((num_blocks, 2 * m.kv_heads, block_size, m.dim), dtype=self.dtype, device=dev),
                            torch.zeros((num_blocks, m.kv_heads, block_size, m.vdim), dtype=self.dtype, device=dev)))
            elif kind == "latent_attention":
                out.append((torch.zeros((num_blocks, 1, block_size, m.kv_rank + m.rot_dim), dtype=self.dtype, device=dev),))
            else:
                C = 2 * m.kv_heads * m.dim + m.heads * m.vdim
                out.append((torch.zeros((max(num_slots, 1), m.heads, m.dim, m.vdim), dtype=torch.float32, device=dev),
                            torch.zeros((max(num_slots, 1), max(m.conv - 1, 1), C), dtype=torch.float32, device=dev)))
        return out

    def activation_bytes_per_token(self) -> int:
        W, widest = self.cfg.hidden_size, 2 * self.cfg.hidden_size
        for l in self.cfg.layers:
            m = l.mixer
            if l.type == "attention":
                n = 2 * (m.heads + m.kv_heads) * m.dim + m.kv_heads * m.vdim + m.heads * m.vdim + 2 * (
                    2 * m.heads * (m.dim + m.vdim))
            elif l.type == "latent_attention":
                n = 2 * m.q_rank + m.kv_rank + m.rot_dim + m.heads * (m.dim + m.rot_dim) + 4 * m.heads * (
                    m.kv_rank + m.rot_dim) + 2 * m.heads * m.vdim
            else:
                n = 4 * (2 * m.kv_heads * m.dim + 2 * m.heads * m.vdim) + 2 * m.heads
            if l.mlp is not None:
                n = max(n, 3 * l.mlp.ff)
            widest = max(widest, n)
        return 4 * W * 6 + 4 * widest

    # ------------------------------------------------------------------ forward
    @torch.inference_mode()
    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor, md, caches: List[tuple]) -> torch.Tensor:
        """The fp32 stream [T, W] after the last layer run, for the step described by ``md``
        (ops/attention.py AttnMetadata: the whole-batch fields)."""
        cfg, eps, dt = self.cfg, self.cfg.rms_eps, self.dtype
        if positions.numel() and self._max_pos == 0:
            raise RuntimeError("Nopunex: reserve_positions(max_model_len) has not been called")
        runs = cfg.runs
        x0 = sw_ops.embed_rows_f32(self.embed, input_ids)
        x = x0.clone() if cfg.looped else x0
        h = None
        for r, (li, t, first) in enumerate(runs):
            L = self.layers[li]
            if first:  # a pass of the repeated block starts: re-project the stream joined with the embedding
                y = _project(sw_ops.join_cast(x, x0, dt), self.loop_in, self.loop_in_p, partial=True)
                h = sw_ops.sandwich_step(x, y, None, L.norm1, eps, dt, replace=True, add=self.loop_step[t])
            elif h is None:
                h = sw_ops.sandwich_step(x, None, None, L.norm1, eps, dt)
            y = L.mix(h, positions, md, caches[r], eps)
            nxt = None
            if r + 1 < len(runs) and not runs[r + 1][2]:
                nxt = self.layers[runs[r + 1][0]].norm1
            if L.mlp is not None:
                h2 = sw_ops.sandwich_step(x, y, L.norm1b, L.norm2, eps, dt)
                h = sw_ops.sandwich_step(x, L.mlp(h2), L.norm2b, nxt, eps, dt)
            else:
                h = sw_ops.sandwich_step(x, y, L.norm1b, nxt, eps, dt)
        return x

    def compute_logits(self, rows: torch.Tensor) -> torch.Tensor:
        """fp32 logits of stream rows [n, W]: the final norm, the head, the logit scale."""
        act = sw_ops.sandwich_step(rows.contiguous(), None, None, self.final_norm, self.cfg.rms_eps, self.dtype)
        logits = gemm.linear(act, self.head).float()
        return sw_ops.scale_(logits, self.cfg.logit_scale)
