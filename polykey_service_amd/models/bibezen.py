"""Bibezen decoder: pre-norm layers on one or several fp32 residual streams (hyper-connections) with
scaled sublayer outputs; the mixer's input passes a short causal filter with a skip; mixers are wkv
time mixing, a selective scan, or pooled-window attention beside wkv; feed-forwards are a clamped
GLU or a softmax-routed mixture of SiLU experts with a shared expert.

Per layer, for the step's tokens (xs: fp32 streams [T, S, W]; a = the model's dtype, bf16 or fp32;
norms, the streams, rotations, scores, softmax, routers, step sizes, decays and recurrent states
are fp32):

    h   = N1(sum_s in1[s] xs[s]) -> a ;  h <- h + filter(h)                   HIP  hyper.hip, short_conv.hip
    wkv:       mixes of h with the previous token's h, one per projection      HIP  wkv.hip
               r, k, v, g = mix_n @ W_n^T ; z = tanh(mix_w @ W1^T) @ W2^T      hipBLASLt / decode GEMM
               o = (S + diag(u) k v^T)^T r ; S <- diag(exp(-exp(z + w0))) S + k v^T   (state [H, D, D] fp32 per slot)
               o = unit_rms_per_head(o) * w * silu(g)                          HIP  head_norm_gate
    mamba1:    x | z = h @ Win^T ; x = silu(filter(x) + b) ; dt | B | C = x @ Wx^T ; d = dt @ Wdt^T
               S <- exp(softplus(d + b_dt) A) S + softplus(.) x B ; y = S C + D x ; y silu(z)     HIP  scan.hip
    parallel:  left  q | k | v = filter(h @ [Wq; Wk; Wv]^T + bias) ; q, k unit RMS per head times a
                     weight, turned by the position ; k, v -> paged caches ; block means -> their pages
                     softmax over the window's keys and the block means behind it, capped scores, a sink,
                     the heads' weights mixed by `talk`                        HIP  pooled_attention.hip
               right wkv as above
               o = [left_scale * left | right_scale * right] -> one output projection
    y   = o @ Wo^T
    xs'[t] = sum_s mix1[s, t] xs[s] + m out1[t] y ;  h2 = N2(sum_t in2[t] xs'[t])        (one kernel)
    dense:     f = (g' sigmoid(1.702 g') (u' + 1)) @ Wdown^T,  g' = min(h2 Wgate^T, L), u' = clamp(h2 Wup^T, -L, L)
    moe:       z = Wr h2 (fp32) ; top experts by z, weights softmax over the chosen z
               f = sum_e w_e down_e(silu(gate_e h2) * up_e h2) + shared(h2)
    xs''[t] = sum_s mix2[s, t] xs'[s] + m out2[t] f ; the next layer's h                 (one kernel)

and logits = embed @ N_final(sum_s xs[s]), N_w(u) = u / sqrt(mean(u^2) + eps) * (1 + w).  A model
without ``streams`` is the same with S = 1 and unit coefficients.  Tensor parallelism is not
implemented for this family.
"""
from __future__ import annotations

from typing import List, Optional

import torch
from torch import nn

from ..ops import gemm
from ..ops import hyper as hyper_ops
from ..ops import masked_attention as ma_ops
from ..ops import moe as moe_ops
from ..ops import pooled_attention as pa_ops
from ..ops import sandwich as sw_ops
from ..ops import scan as scan_ops
from ..ops import short_conv as conv_ops
from ..ops import wkv as wkv_ops
from ..parallel.state import ParallelState
from .config import BibezenConfig, ClampedFFSpec, SoftmaxMoESpec
from .kivezen import _p, _packed, _project
from .nopunex import _pad_rows
from .weights import SafetensorsIndex, random_full


def _f32(t: torch.Tensor, device) -> nn.Parameter:
    return _p(t.to(device=device, dtype=torch.float32))


def _project_into(x: torch.Tensor, w: torch.Tensor, packed: Optional[torch.Tensor], out: torch.Tensor) -> torch.Tensor:
    """x @ w^T written to ``out`` (a plane of a larger buffer): decode-sized rows on the
    weight-streaming GEMM (split-K slabs summed into ``out``), else the library GEMM."""
    if gemm.skinny_ok(x, w):
        S = gemm.choose_split(w.shape[0], x.shape[1], x.shape[0])
        if S > 1:
            ws = torch.empty(S * x.shape[0] * w.shape[0], dtype=torch.float32, device=x.device)
            return gemm.reduce_partial(gemm.linear_partial(x, w, ws, S, packed=packed), out)
    return gemm.linear(x, w, out=out, packed=packed)


class WkvMixer(nn.Module):
    """Weights of one wkv time-mixing branch.  ``activation`` leaves the normed, gated head outputs
    (times ``post``) for the output projection of whoever owns the branch."""

    def __init__(self, spec, width: int):
        super().__init__()
        self.spec, self.width = spec, width
        self.mu = None       # [5, W] fp32: r, k, v, g, w
        self.w_in = None     # r, k, v, g: four [H*D, W]
        self.w_in_p = [None] * 4
        self.w1 = self.w2 = None    # [R, W], [H*D, R]
        self.w0 = self.u = self.norm_w = None   # [H*D] fp32
        self.w_o = self.w_o_p = None            # [W, H*D]

    def pack(self) -> None:
        self.w_o_p = _packed(self.w_o) if self.w_o is not None else None
        self.w_in_p = [_packed(w) for w in self.w_in]

    def set(self, get, dtype, device, own_output: bool = True) -> None:
        s, W = self.spec, self.width
        n = s.heads * s.dim
        ws = [get(x) for x in "rkvg"]
        assert all(w.shape == (n, W) for w in ws) and get("w1").shape[1] == W and get("w2").shape == (n, get("w1").shape[0])
        self.mu = _f32(torch.stack([get("mu." + x).reshape(W) for x in "rkvgw"]), device)
        self.w_in = nn.ParameterList([_p(w.to(device=device, dtype=dtype)) for w in ws])
        self.w1, self.w2 = _p(get("w1").to(device=device, dtype=dtype)), _p(get("w2").to(device=device, dtype=dtype))
        self.w0, self.u, self.norm_w = (_f32(get(x).reshape(n), device) for x in ("w0", "u", "norm"))
        if own_output:
            assert get("o").shape == (W, n)
            self.w_o = _p(get("o").to(device=device, dtype=dtype))

    def activation(self, h, positions, md, cache: dict, eps: float, post: float = 1.0, out=None):
        s = self.spec
        T, n = h.shape[0], s.heads * s.dim
        mixes = wkv_ops.shift_mix(h, self.mu, cache["prev"], md.token_seq, md.cu_q, md.num_seqs, positions, md.state_slots)
        rkvg = torch.empty((4, T, n), dtype=h.dtype, device=h.device)
        for i in range(4):       # one projection per mix (a batched library GEMM returned NaN at 8192 x 2048 x 2048 bf16)
            _project_into(mixes[i], self.w_in[i], self.w_in_p[i], rkvg[i])
        z = gemm.linear(wkv_ops.tanh_(gemm.linear(mixes[4], self.w1)), self.w2)
        o = wkv_ops.wkv_recurrence(rkvg, z, self.w0, self.u, cache["wkv"], md.cu_q, md.num_seqs, positions,
                                   md.state_slots, s.heads, s.dim)
        return ma_ops.head_norm_gate(o, s.heads, s.dim, eps, rkvg[3], ma_ops.GATE_SILU, h.dtype, weight=self.norm_w,
                                     post=post, out=out)

    def forward(self, h, positions, md, cache: dict, eps: float):
        return _project(self.activation(h, positions, md, cache, eps), self.w_o, self.w_o_p, partial=True)

    def state(self, slots: int, device) -> dict:
        s = self.spec
        return {"wkv": torch.zeros((slots, s.heads, s.dim, s.dim), dtype=torch.float32, device=device),
                "prev": torch.zeros((slots, self.width), dtype=torch.float32, device=device)}

    def state_floats(self) -> int:
        return self.spec.heads * self.spec.dim ** 2 + self.width


class SelectiveScanMixer(nn.Module):
    """Weights of one selective-scan mixer."""

    def __init__(self, spec, width: int):
        super().__init__()
        self.spec, self.width = spec, width
        self.w_in = self.w_x = self.w_dt = self.w_o = None   # [2I, W], [R + 2N, I], [I, R], [W, I]
        self.taps = self.conv_b = self.dt_b = self.A = self.D = None   # fp32: [I, K], [I], [I], [I, N], [I]
        self.w_in_p = self.w_o_p = None

    def pack(self) -> None:
        self.w_in_p, self.w_o_p = _packed(self.w_in), _packed(self.w_o)

    def set(self, get, has, dtype, device) -> None:
        s, W = self.spec, self.width
        I, N, R, K = s.inner, s.state, s.dt_rank, s.conv
        assert get("in").shape == (2 * I, W) and get("x").shape == (R + 2 * N, I) and get("dt").shape == (I, R)
        assert get("o").shape == (W, I) and get("conv").shape == (I, K) and get("A_log").shape == (I, N)
        to = lambda n: _p(get(n).to(device=device, dtype=dtype))
        self.w_in, self.w_x, self.w_dt, self.w_o = to("in"), to("x"), to("dt"), to("o")
        self.taps = _f32(get("conv"), device)
        self.conv_b = _f32(get("conv.b").reshape(I), device) if has("conv.b") else None
        self.dt_b, self.D = _f32(get("dt.b").reshape(I), device), _f32(get("D").reshape(I), device)
        self.A = _p((-torch.exp(get("A_log").double())).float().to(device))

    def forward(self, h, positions, md, cache: dict, eps: float):
        s = self.spec
        I, N, R = s.inner, s.state, s.dt_rank
        seq = (md.cu_q, md.num_seqs, positions, md.state_slots)
        xz = _project(h, self.w_in, self.w_in_p)
        x = conv_ops.causal_conv(xz[:, :I], self.taps, self.conv_b, cache.get("conv"), *seq, md.token_seq,
                                 act=conv_ops.ACT_SILU)
        low = gemm.linear(x, self.w_x)
        d = gemm.linear(low[:, :R].contiguous(), self.w_dt)
        y = scan_ops.selective_scan(x, d, self.dt_b, self.A, low[:, R:], self.D, xz[:, I:2 * I], cache["scan"], *seq)
        return _project(y, self.w_o, self.w_o_p, partial=True)

    def state(self, slots: int, device) -> dict:
        s = self.spec
        out = {"scan": torch.zeros((slots, s.inner, s.state), dtype=torch.float32, device=device)}
        if s.conv > 1:
            out["conv"] = torch.zeros((slots, s.conv - 1, s.inner), dtype=torch.float32, device=device)
        return out

    def state_floats(self) -> int:
        return self.spec.inner * (self.spec.state + max(self.spec.conv - 1, 0))


class ParallelMixer(nn.Module):
    """Pooled-window attention (left) beside wkv (right); one output projection over both
    branches' scaled activations."""

    def __init__(self, spec, width: int):
        super().__init__()
        self.spec, self.width = spec, width
        self.right = WkvMixer(spec.right, width)
        self.w_in = self.w_in_p = None    # [H*D | G*D | G*V (+ padding), W]
        self.bias = None     # [C] fp32 or None
        self.taps = None     # [C, K] fp32 (a single column of ones without a filter)
        self.q_norm = self.k_norm = self.sink = self.talk = None
        self.table = None
        self.w_o = self.w_o_p = None      # [W, H*V + Hr*Dr]

    def pack(self) -> None:
        self.w_in_p, self.w_o_p = _packed(self.w_in), _packed(self.w_o)

    @property
    def channels(self) -> int:
        s = self.spec.left
        return (s.heads + s.kv_heads) * s.dim + s.kv_heads * s.vdim

    def set(self, get, has, dtype, device) -> None:
        s, W = self.spec.left, self.width
        H, G, D, V = s.heads, s.kv_heads, s.dim, s.vdim
        g = lambda n: get("left." + n)
        q, k, v = g("q"), g("k"), g("v")
        assert q.shape == (H * D, W) and k.shape == (G * D, W) and v.shape == (G * V, W) and g("o").shape == (W, H * V)
        self.w_in = _p(_pad_rows(torch.cat([q, k, v], 0)).to(device=device, dtype=dtype))
        C = self.channels
        if has("left.q.b"):
            self.bias = _f32(torch.cat([g(n + ".b").reshape(-1) for n in "qkv"]), device)
            assert self.bias.numel() == C
        if s.conv > 1 or has("left.q.conv"):
            self.taps = _f32(torch.cat([g(n + ".conv") for n in "qkv"], 0), device)
            assert self.taps.shape == (C, max(s.conv, 1))
        else:
            self.taps = _p(torch.ones((C, 1), dtype=torch.float32, device=device))
        self.q_norm = _f32(g("q.norm").reshape(D), device) if has("left.q.norm") else None
        self.k_norm = _f32(g("k.norm").reshape(D), device) if has("left.k.norm") else None
        self.sink = _f32(g("sink").reshape(H), device) if has("left.sink") else None
        self.talk = _f32(g("talk").reshape(H, H), device) if has("left.talk") else None
        self.right.set(lambda n: get("right." + n), dtype, device, own_output=False)
        ro = get("right.o")
        assert ro.shape == (W, self.spec.right.heads * self.spec.right.dim)
        self.w_o = _p(torch.cat([g("o"), ro], 1).to(device=device, dtype=dtype))

    def forward(self, h, positions, md, cache: dict, eps: float):
        p, s = self.spec, self.spec.left
        H, G, D, V = s.heads, s.kv_heads, s.dim, s.vdim
        T, C, nl = h.shape[0], self.channels, s.heads * s.vdim
        a = torch.empty((T, self.w_o.shape[1]), dtype=h.dtype, device=h.device)
        proj = _project(h, self.w_in, self.w_in_p)
        qkv = conv_ops.causal_conv(proj[:, :C], self.taps, None, cache.get("conv"), md.cu_q, md.num_seqs, positions,
                                   md.state_slots, md.token_seq, in_bias=self.bias)
        kc, vc = cache["k"], cache["v"]
        q = ma_ops.rotate_cache(qkv, positions, md.slot_mapping, self.table, True, kc, vc, H, G, G, D, V,
                                q_norm=self.q_norm, k_norm=self.k_norm, eps=eps)
        pooled = s.window > 0 and s.pool > 0
        if pooled:
            pa_ops.pool_update(kc, vc, cache["kp"], cache["vp"], positions, md.token_seq, md.block_tables, s.pool,
                               md.slot_mapping)
        o = pa_ops.pooled_attention(q, kc, vc, cache.get("kp"), cache.get("vp"), md.block_tables, md.cu_q, md.context_lens,
                                    md.num_seqs, s.scale, s.softcap, s.window, s.pool if pooled else 0, self.sink,
                                    all_values=self.talk is not None)
        pa_ops.mix_heads(o, self.talk, p.left_scale, h.dtype, out=a[:, :nl])
        self.right.activation(h, positions, md, cache, eps, post=p.right_scale, out=a[:, nl:])
        return _project(a, self.w_o, self.w_o_p, partial=True)

    def state(self, slots: int, device) -> dict:
        out = self.right.state(slots, device)
        if self.spec.left.conv > 1:
            out["conv"] = torch.zeros((slots, self.spec.left.conv - 1, self.channels), dtype=torch.float32, device=device)
        return out

    def state_floats(self) -> int:
        return self.right.state_floats() + max(self.spec.left.conv - 1, 0) * self.channels


class ClampedFF(nn.Module):
    def __init__(self, spec: ClampedFFSpec):
        super().__init__()
        self.spec = spec
        self.w_in = self.down = self.w_in_p = self.down_p = None   # [gate | up rows, W], [W, F]

    def set(self, gate, up, down, dtype, device) -> None:
        assert gate.shape == up.shape == (self.spec.ff, down.shape[0]) and down.shape[1] == self.spec.ff
        self.w_in = _p(torch.cat([gate, up], 0).to(device=device, dtype=dtype))
        self.down = _p(down.to(device=device, dtype=dtype))

    def pack(self) -> None:
        self.w_in_p, self.down_p = _packed(self.w_in), _packed(self.down)

    def forward(self, h, h32):
        a = moe_ops.clamped_glu(_project(h, self.w_in, self.w_in_p, partial=True), self.spec.limit, dtype=h.dtype)
        return _project(a, self.down, self.down_p, partial=True)


class SoftmaxMoE(nn.Module):
    """fp32 router, SiLU-gated experts and the ungated shared expert."""

    def __init__(self, spec: SoftmaxMoESpec):
        super().__init__()
        self.spec = spec
        self.router = None
        self.gate = self.up = self.down = None
        self.w13 = self.w2 = self.w13_p = self.w2_p = None
        self.sh_in = self.sh_down = self.sh_in_p = self.sh_down_p = None

    def set(self, router, gates, ups, downs, shared, dtype, device) -> None:
        to = lambda ts: _p(torch.stack(ts).to(device=device, dtype=dtype))
        E, (F_, W) = len(gates), gates[0].shape
        assert router.shape == (E, W) and ups[0].shape == (F_, W) and downs[0].shape == (W, F_) and F_ == self.spec.ff
        self.router = _f32(router, device)
        if shared is not None:
            sgate, sup, sdown = shared
            assert sgate.shape == sup.shape == (self.spec.shared_ff, W) and sdown.shape == (W, self.spec.shared_ff)
            self.sh_in = _p(torch.cat([sgate, sup], 0).to(device=device, dtype=dtype))
            self.sh_down = _p(sdown.to(device=device, dtype=dtype))
        if moe_ops.mfma_experts_ok(E, F_, W, dtype, torch.device(device)):
            self.w13 = to([gemm.interleave_gate_up(g, u) for g, u in zip(gates, ups)])
            self.w2 = to(downs)
        else:
            self.gate, self.up, self.down = to(gates), to(ups), to(downs)

    def pack(self) -> None:
        if self.sh_in is not None:
            self.sh_in_p, self.sh_down_p = _packed(self.sh_in), _packed(self.sh_down)
        if self.w13 is not None and self.w13_p is None:
            E, N, K = self.w13.shape
            self.w13_p = gemm.pack_weight(self.w13.view(E * N, K)).view(E, N, K)
            E, N, K = self.w2.shape
            self.w2_p = gemm.pack_weight(self.w2.view(E * N, K)).view(E, N, K)

    def forward(self, h, h32) -> hyper_ops.ExpertSum:
        s = self.spec
        ids, wts = moe_ops.route_topk_softmax(moe_ops.router_logits(h32, self.router), s.experts, s.top)
        y, inv = moe_ops.silu_experts(h, ids, self.gate, self.up, self.down, self.w13, self.w2, self.w13_p, self.w2_p)
        out = hyper_ops.ExpertSum(y, inv, wts, s.top)
        if self.sh_in is not None:
            a = sw_ops.silu_mul(_project(h, self.sh_in, self.sh_in_p, partial=True), s.shared_ff, h.dtype)
            out.shared = _project(a, self.sh_down, self.sh_down_p)
        return out


_MIXERS = {"wkv": WkvMixer, "mamba1": SelectiveScanMixer, "parallel": ParallelMixer}


class BibezenLayer(nn.Module):
    def __init__(self, spec, width: int):
        super().__init__()
        self.kind = spec.type
        self.mix = _MIXERS[spec.type](spec.mixer, width)
        self.mlp = None
        if isinstance(spec.mlp, ClampedFFSpec):
            self.mlp = ClampedFF(spec.mlp)
        elif spec.mlp is not None:
            self.mlp = SoftmaxMoE(spec.mlp)
        self.norm1 = self.norm2 = None      # [W] fp32, 1 + the stored weight
        self.hc1 = self.hc2 = None          # (a_in [S], mix [S, S], m * a_out [S]) fp32
        self.canon = None                   # [W, taps] fp32 or None


class BibezenForCausalLM(nn.Module):
    # engine hooks (engine/model_runner.py): this family owns its cache and state layouts
    supports_graphs = True

    def __init__(self, cfg: BibezenConfig, st: ParallelState, dtype: torch.dtype, device: torch.device):
        super().__init__()
        if st.tp_size > 1 or getattr(st, "ep_size", 1) > 1:
            raise ValueError("Bibezen runs on one GPU (no TP / EP sharding for this family)")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"Bibezen runs in bfloat16 or float32, not {dtype}")
        self.cfg, self.st, self.dtype, self.device = cfg, st, dtype, device
        self.S = max(cfg.streams, 1)
        self.needs_state = cfg.needs_state
        self.layers = nn.ModuleList(BibezenLayer(l, cfg.hidden_size) for l in cfg.layers)
        self.embed = self.final_norm = self.sum_in = None
        self._max_pos = 0

    # ------------------------------------------------------------------ weights
    def _hc(self, p: str, get, has):
        S, dev, m = self.S, self.device, self.cfg.residual_mult
        if self.cfg.streams:
            f = lambda n, shape: get(p + n).double().reshape(shape)
            return (_f32(f("in", (S,)), dev), _f32(f("mix", (S, S)), dev), _f32(f("out", (S,)) * m, dev))
        one = lambda *shape: torch.ones(shape, dtype=torch.float64)
        return _f32(one(1), dev), _f32(one(1, 1), dev), _f32(one(1) * m, dev)

    def _norm(self, get, name: str) -> nn.Parameter:
        w = get(name)
        assert w.numel() == self.cfg.hidden_size, name
        return _f32(1.0 + w.double().reshape(-1), self.device)

    def _set_layer(self, i: int, get, has) -> None:
        cfg, L, spec = self.cfg, self.layers[i], self.cfg.layers[i]
        p, dev, dt, W = f"l{i}.", self.device, self.dtype, self.cfg.hidden_size
        mget, mhas = (lambda n: get(p + "mix." + n)), (lambda n: has(p + "mix." + n))
        if L.kind == "wkv":
            L.mix.set(mget, dt, dev)
        else:
            L.mix.set(mget, mhas, dt, dev)
        L.norm1, L.hc1 = self._norm(get, p + "norm1"), self._hc(p + "hc1.", get, has)
        if cfg.canon_taps > 0 and has(p + "canon1"):
            L.canon = _f32(get(p + "canon1"), dev)
            assert L.canon.shape == (W, cfg.canon_taps)
        f = spec.mlp
        if f is None:
            return
        L.norm2, L.hc2 = self._norm(get, p + "norm2"), self._hc(p + "hc2.", get, has)
        if isinstance(f, ClampedFFSpec):
            L.mlp.set(get(p + "mlp.gate"), get(p + "mlp.up"), get(p + "mlp.down"), dt, dev)
        else:
            part = lambda n: [get(p + f"mlp.e{e}.{n}") for e in range(f.experts)]
            shared = tuple(get(p + "mlp.shared." + n) for n in ("gate", "up", "down")) if f.shared_ff else None
            L.mlp.set(get(p + "mlp.router"), part("gate"), part("up"), part("down"), shared, dt, dev)

    def load_hf(self, path: str) -> "BibezenForCausalLM":
        """Load a checkpoint folder (safetensors; tensors under the design's own names)."""
        idx = SafetensorsIndex(path)
        return self._load(idx.get, idx.has)

    def load_state(self, tensors: dict) -> "BibezenForCausalLM":
        """The same from a dict name -> tensor (tests)."""
        return self._load(tensors.__getitem__, tensors.__contains__)

    def _load(self, get, has) -> "BibezenForCausalLM":
        dev = self.device
        self.embed = _p(get("embed").to(device=dev, dtype=self.dtype))
        assert self.embed.shape == (self.cfg.vocab_size, self.cfg.hidden_size)
        self.final_norm = self._norm(get, "final.norm")
        self.sum_in = _p(torch.ones(self.S, dtype=torch.float32, device=dev))
        for i in range(len(self.layers)):
            self._set_layer(i, get, has)
        if self._max_pos:
            self._build_tables()
        return self

    def random_state(self, seed: int = 0) -> dict:
        """Random bf16-representable tensors under the checkpoint names (norm weights near 0, stream
        mixes near the identity, decays spread over fast and slow channels)."""
        cfg, W, std, S = self.cfg, self.cfg.hidden_size, self.cfg.init_std, self.cfg.streams
        r = lambda name, shape, s=std: random_full(name, shape, s, seed, self.device, torch.bfloat16)
        out = {"embed": r("embed", (cfg.vocab_size, W), W ** -0.5), "final.norm": r("final.norm", (W,), 0.1)}

        def wkv(p, m):
            n = m.heads * m.dim
            R = m.decay_rank or max(16, W // 64)
            for x in "rkvgw":
                out[p + "mu." + x] = (0.5 + r(p + "mu." + x, (W,), 0.2)).bfloat16()
            for x in "rkvg":
                out[p + x] = r(p + x, (n, W), W ** -0.5)
            out[p + "w1"], out[p + "w2"] = r(p + "w1", (R, W), W ** -0.5), r(p + "w2", (n, R), 0.3)
            out[p + "w0"] = (-1.5 + r(p + "w0", (n,), 1.5)).bfloat16()
            out[p + "u"] = r(p + "u", (m.heads, m.dim), 0.5)
            out[p + "norm"] = (1 + r(p + "norm", (n,), 0.1)).bfloat16()

        for i, l in enumerate(cfg.layers):
            p, m = f"l{i}.", l.mixer
            for q in ["1"] + (["2"] if l.mlp is not None else []):
                out[p + "norm" + q] = r(p + "norm" + q, (W,), 0.1)
                if S:
                    out[p + f"hc{q}.in"] = (1.0 / S + r(p + f"hc{q}.in", (S,), 0.1)).bfloat16()
                    out[p + f"hc{q}.out"] = (1 + r(p + f"hc{q}.out", (S,), 0.2)).bfloat16()
                    out[p + f"hc{q}.mix"] = (torch.eye(S, device=self.device) + r(p + f"hc{q}.mix", (S, S), 0.1)).bfloat16()
            if cfg.canon_taps:
                out[p + "canon1"] = r(p + "canon1", (W, cfg.canon_taps), 0.2)
            if l.type == "wkv":
                wkv(p + "mix.", m)
                out[p + "mix.o"] = r(p + "mix.o", (W, m.heads * m.dim), (m.heads * m.dim) ** -0.5)
            elif l.type == "mamba1":
                I, N, R, K = m.inner, m.state, m.dt_rank, m.conv
                t = lambda n, shape, s: out.__setitem__(p + "mix." + n, r(p + "mix." + n, shape, s))
                t("in", (2 * I, W), W ** -0.5), t("conv", (I, K), 0.4), t("conv.b", (I,), 0.1), t("x", (R + 2 * N, I), I ** -0.5)
                t("dt", (I, R), R ** -0.5), t("D", (I,), 0.5), t("o", (W, I), I ** -0.5)
                out[p + "mix.dt.b"] = (-2.0 + r(p + "mix.dt.b", (I,), 1.0)).bfloat16()
                out[p + "mix.A_log"] = (torch.log(torch.arange(1, N + 1, device=self.device).float())[None, :]
                                        + r(p + "mix.A_log", (I, N), 0.2)).bfloat16()
            else:
                a, q = m.left, p + "mix.left."
                H, G, D, V = a.heads, a.kv_heads, a.dim, a.vdim
                for n, rows in (("q", H * D), ("k", G * D), ("v", G * V)):
                    out[q + n] = r(q + n, (rows, W), W ** -0.5)
                    out[q + n + ".b"] = r(q + n + ".b", (rows,), 0.1)
                    if a.conv > 0:
                        out[q + n + ".conv"] = r(q + n + ".conv", (rows, a.conv), 0.5)
                out[q + "q.norm"] = (1 + r(q + "q.norm", (D,), 0.1)).bfloat16()
                out[q + "k.norm"] = (1 + r(q + "k.norm", (D,), 0.1)).bfloat16()
                out[q + "talk"] = (torch.eye(H, device=self.device) + r(q + "talk", (H, H), 0.2)).bfloat16()
                out[q + "sink"] = r(q + "sink", (H,), 1.0)
                out[q + "o"] = r(q + "o", (W, H * V), (H * V) ** -0.5)
                wkv(p + "mix.right.", m.right)
                nr = m.right.heads * m.right.dim
                out[p + "mix.right.o"] = r(p + "mix.right.o", (W, nr), nr ** -0.5)
            f = l.mlp
            if isinstance(f, ClampedFFSpec):
                for n, shape, s in (("gate", (f.ff, W), W ** -0.5), ("up", (f.ff, W), W ** -0.5), ("down", (W, f.ff), f.ff ** -0.5)):
                    out[p + "mlp." + n] = r(p + "mlp." + n, shape, s)
            elif f is not None:
                out[p + "mlp.router"] = r(p + "mlp.router", (f.experts, W), 0.5)
                for n in [f"e{e}" for e in range(f.experts)] + (["shared"] if f.shared_ff else []):
                    ff = f.shared_ff if n == "shared" else f.ff
                    out[p + f"mlp.{n}.gate"] = r(p + f"mlp.{n}.gate", (ff, W), W ** -0.5)
                    out[p + f"mlp.{n}.up"] = r(p + f"mlp.{n}.up", (ff, W), W ** -0.5)
                    out[p + f"mlp.{n}.down"] = r(p + f"mlp.{n}.down", (W, ff), ff ** -0.5)
        return out

    def init_random(self, seed: int = 0) -> "BibezenForCausalLM":
        return self.load_state(self.random_state(seed))

    def pack_decode_weights(self) -> None:
        """Block-packed copies of the projections and expert weights for the decode GEMM (engine hook)."""
        for L in self.layers:
            L.mix.pack()
            if L.mlp is not None:
                L.mlp.pack()

    def to(self, device, *a, **k):  # keeps the fp32 tensors fp32 (no dtype argument)
        super().to(device)
        self.device = torch.device(device)
        for L in self.layers:
            for n in ("hc1", "hc2"):
                if getattr(L, n) is not None:
                    setattr(L, n, tuple(t.to(device) for t in getattr(L, n)))
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
            rot = L.mix.spec.left.rot if L.kind == "parallel" else None
            if rot is None:
                continue
            if rot not in made:
                made[rot] = ma_ops.table_for(rot, self._max_pos, self.device)
            L.mix.table = made[rot]

    def _paged_row(self, l) -> int:
        """Cached numbers per token of a layer: keys and values, and as many again for the pages of block means."""
        if l.type != "parallel":
            return 0
        a = l.mixer.left
        return a.kv_heads * (a.dim + a.vdim) * (2 if (a.window > 0 and a.pool > 0) else 1)

    def cache_bytes_per_block(self, block_size: int) -> int:
        esz = 2 if self.dtype == torch.bfloat16 else 4
        return max(sum(self._paged_row(l) for l in self.cfg.layers) * block_size * esz, 1)

    def state_bytes_per_slot(self) -> int:
        W, taps = self.cfg.hidden_size, self.cfg.canon_taps
        return 4 * sum(L.mix.state_floats() + max(taps - 1, 0) * W for L in self.layers)

    def alloc_cache(self, num_blocks: int, block_size: int, num_slots: int) -> List[dict]:
        """Per layer a dict: the mixer's state tensors ([slots, ...] fp32), ``canon`` [slots, taps - 1, W]
        fp32, and for a parallel mixer the paged ``k`` / ``v`` [blocks, G, block_size, D | V] with
        the pages of block means ``kp`` / ``vp`` of the same geometry."""
        out, dev, slots = [], self.device, max(num_slots, 1)
        for L, l in zip(self.layers, self.cfg.layers):
            c = L.mix.state(slots, dev)
            if L.canon is not None and self.cfg.canon_taps > 1:
                c["canon"] = torch.zeros((slots, self.cfg.canon_taps - 1, self.cfg.hidden_size), dtype=torch.float32, device=dev)
            if l.type == "parallel":
                a = l.mixer.left
                page = lambda w: torch.zeros((num_blocks, a.kv_heads, block_size, w), dtype=self.dtype, device=dev)
                c["k"], c["v"] = page(a.dim), page(a.vdim)
                if a.window > 0 and a.pool > 0:
                    c["kp"], c["vp"] = page(a.dim), page(a.vdim)
            out.append(c)
        return out

    def activation_bytes_per_token(self) -> int:
        W, widest = self.cfg.hidden_size, 0
        for l in self.cfg.layers:
            m = l.mixer
            wk = lambda s: 5 * W + 10 * s.heads * s.dim
            if l.type == "wkv":
                n = wk(m)
            elif l.type == "mamba1":
                n = 6 * m.inner + m.dt_rank + 2 * m.state
            else:
                a = m.left
                n = wk(m.right) + 3 * ((a.heads + a.kv_heads) * a.dim + a.kv_heads * a.vdim) + 2 * a.heads * a.kv_heads * a.vdim
            f = l.mlp
            if isinstance(f, ClampedFFSpec):
                n = max(n, 3 * f.ff)
            elif f is not None:
                n = max(n, f.top * (3 * f.ff + 2 * W) + 3 * f.shared_ff + f.experts)
            widest = max(widest, n)
        return 4 * W * (self.S + 4) + 4 * widest

    # ------------------------------------------------------------------ forward
    @torch.inference_mode()
    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor, md, caches: List[dict]) -> torch.Tensor:
        """The fp32 streams [T, S, W] after the last layer, for the step described by ``md``
        (ops/attention.py AttnMetadata: the whole-batch fields)."""
        cfg, eps, dt = self.cfg, self.cfg.rms_eps, self.dtype
        if positions.numel() and self._max_pos == 0:
            raise RuntimeError("Bibezen: reserve_positions(max_model_len) has not been called")
        xs = hyper_ops.spread_rows(self.embed, input_ids, self.S, cfg.embed_scale)
        L0 = self.layers[0]
        h, _ = hyper_ops.hyper_step(xs, None, None, (L0.hc1[0], L0.norm1), eps, dt)
        for i, L in enumerate(self.layers):
            cache = caches[i]
            if L.canon is not None:
                h = conv_ops.causal_conv(h, L.canon, None, cache.get("canon"), md.cu_q, md.num_seqs, positions,
                                         md.state_slots, md.token_seq, residual=True)
            y = L.mix(h, positions, md, cache, eps)
            close = L.hc1[1:]
            if L.mlp is not None:
                h, h32 = hyper_ops.hyper_step(xs, y, close, (L.hc2[0], L.norm2), eps, dt,
                                              want_f32=isinstance(L.mlp, SoftmaxMoE))
                y, close = L.mlp(h, h32), L.hc2[1:]
            nxt = self.layers[i + 1] if i + 1 < len(self.layers) else None
            h, _ = hyper_ops.hyper_step(xs, y, close, (nxt.hc1[0], nxt.norm1) if nxt is not None else None, eps, dt)
        return xs

    def compute_logits(self, rows: torch.Tensor) -> torch.Tensor:
        """fp32 logits of stream rows [n, S, W]: the streams' sum, the final norm, the embedding table."""
        act, _ = hyper_ops.hyper_step(rows.contiguous(), None, None, (self.sum_in, self.final_norm), self.cfg.rms_eps,
                                      self.dtype)
        return gemm.linear(act, self.embed).float()
