"""Model architecture presets (public HF configs; SURVEY.md §2.3 "Model constants").

The reference has no models; these are the north-star families (``BASELINE.json:8-11``):
Llama-3-8B, Llama-3-70B and Mixtral-8x7B, plus tiny variants with the same structure used by
tests (head_dim stays 128 because the attention kernels are specialised for it).
"""
from __future__ import annotations

import dataclasses
import json
import os
from typing import Dict, Optional


@dataclasses.dataclass(frozen=True)
class ModelConfig:
    name: str
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_layers: int
    num_heads: int
    num_kv_heads: int
    head_dim: int = 128
    rope_theta: float = 500000.0
    rms_eps: float = 1e-5
    max_position: int = 8192
    num_experts: int = 0          # 0 → dense MLP
    experts_per_token: int = 2
    tie_embeddings: bool = False
    rope_scaling: Optional[dict] = None
    bos_token_id: int = 128000
    eos_token_id: int = 128001
    init_std: float = 0.02
    # random-init std of the MoE router (None: init_std).  The tiny test MoEs use a wide router so
    # top-2 routing has no near-ties that bf16 reduction-order noise could flip between TP layouts
    router_init_std: Optional[float] = None

    @property
    def is_moe(self) -> bool:
        return self.num_experts > 0

    @property
    def q_size(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_kv_heads * self.head_dim

    def num_params(self) -> int:
        H, I, L, V = self.hidden_size, self.intermediate_size, self.num_layers, self.vocab_size
        attn = H * (self.q_size + 2 * self.kv_size) + self.q_size * H
        mlp = 3 * H * I * (self.num_experts or 1) + (H * self.num_experts if self.is_moe else 0)
        emb = V * H * (1 if self.tie_embeddings else 2)
        return L * (attn + mlp + 2 * H) + emb + H

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        return 2 * self.num_layers * self.kv_size * dtype_bytes


PRESETS: Dict[str, ModelConfig] = {
    "llama3-8b": ModelConfig("llama3-8b", 128256, 4096, 14336, 32, 32, 8),
    "llama3-70b": ModelConfig("llama3-70b", 128256, 8192, 28672, 80, 64, 8),
    "mixtral-8x7b": ModelConfig("mixtral-8x7b", 32000, 4096, 14336, 32, 32, 8, rope_theta=1e6,
                                max_position=32768, num_experts=8, experts_per_token=2,
                                bos_token_id=1, eos_token_id=2),
    # test-sized models with the real structure (GQA groups 4 and 8, MoE top-2)
    "tiny-llama": ModelConfig("tiny-llama", 1024, 512, 1024, 2, 4, 1, max_position=2048, init_std=0.05,
                              bos_token_id=1, eos_token_id=2),
    "tiny-llama-gqa4": ModelConfig("tiny-llama-gqa4", 1024, 1024, 2048, 2, 8, 2, max_position=2048,
                                   init_std=0.05, bos_token_id=1, eos_token_id=2),
    "tiny-mixtral": ModelConfig("tiny-mixtral", 1024, 512, 768, 2, 8, 2, rope_theta=1e6, max_position=2048,
                                num_experts=4, experts_per_token=2, init_std=0.05, bos_token_id=1,
                                eos_token_id=2, router_init_std=0.5),
    # the 70B TP=8 per-rank shape at test size: 8 KV heads (one per rank at TP=8), GQA group 8,
    # vocab not divisible by 8 (padded shards, like 128256 / 8 = 16032 rows), hidden % 1024 == 0
    "tiny-llama-g8": ModelConfig("tiny-llama-g8", 1003, 1024, 2048, 2, 64, 8, max_position=2048, init_std=0.05,
                                 bos_token_id=1, eos_token_id=2),
    # Mixtral's expert count and attention shape (8 experts: one per rank at EP=8, 8 KV heads)
    "tiny-mixtral-e8": ModelConfig("tiny-mixtral-e8", 1000, 1024, 1024, 2, 32, 8, rope_theta=1e6,
                                   max_position=2048, num_experts=8, experts_per_token=2, init_std=0.05,
                                   bos_token_id=1, eos_token_id=2, router_init_std=0.5),
    "small-llama": ModelConfig("small-llama", 32000, 2048, 5632, 8, 16, 4, init_std=0.02,
                               bos_token_id=1, eos_token_id=2),
}


@dataclasses.dataclass(frozen=True)
class LatentAttentionSpec:
    """Attention whose keys and values are expanded from one cached low-rank latent per token.
    Optional parts (0 / None: absent): queries through a normed latent of ``q_rank`` numbers; one
    rotated key part of ``rot_dim`` numbers per token shared by all heads (cached beside the
    latent) against ``rot_dim`` rotated query numbers per head; a sliding window of ``window``
    positions; one learned sink logit per head in the softmax denominator."""
    heads: int
    dim: int        # unrotated query / key size per head
    vdim: int       # value size per head
    kv_rank: int    # size of the cached latent
    scale: float
    q_rank: int = 0
    rot_dim: int = 0
    rot: Optional["RotarySpec"] = None
    window: int = 0
    sink: bool = False


@dataclasses.dataclass(frozen=True)
class SigmoidMoESpec:
    """Experts chosen by the largest sigmoid(router) scores; the score scales the expert's input."""
    experts: int
    top: int
    ff: int


@dataclasses.dataclass(frozen=True)
class LayerSpec:
    type: str
    mixer: object    # the mixer's spec (LatentAttentionSpec, SinkAttentionSpec, LightningSpec)
    mlp: object      # the feed-forward's spec, None: no feed-forward


@dataclasses.dataclass(frozen=True)
class SapapelConfig:
    """Sapapel: post-norm layers (one scalar gain per norm, alpha-scaled skip path) with a token
    shift in front of each mixer, a learned average over all earlier layers' outputs behind each
    layer, latent attention without positions and a sigmoid-routed MoE.  Read from a checkpoint
    folder's config.json ("architecture": "Sapapel"); every size comes from there."""
    name: str
    vocab_size: int
    hidden_size: int
    layers: tuple
    alpha: float
    rms_eps: float
    max_position: int = 1 << 20     # no positional encoding: bounded by the cache only
    bos_token_id: int = 0
    eos_token_id: int = -1          # the checkpoint names no end token
    init_std: float = 0.05
    family: str = "sapapel"
    is_moe: bool = False            # not the Mixtral expert-parallel family (engine lockstep paths)
    experts_per_token: int = 0
    needs_state: bool = True        # per-sequence token-shift state beside the paged cache

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    def num_params(self) -> int:
        W, n = self.hidden_size, 2 * self.vocab_size * self.hidden_size
        for l in self.layers:
            m = l.mixer
            n += W * (m.heads * m.dim + m.kv_rank + 2 * m.heads * m.vdim) + m.kv_rank * m.heads * (m.dim + m.vdim)
            if l.mlp is not None:
                n += l.mlp.experts * (3 * l.mlp.ff * W + W)
        return n

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        return sum(l.mixer.kv_rank for l in self.layers) * dtype_bytes

    @classmethod
    def from_json(cls, c: dict, name: str = "sapapel") -> "SapapelConfig":
        layers = []
        for l in c["layers"]:
            if l["type"] != "latent_attention":
                raise ValueError(f"Sapapel: unknown mixer type {l['type']!r}")
            m = l["mixer"]
            mixer = LatentAttentionSpec(int(m["heads"]), int(m["dim"]), int(m["vdim"]), int(m["kv_rank"]),
                                        float(m["scale"]))
            f = l.get("mlp")
            mlp = None
            if f is not None:
                if f.get("kind") != "moe":
                    raise ValueError(f"Sapapel: unknown feed-forward kind {f.get('kind')!r}")
                mlp = SigmoidMoESpec(int(f["router"]["experts"]), int(f["router"]["top"]), int(f["expert"]["ff"]))
            layers.append(LayerSpec(l["type"], mixer, mlp))
        return cls(name=name, vocab_size=int(c["vocab"]), hidden_size=int(c["width"]), layers=tuple(layers),
                   alpha=float(c["postln_alpha"]), rms_eps=float(c["norm"]["eps"]))

    @classmethod
    def uniform(cls, name: str, vocab: int, width: int, n_layers: int, heads: int, dim: int, vdim: int, kv_rank: int,
                ff: int, experts: int, top: int, alpha: float = 2.0, eps: float = 1e-6) -> "SapapelConfig":
        l = LayerSpec("latent_attention", LatentAttentionSpec(heads, dim, vdim, kv_rank, dim ** -0.5),
                      SigmoidMoESpec(experts, top, ff))
        return cls(name=name, vocab_size=vocab, hidden_size=width, layers=(l,) * n_layers, alpha=alpha, rms_eps=eps)


@dataclasses.dataclass(frozen=True)
class RotarySpec:
    """Rotation of coordinate pairs of the first ``dims`` coordinates by position * base^(-2i/dims):
    pair i is (2i, 2i+1) (``halves`` False) or (i, i + dims/2) (``halves`` True); ``scaling`` =
    (factor, original, fast, slow) stretches the slow pairs (YaRN) and scales cos / sin by
    0.1 ln(factor) + 1."""
    dims: int
    base: float
    scaling: Optional[tuple] = None
    halves: bool = False


@dataclasses.dataclass(frozen=True)
class SinkAttentionSpec:
    """Grouped-query softmax attention with unit-RMS rotated queries / keys, position-rotated values,
    a tanh cap on the scores (0: none) and ``sink`` extra exp(0) terms in the softmax denominator."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: float = 0.0
    rot: Optional[RotarySpec] = None
    sink: float = 1.0


@dataclasses.dataclass(frozen=True)
class LightningSpec:
    """Linear attention with one constant decay per head and a [dim, vdim] fp32 state per head."""
    heads: int
    dim: int
    vdim: int
    decay: tuple


@dataclasses.dataclass(frozen=True)
class DenseFFSpec:
    ff: int


@dataclasses.dataclass(frozen=True)
class ClampedMoESpec:
    """Experts with clamped gate / up products, chosen by the largest router logits and weighted by
    the softmax over the chosen logits; optionally one shared expert behind a sigmoid gate."""
    experts: int
    top: int
    ff: int
    limit: float
    shared_ff: int = 0
    shared_limit: float = 0.0


@dataclasses.dataclass(frozen=True)
class KivezenConfig:
    """Kivezen: pre-norm layers on ``streams`` fp32 residual streams (hyper-connections; 0: the one
    plain residual), each layer a sink-softmax attention or a lightning (decayed linear) attention
    mixer and a dense GELU or clamped-GLU MoE feed-forward; layers ``loop[0]..loop[1]-1`` run
    ``loop[2]`` times in a row with the same weights and a cache / state per pass.  Read from a
    checkpoint folder's config.json ("architecture": "Kivezen")."""
    name: str
    vocab_size: int
    hidden_size: int
    layers: tuple
    rms_eps: float
    streams: int = 0
    loop: tuple = (0, 0, 1)
    logit_softcap: float = 0.0
    max_position: int = 1 << 20     # the rotation tables are built for the engine's max_model_len
    bos_token_id: int = 0
    eos_token_id: int = -1
    init_std: float = 0.05
    family: str = "kivezen"
    is_moe: bool = False            # not the Mixtral expert-parallel family (engine lockstep paths)
    experts_per_token: int = 0

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @property
    def runs(self) -> tuple:
        """Layer index of every layer run, in execution order (a looped layer appears once per pass)."""
        a, b, times = self.loop
        n = len(self.layers)
        return tuple(range(a)) + tuple(range(a, b)) * times + tuple(range(b, n))

    @property
    def needs_state(self) -> bool:
        return any(l.type == "lightning" for l in self.layers)

    def num_params(self) -> int:
        W, n = self.hidden_size, 2 * self.vocab_size * self.hidden_size
        for l in self.layers:
            m = l.mixer
            if l.type == "attention":
                n += W * (m.heads * m.dim + m.kv_heads * (m.dim + m.vdim) + m.heads * m.vdim)
            else:
                n += W * m.heads * (2 * m.dim + 3 * m.vdim)
            f = l.mlp
            if isinstance(f, DenseFFSpec):
                n += 2 * W * f.ff
            elif f is not None:
                n += f.experts * (3 * f.ff * W + W) + 3 * f.shared_ff * W
        return n

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        return sum(self.layers[i].mixer.kv_heads * (self.layers[i].mixer.dim + self.layers[i].mixer.vdim)
                   for i in self.runs if self.layers[i].type == "attention") * dtype_bytes

    @classmethod
    def from_json(cls, c: dict, name: str = "kivezen") -> "KivezenConfig":
        layers = []
        for l in c["layers"]:
            m = l["mixer"]
            if l["type"] == "attention":
                rot = None
                if m.get("rot"):
                    sc = m["rot"].get("scaling")
                    rot = RotarySpec(int(m["rot"]["dims"]), float(m["rot"]["base"]),
                                     (float(sc["factor"]), float(sc["original"]), float(sc["fast"]), float(sc["slow"]))
                                     if sc else None)
                mixer = SinkAttentionSpec(int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]),
                                          int(m.get("vdim", m["dim"])), float(m["scale"]), float(m.get("softcap") or 0.0),
                                          rot)
            elif l["type"] == "lightning":
                mixer = LightningSpec(int(m["heads"]), int(m["dim"]), int(m.get("vdim", m["dim"])),
                                      tuple(float(d) for d in m["decay"]))
                if len(mixer.decay) != mixer.heads:
                    raise ValueError("Kivezen: a lightning mixer needs one decay per head")
            else:
                raise ValueError(f"Kivezen: unknown mixer type {l['type']!r}")
            f = l.get("mlp")
            mlp = None
            if f is not None:
                if f.get("kind") == "dense":
                    mlp = DenseFFSpec(int(f["ff"]))
                elif f.get("kind") == "moe":
                    sh = f.get("shared") or {}
                    mlp = ClampedMoESpec(int(f["router"]["experts"]), int(f["router"]["top"]), int(f["expert"]["ff"]),
                                         float(f["expert"]["limit"]), int(sh.get("ff", 0)), float(sh.get("limit", 0.0)))
                else:
                    raise ValueError(f"Kivezen: unknown feed-forward kind {f.get('kind')!r}")
            layers.append(LayerSpec(l["type"], mixer, mlp))
        lp = c.get("loop") or {}
        loop = (int(lp.get("start", 0)), int(lp.get("stop", 0)), int(lp.get("times", 1)))
        if not (0 <= loop[0] <= loop[1] <= len(layers)) or loop[2] < 1:
            raise ValueError(f"Kivezen: loop {loop} does not fit {len(layers)} layers")
        return cls(name=name, vocab_size=int(c["vocab"]), hidden_size=int(c["width"]), layers=tuple(layers),
                   rms_eps=float(c["norm"]["eps"]), streams=int(c.get("streams") or 0), loop=loop,
                   logit_softcap=float(c.get("logit_softcap") or 0.0))

    @classmethod
    def uniform(cls, name: str, vocab: int, width: int, pattern: str, heads: int, kv_heads: int, dim: int, ff: int,
                experts: int, top: int, expert_ff: int, streams: int = 2, loop: tuple = (0, 0, 1)) -> "KivezenConfig":
        """``pattern``: one letter per layer, A attention / L lightning, upper case with the MoE
        feed-forward (and a shared expert of ``expert_ff``), lower case with the dense one."""
        rot = RotarySpec(dim, 10000.0, (8.0, 4096.0, 32.0, 1.0))
        layers = []
        for ch in pattern:
            if ch in "Aa":
                mixer = SinkAttentionSpec(heads, kv_heads, dim, dim, dim ** -0.5, 30.0, rot)
            else:
                mixer = LightningSpec(heads, dim, dim, tuple(1.0 - 2.0 ** (-1 - 6 * h / max(heads - 1, 1))
                                                             for h in range(heads)))
            mlp = ClampedMoESpec(experts, top, expert_ff, 7.0, expert_ff, 7.0) if ch.isupper() else DenseFFSpec(ff)
            layers.append(LayerSpec("attention" if ch in "Aa" else "lightning", mixer, mlp))
        return cls(name=name, vocab_size=vocab, hidden_size=width, layers=tuple(layers), rms_eps=1e-5,
                   streams=streams, loop=loop, logit_softcap=50.0)


@dataclasses.dataclass(frozen=True)
class DiffAttentionSpec:
    """Grouped-query differential attention: two softmax maps per head over the same values, the
    second subtracted with one learned factor (offset ``diff``), the difference set to unit RMS per
    head and scaled by 1 - ``diff``, then gated by a sigmoid of the mixer's input.  ``chunk`` > 0:
    a key is visible only inside the query's block of ``chunk`` positions (counted from 0)."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    diff: float
    rot: Optional[RotarySpec] = None
    chunk: int = 0


@dataclasses.dataclass(frozen=True)
class DeltaSpec:
    """Gated delta rule: per head a [dim, vdim] fp32 memory that decays by a data-dependent gate,
    is corrected along the new unit key towards the new value, and is read with the unit query;
    q, k, v pass a causal per-channel filter of ``conv`` taps and SiLU first."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int


@dataclasses.dataclass(frozen=True)
class GatedFFSpec:
    """down(silu(gate x) * (up x))."""
    ff: int


@dataclasses.dataclass(frozen=True)
class NopunexConfig:
    """Nopunex: an fp32 residual stream with a layer norm (weight and bias) before and after every
    sublayer; mixers are differential chunked attention, windowed latent attention with a sink, or
    the gated delta rule; SiLU-gated dense feed-forwards (or none).  Layers ``loop[0]..loop[1]-1``
    run ``loop[2]`` times in a row with the same weights and a cache / state per pass; every pass
    starts from a projection of the stream joined with the embedding, plus a per-pass vector
    (``looped`` False: no such block).  Read from a checkpoint folder's config.json
    ("architecture": "Nopunex")."""
    name: str
    vocab_size: int
    hidden_size: int
    layers: tuple
    rms_eps: float                  # eps of every norm of a layer
    loop: tuple = (0, 0, 1)
    looped: bool = False
    logit_scale: float = 1.0
    max_position: int = 1 << 20     # the rotation tables are built for the engine's max_model_len
    bos_token_id: int = 0
    eos_token_id: int = -1
    init_std: float = 0.05
    family: str = "nopunex"
    is_moe: bool = False
    experts_per_token: int = 0

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @property
    def runs(self) -> tuple:
        """(layer index, pass number or -1, first of its pass) of every layer run, in order."""
        n = len(self.layers)
        if not self.looped:
            return tuple((i, -1, False) for i in range(n))
        a, b, times = self.loop
        out = [(i, -1, False) for i in range(a)]
        for t in range(times):
            out += [(i, t, i == a) for i in range(a, b)]
        return tuple(out + [(i, -1, False) for i in range(b, n)])

    @property
    def needs_state(self) -> bool:
        return any(l.type == "delta" for l in self.layers)

    def num_params(self) -> int:
        W, n = self.hidden_size, 2 * self.vocab_size * self.hidden_size
        if self.looped:
            n += 2 * W * W
        for l in self.layers:
            m = l.mixer
            if l.type == "attention":
                n += W * (2 * m.heads * m.dim + 2 * m.kv_heads * m.dim + m.kv_heads * m.vdim + 2 * m.heads * m.vdim)
            elif l.type == "latent_attention":
                n += W * (m.q_rank + m.kv_rank + m.rot_dim) + m.q_rank * m.heads * (m.dim + m.rot_dim)
                n += m.kv_rank * m.heads * (m.dim + m.vdim) + W * m.heads * m.vdim
            else:
                n += W * (2 * m.kv_heads * m.dim + 3 * m.heads * m.vdim + 2 * m.heads)
            if l.mlp is not None:
                n += 3 * W * l.mlp.ff
        return n

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        n = 0
        for i, _, _ in self.runs:
            m = self.layers[i].mixer
            if self.layers[i].type == "attention":
                n += m.kv_heads * (2 * m.dim + m.vdim)
            elif self.layers[i].type == "latent_attention":
                n += m.kv_rank + m.rot_dim
        return n * dtype_bytes

    @staticmethod
    def _rot(r: Optional[dict]) -> Optional[RotarySpec]:
        if not r:
            return None
        sc = r.get("scaling")
        return RotarySpec(int(r["dims"]), float(r["base"]),
                          (float(sc["factor"]), float(sc["original"]), float(sc["fast"]), float(sc["slow"])) if sc else None,
                          halves=True)

    @classmethod
    def from_json(cls, c: dict, name: str = "nopunex") -> "NopunexConfig":
        layers = []
        for l in c["layers"]:
            m = l["mixer"]
            size = int((m.get("mask") or {}).get("size", 0))
            if l["type"] == "attention":
                mixer = DiffAttentionSpec(int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]),
                                          int(m.get("vdim", m["dim"])), float(m["scale"]), float(m["diff"]),
                                          cls._rot(m.get("rot")), size)
                if mixer.heads % mixer.kv_heads:
                    raise ValueError("Nopunex: attention heads must be a multiple of kv_heads")
            elif l["type"] == "latent_attention":
                mixer = LatentAttentionSpec(int(m["heads"]), int(m["dim"]), int(m["vdim"]), int(m["kv_rank"]),
                                            float(m["scale"]), int(m["q_rank"]), int(m["rot_dim"]), cls._rot(m.get("rot")),
                                            size, True)
                if mixer.rot is not None and mixer.rot.dims > mixer.rot_dim:
                    raise ValueError("Nopunex: rot.dims exceeds rot_dim")
            elif l["type"] == "delta":
                mixer = DeltaSpec(int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]), int(m["vdim"]),
                                  int(m["conv"]))
                if mixer.heads % mixer.kv_heads or mixer.conv < 1:
                    raise ValueError("Nopunex: delta heads must be a multiple of kv_heads, conv >= 1")
            else:
                raise ValueError(f"Nopunex: unknown mixer type {l['type']!r}")
            f = l.get("mlp")
            mlp = None
            if f is not None:
                if f.get("kind") != "dense":
                    raise ValueError(f"Nopunex: unknown feed-forward kind {f.get('kind')!r}")
                mlp = GatedFFSpec(int(f["ff"]))
            layers.append(LayerSpec(l["type"], mixer, mlp))
        lp = c.get("loop")
        loop = (int(lp["start"]), int(lp["stop"]), int(lp["times"])) if lp else (0, 0, 1)
        if not (0 <= loop[0] <= loop[1] <= len(layers)) or loop[2] < 1:
            raise ValueError(f"Nopunex: loop {loop} does not fit {len(layers)} layers")
        return cls(name=name, vocab_size=int(c["vocab"]), hidden_size=int(c["width"]), layers=tuple(layers),
                   rms_eps=float(c["norm"]["eps"]), loop=loop, looped=bool(lp) and loop[1] > loop[0],
                   logit_scale=float(c.get("logit_scale", 1.0)))

    @classmethod
    def uniform(cls, name: str, vocab: int, width: int, pattern: str, heads: int, kv_heads: int, dim: int, ff: int,
                kv_rank: int = 512, q_rank: int = 1024, rot_dim: int = 64, window: int = 1024, chunk: int = 1024,
                loop: Optional[tuple] = None) -> "NopunexConfig":
        """``pattern``: one letter per layer, A differential attention / M latent attention /
        D delta rule; lower case: without a feed-forward."""
        layers = []
        for ch in pattern:
            up = ch.upper()
            if up == "A":
                mixer = DiffAttentionSpec(heads, kv_heads, dim, dim, dim ** -0.5, 0.3,
                                          RotarySpec(dim // 2, 1e6, None, True), chunk)
            elif up == "M":
                mixer = LatentAttentionSpec(heads, dim, dim, kv_rank, (dim + rot_dim) ** -0.5, q_rank, rot_dim,
                                            RotarySpec(rot_dim, 5e5, (8.0, 4096.0, 32.0, 1.0), True), window, True)
            else:
                mixer = DeltaSpec(heads, kv_heads, dim, dim, 4)
            layers.append(LayerSpec({"A": "attention", "M": "latent_attention", "D": "delta"}[up], mixer,
                                    GatedFFSpec(ff) if ch.isupper() else None))
        return cls(name=name, vocab_size=vocab, hidden_size=width, layers=tuple(layers), rms_eps=1e-5,
                   loop=loop or (0, 0, 1), looped=loop is not None, logit_scale=1.0)


@dataclasses.dataclass(frozen=True)
class PooledWindowAttentionSpec:
    """Grouped-query softmax attention whose projections (with biases) pass a causal per-channel
    filter of ``conv`` taps (0 / 1: none), then a weighted unit RMS per head on q and k (``qk_norm``)
    and a rotation.  A query sees the last ``window`` single keys (0: all) and, behind the window,
    the mean key / value of every complete block of ``pool`` positions (0: none) that ended before
    the window; scores are capped by tanh (``softcap`` 0: none); the denominator holds one learned
    sink term per head (``sink``); the heads' softmax weights are mixed by an [H, H] matrix (``talk``)
    before they meet the values of each head's own key / value head."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: float = 0.0
    rot: Optional[RotarySpec] = None
    window: int = 0
    pool: int = 0
    conv: int = 0
    qk_norm: bool = True
    sink: bool = True
    talk: bool = True
    bias: bool = True


@dataclasses.dataclass(frozen=True)
class WkvSpec:
    """Time mixing with a [dim, dim] fp32 state per head that decays per key channel by a
    data-dependent factor exp(-exp(.)) from a low-rank projection (``decay_rank``), a bonus for the
    current token, inputs mixed with the previous token's, unit RMS per head and a SiLU gate."""
    heads: int
    dim: int
    decay_rank: int = 0     # read from the checkpoint's tensor shapes when 0


@dataclasses.dataclass(frozen=True)
class SelectiveScanSpec:
    """State-space mixer with input-dependent step sizes: ``inner`` channels, each with a diagonal
    state of ``state`` numbers, a causal filter of ``conv`` taps and SiLU in front, a gate behind."""
    inner: int
    state: int
    dt_rank: int
    conv: int


@dataclasses.dataclass(frozen=True)
class ParallelSpec:
    """Two mixers reading the same input, their outputs summed with fixed weights."""
    left: PooledWindowAttentionSpec
    right: WkvSpec
    left_scale: float = 1.0
    right_scale: float = 1.0


@dataclasses.dataclass(frozen=True)
class ClampedFFSpec:
    """down(min(g, limit) sigmoid(1.702 min(g, limit)) (clamp(u, -limit, limit) + 1)), g = gate x, u = up x."""
    ff: int
    limit: float


@dataclasses.dataclass(frozen=True)
class SoftmaxMoESpec:
    """SiLU-gated experts chosen by the largest fp32 router logits, weighted by the softmax over the
    chosen logits, plus an ungated shared expert of ``shared_ff`` (0: none)."""
    experts: int
    top: int
    ff: int
    shared_ff: int = 0


@dataclasses.dataclass(frozen=True)
class BibezenConfig:
    """Bibezen: pre-norm layers (norm weights stored around zero) on ``streams`` fp32 residual
    streams (hyper-connections; 0: the one plain residual) with sublayer outputs scaled by
    ``residual_mult``; the mixer's input passes h + filter(h) over ``canon_taps`` positions (0: not);
    mixers are ``wkv``, ``mamba1`` (selective scan) or ``parallel`` (pooled-window attention beside
    wkv); feed-forwards are a clamped GLU, a softmax-routed mixture with a shared expert, or none.
    The embedding rows are scaled by ``embed_scale``; the logits reuse the embedding table.  Read
    from a checkpoint folder's config.json ("architecture": "Bibezen")."""
    name: str
    vocab_size: int
    hidden_size: int
    layers: tuple
    rms_eps: float
    streams: int = 0
    residual_mult: float = 1.0
    embed_scale: float = 1.0
    canon_taps: int = 0
    max_position: int = 1 << 20
    bos_token_id: int = 0
    eos_token_id: int = -1
    init_std: float = 0.05
    family: str = "bibezen"
    is_moe: bool = False
    experts_per_token: int = 0

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @property
    def runs(self) -> tuple:
        return tuple(range(len(self.layers)))

    @property
    def needs_state(self) -> bool:
        return True     # every mixer keeps per-sequence state (filters, previous rows, recurrences)

    def num_params(self) -> int:
        W, n = self.hidden_size, self.vocab_size * self.hidden_size + self.hidden_size

        def wkv(m, own_output=True):
            c, r = m.heads * m.dim, m.decay_rank or max(16, W // 64)
            return (5 if own_output else 4) * c * W + r * (W + c) + 5 * W + 3 * c

        def left(m):
            c = (m.heads + m.kv_heads) * m.dim + m.kv_heads * m.vdim
            return c * (W + 1 + max(m.conv, 0)) + 2 * m.dim + m.heads * (m.heads + 1) + W * m.heads * m.vdim

        for l in self.layers:
            m = l.mixer
            n += W * (2 if l.mlp is not None else 1) + max(self.streams, 0) * (self.streams + 2) * (2 if l.mlp is not None else 1)
            n += W * self.canon_taps
            if l.type == "wkv":
                n += wkv(m)
            elif l.type == "mamba1":
                n += 3 * W * m.inner + m.inner * (m.conv + 3 + m.state + 2 * m.dt_rank + 2 * m.state)
            else:
                n += left(m.left) + wkv(m.right, False) + W * m.right.heads * m.right.dim
            f = l.mlp
            if isinstance(f, ClampedFFSpec):
                n += 3 * W * f.ff
            elif f is not None:
                n += f.experts * (3 * f.ff * W + W) + 3 * f.shared_ff * W
        return n

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        """Paged bytes per token: keys and values of every attention branch and the pages of their block means."""
        return sum(2 * l.mixer.left.kv_heads * (l.mixer.left.dim + l.mixer.left.vdim) for l in self.layers
                   if l.type == "parallel") * dtype_bytes

    @staticmethod
    def _left(m: dict) -> PooledWindowAttentionSpec:
        r, mask = m.get("rot"), m.get("mask") or {}
        rot = RotarySpec(int(r["dims"]), float(r["base"]), None, halves=True) if r else None
        s = PooledWindowAttentionSpec(int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]),
                                      int(m.get("vdim", m["dim"])), float(m["scale"]), float(m.get("softcap") or 0.0), rot,
                                      int(mask.get("size") or 0), int(mask.get("pool") or 0), int(m.get("conv") or 0))
        if s.heads % s.kv_heads or (rot is not None and (rot.dims % 2 or rot.dims > s.dim)):
            raise ValueError("Bibezen: heads must be a multiple of kv_heads and rot.dims even and at most dim")
        return s

    @classmethod
    def from_json(cls, c: dict, name: str = "bibezen") -> "BibezenConfig":
        layers = []
        for l in c["layers"]:
            m = l["mixer"]
            if l["type"] == "wkv":
                mixer = WkvSpec(int(m["heads"]), int(m["dim"]))
            elif l["type"] == "mamba1":
                mixer = SelectiveScanSpec(int(m["inner"]), int(m["state"]), int(m["dt_rank"]), int(m["conv"]))
            elif l["type"] == "parallel":
                mixer = ParallelSpec(cls._left(m["left"]), WkvSpec(int(m["right"]["heads"]), int(m["right"]["dim"])),
                                     float(m.get("left_scale", 1.0)), float(m.get("right_scale", 1.0)))
            else:
                raise ValueError(f"Bibezen: unknown mixer type {l['type']!r}")
            f = l.get("mlp")
            mlp = None
            if f is not None:
                if f.get("kind") == "dense":
                    mlp = ClampedFFSpec(int(f["ff"]), float(f["limit"]))
                elif f.get("kind") == "moe":
                    mlp = SoftmaxMoESpec(int(f["router"]["experts"]), int(f["router"]["top"]), int(f["expert"]["ff"]),
                                         int((f.get("shared") or {}).get("ff", 0)))
                    if not 1 <= mlp.top <= mlp.experts:
                        raise ValueError("Bibezen: top must lie between 1 and the number of experts")
                else:
                    raise ValueError(f"Bibezen: unknown feed-forward kind {f.get('kind')!r}")
            layers.append(LayerSpec(l["type"], mixer, mlp))
        return cls(name=name, vocab_size=int(c["vocab"]), hidden_size=int(c["width"]), layers=tuple(layers),
                   rms_eps=float(c["norm"]["eps"]), streams=int(c.get("streams") or 0),
                   residual_mult=float(c.get("residual_mult", 1.0)),
                   embed_scale=float((c.get("embedding") or {}).get("scale", 1.0)),
                   canon_taps=int((c.get("canon") or {}).get("taps") or 0))

    @classmethod
    def uniform(cls, name: str, vocab: int, width: int, pattern: str, heads: int, kv_heads: int, dim: int, ff: int,
                experts: int = 16, top: int = 2, expert_ff: int = 1536, streams: int = 2, window: int = 1024,
                pool: int = 64, state: int = 16) -> "BibezenConfig":
        """``pattern``: one letter per layer, W wkv / S selective scan / P parallel; upper case with
        the mixture feed-forward (and a shared expert of ``expert_ff``), lower case with the dense one."""
        layers = []
        for ch in pattern:
            up = ch.upper()
            if up == "W":
                mixer = WkvSpec(heads, dim)
            elif up == "S":
                mixer = SelectiveScanSpec(2 * width, state, max(width // 16, 1), 4)
            else:
                left = PooledWindowAttentionSpec(heads, kv_heads, dim, dim, dim ** -0.5, 30.0,
                                                 RotarySpec(dim // 2, 1e6, None, True), window, pool, 4)
                mixer = ParallelSpec(left, WkvSpec(heads, dim), 1.0, 1.0)
            mlp = SoftmaxMoESpec(experts, top, expert_ff, expert_ff) if ch.isupper() else ClampedFFSpec(ff, 7.0)
            layers.append(LayerSpec({"W": "wkv", "S": "mamba1", "P": "parallel"}[up], mixer, mlp))
        return cls(name=name, vocab_size=vocab, hidden_size=width, layers=tuple(layers), rms_eps=1e-5, streams=streams,
                   residual_mult=0.5, embed_scale=float(width) ** 0.5, canon_taps=3)


# config.json "architecture" -> reader (checkpoints that are not HF Llama / Mixtral folders)
ARCHITECTURES = {"Sapapel": SapapelConfig.from_json, "Kivezen": KivezenConfig.from_json,
                 "Nopunex": NopunexConfig.from_json, "Bibezen": BibezenConfig.from_json}

PRESETS["tiny-sapapel"] = SapapelConfig.uniform("tiny-sapapel", 512, 128, 3, 4, 16, 32, 48, 64, 6, 2)
# speed measurements (random weights): layer shapes of small production MoE models, and the
# Mixtral-family model of the same width, depth, heads, experts and expert size beside each
PRESETS["sapapel-2k"] = SapapelConfig.uniform("sapapel-2k", 32000, 2048, 8, 16, 128, 128, 512, 1536, 16, 2)
PRESETS["sapapel-4k"] = SapapelConfig.uniform("sapapel-4k", 32000, 4096, 4, 32, 128, 128, 512, 2048, 8, 2)
PRESETS["mixtral-2k"] = ModelConfig("mixtral-2k", 32000, 2048, 1536, 8, 16, 4, rope_theta=1e6, num_experts=16,
                                    experts_per_token=2, bos_token_id=1, eos_token_id=2, router_init_std=0.5)
PRESETS["mixtral-4k"] = ModelConfig("mixtral-4k", 32000, 4096, 2048, 4, 32, 8, rope_theta=1e6, num_experts=8,
                                    experts_per_token=2, bos_token_id=1, eos_token_id=2, router_init_std=0.5)


PRESETS["tiny-kivezen"] = KivezenConfig.uniform("tiny-kivezen", 512, 128, "LAa", 4, 2, 32, 256, 6, 2, 64, loop=(1, 3, 2))
# speed measurements beside mixtral-2k / mixtral-4k: the same width, depth, heads, KV heads, experts
# and expert size; every fourth mixer is a lightning layer, every layer has the MoE with a shared expert
PRESETS["kivezen-2k"] = KivezenConfig.uniform("kivezen-2k", 32000, 2048, "LAAALAAA", 16, 4, 128, 4096, 16, 2, 1536)
PRESETS["kivezen-4k"] = KivezenConfig.uniform("kivezen-4k", 32000, 4096, "LAAA", 32, 8, 128, 8192, 8, 2, 2048)


PRESETS["tiny-nopunex"] = NopunexConfig.uniform("tiny-nopunex", 512, 128, "AdMA", 4, 2, 32, 256, kv_rank=48, q_rank=64,
                                                rot_dim=8, window=40, chunk=24, loop=(1, 3, 2))
# speed measurements beside kivezen-2k / kivezen-4k (the closest family: fp32 stream, a recurrent
# mixer among attention layers): the same width, depth, heads, KV heads and head size, dense
# feed-forwards of the MoE's active size
PRESETS["nopunex-2k"] = NopunexConfig.uniform("nopunex-2k", 32000, 2048, "DAMADAMA", 16, 4, 128, 4608)
PRESETS["nopunex-4k"] = NopunexConfig.uniform("nopunex-4k", 32000, 4096, "DAMA", 32, 8, 128, 6144)


PRESETS["tiny-bibezen"] = BibezenConfig.uniform("tiny-bibezen", 512, 128, "wPSp", 4, 2, 32, 256, 6, 2, 64, window=40, pool=8)
# speed measurements beside kivezen-2k / kivezen-4k (the closest family: fp32 hyper-connection
# streams, a recurrent mixer among attention layers, a softmax-routed mixture with a shared expert):
# the same width, depth, heads, KV heads, head size, experts and expert size
PRESETS["bibezen-2k"] = BibezenConfig.uniform("bibezen-2k", 32000, 2048, "WPPPSPPP", 16, 4, 128, 4096, 16, 2, 1536)
PRESETS["bibezen-4k"] = BibezenConfig.uniform("bibezen-4k", 32000, 4096, "WPSP", 32, 8, 128, 8192, 8, 2, 2048)


def get_config(name_or_path: str):
    if name_or_path in PRESETS:
        return PRESETS[name_or_path]
    path = os.path.join(name_or_path, "config.json") if os.path.isdir(name_or_path) else name_or_path
    if os.path.isfile(path):
        with open(path) as f:
            arch = json.load(f).get("architecture")
        if arch in ARCHITECTURES:
            with open(path) as f:
                return ARCHITECTURES[arch](json.load(f), os.path.basename(os.path.dirname(os.path.abspath(path))) or arch)
        return from_hf_config(path)
    raise KeyError(f"unknown model {name_or_path!r}; presets: {sorted(PRESETS)}")


def from_hf_config(path: str) -> ModelConfig:
    with open(path) as f:
        c = json.load(f)
    nh = c["num_attention_heads"]
    eos = c.get("eos_token_id", 2)
    return ModelConfig(
        name=c.get("_name_or_path", os.path.basename(os.path.dirname(path)) or "hf-model"),
        vocab_size=c["vocab_size"], hidden_size=c["hidden_size"], intermediate_size=c["intermediate_size"],
        num_layers=c["num_hidden_layers"], num_heads=nh, num_kv_heads=c.get("num_key_value_heads", nh),
        head_dim=c.get("head_dim", c["hidden_size"] // nh), rope_theta=c.get("rope_theta", 10000.0),
        rms_eps=c.get("rms_norm_eps", 1e-5), max_position=c.get("max_position_embeddings", 8192),
        num_experts=c.get("num_local_experts", 0), experts_per_token=c.get("num_experts_per_tok", 2),
        tie_embeddings=c.get("tie_word_embeddings", False), rope_scaling=c.get("rope_scaling"),
        bos_token_id=c.get("bos_token_id", 1) or 1, eos_token_id=eos[0] if isinstance(eos, list) else eos)
