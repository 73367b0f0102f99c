"""Nopunex through the framework (checkpoint loader, scheduler, block manager and state slots,
model runner, kernels) against the plain per-sequence model of tests/oracle_nopunex.py.

Every test builds its own small configuration and random weights, writes them as a checkpoint
folder and loads that through the engine, or drives one mixer with hand-made inputs over a
hand-made paged cache.  The same tests run on the CPU (the ops' PyTorch compositions) and, marked
gpu, on the HIP kernels."""
import json
import os
import random
import sys
from types import SimpleNamespace

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import oracle_nopunex as O  # noqa: E402

from polykey_service_amd.engine import EngineConfig, LLMEngine, SamplingParams  # noqa: E402
from polykey_service_amd.models.config import NopunexConfig  # noqa: E402
from polykey_service_amd.parallel.state import ParallelState  # noqa: E402

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
BS = 32


def checkpoint(tmp_path, cfg, w, name="m"):
    from safetensors.torch import save_file
    d = tmp_path / name
    d.mkdir()
    (d / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in w.items()}, str(d / "model.safetensors"))
    return str(d)


def engine(path, device, dtype="float32", pool_tokens=512, max_seqs=4, budget=512, graphs=False, max_len=None):
    cfg = EngineConfig(model_path=path, dtype=dtype, block_size=BS, max_num_seqs=max_seqs, max_num_batched_tokens=budget,
                       max_model_len=max_len or pool_tokens, num_kv_blocks=pool_tokens // BS, watermark=0.0,
                       hip_graphs=graphs, device=device, graph_batch_sizes=(1, 2, 4))
    return LLMEngine(cfg, ParallelState(device=torch.device(device)))


def replay(eng, steps):
    """steps: list of lists of (id, tokens, want, end?) -> {id: {position: logits row}}."""
    got, at = {}, {}
    for step in steps:
        ends = [e[0] for e in step if len(e) > 3 and e[3]]
        lg = eng.replay_step([(e[0], e[1], e[2]) for e in step], ends)
        r = 0
        for e in step:
            base = at.get(e[0], 0)
            for wpos in e[2]:
                got.setdefault(e[0], {})[base + wpos] = lg[r]
                r += 1
            at[e[0]] = base + len(e[1])
            if e[0] in ends:
                at.pop(e[0])
    return got


def cut(rid, toks, sizes, end=True):
    """The request in portions of the given sizes (the rest one token at a time), all places wanted."""
    out, i = [], 0
    sizes = list(sizes)
    while i < len(toks):
        n = min(sizes.pop(0) if sizes else 1, len(toks) - i)
        out.append((rid, toks[i:i + n], list(range(n)), end and i + n == len(toks)))
        i += n
    return out


def close(a, b, tol=3e-4):
    torch.testing.assert_close(a.float(), b.float(), rtol=tol, atol=tol)


def rand_tokens(n, vocab, seed):
    return random.Random(seed).choices(range(vocab), k=n)


def rows_of(got, rid, n):
    return torch.stack([got[rid][i] for i in range(n)])


@pytest.fixture
def small(tmp_path):
    # attention, then (delta without feed-forward, latent attention) twice, then attention
    cfg = O.make_config(loop=(1, 3, 2))
    w = O.random_model(cfg, seed=3)
    return cfg, w, checkpoint(tmp_path, cfg, w)


# ------------------------------------------------------------------ mixers over a hand-made cache
class Feed:
    """One sequence fed to a mixer module in portions: pages, slots and step metadata by hand."""

    def __init__(self, dev, pages, slot=1, n_slots=3):
        self.dev, self.pages, self.slot, self.at = dev, pages, slot, 0

    def step(self, c):
        i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=self.dev)
        at = self.at
        pos = torch.arange(at, at + c, dtype=torch.int32, device=self.dev)
        md = SimpleNamespace(slot_mapping=i32([self.pages[p // BS] * BS + p % BS for p in range(at, at + c)]),
                             block_tables=i32([self.pages]), cu_q=i32([0, c]), context_lens=i32([at + c]), num_seqs=1,
                             state_slots=i32([self.slot]), token_seq=i32([0] * c), num_decode=1 if (c == 1 and at) else 0)
        self.at += c
        return pos, md


def _table(spec, n, dev):
    from polykey_service_amd.ops import masked_attention as ma
    return ma.table_for(spec.rot, n + 3, dev) if spec.rot is not None else None


def _mixer(kind, m, w, W, dev, n, dtype=torch.float32):
    """The framework's mixer module of ``kind`` holding the oracle's weights, and its cache."""
    from polykey_service_amd.models import nopunex as N
    cfg = NopunexConfig.from_json({"vocab": 4, "width": W, "norm": {"eps": 1e-5},
                                   "layers": [{"type": kind, "mixer": m, "mlp": None}]})
    spec = cfg.layers[0].mixer
    mod = N._MIXERS[kind](spec, W)
    g = lambda n_: w[n_].float()
    if kind == "attention":
        mod.set(g("q"), g("k"), g("v"), g("g"), g("o"), g("lq1"), g("lk1"), g("lq2"), g("lk2"), dtype, dev)
    elif kind == "latent_attention":
        mod.set(g("dq"), g("dq.norm"), g("uq"), g("dkv"), g("dkv.norm"), g("uk"), g("uv"), g("sink"), g("o"), dtype, dev)
    else:
        mod.set(g("q"), g("k"), g("v"), g("a"), g("b"), g("g"), g("o"), g("q.conv"), g("k.conv"), g("v.conv"),
                g("A_log"), g("dt_bias"), g("norm"), dtype, dev)
    if kind != "delta":
        mod.table = _table(spec, n, dev)
    return mod, spec


def _weights(kind, m, W, seed):
    cfg = {"vocab": 4, "width": W, "norm": {"eps": 1e-5}, "layers": [{"type": kind, "mixer": m, "mlp": None}]}
    return {k[len("l0.mix."):]: v for k, v in O.random_model(cfg, seed, std=0.4).items() if k.startswith("l0.mix.")}


def _feed(mod, cache, h, portions, pages, dev, slot=1, dtype=torch.float32):
    feed, outs = Feed(dev, pages, slot), []
    for c in portions:
        pos, md = feed.step(c)
        y = mod(h[feed.at - c:feed.at].to(dev).to(dtype), pos, md, cache, 1e-5)
        outs.append((y.view().sum(0) if hasattr(y, "view") and not isinstance(y, torch.Tensor) else y).float().cpu())
    return torch.cat(outs)


def _attn_cache(spec, nb, dev, dtype=torch.float32):
    return (torch.zeros(nb, 2 * spec.kv_heads, BS, spec.dim, device=dev, dtype=dtype),
            torch.zeros(nb, spec.kv_heads, BS, spec.vdim, device=dev, dtype=dtype))


def test_rotation_tables_match_the_frequency_rule():
    from polykey_service_amd.models.config import RotarySpec
    from polykey_service_amd.ops import masked_attention as ma
    for dims, base, sc in [(8, 1000.0, None), (40, 30000.0, (6.0, 1024, 24.0, 1.5)), (6, 10.0, (2.0, 16, 4.0, 0.5))]:
        rot = {"dims": dims, "base": base}
        if sc:
            rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), sc))
        want, mag = O.rotary_frequencies(rot)
        tab = ma.table_for(RotarySpec(dims, base, sc, True), 70, "cpu")
        ang = torch.arange(70, dtype=torch.float64)[:, None] * want
        close(tab[..., 0], torch.cos(ang) * mag, 1e-6)
        close(tab[..., 1], torch.sin(ang) * mag, 1e-6)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("T,W", [(9, 40), (9, 42), (700, 2056), (5, 4100)])
def test_sandwich_step(device, T, W):
    """Closing a sublayer behind its norm and opening the next equals the layer-norm equations, at
    widths held in registers and in LDS; the re-projection form replaces the stream."""
    from polykey_service_amd.ops import sandwich as sw
    dev = torch.device(device)
    x, y = torch.randn(T, W) * 3 + 1, torch.randn(T, W) * 2 - 0.5
    pw, pb, ow, ob, add = (torch.randn(W) for _ in range(5))
    new = x.double() + O.layer_norm(y.double(), pw.double(), pb.double(), 1e-5)
    want = O.layer_norm(new, ow.double(), ob.double(), 1e-5)
    xd = x.to(dev).clone()
    act = sw.sandwich_step(xd, y.to(dev), (pw.to(dev), pb.to(dev)), (ow.to(dev), ob.to(dev)), 1e-5, torch.float32)
    close(xd.cpu(), new, 1e-5)
    close(act.cpu(), want, 1e-4)
    pick = torch.tensor([T - 2, 0, 3], dtype=torch.int32)
    act2 = sw.sandwich_step(xd, None, None, (ow.to(dev), ob.to(dev)), 1e-5, torch.float32, rows=pick.to(dev))
    close(act2.cpu(), want[pick.long()], 1e-4)
    xd = x.to(dev).clone()
    act3 = sw.sandwich_step(xd, y.to(dev), None, (ow.to(dev), ob.to(dev)), 1e-5, torch.float32, replace=True, add=add.to(dev))
    close(xd.cpu(), y + add, 1e-6)
    close(act3.cpu(), O.layer_norm((y + add).double(), ow.double(), ob.double(), 1e-5), 1e-4)
    xd = x.to(dev).clone()
    assert sw.sandwich_step(xd, y.to(dev), None, None, 1e-5) is None
    close(xd.cpu(), x + y, 1e-6)
    close(sw.join_cast(x.to(dev), y.to(dev), torch.float32).cpu(), torch.cat([x, y], -1), 0)
    close(sw.silu_mul(torch.cat([x, y], -1).to(dev), W, torch.float32).cpu(), O.silu(x.double()) * y.double(), 1e-5)
    close(sw.scale_(x.to(dev).clone(), 1.75).cpu(), x * 1.75, 1e-6)


@pytest.mark.gpu
def test_sandwich_step_sums_split_k_slabs():
    from polykey_service_amd.ops import gemm
    from polykey_service_amd.ops import sandwich as sw
    dev, T, W, S = torch.device("cuda"), 6, 200, 3
    slabs, x = torch.randn(S, T, W, device=dev), torch.randn(T, W, device=dev)
    pw, pb = torch.randn(W, device=dev), torch.randn(W, device=dev)
    want = x.double() + O.layer_norm(slabs.double().sum(0), pw.double(), pb.double(), 1e-5)
    sw.sandwich_step(x, gemm.Partial(slabs.view(-1), S, T, W), (pw, pb), None, 1e-5)
    close(x.cpu(), want.cpu(), 1e-5)
    gu = torch.randn(S, T, 2 * W, device=dev)
    got = sw.silu_mul(gemm.Partial(gu.view(-1), S, T, 2 * W), W, torch.float32)
    g = gu.double().sum(0)
    close(got.cpu(), (O.silu(g[:, :W]) * g[:, W:]).cpu(), 1e-5)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,G,D,V,rd,chunk", [(4, 2, 8, 12, 6, 16), (3, 3, 16, 4, 16, 40), (6, 1, 6, 34, 2, 7),
                                             (2, 1, 24, 24, 0, 33), (2, 2, 70, 20, 8, 1)])
def test_differential_attention_mixer(device, H, G, D, V, rd, chunk):
    """Two maps per head on regrouped query rows, partial rotation in the halves layout, blocks of
    visible keys that straddle pages, the learned factor, the head norm and the gate: prompt
    portions and single decoded tokens over shuffled pages against the plain rule."""
    dev, n, W = torch.device(device), 75, 20
    m = O.make_config(pattern="a", heads=H, kv_heads=G, dim=D, vdim=V, rot_dims=rd, chunk=chunk)["layers"][0]["mixer"]
    w = _weights("attention", m, W, seed=H)
    h = torch.randn(n, W)
    want = O.diff_attention(h.double(), w, "", m, 1e-5).float()
    mod, spec = _mixer("attention", m, w, W, dev, n)
    got = _feed(mod, _attn_cache(spec, 8, dev), h, [31, 2, 33, 1, 1, 7], [5, 0, 3], dev)
    close(got, want, 3e-4)


def _one_key_attention(dev, chunk, key, qpos, n, decoded):
    """Differential attention whose second map is silent and whose first map has one key standing
    far above the rest: returns the per-head mean of (framework, plain rule) rows at ``qpos``."""
    H, G, D, V = 2, 1, 8, 6
    W = 2 * H * D + 2 * G * D + G * V + H * V
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "scale": 6.0, "diff": 0.25, "mask": {"size": chunk}}
    eye = torch.eye(W, dtype=torch.float64)
    o = 0
    w = {}
    for name, rows in (("q", 2 * H * D), ("k", 2 * G * D), ("v", G * V), ("g", H * V)):
        w[name], o = eye[o:o + rows], o + rows
    w["o"] = eye[:, :H * V]                                     # the heads land in the first output columns
    z = torch.zeros(D, dtype=torch.float64)
    w.update({"lq1": z, "lk1": z, "lq2": z, "lk2": z})       # lambda = diff
    torch.manual_seed(11)
    h = torch.randn(n, W) * 0.3
    h[:, -H * V:] = 30.0                                        # gate wide open
    u = torch.randn(D)
    for a in range(H):
        h[qpos, a * 2 * D:a * 2 * D + D] = u                   # first map of both heads asks for u
    h[key, 2 * H * D:2 * H * D + D] = u                        # first-map key answers
    vcols = slice(2 * H * D + 2 * G * D, 2 * H * D + 2 * G * D + G * V)
    h[:, vcols] = -(0.5 + 0.1 * torch.rand(n, G * V))             # every other value is negative
    h[key, 2 * H * D + 2 * G * D:2 * H * D + 2 * G * D + G * V] = torch.linspace(20.0, 60.0, V)
    want = O.diff_attention(h.double(), w, "", m, 1e-5).float()
    mod, spec = _mixer("attention", m, w, W, dev, n)
    portions = [qpos - 5] + ([1] * (n - qpos + 5) if decoded else [n - qpos + 5])
    got = _feed(mod, _attn_cache(spec, 9, dev), h, portions, [6, 2, 4, 0, 5, 1, 3, 7], dev)
    return got[qpos], want[qpos]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("where", ["block_first", "before_block", "page_last", "page_first", "self", "next"])
@pytest.mark.parametrize("decoded", [False, True])
def test_attention_sees_its_block_only(device, where, decoded):
    """One key's score stands far above the rest: its value shapes the output when it lies in the
    query's block of positions (the block's first position, either side of a page border, the
    query's own) and leaves no trace when it is the last position of the block before or the
    query's successor; for a prompt portion and for decoded tokens."""
    chunk, n = 80, 230                                          # blocks 0-79, 80-159, 160-229: borders inside pages
    qpos = 222
    key = {"block_first": 160, "before_block": 159, "page_last": 191, "page_first": 192, "self": qpos, "next": qpos + 1}[where]
    got, want = _one_key_attention(torch.device(device), chunk, key, qpos, n, decoded)
    close(got, want, 5e-4)
    if where in ("before_block", "next"):                       # the key's value is the only positive one
        assert float(got[:12].max()) < 0.0
    else:
        assert float(got[:12].min()) > 0.0


MIX = {"attention": O.diff_attention, "latent_attention": O.latent_attention}


def _latent_case(H, D, Dr, V, R, Q, window, W, scaling=(4.0, 64, 8.0, 1.0)):
    return O.make_config(pattern="m", heads=H, dim=D, rot_dim=Dr, vdim=V, kv_rank=R, q_rank=Q, window=window,
                         scaling=scaling)["layers"][0]["mixer"]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,D,Dr,V,R,Q,window", [(4, 8, 6, 12, 20, 28, 24), (3, 16, 4, 4, 9, 70, 40), (1, 6, 16, 34, 33, 5, 1),
                                                (5, 12, 2, 8, 64, 16, 200)])
def test_latent_attention_mixer(device, H, D, Dr, V, R, Q, window):
    """Query latent, cached latent and shared rotated key part, folded queries, the sliding window,
    the sink: prompt portions and decoded tokens over shuffled pages against the plain rule (which
    expands keys and values per head)."""
    dev, n, W = torch.device(device), 75, 24
    m = _latent_case(H, D, Dr, V, R, Q, window, W, (4.0, 64, 8.0, 1.0) if H != 3 else None)
    w = _weights("latent_attention", m, W, seed=D)
    h = torch.randn(n, W)
    want = O.latent_attention(h.double(), w, "", m, 1e-5).float()
    mod, spec = _mixer("latent_attention", m, w, W, dev, n)
    cache = (torch.zeros(8, 1, BS, R + Dr, device=dev),)
    got = _feed(mod, cache, h, [31, 2, 33, 1, 1, 7], [5, 0, 3], dev)
    close(got, want, 3e-4)


@pytest.mark.gpu
@pytest.mark.parametrize("kind,m", [
    ("attention", dict(heads=8, kv_heads=2, dim=64, vdim=64, rot_dims=32, chunk=100)),
    ("attention", dict(heads=4, kv_heads=4, dim=128, vdim=128, rot_dims=128, chunk=70)),
    ("attention", dict(heads=6, kv_heads=1, dim=64, vdim=128, rot_dims=0, chunk=1000)),
    ("attention", dict(heads=2, kv_heads=1, dim=128, vdim=64, rot_dims=64, chunk=32)),
    ("latent_attention", dict(heads=4, dim=24, rot_dim=32, vdim=24, kv_rank=64, q_rank=40, window=75)),
    ("latent_attention", dict(heads=20, dim=32, rot_dim=64, vdim=16, kv_rank=128, q_rank=32, window=64)),
    ("latent_attention", dict(heads=2, dim=64, rot_dim=64, vdim=64, kv_rank=256, q_rank=48, window=1)),
    ("latent_attention", dict(heads=16, dim=32, rot_dim=64, vdim=24, kv_rank=512, q_rank=40, window=90)),
    ("latent_attention", dict(heads=5, dim=48, rot_dim=32, vdim=40, kv_rank=256, q_rank=64, window=33)),
    ("latent_attention", dict(heads=3, dim=16, rot_dim=32, vdim=16, kv_rank=128, q_rank=32, window=400))])
def test_matrix_core_attention(kind, m):
    """bf16 at head sizes the MFMA kernel tiles: prompt portions that start and end inside 32-key
    tiles, bands whose edges lie inside tiles, decoded tokens; against the plain rule and the FMA kernel."""
    from polykey_service_amd.ops import native
    dev, n, W = torch.device("cuda"), 330, 64
    mm = O.make_config(pattern="a" if kind == "attention" else "m", **m)["layers"][0]["mixer"]
    w = {k: v.bfloat16().double() for k, v in _weights(kind, mm, W, seed=m["heads"]).items()}
    torch.manual_seed(1)
    h = (torch.randn(n, W) * 0.5).bfloat16().float()
    want = MIX[kind](h.double(), w, "", mm, 1e-5).float()
    pages = [9, 3, 0, 7, 5, 1, 8, 2, 6, 4, 10]
    portions = [150, 2, 37, 120] + [1] * 21

    def run():
        mod, spec = _mixer(kind, mm, w, W, dev, n, torch.bfloat16)
        if kind == "attention":
            cache = _attn_cache(spec, 12, dev, torch.bfloat16)
        else:
            cache = (torch.zeros(12, 1, BS, spec.kv_rank + spec.rot_dim, device=dev, dtype=torch.bfloat16),)
        return _feed(mod, cache, h, portions, pages, dev, dtype=torch.bfloat16)
    got = run()
    native.call("pkm_set_masked_mfma", 0)
    try:
        fma = run()
    finally:
        native.call("pkm_set_masked_mfma", 1)
    scale = float(want.pow(2).mean().sqrt())
    assert float((fma - want).pow(2).mean(-1).sqrt().max()) < 0.05 * scale
    assert float((got - want).pow(2).mean(-1).sqrt().max()) < 0.05 * scale
    assert float((got - fma).pow(2).mean(-1).sqrt().max()) < 0.03 * scale


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("back", [0, 1, 63, 64, 87, 88, 89])
@pytest.mark.parametrize("decoded", [False, True])
def test_window_keeps_its_last_keys_only(device, back, decoded):
    """A sliding window of 88: a token ``back`` positions behind the query carries a value nothing
    else has and a key the query matches; it shows for back <= 87 and not beyond, in a prompt
    portion and for decoded tokens (the window's edge lies inside a page)."""
    from polykey_service_amd.ops import masked_attention as ma
    dev = torch.device(device)
    H, D, V, n, window, qpos = 2, 8, 6, 180, 88, 170
    torch.manual_seed(5)
    kc = torch.zeros(8, 1, BS, D, device=dev)
    vc = torch.zeros(8, 1, BS, V, device=dev)
    pages = [6, 2, 4, 0, 5, 1]
    k, v, q = torch.randn(n, 1, D) * 0.2, torch.randn(n, 1, V) * 0.1, torch.randn(n, H, D) * 0.2
    u = torch.randn(D)
    q[qpos], k[qpos - back, 0], v[qpos - back, 0] = u * 3.0, u * 3.0, 50.0
    for p in range(n):
        kc[pages[p // BS], 0, p % BS], vc[pages[p // BS], 0, p % BS] = k[p, 0].to(dev), v[p, 0].to(dev)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
    a, b = (qpos, qpos + 1) if decoded else (qpos - 20, qpos + 5)
    sink = torch.tensor([0.3, -0.2], device=dev)
    o = ma.masked_attention(q[a:b].to(dev), kc, vc, V, i32([pages]), i32([0, b - a]), i32([b]), 1, 1.0, window=window,
                            sink=sink).cpu()[qpos - a]
    sc = torch.einsum("hd,jd->hj", q[qpos].double(), k[:qpos + 1, 0].double())
    lo = max(0, qpos - window + 1)
    e = torch.exp(sc[:, lo:])
    want = (e / (e.sum(-1, keepdim=True) + torch.exp(sink.cpu().double())[:, None])) @ v[lo:qpos + 1, 0].double()
    close(o, want, 3e-4)
    assert (float(o.min()) > 25.0) == (back <= 87)


@pytest.mark.parametrize("device", DEVICES)
def test_sink_takes_its_share(device):
    """With scores near zero a sink logit s holds exp(s) / (keys + exp(s)) of the weight."""
    from polykey_service_amd.ops import masked_attention as ma
    dev = torch.device(device)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
    kc, vc = torch.zeros(2, 1, BS, 4, device=dev), torch.zeros(2, 1, BS, 4, device=dev)
    v = torch.randn(3, 4)
    vc[1, 0, :3] = v.to(dev)
    q = torch.zeros(3, 2, 4, device=dev)
    sink = torch.tensor([0.0, 1.2], device=dev)
    o = ma.masked_attention(q, kc, vc, 4, i32([[1]]), i32([0, 3]), i32([3]), 1, 1.0, sink=sink).cpu()
    close(o[0, 0], v[0] / 2, 1e-5)
    close(o[2, 0], v.sum(0) / 4, 1e-5)
    close(o[2, 1], v.sum(0) / (3 + float(torch.exp(torch.tensor(1.2)))), 1e-5)
    close(ma.masked_attention(q, kc, vc, 4, i32([[1]]), i32([0, 3]), i32([3]), 1, 1.0).cpu()[2, 0], v.mean(0), 1e-5)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,G,D,V,K", [(3, 3, 6, 10, 3), (4, 2, 20, 3, 4), (2, 1, 33, 17, 2), (2, 2, 5, 70, 1), (1, 1, 130, 8, 5)])
def test_delta_mixer(device, H, G, D, V, K):
    """The filter and the recurrence in portions down to one token (state and the filter's last
    inputs carried in a slot, the slot reused by a new sequence) against the token-by-token rule,
    with grouped query / key heads and filters of one to five taps."""
    dev, n, W = torch.device(device), 70, 16
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "conv": K}
    w = _weights("delta", m, W, seed=D)
    mod, spec = _mixer("delta", m, w, W, dev, n)
    C = 2 * G * D + H * V
    cache = (torch.full((3, H, D, V), 7.0, device=dev), torch.full((3, max(K - 1, 1), C), -3.0, device=dev))
    for seq in range(2):
        torch.manual_seed(seq)
        h = torch.randn(n, W)
        want = O.delta(h.double(), w, "", m, 1e-5).float()
        got = _feed(mod, cache, h, [1, 1, 31, 2, 1, 1, 30, 3], [4, 1, 2], dev)
        close(got, want, 3e-4)
    assert float((cache[0][0] - 7.0).abs().max()) == 0.0 and float((cache[1][2] + 3.0).abs().max()) == 0.0


@pytest.mark.parametrize("device", DEVICES)
def test_delta_rule_remembers_and_overwrites(device):
    """A key written 300 tokens back is still read when the gate stays near 1; writing the same
    key again with beta near 1 replaces its value; a head whose gate is small has lost it."""
    from polykey_service_amd.ops import delta as dl
    dev, H, D, V, n = torch.device(device), 2, 4, 4, 330
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
    e0 = torch.zeros(D)
    e0[0] = 1.0
    qkv = torch.zeros(n, 2 * H * D + H * V)
    qkv[:, H * D:2 * H * D] = torch.tensor([0.0, 1.0, 0.0, 0.0]).repeat(H)      # silent tokens write along e1 ...
    ab = torch.zeros(n, 2 * H)
    ab[:, 0], ab[:, 1] = -30.0, 3.0                                              # head 0 keeps (gate ~ 1), head 1 forgets
    ab[:, H:] = -30.0                                                            # ... with beta ~ 0
    for t, val in ((20, 3.0), (200, 5.0)):
        qkv[t, H * D:2 * H * D] = e0.repeat(H)
        qkv[t, 2 * H * D:] = val
        ab[t, H:] = 30.0
    qkv[150, :H * D] = e0.repeat(H)
    qkv[320, :H * D] = e0.repeat(H)
    state = torch.zeros(1, H, D, V, device=dev)
    a_log, dt_bias = torch.zeros(H, device=dev), torch.zeros(H, device=dev)
    outs, at = [], 0
    for c in [100, 150, 60, 2] + [1] * 18:
        pos = torch.arange(at, at + c, dtype=torch.int32, device=dev)
        outs.append(dl.delta_rule(qkv[at:at + c].to(dev).contiguous(), ab[at:at + c].to(dev), a_log, dt_bias, state,
                                  i32([0, c]), 1, pos, i32([0]), H, D, H, V).cpu())
        at += c
    o = torch.cat(outs)
    close(o[150, 0], torch.full((V,), 3.0), 1e-3)
    close(o[320, 0], torch.full((V,), 5.0), 1e-3)
    assert float(o[320, 1].abs().max()) < 1e-3


# ------------------------------------------------------------------ the whole model through the engine
@pytest.mark.parametrize("device", DEVICES)
def test_prompt_logits_match_the_plain_model(device, small):
    cfg, w, path = small
    eng = engine(path, device)
    toks = rand_tokens(100, cfg["vocab"], 1)
    got = replay(eng, [[("a", toks, list(range(100)), True)]])
    close(rows_of(got, "a", 100), O.forward(cfg, w, toks), 5e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_layer_streams_match_the_plain_model(device, small):
    """The residual stream after the last layer run of a model cut after 1, 2, ... layers."""
    cfg, w, _ = small
    from polykey_service_amd.models import build_model
    toks = rand_tokens(40, cfg["vocab"], 2)
    outs = []
    O.forward(cfg, w, toks, outs)
    dev = torch.device(device)
    mc = NopunexConfig.from_json(cfg)
    model = build_model(mc, ParallelState(device=dev), torch.float32, dev).load_state({k: v.float() for k, v in w.items()})
    model.reserve_positions(64)
    caches = model.alloc_cache(2, BS, 1)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
    md = SimpleNamespace(slot_mapping=i32(list(range(BS, 2 * BS)) + list(range(8))), block_tables=i32([[1, 0]]), cu_q=i32([0, 40]),
                         context_lens=i32([40]), num_seqs=1, state_slots=i32([0]), token_seq=i32([0] * 40), num_decode=0)
    x = model(i32(toks), i32(list(range(40))), md, caches)
    close(x.cpu(), outs[-1], 5e-4)
    assert len(outs) == len(mc.runs) == 6


@pytest.mark.parametrize("device", DEVICES)
def test_decoding_equals_prefill(device, small):
    cfg, w, path = small
    eng = engine(path, device)
    toks = rand_tokens(90, cfg["vocab"], 3)
    want = O.forward(cfg, w, toks)
    got = replay(eng, [[s] for s in cut("a", toks, [50])])
    close(rows_of(got, "a", 90), want, 5e-4)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("sizes", [[2, 2, 2, 3, 40, 2, 17], [33, 31, 1, 1, 2], [7] * 14])
def test_portions_of_any_size(device, small, sizes):
    cfg, w, path = small
    eng = engine(path, device)
    toks = rand_tokens(100, cfg["vocab"], 4)
    got = replay(eng, [[s] for s in cut("a", toks, sizes)])
    close(rows_of(got, "a", 100), O.forward(cfg, w, toks), 5e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_mixed_batches_and_reused_pages_and_slots(device, small):
    """Four live requests of unequal lengths, portions beside decoded tokens, a pool that only
    holds them because finished requests give their pages and state slots back."""
    cfg, w, path = small
    eng = engine(path, device, pool_tokens=384, max_seqs=4, budget=384)
    lens = {"a": 120, "b": 37, "c": 64, "d": 90, "e": 70, "f": 33}
    toks = {k: rand_tokens(n, cfg["vocab"], 10 + i) for i, (k, n) in enumerate(lens.items())}
    plans = {"a": cut("a", toks["a"], [40, 30, 2, 2, 30]), "b": cut("b", toks["b"], [30]), "c": cut("c", toks["c"], [2, 50]),
             "d": cut("d", toks["d"], [64, 20]), "e": cut("e", toks["e"], [33, 33]), "f": cut("f", toks["f"], [31])}
    order = [["a", "b", "c"], ["a", "b", "c", "d"]]
    steps, live, waiting = [], ["a", "b", "c", "d"], ["e", "f"]
    while live:
        step = []
        for rid in list(live):
            step.append(plans[rid].pop(0))
            if not plans[rid]:
                live.remove(rid)
                if waiting:
                    live.append(waiting.pop(0))
        steps.append(step)
    got = replay(eng, steps)
    for rid, n in lens.items():
        close(rows_of(got, rid, n), O.forward(cfg, w, toks[rid]), 5e-4)
    assert eng.scheduler.bm.num_free_state_slots == 4


@pytest.mark.parametrize("device", DEVICES)
def test_long_decoding_past_windows_and_blocks(device, tmp_path):
    """One-token steps across several windows, blocks and pages, with other sizes: grouped delta
    heads, one key / value head, no loop, a feed-forward everywhere."""
    cfg = O.make_config(vocab=50, width=40, pattern="DMA", heads=4, kv_heads=1, dim=6, vdim=10, rot_dims=4, ff=24, chunk=20,
                        window=13, kv_rank=12, q_rank=10, rot_dim=4, conv=2, logit_scale=1.0)
    w = O.random_model(cfg, seed=8)
    eng = engine(checkpoint(tmp_path, cfg, w), device)
    toks = rand_tokens(110, cfg["vocab"], 5)
    got = replay(eng, [[s] for s in cut("a", toks, [3])])
    close(rows_of(got, "a", 110), O.forward(cfg, w, toks), 5e-4)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("kw", [dict(pattern="aM", loop=(0, 2, 3), heads=2, kv_heads=2, dim=16, vdim=16, rot_dims=16, chunk=32,
                                     window=32, rot_dim=8, kv_rank=16, q_rank=16, conv=4),
                                dict(pattern="DdA", loop=(1, 2, 1), heads=6, kv_heads=3, dim=4, vdim=6, rot_dims=2, chunk=5,
                                     window=3, rot_dim=2, width=36, scaling=None),
                                dict(pattern="MAD", loop=(2, 3, 2), heads=1, kv_heads=1, dim=10, vdim=7, rot_dims=0, chunk=64,
                                     window=64, rot_dim=10, kv_rank=7, q_rank=50, conv=1)])
def test_other_sizes_and_loop_positions(device, tmp_path, kw):
    """Loops at the start, over one layer once, and at the end; sizes that the small model makes
    equal are unequal here and the other way round; no rotation, full rotation, one head."""
    cfg = O.make_config(**kw)
    w = O.random_model(cfg, seed=9)
    eng = engine(checkpoint(tmp_path, cfg, w), device)
    toks = rand_tokens(80, cfg["vocab"], 6)
    got = replay(eng, [[s] for s in cut("a", toks, [30, 2, 35])])
    close(rows_of(got, "a", 80), O.forward(cfg, w, toks), 5e-4)


def _drawn_config(seed):
    """A configuration drawn from the seed: layer order, loop, head counts and every size."""
    r = random.Random(seed)
    kv = r.choice([1, 2, 3, 4])
    heads = kv * r.choice([1, 2, 3, 4])
    nl = r.randint(3, 6)
    pattern = "".join(r.choice("AMD") if r.random() < 0.75 else r.choice("amd") for _ in range(nl))
    a = r.randint(0, nl - 1)
    loop = (a, r.randint(a + 1, nl), r.randint(1, 3)) if r.random() < 0.8 else None
    dim = r.choice([16, 24, 40, 64, 80])
    return O.make_config(vocab=r.randint(100, 300), width=r.choice([64, 96, 160]), pattern=pattern, heads=heads, kv_heads=kv,
                         dim=dim, vdim=r.choice([16, 24, 48, 72, 128]), rot_dims=r.choice([0, 2, dim // 4 * 2, dim]),
                         ff=r.choice([64, 100, 200]), chunk=r.choice([16, 30, 100]), window=r.choice([8, 31, 100]),
                         kv_rank=r.choice([32, 48, 80, 128]), q_rank=r.choice([32, 72, 136]), rot_dim=r.choice([8, 24, 32, 64]),
                         conv=r.randint(2, 5), loop=loop, diff=r.choice([0.2, 0.35]),
                         scaling=r.choice([None, (4.0, 64, 8.0, 1.0)]), logit_scale=r.choice([1.0, 2.0, 0.5]))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("seed", [1, 2, 3, 4, 5, 6])
def test_drawn_configurations_in_mixed_steps(device, tmp_path, seed):
    """Layer orders, loops and sizes drawn at random, three unequal requests in steps drawn at
    random (a request may sit out a step), against the plain model."""
    cfg = _drawn_config(seed)
    w = O.random_model(cfg, seed=seed, std=0.1)
    r = random.Random(100 + seed)
    lens = {"a": r.randint(100, 200), "b": r.randint(2, 60), "c": r.randint(40, 150)}
    toks = {k: rand_tokens(n, cfg["vocab"], seed * 7 + i) for i, (k, n) in enumerate(lens.items())}
    plans = {k: cut(k, toks[k], [r.choice([2, 3, 17, 33, 64]) for _ in range(r.randint(1, 5))]) for k in lens}
    steps, live = [], list(lens)
    while live:
        step = []
        for rid in list(live):
            if r.random() < 0.85 or len(live) == 1:
                step.append(plans[rid].pop(0))
                if not plans[rid]:
                    live.remove(rid)
        if step:
            steps.append(step)
    got = replay(engine(checkpoint(tmp_path, cfg, w), device), steps)
    for rid, n in lens.items():
        want = O.forward(cfg, w, toks[rid])
        err = (rows_of(got, rid, n).double() - want).pow(2).mean(-1).sqrt() / want.pow(2).mean(-1).sqrt()
        assert float(err.max()) < 1e-3, (rid, cfg["layers"])


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_the_engine(device, small):
    """add_request / step with the scheduler's own batching: two prompts generated together equal
    the plain model's argmax continuation (steps whose top two logits nearly tie are skipped)."""
    cfg, w, path = small
    eng = engine(path, device, graphs=device == "cuda")
    prompts = [rand_tokens(45, cfg["vocab"], 20), rand_tokens(9, cfg["vocab"], 21)]
    outs = eng.generate(prompts, SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True))
    for p, out in zip(prompts, outs):
        assert len(out) == 12
        seq = list(p)
        for tok in out:
            lg = O.forward(cfg, w, seq)[-1]
            top = torch.topk(lg, 2).values
            if float(top[0] - top[1]) > 1e-2:
                assert int(lg.argmax()) == tok
            seq.append(tok)


@pytest.mark.parametrize("device", DEVICES)
def test_preset_with_random_weights_generates(device):
    """The registry's small preset with seeded random weights (no checkpoint folder) through
    add_request / step; the same seed gives the same tokens again."""
    outs = []
    for _ in range(2):
        cfg = EngineConfig(model="tiny-nopunex", dtype="float32", block_size=BS, max_num_seqs=2, max_num_batched_tokens=64,
                           max_model_len=128, num_kv_blocks=8, watermark=0.0, hip_graphs=False, device=device, seed=5)
        eng = LLMEngine(cfg, ParallelState(device=torch.device(device)))
        outs.append(eng.generate([list(range(3, 40)), [7, 8, 9]], SamplingParams(max_tokens=6, temperature=0.0, ignore_eos=True)))
    assert outs[0] == outs[1] and all(len(o) == 6 for o in outs[0])


@pytest.mark.gpu
def test_bfloat16_stays_near_the_plain_model(small):
    """The serving precision: bf16 projections and caches, fp32 stream / norms / scores / state.
    Rounding alone moves this small random model's logits by a few percent (a position where the
    two attention maps nearly cancel by more), so the kernels are also held against the ops'
    PyTorch compositions rounding at the same places."""
    cfg, w, path = small
    toks = rand_tokens(100, cfg["vocab"], 7)
    want = O.forward(cfg, w, toks).float()
    steps = [[s] for s in cut("a", toks, [60, 20])]
    got = rows_of(replay(engine(path, "cuda", dtype="bfloat16", graphs=True), steps), "a", 100)
    ref = rows_of(replay(engine(path, "cpu", dtype="bfloat16"), steps), "a", 100)
    rel = lambda a, b: (a - b).pow(2).mean(-1).sqrt() / b.pow(2).mean(-1).sqrt()
    assert float(rel(got, want).mean()) < 0.1 and float(rel(got, want).median()) < 0.08
    assert float(rel(got, ref).mean()) < 0.03


@pytest.mark.gpu
def test_matrix_core_sizes_in_mixed_batches(tmp_path):
    """A bf16 model at sizes the matrix-core attention kernel tiles: unequal live requests, prompt
    portions beside decoded tokens (whose bands are cut into runs and merged), decode graphs;
    against the ops' compositions at the same precision and the plain model."""
    cfg = O.make_config(vocab=120, width=128, pattern="AMDA", heads=4, kv_heads=2, dim=64, vdim=64, rot_dims=32, ff=128,
                        chunk=100, window=150, kv_rank=128, q_rank=64, rot_dim=32, conv=4, loop=(1, 3, 2))
    w = O.random_model(cfg, seed=12, std=0.12)
    path = checkpoint(tmp_path, cfg, w)
    lens = {"a": 300, "b": 170, "c": 230, "d": 40}
    toks = {k: rand_tokens(n, cfg["vocab"], 30 + i) for i, (k, n) in enumerate(lens.items())}
    plans = {"a": cut("a", toks["a"], [200, 60]), "b": cut("b", toks["b"], [2, 150]), "c": cut("c", toks["c"], [64, 64, 90]),
             "d": cut("d", toks["d"], [33])}
    steps, live = [], list(lens)
    while live:
        step = []
        for rid in list(live):
            step.append(plans[rid].pop(0))
            if not plans[rid]:
                live.remove(rid)
        steps.append(step)
    got = replay(engine(path, "cuda", dtype="bfloat16", pool_tokens=1024, budget=1024, graphs=True), steps)
    ref = replay(engine(path, "cpu", dtype="bfloat16", pool_tokens=1024, budget=1024), steps)
    rel = lambda a, b: (a - b).pow(2).mean(-1).sqrt() / b.pow(2).mean(-1).sqrt()
    for rid, n in lens.items():
        g, r = rows_of(got, rid, n), rows_of(ref, rid, n)
        assert float(rel(g, r).mean()) < 0.03, rid
        assert float(rel(g, O.forward(cfg, w, toks[rid]).float()).median()) < 0.1, rid
