"""Bibezen through the framework (checkpoint loader, scheduler, block manager and state slots,
model runner, kernels) against the plain per-sequence model of tests/oracle_bibezen.py.

Every test builds its own small configuration and random weights, writes them as a checkpoint
folder and loads that through the engine, or drives one op or mixer with hand-made inputs over a
hand-made paged cache and hand-made state slots.  The same tests run on the CPU (the ops' PyTorch
compositions) and, marked gpu, on the HIP kernels."""
import json
import os
import random
import sys
from types import SimpleNamespace

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import oracle_bibezen as O  # noqa: E402

from polykey_service_amd.engine import EngineConfig, LLMEngine, SamplingParams  # noqa: E402
from polykey_service_amd.models.config import BibezenConfig  # noqa: E402
from polykey_service_amd.parallel.state import ParallelState  # noqa: E402

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
BS = 32
D64 = torch.float64


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
    torch.testing.assert_close(a.float().cpu(), b.float().cpu(), rtol=tol, atol=tol)


def rand_tokens(n, vocab, seed):
    return random.Random(seed).choices(range(vocab), k=n)


def rows_of(got, rid, n):
    return torch.stack([got[rid][i] for i in range(n)])


def logits_of(cfg, w, toks):
    return O.forward(cfg, w, toks)[0]


@pytest.fixture
def small(tmp_path):
    # wkv + clamped GLU, parallel + mixture, selective scan + mixture, parallel without a feed-forward
    cfg = O.make_config()
    w = O.random_model(cfg, seed=3)
    return cfg, w, checkpoint(tmp_path, cfg, w)


def i32(v, dev):
    return torch.tensor(v, dtype=torch.int32, device=dev)


class Feed:
    """One sequence fed in portions: pages, slot and step metadata by hand."""

    def __init__(self, dev, pages, slot=1):
        self.dev, self.pages, self.slot, self.at = dev, pages, slot, 0

    def step(self, c):
        dev, at = self.dev, self.at
        pos = torch.arange(at, at + c, dtype=torch.int32, device=dev)
        md = SimpleNamespace(slot_mapping=i32([self.pages[p // BS] * BS + p % BS for p in range(at, at + c)], dev),
                             block_tables=i32([self.pages], dev), cu_q=i32([0, c], dev), context_lens=i32([at + c], dev),
                             num_seqs=1, state_slots=i32([self.slot], dev), token_seq=i32([0] * c, dev),
                             num_decode=1 if (c == 1 and at) else 0)
        self.at += c
        return pos, md


def full(y):
    """A projection's result: a tensor, or the decode GEMM's unreduced slabs."""
    return (y if isinstance(y, torch.Tensor) else y.view().sum(0)).float().cpu()


# ------------------------------------------------------------------ single mechanisms
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("K,C,act,residual,bias,in_bias", [(1, 7, 0, False, False, True), (2, 300, 1, False, True, False),
                                                           (3, 40, 0, True, False, False), (4, 33, 1, False, True, True),
                                                           (6, 5, 0, False, False, False)])
def test_causal_filter_in_portions_with_a_dirty_slot(device, K, C, act, residual, bias, in_bias):
    from polykey_service_amd.ops import short_conv as sc
    dev = torch.device(device)
    g = torch.Generator().manual_seed(K * 100 + C)
    x, taps = torch.randn((50, C + 3), generator=g), torch.randn((C, K), generator=g)
    b, ib = (torch.randn(C, generator=g) if bias else None), (torch.randn(C, generator=g) if in_bias else None)
    xin = x[:, 2:2 + C].double() + (ib.double() if in_bias else 0)
    want = O.causal_filter(xin, taps.double(), b.double() if bias else None)
    if act:
        want = O.silu(want)
    if residual:
        want = want + xin
    state = torch.full((3, max(K - 1, 1), C), 7.0, device=dev) if K > 1 else None   # an earlier owner's rows
    outs, at = [], 0
    to = lambda t: None if t is None else t.to(dev)
    for c in [1, 2, 1, 5, 17, 1, 1, 22]:
        feed = Feed(dev, [0, 1])
        feed.at = at
        pos, md = feed.step(c)
        outs.append(sc.causal_conv(x[at:at + c].to(dev)[:, 2:2 + C], taps.to(dev), to(b), state, md.cu_q, 1, pos, md.state_slots,
                                   md.token_seq, act=act, residual=residual, in_bias=to(ib)))
        at += c
    close(torch.cat(outs), want, 1e-4)


def _one_layer(kind, mixer, W, mlp=None):
    return {"vocab": 4, "width": W, "norm": {"eps": 1e-5}, "layers": [{"type": kind, "mixer": mixer, "mlp": mlp}]}


def _mixer(kind, m, W, dev, seed, n, dtype=torch.float32):
    """The framework's mixer module of ``kind`` with the oracle's random weights, its cache, the weights."""
    from polykey_service_amd.models import bibezen as B
    from polykey_service_amd.ops import masked_attention as ma
    cfg = _one_layer(kind, m, W)
    w = {k[len("l0.mix."):]: v for k, v in O.random_model(cfg, seed, std=0.3).items() if k.startswith("l0.mix.")}
    spec = BibezenConfig.from_json(cfg).layers[0].mixer
    mod = B._MIXERS[kind](spec, W)
    if kind == "wkv":
        mod.set(w.__getitem__, dtype, dev)
    else:
        mod.set(w.__getitem__, w.__contains__, dtype, dev)
    cache = mod.state(3, dev)
    for t in cache.values():
        t.fill_(5.0)                        # whatever an earlier owner of the slot left
    if kind == "parallel":
        a = spec.left
        nb = (n + BS - 1) // BS + 3
        for name, wd in (("k", a.dim), ("v", a.vdim), ("kp", a.dim), ("vp", a.vdim)):
            cache[name] = torch.full((nb, a.kv_heads, BS, wd), 3.0, device=dev, dtype=dtype)
        if a.rot is not None:
            mod.table = ma.table_for(a.rot, n + 3, dev)
    return mod, cache, w


def _feed(mod, cache, h, portions, pages, dev):
    feed, outs = Feed(dev, pages), []
    for c in portions:
        pos, md = feed.step(c)
        outs.append(full(mod(h[feed.at - c:feed.at].to(dev), pos, md, cache, 1e-5)))
    return torch.cat(outs)


PORTIONS = [3, 1, 1, 30, 2, 40, 1, 1, 1, 17]      # 97 tokens over shuffled pages


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,D", [(3, 12), (1, 40), (2, 64), (5, 7), (2, 70)])
def test_wkv_mixer(device, H, D):
    dev, W, n = torch.device(device), 36, sum(PORTIONS)
    m = {"heads": H, "dim": D}
    mod, cache, w = _mixer("wkv", m, W, dev, 11, n)
    h = torch.randn((n, W), generator=torch.Generator().manual_seed(1))
    want = O.wkv(h.double(), {k: v.double() for k, v in w.items()}, m, 1e-5)
    close(_feed(mod, cache, h, PORTIONS, [4, 0, 2, 1], dev), want, 5e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_wkv_state_keeps_a_far_token_with_slow_decay_and_loses_it_with_fast(device):
    """One head, value v0 written at position 0 along key channel 0; r reads channel 0 at the end."""
    from polykey_service_amd.ops import wkv as wk
    dev = torch.device(device)
    n, D = 300, 8
    rkv = torch.zeros((3, n, D))
    rkv[1, 0, 0], rkv[2, 0, :] = 1.0, torch.arange(1, D + 1).float()
    rkv[0, -1, 0] = 1.0
    for z0, keep in ((-9.0, True), (1.0, False)):          # w = exp(-exp(z0)): 0.99988 or 0.066 per step
        state = torch.full((2, 1, D, D), 9.0, device=dev)
        feed, outs = Feed(dev, [0] * 10), []
        for c in [100, 1, 1, 198]:
            pos, md = feed.step(c)
            sl = slice(feed.at - c, feed.at)
            outs.append(wk.wkv_recurrence(rkv[:, sl].contiguous().to(dev), torch.full((c, D), z0, device=dev),
                                          torch.zeros(D, device=dev), torch.zeros(D, device=dev), state, md.cu_q, 1, pos,
                                          md.state_slots, 1, D))
        o = torch.cat(outs).cpu()[-1, 0]
        want = torch.arange(1, D + 1).float() * torch.exp(-torch.exp(torch.tensor(z0))) ** (n - 2)
        close(o, want, 1e-4)
        assert (float(o[-1]) > 5.0) == keep


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("I,N,R,K", [(40, 6, 5, 4), (70, 16, 3, 2), (9, 33, 1, 1), (130, 1, 8, 3)])
def test_selective_scan_mixer(device, I, N, R, K):
    dev, W, n = torch.device(device), 28, sum(PORTIONS)
    m = {"inner": I, "state": N, "dt_rank": R, "conv": K}
    mod, cache, w = _mixer("mamba1", m, W, dev, 12, n)
    h = torch.randn((n, W), generator=torch.Generator().manual_seed(2))
    want = O.selective_scan(h.double(), {k: v.double() for k, v in w.items()}, m)
    close(_feed(mod, cache, h, PORTIONS, [0, 1, 2, 3], dev), want, 5e-4)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,G,D,V,rd,window,pool,conv,cap", [(4, 2, 16, 8, 8, 24, 5, 3, 15.0), (3, 3, 8, 20, 8, 40, 40, 2, 0.0),
                                                             (6, 1, 6, 34, 2, 7, 1, 4, 5.0), (2, 2, 36, 4, 0, 0, 0, 0, 30.0),
                                                             (1, 1, 70, 12, 70, 33, 32, 1, 50.0)])
def test_parallel_mixer(device, H, G, D, V, rd, window, pool, conv, cap):
    dev, W, n = torch.device(device), 30, sum(PORTIONS)
    left = {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "scale": D ** -0.5, "softcap": cap, "conv": conv,
            "mask": {"size": window, "pool": pool}}
    if rd:
        left["rot"] = {"dims": rd, "base": 500.0}
    m = {"left": left, "right": {"heads": 2, "dim": 10}, "left_scale": 0.6, "right_scale": 1.3}
    mod, cache, w = _mixer("parallel", m, W, dev, 13, n)
    h = torch.randn((n, W), generator=torch.Generator().manual_seed(3))
    want = O.parallel(h.double(), {k: v.double() for k, v in w.items()}, m, 1e-5)
    close(_feed(mod, cache, h, PORTIONS, [5, 0, 3, 1], dev), want, 5e-4)


def _probe_attention(dev, window, pool, key, qpos, decoded, H=2, G=1, D=8, V=4, talk=None, sink=None, cap=0.0):
    """Keys and values written by hand; key ``key`` points along the query, the others are small.
    Returns (the framework's output at ``qpos``, the plain rule's) [H, V]."""
    from polykey_service_amd.ops import pooled_attention as pa
    n = qpos + 1
    g = torch.Generator().manual_seed(5)
    k, v = 0.05 * torch.randn((n, G, D), generator=g), torch.randn((n, G, V), generator=g)
    q = 0.05 * torch.randn((n, H, D), generator=g)
    k[key, :, 0], q[qpos, :, 0] = 6.0, 6.0
    pages = [3, 0, 5, 1, 2, 4][: (n + BS - 1) // BS + 1]
    kc, vc = torch.zeros((6, G, BS, D), device=dev), torch.zeros((6, G, BS, V), device=dev)
    kp, vp = torch.full_like(kc, 9.0), torch.full_like(vc, 9.0)
    portions = [qpos, 1] if decoded else [max(qpos - 6, 1), n - max(qpos - 6, 1)]
    feed, out = Feed(dev, pages), None
    for c in [c for c in portions if c > 0]:
        pos, md = feed.step(c)
        sl = md.slot_mapping.long()
        kc[sl // BS, :, sl % BS] = k[feed.at - c:feed.at].to(dev)
        vc[sl // BS, :, sl % BS] = v[feed.at - c:feed.at].to(dev)
        pa.pool_update(kc, vc, kp, vp, pos, md.token_seq, md.block_tables, pool)
        o = pa.pooled_attention(q[feed.at - c:feed.at].contiguous().to(dev), kc, vc, kp, vp, md.block_tables, md.cu_q,
                                md.context_lens, 1, 1.0, cap, window, pool, None if sink is None else sink.to(dev),
                                all_values=talk is not None)
        out = pa.mix_heads(o, None if talk is None else talk.to(dev), 1.0, torch.float32)
    want = O.pooled_softmax(q.double(), k.double(), v.double(), 1.0, cap, window, pool,
                            None if sink is None else sink.double(), None if talk is None else talk.double())
    return out[-1].view(H, V).cpu(), want[qpos], v[key, 0]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("decoded", [False, True])
@pytest.mark.parametrize("back,sees", [(0, "key"), (1, "key"), (39, "key"), (40, "none"), (41, "none"), (44, "mean"), (45, "mean"),
                                        (46, "mean"), (100, "mean")])
def test_window_edge_and_the_first_block_behind_it(device, decoded, back, sees):
    """Window 40, blocks of 6, query at 100: keys 61..100 are seen as they are; blocks 0..9 (keys
    0..59) as their means; key 60 (block 10 ends at 65 > 60) not at all."""
    window, pool, qpos = 40, 6, 100
    key = qpos - back
    got, want, val = _probe_attention(torch.device(device), window, pool, key, qpos, decoded)
    close(got, want, 1e-4)
    if sees == "key":
        close(got[0], val, 1e-2)                       # the one large score takes all the weight
    else:
        assert float((got[0] - val).abs().max()) > 0.2


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("decoded", [False, True])
@pytest.mark.parametrize("qpos", [63, 64, 65, 69, 70, 71])
def test_a_block_is_seen_from_the_position_that_completes_the_gap(device, decoded, qpos):
    """Window 34, blocks of 12: block 2 (keys 24..35) is seen from query 69 on (35 <= q - 34); its
    keys leave the window one by one from query 58 on, so key 30 is invisible for queries 64..68."""
    got, want, _ = _probe_attention(torch.device(device), 34, 12, 30, qpos, decoded, H=4, G=2,
                                    talk=torch.eye(4) + 0.1 * torch.ones((4, 4)), sink=torch.tensor([0.5, -1.0, 2.0, 0.0]),
                                    cap=20.0)
    close(got, want, 1e-4)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("key,qpos", [(0, 0), (0, 1), (31, 32), (32, 32), (32, 33), (0, 95), (63, 64), (64, 127)])
def test_first_tokens_and_page_borders_without_a_window(device, key, qpos):
    for decoded in ([False] if qpos == 0 else [False, True]):
        got, want, val = _probe_attention(torch.device(device), 0, 0, key, qpos, decoded)
        close(got, want, 1e-4)
        close(got[0], val, 1e-2)


@pytest.mark.parametrize("device", DEVICES)
def test_sink_takes_its_share_and_heads_are_mixed(device):
    """All scores zero: n keys and a sink of logit s leave weight 1 / (n + e^s) on each key; head h
    then reads sum_g talk[h, g] of those weights times the mean-free values of its own value head."""
    from polykey_service_amd.ops import pooled_attention as pa
    dev = torch.device(device)
    n, H, G, D, V = 5, 4, 2, 4, 3
    kc, vc = torch.zeros((1, G, BS, D), device=dev), torch.zeros((1, G, BS, V), device=dev)
    vals = torch.randn((n, G, V), generator=torch.Generator().manual_seed(1))
    vc[0, :, :n] = vals.transpose(0, 1).to(dev)
    sink = torch.tensor([0.0, 1.0, -2.0, 3.0])
    talk = torch.randn((H, H), generator=torch.Generator().manual_seed(2))
    o = pa.pooled_attention(torch.zeros((1, H, D), device=dev), kc, vc, None, None, i32([[0]], dev), i32([0, 1], dev),
                            i32([n], dev), 1, 1.0, 0.0, 0, 0, sink.to(dev), all_values=True)
    got = pa.mix_heads(o, talk.to(dev), 2.0, torch.float32).view(H, V).cpu()
    share = 1.0 / (n + torch.exp(sink))                                         # [H]
    want = torch.stack([2.0 * (talk[h] * share).sum() * vals[:, h // 2].sum(0) for h in range(H)])
    close(got, want, 1e-4)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("S,W,T", [(0, 40, 9), (1, 42, 5), (2, 64, 700), (3, 36, 4)])
def test_stream_step_with_scaled_outputs_and_an_ungated_shared_row(device, S, W, T):
    """hyper_step closing a mixture whose shared expert has no gate, with residual_mult folded into
    the output coefficients; spread_rows with the embedding scale."""
    from polykey_service_amd.ops import hyper as hy
    dev = torch.device(device)
    g = torch.Generator().manual_seed(S * 10 + W)
    n = max(S, 1)
    table, ids = torch.randn((11, W), generator=g), torch.randint(0, 11, (T,), generator=g).to(torch.int32)
    xs = hy.spread_rows(table.to(dev), ids.to(dev), n, 1.75)
    close(xs[:, n - 1], table[ids.long()] * 1.75, 1e-6)
    top, rows = 2, 3 * T
    y, shared = torch.randn((rows, W), generator=g), torch.randn((T, W), generator=g)
    inv = torch.randint(0, rows, (T * top,), generator=g).to(torch.int32)
    wts = torch.rand((T, top), generator=g)
    mix, a_out, a_in, nw = torch.randn((n, n), generator=g), torch.randn(n, generator=g), torch.randn(n, generator=g), torch.randn(W, generator=g)
    es = hy.ExpertSum(y.to(dev), inv.to(dev), wts.to(dev), top, shared=shared.to(dev))
    x0 = xs.cpu().double()
    act, _ = hy.hyper_step(xs, es, (mix.to(dev), (0.5 * a_out).to(dev)), (a_in.to(dev), nw.to(dev)), 1e-5, torch.float32)
    f = (y[inv.long()].view(T, top, W).double() * wts[..., None].double()).sum(1) + shared.double()
    x1 = torch.einsum("st,nsw->ntw", mix.double(), x0) + 0.5 * a_out.double()[None, :, None] * f[:, None, :]
    close(xs, x1, 1e-4)
    u = torch.einsum("s,nsw->nw", a_in.double(), x1)
    close(act, O.unit(u, 1e-5) * nw.double(), 2e-4)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("E,top,F_,Fs", [(5, 2, 24, 32), (16, 3, 8, 0), (3, 3, 40, 8), (2, 1, 16, 16)])
def test_mixture_block(device, E, top, F_, Fs):
    from polykey_service_amd.models import bibezen as B
    from polykey_service_amd.models.config import SoftmaxMoESpec
    dev, W, T = torch.device(device), 32, 50
    f = {"kind": "moe", "router": {"experts": E, "top": top}, "expert": {"ff": F_}}
    if Fs:
        f["shared"] = {"ff": Fs}
    cfg = _one_layer("wkv", {"heads": 1, "dim": 4}, W, f)
    w = {k[len("l0.mlp."):]: v for k, v in O.random_model(cfg, 21).items() if k.startswith("l0.mlp.")}
    mod = B.SoftmaxMoE(SoftmaxMoESpec(E, top, F_, Fs))
    part = lambda n: [w[f"e{e}.{n}"] for e in range(E)]
    mod.set(w["router"], part("gate"), part("up"), part("down"),
            tuple(w["shared." + n] for n in ("gate", "up", "down")) if Fs else None, torch.float32, dev)
    h = torch.randn((T, W), generator=torch.Generator().manual_seed(4))
    want = O.moe_ff(h.double(), {k: v.double() for k, v in w.items()}, f)
    close(mod(h.to(dev), h.to(dev)).total(), want, 3e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_router_ties_go_to_the_lower_expert(device):
    from polykey_service_amd.ops import moe
    z = torch.tensor([[1.0, 3.0, 3.0, 0.0], [2.0, 2.0, 2.0, 2.0]], device=torch.device(device))
    ids, wts = moe.route_topk_softmax(z, 4, 2)
    assert ids.cpu().tolist() == [[1, 2], [0, 1]]
    close(wts, torch.full((2, 2), 0.5), 1e-6)


@pytest.mark.parametrize("device", DEVICES)
def test_clamped_feed_forward(device):
    from polykey_service_amd.models import bibezen as B
    from polykey_service_amd.models.config import ClampedFFSpec
    dev, W, F_ = torch.device(device), 24, 40
    g = torch.Generator().manual_seed(6)
    w = {n: torch.randn(s, generator=g) for n, s in (("gate", (F_, W)), ("up", (F_, W)), ("down", (W, F_)))}
    mod = B.ClampedFF(ClampedFFSpec(F_, 1.25))
    mod.set(w["gate"], w["up"], w["down"], torch.float32, dev)
    h = torch.randn((30, W), generator=g)
    want = O.dense_ff(h.double(), {k: v.double() for k, v in w.items()}, {"limit": 1.25})
    close(full(mod(h.to(dev), None)), want, 3e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_head_norm_before_the_rotation(device):
    from polykey_service_amd.ops import masked_attention as ma
    from polykey_service_amd.models.config import RotarySpec
    dev = torch.device(device)
    T, QH, KH, D, V = 7, 3, 1, 12, 5
    g = torch.Generator().manual_seed(7)
    proj = torch.randn((T, (QH + KH) * D + KH * V + 2), generator=g)
    qn, kn = torch.randn(D, generator=g), torch.randn(D, generator=g)
    table = ma.table_for(RotarySpec(8, 100.0, None, True), 40, dev)
    kc, vc = torch.zeros((2, KH, BS, D), device=dev), torch.zeros((2, KH, BS, V), device=dev)
    pos = torch.arange(20, 20 + T, dtype=torch.int32)
    q = ma.rotate_cache(proj.to(dev)[:, :(QH + KH) * D + KH * V], pos.to(dev), pos.to(dev), table, True, kc, vc, QH, KH, KH,
                        D, V, q_norm=qn.to(dev), k_norm=kn.to(dev), eps=1e-3)
    qq = proj[:, :QH * D].view(T, QH, D).double()
    kk = proj[:, QH * D:(QH + KH) * D].view(T, KH, D).double()
    turn = lambda x: O.rotate_halves(torch.cat([torch.zeros((20,) + x.shape[1:], dtype=D64), x]), 8, 100.0)[20:]
    close(q, turn(O.unit(qq, 1e-3) * qn.double()), 1e-4)
    close(kc[0, :, 20:20 + T].transpose(0, 1), turn(O.unit(kk, 1e-3) * kn.double()), 1e-4)
    close(vc[0, 0, 20:20 + T], proj[:, (QH + KH) * D:(QH + KH) * D + V], 1e-6)


# ------------------------------------------------------------------ the whole model through the engine
@pytest.mark.parametrize("device", DEVICES)
def test_prompt_logits_and_layer_streams_match_the_plain_model(device, small):
    cfg, w, path = small
    eng = engine(path, device)
    assert eng.model.embed.device.type == device
    toks = rand_tokens(100, cfg["vocab"], 1)
    want, layers = O.forward(cfg, w, toks)
    got = replay(eng, [[("a", toks, list(range(100)), True)]])
    close(rows_of(got, "a", 100), want, 5e-4)
    # the streams' sum after the last layer, through the model's own forward
    dev = torch.device(device)
    md = SimpleNamespace(slot_mapping=i32(list(range(100)), dev), block_tables=i32([[0, 1, 2, 3]], dev), cu_q=i32([0, 100], dev),
                         context_lens=i32([100], dev), num_seqs=1, state_slots=i32([0], dev), token_seq=i32([0] * 100, dev),
                         num_decode=0)
    xs = eng.model(i32(toks, dev), i32(list(range(100)), dev), md, eng.model.alloc_cache(4, BS, 1))
    close(xs.sum(1), layers[-1], 5e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_decoding_equals_prefill(device, small):
    cfg, w, path = small
    eng = engine(path, device)
    toks = rand_tokens(90, cfg["vocab"], 3)
    got = replay(eng, [[s] for s in cut("a", toks, [50])])
    close(rows_of(got, "a", 90), logits_of(cfg, w, toks), 5e-4)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("sizes", [[2, 2, 2, 3, 40, 2, 17], [33, 31, 1, 1, 2], [7] * 14, [1, 1, 1, 2, 64]])
def test_portions_of_any_size(device, small, sizes):
    cfg, w, path = small
    eng = engine(path, device)
    toks = rand_tokens(100, cfg["vocab"], 4)
    got = replay(eng, [[s] for s in cut("a", toks, sizes)])
    close(rows_of(got, "a", 100), logits_of(cfg, w, toks), 5e-4)


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
        close(rows_of(got, rid, n), logits_of(cfg, w, toks[rid]), 5e-4)
    assert eng.scheduler.bm.num_free_state_slots == 4


@pytest.mark.parametrize("device", DEVICES)
def test_long_decoding_past_windows_blocks_and_pages(device, tmp_path):
    """One-token steps across several windows, blocks and pages, with other sizes: one key / value
    head, a block as long as the window, no streams, no input filter, two experts of which both are used."""
    cfg = O.make_config(pattern=("parallel:moe", "mamba1:dense", "wkv:none"), vocab=50, width=40, streams=0, heads=4, kv_heads=1,
                        dim=6, vdim=10, rot_dims=4, window=13, pool=13, conv=2, wheads=1, wdim=20, inner=24, state=3,
                        dt_rank=2, mconv=2, experts=2, top=2, eff=12, shared=0, taps=0, mult=1.0, scale=1.0)
    w = O.random_model(cfg, seed=8)
    eng = engine(checkpoint(tmp_path, cfg, w), device)
    toks = rand_tokens(110, cfg["vocab"], 5)
    got = replay(eng, [[s] for s in cut("a", toks, [3])])
    close(rows_of(got, "a", 110), logits_of(cfg, w, toks), 5e-4)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("kw", [
    dict(pattern=("mamba1:none", "parallel:dense"), heads=2, kv_heads=2, dim=16, vdim=16, rot_dims=16, window=32, pool=1, conv=1, streams=1),
    dict(pattern=("parallel:moe",), heads=6, kv_heads=3, dim=12, vdim=5, rot_dims=0, window=20, pool=7, conv=5, streams=3, top=1, taps=2),
    dict(pattern=("wkv:moe", "wkv:dense", "mamba1:moe"), wheads=1, wdim=40, streams=4, experts=9, top=4, taps=5, mult=1.5),
    dict(pattern=("parallel:none", "parallel:moe"), heads=3, kv_heads=1, dim=20, vdim=24, rot_dims=6, window=64, pool=32, conv=0,
         softcap=0.0, taps=1)])
def test_other_sizes(device, tmp_path, kw):
    cfg = O.make_config(**kw)
    w = O.random_model(cfg, seed=9)
    eng = engine(checkpoint(tmp_path, cfg, w), device)
    toks = rand_tokens(120, cfg["vocab"], 6)
    got = replay(eng, [[s] for s in cut("a", toks, [31, 2, 70])])
    close(rows_of(got, "a", 120), logits_of(cfg, w, toks), 5e-4)


def _drawn_config(seed):
    r = random.Random(seed)
    kv = r.choice([1, 2, 3])
    kinds, ffs = ["wkv", "mamba1", "parallel"], ["dense", "moe", "none"]
    pattern = tuple(f"{r.choice(kinds)}:{r.choice(ffs)}" for _ in range(r.randint(2, 4))) + ("parallel:moe",)
    dim = r.choice([4, 6, 10, 16])
    experts = r.randint(2, 7)
    return O.make_config(pattern=pattern, vocab=r.randint(40, 90), width=r.choice([24, 36, 50]), streams=r.choice([0, 2, 3]),
                         heads=kv * r.choice([1, 2]), kv_heads=kv, dim=dim, vdim=r.choice([3, 8, 12]),
                         rot_dims=r.choice([0, 2, dim]), window=r.choice([9, 33, 70]), pool=r.choice([1, 4, 11]),
                         conv=r.choice([0, 2, 4]), softcap=r.choice([0.0, 8.0]), wheads=r.randint(1, 3), wdim=r.choice([5, 8, 17]),
                         inner=r.choice([20, 33]), state=r.choice([2, 5, 9]), dt_rank=r.randint(1, 4), mconv=r.randint(1, 4),
                         ff=r.choice([20, 44]), experts=experts, top=r.randint(1, experts), eff=r.choice([8, 20]),
                         shared=r.choice([0, 12]), taps=r.choice([0, 2, 3, 4]), mult=r.choice([0.5, 1.0]))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("seed", [1, 2, 3, 4, 5, 6])
def test_drawn_configurations_in_mixed_steps(device, tmp_path, seed):
    """Layer orders and sizes drawn at random, three unequal requests in steps drawn at random (a
    request may sit out a step), against the plain model."""
    cfg = _drawn_config(seed)
    w = O.random_model(cfg, seed=seed)
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
        want = logits_of(cfg, w, toks[rid])
        err = (rows_of(got, rid, n).double().cpu() - want).pow(2).mean(-1).sqrt() / want.pow(2).mean(-1).sqrt()
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
            lg = logits_of(cfg, w, seq)[-1]
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
        cfg = EngineConfig(model="tiny-bibezen", dtype="float32", block_size=BS, max_num_seqs=2, max_num_batched_tokens=64,
                           max_model_len=128, num_kv_blocks=8, watermark=0.0, hip_graphs=False, device=device, seed=5)
        eng = LLMEngine(cfg, ParallelState(device=torch.device(device)))
        outs.append(eng.generate([list(range(3, 40)), [7, 8, 9]], SamplingParams(max_tokens=6, temperature=0.0, ignore_eos=True)))
    assert outs[0] == outs[1] and all(len(o) == 6 for o in outs[0])


@pytest.mark.gpu
def test_bfloat16_stays_near_the_plain_model(small):
    """The serving precision: bf16 projections and caches, fp32 streams / norms / scores / states.
    The kernels are also held against the ops' PyTorch compositions rounding at the same places."""
    cfg, w, path = small
    toks = rand_tokens(100, cfg["vocab"], 7)
    want = logits_of(cfg, w, toks).float()
    steps = [[s] for s in cut("a", toks, [60, 20])]
    got = rows_of(replay(engine(path, "cuda", dtype="bfloat16", graphs=True), steps), "a", 100).cpu()
    ref = rows_of(replay(engine(path, "cpu", dtype="bfloat16"), steps), "a", 100)
    rel = lambda a, b: (a - b).pow(2).mean(-1).sqrt() / b.pow(2).mean(-1).sqrt()
    assert float(rel(got, want).mean()) < 0.1 and float(rel(got, want).median()) < 0.08
    assert float(rel(got, ref).mean()) < 0.03


@pytest.mark.gpu
def test_aligned_sizes_in_mixed_batches_with_decode_graphs(tmp_path):
    """A bf16 model at sizes the decode GEMM and the grouped expert GEMMs tile (width and expert size
    multiples of 256): unequal live requests, prompt portions beside decoded tokens, decode graphs;
    against the ops' compositions at the same precision and the plain model."""
    cfg = O.make_config(pattern=("wkv:moe", "parallel:dense", "mamba1:moe", "parallel:moe"), vocab=120, width=256, heads=4,
                        kv_heads=2, dim=64, vdim=64, rot_dims=32, window=100, pool=16, conv=4, wheads=4, wdim=64, inner=512,
                        state=16, dt_rank=16, ff=512, experts=4, top=2, eff=256, shared=256)
    w = O.random_model(cfg, seed=12)
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
        g, r = rows_of(got, rid, n).cpu(), rows_of(ref, rid, n)
        assert float(rel(g, r).mean()) < 0.03, rid
        assert float(rel(g, logits_of(cfg, w, toks[rid]).float()).median()) < 0.1, rid


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,D,V,window,pool,talk", [(4, 2, 64, 64, 100, 16, True), (8, 2, 128, 128, 70, 7, True), (2, 2, 32, 8, 0, 0, False),
                                                      (6, 3, 96, 40, 33, 33, True), (16, 4, 128, 128, 200, 64, True), (16, 8, 64, 128, 150, 10, True), (6, 2, 96, 48, 50, 9, True)])
def test_matrix_core_attention_matches_the_fma_tiles(H, G, D, V, window, pool, talk):
    """bf16 at sizes the matrix-core kernel takes: prompt portions and decoded tokens (their key tiles cut into runs
    and merged) against the FMA kernel on the same caches, and against the plain rule."""
    from polykey_service_amd.ops import native
    from polykey_service_amd.ops import pooled_attention as pa
    dev, n = torch.device("cuda"), 300
    g = torch.Generator().manual_seed(H * 100 + D)
    bf = torch.bfloat16
    q = torch.randn((n, H, D), generator=g).to(bf)
    k = (0.5 * torch.randn((n, G, D), generator=g)).to(bf)
    v = torch.randn((n, G, V), generator=g).to(bf)
    sink = torch.randn(H, generator=g)
    tk = (torch.eye(H) + 0.2 * torch.randn((H, H), generator=g)) if talk else None
    pages = [7, 2, 11, 0, 5, 9, 3, 1, 10, 4, 6, 8]
    outs = {}
    for mfma in (1, 0):
        native.mixers().pkm_set_pooled_mfma(mfma)
        try:
            kc, vc = torch.zeros((12, G, BS, D), device=dev, dtype=bf), torch.zeros((12, G, BS, V), device=dev, dtype=bf)
            kp, vp = torch.full_like(kc, 9.0), torch.full_like(vc, 9.0)
            feed, got = Feed(dev, pages), []
            for c in [150, 1, 1, 40, 2, 1, 1, 1, 103]:
                pos, md = feed.step(c)
                sl = md.slot_mapping.long()
                kc[sl // BS, :, sl % BS] = k[feed.at - c:feed.at].to(dev)
                vc[sl // BS, :, sl % BS] = v[feed.at - c:feed.at].to(dev)
                pa.pool_update(kc, vc, kp, vp, pos, md.token_seq, md.block_tables, pool, md.slot_mapping)
                o = pa.pooled_attention(q[feed.at - c:feed.at].contiguous().to(dev), kc, vc, kp, vp, md.block_tables, md.cu_q,
                                        md.context_lens, 1, D ** -0.5, 12.0, window, pool, sink.to(dev), all_values=talk)
                got.append(pa.mix_heads(o, None if tk is None else tk.to(dev), 1.0, torch.float32).cpu())
            outs[mfma] = torch.cat(got).view(n, H, V)
        finally:
            native.mixers().pkm_set_pooled_mfma(1)
    # the block means are rounded to bf16 in the cache; the plain rule keeps them exact
    want = O.pooled_softmax(q.double(), k.double(), v.double(), D ** -0.5, 12.0, window, pool, sink.double(),
                            None if tk is None else tk.double())
    close(outs[1], outs[0], 2e-3)
    close(outs[1], want, 4e-2)
