"""The Sizudra decoder through the library against the plain implementation (plain_sizudra.py): each mechanism alone,
then whole models through Engine.step and generate() with every way of cutting and batching, on configurations made
here."""
import math

import pytest
import torch

import plain_sizudra as plain
import sizudra_common as S
from tq_kv_amd import Engine, GenerationParams, Model, generate
from tq_kv_amd.cache import PAGE, Cache
from tq_kv_amd.engine.context import StepContext
from tq_kv_amd.parts import BuildEnv, PartSpec

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda")
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
TOL = {"float32": dict(atol=2e-5, rtol=2e-5), "bfloat16": dict(atol=3e-2, rtol=3e-2)}
DTYPES = ["float32", "bfloat16"]


@pytest.fixture(autouse=True)
def _seeded():
    torch.manual_seed(4321)


def load(part, tensors, dtype):
    part.load({k: v.to(DT[dtype]).to(DEV) for k, v in tensors.items()})
    return {k: v.to(DT[dtype]).float() for k, v in tensors.items()}


def rand_weights(part, seed, gain=None):
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, s in part.tensors().items():
        if len(s.shape) == 2:
            out[name] = torch.randn(*s.shape, generator=g) * (gain or {}).get(name, 1.0) / s.shape[1] ** 0.5
        elif len(s.shape) == 0:
            out[name] = 0.25 + 0.5 * torch.rand((), generator=g)
        else:
            out[name] = (gain or {}).get(name, 1.0 if s.init == "one_plus_normal" else 0.0) + 0.3 * torch.randn(*s.shape, generator=g)
    return out


# ---- each mechanism alone ------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows", [1, 9, 40, 200])
def test_feed_forward_of_one_product_and_its_square(dtype, rows):
    env = BuildEnv(DEV, DT[dtype])
    ff = env.build("feed_forward", PartSpec("activated", {"hidden": 96, "inter": 72, "gate": "relu2", "names": {"up": "a", "down": "b"}}))
    assert sorted(ff.tensors()) == ["a", "b"]
    w = load(ff, rand_weights(ff, 2, {"a": 2.0}), dtype)
    x = torch.randn(rows, 96).to(DT[dtype])
    want = plain.expert(x.float(), {"up": w["a"], "down": w["b"]}, "", DT[dtype])
    torch.testing.assert_close(ff.forward(x.to(DEV), None).float().cpu(), want, **TOL[dtype])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows", [1, 9, 40, 200])
def test_dense_feed_forward_with_the_tanh_gelu(dtype, rows):
    env = BuildEnv(DEV, DT[dtype])
    ff = env.build("feed_forward", PartSpec("gated", {"hidden": 80, "inter": 56, "gate": "gelu_tanh", "names": {"gate": "gate", "up": "up", "down": "down"}}))
    w = load(ff, rand_weights(ff, 3, {"gate": 2.0, "up": 2.0}), dtype)
    x = torch.randn(rows, 80).to(DT[dtype])
    torch.testing.assert_close(ff.forward(x.to(DEV), None).float().cpu(), plain.dense_ff(x.float(), w, "", DT[dtype]), **TOL[dtype])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("experts,top,shared", [(6, 2, True), (1, 1, False), (5, 5, True), (70, 3, False)])
@pytest.mark.parametrize("rows", [1, 11, 150, 700])         # tiles of 16, 32 and 64 rows, one and many an expert
def test_routed_experts_without_a_gate_product(dtype, experts, top, shared, rows):
    env = BuildEnv(DEV, DT[dtype])
    hidden, inter = 80, 24
    sh = PartSpec("activated", {"hidden": hidden, "inter": 40, "gate": "relu2", "names": {"up": "up", "down": "down"}}) if shared else None
    ff = env.build("feed_forward", PartSpec("routed_experts", {"hidden": hidden, "inter": inter, "n_experts": experts, "top": top, "router_scale": 1.0,
                                                               "gate": "relu2", "gated": False, "normalize": "chosen", "shared": sh,
                                                               "shared_gate": "shared.sg" if shared else None}))
    assert ff.graph_safe and not any(n.endswith("gate") for n in ff.tensors())
    gain = {n: 1.5 for n in ff.tensors() if n.endswith("up")}
    gain.update({"router": 4.0, "shared.sg": 3.0})
    w = load(ff, rand_weights(ff, 3, gain), dtype)
    cand = torch.randn(4 * rows + 8, hidden).to(DT[dtype]).float()
    zc = (cand @ w["router"].T).sort(-1, descending=True).values
    keep = torch.ones(cand.shape[0], dtype=torch.bool) if top == experts else (zc[:, top - 1] - zc[:, top]) > 0.1
    x = cand[keep][:rows]
    assert x.shape[0] == rows
    mlp = {"router": {"experts": experts, "top": top}, "expert": {"ff": inter}, "shared": {"ff": 40} if shared else None}
    want = plain.moe_ff(x, w, "", mlp, DT[dtype])
    got = ff.forward(x.to(DT[dtype]).to(DEV), None).float().cpu()
    torch.testing.assert_close(got, want, **TOL[dtype])


def test_router_weights_are_the_softmax_over_the_chosen_and_the_shared_expert_is_gated():
    """Every expert gives a constant of its own: the output is the chosen constants weighted by the softmax of their logits alone, plus
    the shared expert's constant times the sigmoid of its gate's product."""
    env = BuildEnv(DEV, torch.float32)
    hidden, inter, experts = 32, 8, 5
    sh = PartSpec("activated", {"hidden": hidden, "inter": 8, "gate": "relu2", "names": {"up": "up", "down": "down"}})
    ff = env.build("feed_forward", PartSpec("routed_experts", {"hidden": hidden, "inter": inter, "n_experts": experts, "top": 2, "router_scale": 1.0,
                                                               "gate": "relu2", "gated": False, "normalize": "chosen", "shared": sh, "shared_gate": "sg"}))
    w = {n: torch.zeros(*s.shape) for n, s in ff.tensors().items()}
    w["router"] = torch.randn(experts, hidden)
    w["sg"] = torch.randn(1, hidden)
    x = torch.randn(6, hidden)
    x[:, 0] = 1.0
    w["router"][:, 0] = 0.0
    w["sg"][:, 0] = 0.0
    consts = [2.0, -1.0, 0.5, 3.0, -4.0]
    for e, c in enumerate(consts):          # up reads x[0] = 1 times sqrt(|c|), squared: |c|; down gives its sign
        w["e%d.up" % e][0, 0] = math.sqrt(abs(c))
        w["e%d.down" % e][:, 0] = math.copysign(1.0, c)
    w["shared.up"][0, 0] = 3.0
    w["shared.down"][:, 0] = 1.0
    load(ff, w, "float32")
    z = x @ w["router"].T
    val, idx = z.topk(2, -1)
    wt = torch.softmax(val, -1)
    want = (wt * torch.tensor(consts)[idx]).sum(-1) + torch.sigmoid(x @ w["sg"].T)[:, 0] * 9.0
    got = ff.forward(x.to(DEV), None).cpu()
    torch.testing.assert_close(got, want[:, None].expand(6, hidden), atol=1e-5, rtol=1e-5)


def step_ctx(cache, items):
    sizes = [(s, len(t)) for s, t in items]
    cache.reserve(sizes)
    return StepContext([(s, cache.length(s), t) for s, t in items], [[] for _ in items], cache, DEV), sizes


def attention_spec(m, hidden, eps, value_mix="none"):
    pos = (PartSpec("rotary", {"theta": m["rot"]["base"], "rot_dim": m["rot"]["dims"], "max_positions": 512, "style": "halves"})
           if m["rot"]["dims"] else PartSpec("none", {"max_positions": 512}))
    mask = m.get("mask")
    return PartSpec("attention", {"hidden": hidden, "n_heads": m["heads"], "n_kv_heads": m["kv_heads"], "head_dim": m["dim"], "value_dim": m["vdim"],
                                  "scale": m["scale"], "qk_norm": True, "eps": eps, "window": mask["size"] if mask else None,
                                  "keep_first": mask["keep_first"] if mask else 0, "cap": m.get("softcap"), "sink": mask is not None,
                                  "value_mix": value_mix, "position": pos,
                                  "names": {"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm", "sink": "sink", "mix": "vmix"}})


SHAPES = [dict(heads=6, kv_heads=3, dim=24, vdim=40, rot_dims=16, window=23, keep_first=5, softcap=6.0),
          dict(heads=1, kv_heads=1, dim=8, vdim=8, rot_dims=2, window=1, keep_first=1, softcap=1.0),
          dict(heads=3, kv_heads=3, dim=10, vdim=14, rot_dims=6, window=130, keep_first=67, softcap=9.0),
          dict(heads=4, kv_heads=1, dim=32, vdim=16, rot_dims=32),
          dict(heads=8, kv_heads=2, dim=64, vdim=64, rot_dims=32, window=64, keep_first=64, softcap=50.0),
          dict(heads=4, kv_heads=4, dim=128, vdim=64, rot_dims=0, window=65, keep_first=3, softcap=30.0),
          dict(heads=16, kv_heads=2, dim=96, vdim=128, rot_dims=64),
          dict(heads=2, kv_heads=1, dim=160, vdim=200, rot_dims=40, window=40, keep_first=0, softcap=25.0)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "h%(heads)dg%(kv_heads)dd%(dim)dv%(vdim)d" % s)
def test_attention_part_with_its_options(dtype, shape):
    """Two sequences in shared steps: one in two portions and then token by token, across a page border and past its
    window; the other whole.  A second mixer mixes its values with those the first one hands on."""
    hidden, eps = 88, 1e-5
    m = S.mixer(**dict(shape, base=40.0, v_mix=True))
    m2 = S.mixer(shape["heads"], shape["kv_heads"], shape["dim"], shape["vdim"], shape["rot_dims"], base=40.0, v_mix=True)
    env = BuildEnv(DEV, DT[dtype])
    att = env.build("mixer", attention_spec(m, hidden, eps, "source"))
    mixed = env.build("mixer", attention_spec(m2, hidden, eps, "mixed"))
    assert att.graph_safe and ("sink" in att.tensors()) == ("mask" in m) and "vmix" in att.tensors()
    gain = {"q.norm": 2.0, "k.norm": 2.0, "sink": 0.5}
    w, w2 = load(att, rand_weights(att, 4, gain), dtype), load(mixed, rand_weights(mixed, 5, gain), dtype)
    cache = Cache([att.cache_need(), mixed.cache_need()], [None, None], 64 * 16, 4, DT[dtype], DEV)
    xs = [torch.randn(n, hidden).to(DT[dtype]) for n in (150, 40)]
    slots = [cache.acquire(), cache.acquire()]
    plan = [[(0, 0, 100), (1, 0, 40)], [(0, 100, 126)]] + [[(0, t, t + 1)] for t in range(126, 150)]
    got, got2 = [[], []], [[], []]
    for step in plan:
        ctx, sizes = step_ctx(cache, [(slots[i], [0] * (b - a)) for i, a, b in step])
        x = torch.cat([xs[i][a:b] for i, a, b in step]).to(DEV)
        y, y2 = att.forward(x, ctx, cache.entry(0)), mixed.forward(x, ctx, cache.entry(1))
        cache.commit(sizes)
        off = 0
        for i, a, b in step:
            got[i].append(y[off:off + b - a])
            got2[i].append(y2[off:off + b - a])
            off += b - a
    low = DT[dtype]
    for i in range(2):
        pos = torch.arange(xs[i].shape[0])
        carried = {}
        out = plain.mixer(xs[i].float(), w, "", m, eps, pos, low, carried)
        S.close(torch.cat(got[i]), out, dtype, "the source, sequence %d" % i, spare=0)
        assert S.row_errors(torch.cat(got[i]), out).max().item() < 0.02        # a mixer alone is held much closer than whole models
        assert "v_first" in carried
        S.close(torch.cat(got2[i]), plain.mixer(xs[i].float(), w2, "", m2, eps, pos, low, carried), dtype, "mixed values, sequence %d" % i, spare=0)


# ---- whole models ----------------------------------------------------------------------------------------
_MODELS = {}
MAKERS = {"mixed": S.config_mixed, "ones": S.config_ones, "odd": S.config_odd, "single": lambda: S.config_single(21, 3),
          "single_page": lambda: S.config_single(64, 64), "single_all": lambda: S.config_single(0, 0, plain_attention=True)}


def model(name, tmp_path_factory, sharp=1.0, change=None):
    key = (name, sharp, change is not None and change.__name__)
    if key not in _MODELS:
        cfg = MAKERS[name]()
        w = S.weights(cfg, seed=11 + len(name), sharp=sharp)
        if change:
            change(cfg, w)
        folder = S.write_folder(str(tmp_path_factory.mktemp("sizudra_%s" % name)), cfg, w)
        _MODELS[key] = (cfg, w, folder, {})
    return _MODELS[key]


def engine(name, dtype, tmp_path_factory, sharp=1.0, max_tokens=4096, slots=8, change=None):
    cfg, w, folder, engines = model(name, tmp_path_factory, sharp, change)
    if dtype not in engines:
        engines[dtype] = Engine(Model.from_dir(folder, dtype=dtype), max_tokens=max_tokens, max_slots=slots)
    return cfg, w, engines[dtype]


def run_cut(eng, toks, cuts):
    """One request alone, its tokens in portions that end at `cuts`; the logits of every position."""
    s = eng.open()
    out, a = [], 0
    for b in list(cuts) + [len(toks)]:
        b = min(b, len(toks))
        if b > a:
            out.append(eng.step([(s, toks[a:b], list(range(b - a)))]))
            a = b
    eng.close(s)
    return torch.cat(out)


def silent_layers(cfg, w):
    """No layer adds anything: what is left is the two embeddings, the final norm and the head."""
    for name in w:
        if name.endswith("mix.o") or name.endswith(".down"):
            w[name] = torch.zeros_like(w[name])


@pytest.mark.parametrize("dtype", DTYPES)
def test_pair_embedding_alone_whole_and_in_portions(dtype, tmp_path_factory):
    cfg, w, eng = engine("odd", dtype, tmp_path_factory, change=silent_layers)
    f = S.as_float(w)
    toks = S.tokens(70, cfg["vocab"], 3)
    big = cfg["embedding"]["bigram"]
    x = plain.embed(torch.tensor(toks), f["embed"], f["bigram"], big["buckets"], big["mul_prev"], big["mul_cur"])
    want = plain.rnd(plain.rms_norm(x, f["final.norm"], cfg["norm"]["eps"]), DT[dtype]) @ f["head"].T
    for cuts in ([], [1], [2, 3, 4], [64], list(range(1, 70))):
        S.close(run_cut(eng, toks, cuts), want, dtype, "cuts %s" % cuts[:4], spare=0)
    # two requests whose pieces meet in one step: each takes its own previous token
    a, b = eng.open(), eng.open()
    eng.step([(a, toks[:5], []), (b, toks[10:12], [])])
    got = eng.step([(b, toks[12:13], [0]), (a, toks[5:9], [0, 3])])
    eng.close(a), eng.close(b)
    first = plain.embed(torch.tensor(toks[10:13]), f["embed"], f["bigram"], big["buckets"], big["mul_prev"], big["mul_cur"])
    want_b = plain.rnd(plain.rms_norm(first, f["final.norm"], cfg["norm"]["eps"]), DT[dtype]) @ f["head"].T
    S.close(got, torch.stack([want_b[2], want[5], want[8]]), dtype, "two requests", spare=0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,sharp", [("mixed", 1.0), ("mixed", 2.0), ("ones", 1.0), ("odd", 2.0)])
def test_whole_prompts_and_every_cut(name, sharp, dtype, tmp_path_factory):
    cfg, w, eng = engine(name, dtype, tmp_path_factory, sharp)
    assert eng.model.spec.architecture == "Sizudra" and eng.model.graph_safe
    toks = S.tokens(200, cfg["vocab"], 5)
    want = S.plain_logits(cfg, w, toks)
    whole = run_cut(eng, toks, [])
    S.close(whole, want, dtype, "whole")
    S.close(whole[:3], want[:3], dtype, "the first tokens", spare=0)
    for cuts in ([64], [63, 65], [1, 3, 128, 130], [150, 152, 154] + list(range(155, 200)), list(range(2, 200, 2)), list(range(1, 200))):
        got = run_cut(eng, toks, cuts)
        S.close(got, want, dtype, "cuts %s" % cuts[:4])
        if dtype == "float32":          # no sum depends on the cut
            assert torch.equal(got, whole), "float32 logits depend on the cut %s" % cuts[:4]


def poison(eng):
    """NaN into every page that no sequence holds: nothing may read them."""
    for g in eng.cache.kv_groups:
        held = {p for pages in g.pages.values() for p in pages if p >= 0}
        free = [p for p in range(g.pool.n) if p not in held]
        if free:
            g.keys[:, torch.tensor(free, device=g.keys.device)] = float("nan")
            g.values[:, torch.tensor(free, device=g.keys.device)] = float("nan")


@pytest.mark.parametrize("dtype", DTYPES)
def test_batches_of_unequal_requests_and_reused_slots(dtype, tmp_path_factory):
    cfg, w, eng = engine("mixed", dtype, tmp_path_factory, 2.0, max_tokens=64 * 12, slots=4)
    reqs = [S.tokens(n, cfg["vocab"], 30 + n) for n in (130, 7, 66, 1, 95, 64, 20)]
    want = [S.plain_logits(cfg, w, t) for t in reqs]
    alone = [run_cut(eng, t, []) for t in reqs]
    # three batches one after the other in a cache that only holds them because ended requests give pages and slots back;
    # what they leave behind is overwritten with NaN as soon as nobody holds it
    for batch in ([0, 1, 2, 3], [4, 5, 6, 1], [2, 0, 4]):
        heads = {i: max(1, len(reqs[i]) - 3 - 5 * k) for k, i in enumerate(batch)}
        slots = {i: eng.open() for i in batch}
        poison(eng)
        got = eng.step([(slots[i], reqs[i][:heads[i]], list(range(heads[i]))) for i in batch])
        off = 0
        for i in batch:
            S.close(got[off:off + heads[i]], want[i][:heads[i]], dtype, "prompt of %d in a batch" % i)
            if dtype == "float32":
                assert torch.equal(got[off:off + heads[i]], alone[i][:heads[i]])
            off += heads[i]
        pos, live = dict(heads), [i for i in batch if heads[i] < len(reqs[i])]
        for i in batch:
            if i not in live:
                eng.close(slots[i])
        while live:
            poison(eng)
            got = eng.step([(slots[i], [reqs[i][pos[i]]], [0]) for i in live])
            for k, i in enumerate(live):
                S.close(got[k:k + 1], want[i][pos[i]:pos[i] + 1], dtype, "request %d decoded at %d" % (i, pos[i]), spare=1.0)
                if dtype == "float32":
                    assert torch.equal(got[k], alone[i][pos[i]])
                pos[i] += 1
            for i in live:
                if pos[i] == len(reqs[i]):
                    eng.close(slots[i])
            live = [i for i in live if pos[i] < len(reqs[i])]
    eng.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,window,keep", [("single", 21, 3), ("single_page", 64, 64), ("single_all", None, 0)])
def test_a_token_reaches_the_logits_exactly_through_the_window_and_the_kept_positions(name, window, keep, dtype, tmp_path_factory):
    """One layer: changing the token at j changes the logits at i if and only if i sees j (or j is i or the token before it, which the
    pair embedding reads).  Queries in a prompt, in a second portion, and decoded one by one; keys at page borders, just inside and
    just outside the window, the last kept and the first not kept, and far away."""
    cfg, w, eng = engine(name, dtype, tmp_path_factory, sharp=3.0)
    n = 200
    toks = S.tokens(n, cfg["vocab"], 8)

    def sees(i, j):
        return j <= i and (window is None or i - j < window or j < keep)

    def logits_of(tokens, how):
        if how == "prompt":
            return run_cut(eng, tokens, [])
        if how == "portions":
            return run_cut(eng, tokens, [61, 63, 130])
        return run_cut(eng, tokens, [100] + list(range(101, n)))

    queries = [130, 150, 191, 199]
    for how in ("prompt", "portions", "decoded"):
        base = logits_of(toks, how)
        S.close(base, S.plain_logits(cfg, w, toks), dtype, how)
        for i in queries:
            edge = i - (window or 0)
            for j in sorted({0, 1, keep - 1, keep, keep + 1, 63, 64, 65, edge - 1, edge, edge + 1, edge + 2, 127, 128, i - 2}):
                if j < 0 or j + 2 > i:
                    continue
                changed = list(toks)
                changed[j] = (toks[j] + 1 + j) % cfg["vocab"]
                got = logits_of(changed[:i + 1], how if i >= 131 or how != "portions" else "prompt")[i]
                # the token after j reads j through the pair embedding: it counts as seen if i sees j + 1
                reached = sees(i, j) or sees(i, j + 1)
                moved = (got - base[i]).abs().max().item()
                if reached:
                    # (a key among many may weigh little: in float32 any weight at all shows, in bfloat16 rounding may hide it)
                    assert moved > 0.0 or dtype == "bfloat16", "%s: query %d does not see the token at %d" % (how, i, j)
                elif not sees(i, j + 1):
                    assert moved == 0.0 if dtype == "float32" else moved < 1e-6, "%s: query %d sees the token at %d (moved %.3g)" % (how, i, j, moved)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,sharp", [("single_all", 3.0), ("odd", 1.0)])
def test_keys_far_away_and_long_decoding(name, sharp, dtype, tmp_path_factory):
    """A prompt of some pages, then a hundred tokens decoded one by one, past the windows.  In the model of one layer that sees everything,
    head norms scaled up make single keys among hundreds carry the output."""
    cfg, w, eng = engine(name, dtype, tmp_path_factory, sharp=sharp)
    toks = S.tokens(700, cfg["vocab"], 21)
    want = S.plain_logits(cfg, w, toks)
    s = eng.open()
    got = [eng.step([(s, toks[:600], [0, 1, 2, 300, 599])])]
    for t in range(600, 700):
        got.append(eng.step([(s, [toks[t]], [0])]))
    eng.close(s)
    rows = [0, 1, 2, 300, 599] + list(range(600, 700))
    S.close(torch.cat(got), want[rows], dtype, "a long sequence")


@pytest.mark.parametrize("dtype", DTYPES)
def test_greedy_generation_through_the_loop(dtype, tmp_path_factory):
    cfg, w, eng = engine("mixed", dtype, tmp_path_factory, 1.0)
    prompts = [S.tokens(n, cfg["vocab"], 50 + n) for n in (1, 9, 70, 33, 128)]
    params = GenerationParams(max_tokens=12, temperature=0.0, repeat_penalty=1.0)
    out = generate(eng, prompts, params, eos_ids=(), max_batch=3)
    for p, o in zip(prompts, out):
        assert len(o) == 12
        # the plain implementation, token by token; a step whose two best logits are closer than rounding may go either way
        seq = list(p)
        for k, t in enumerate(o):
            z = S.plain_logits(cfg, w, seq)[-1]
            best = z.topk(2).values
            if int(z.argmax()) != t:
                assert dtype == "bfloat16" and (best[0] - z[t]).item() < 0.05 * z.std().item(), "token %d of a prompt of %d" % (k, len(p))
            seq.append(t)
    # the same requests again, in another order and batch size, give the same tokens
    again = generate(eng, prompts[::-1], params, eos_ids=(), max_batch=2)
    assert again[::-1] == out or dtype == "bfloat16"


# ---- the programs a user runs ---------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
def test_replay_of_steps_and_the_command_line(dtype, tmp_path_factory):
    """bin/trace_run fed steps on standard input (a request whole, then its last tokens one by one beside a second request, a tensor
    too many in the folder), and bin/tq generate on the same folder: logits and greedy tokens of the plain implementation."""
    import json
    import os
    import subprocess
    import sys

    import numpy as np
    from test_gpu_trace_run import Replay
    root = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..")
    cfg = S.config_odd()
    w = S.weights(cfg, seed=77)
    w["l0.mix.unused"] = torch.zeros(3, dtype=torch.bfloat16)
    folder = S.write_folder(str(tmp_path_factory.mktemp("sizudra_replay")), cfg, w)
    del w["l0.mix.unused"]
    a, b = S.tokens(150, cfg["vocab"], 1), S.tokens(9, cfg["vocab"], 2)
    want_a, want_b = S.plain_logits(cfg, w, a), S.plain_logits(cfg, w, b)
    r = Replay(folder, dtype, str(tmp_path_factory.mktemp("out")), max_tokens=64 * 6)
    got = r.step([("x", a, list(range(150)))], end=["x"])
    S.close(got.view(-1, cfg["vocab"]), want_a, dtype, "whole")
    assert r.step([("y", a[:140], []), ("z", b[:5], [])]) is None
    for t in range(10):
        live = [("y", [a[140 + t]], [0])] + ([("z", [b[5 + t]], [0])] if t < 4 else [])
        got = r.step(live, end=(["y"] if t == 9 else []) + (["z"] if t == 3 else [])).view(-1, cfg["vocab"])
        S.close(got[0:1], want_a[140 + t:141 + t], dtype, "one by one at %d" % t, spare=1.0)
        if t < 4:
            S.close(got[1:2], want_b[5 + t:6 + t], dtype, "the second request at %d" % t, spare=1.0)
    r.finish()
    if dtype != "float32":
        return
    cmd = [sys.executable, os.path.join(root, "bin", "tq"), "--fp32", "generate", folder, "--allow-extra-tensors", "--prompt-ids",
           ",".join(str(t) for t in b), "-n", "5", "-t", "0", "--repeat-penalty", "1.0", "--json"]
    out = subprocess.run(cmd, capture_output=True, text=True)
    assert out.returncode == 0, out.stderr
    tokens = json.loads(out.stdout.strip().splitlines()[-1])["outputs"][0]
    seq = list(b)
    for t in tokens:
        assert int(S.plain_logits(cfg, w, seq)[-1].argmax()) == t
        seq.append(t)


def test_a_model_of_more_windows_than_the_cache_has_groups(tmp_path_factory):
    """Twenty layers with twenty windows: the cache keeps every page in one group, and each layer still sees its own window."""
    cfg = S.config(50, 32, [(S.mixer(2, 1, 8, 8, 4, v_mix=l % 3 == 0, window=3 + 4 * l, keep_first=l % 5), S.dense(24) if l % 2 else None) for l in range(20)])
    w = S.weights(cfg, seed=5)
    eng = Engine(Model.from_dir(S.write_folder(str(tmp_path_factory.mktemp("sizudra_windows")), cfg, w), dtype="float32"), max_tokens=64 * 8, max_slots=2)
    assert len(eng.cache.kv_groups) == 1
    toks = S.tokens(150, cfg["vocab"], 9)
    want = S.plain_logits(cfg, w, toks)
    S.close(run_cut(eng, toks, []), want, "float32", "whole")
    S.close(run_cut(eng, toks, [70] + list(range(100, 150))), want, "float32", "a portion and single tokens")


def test_a_step_of_many_blocks(tmp_path_factory):
    """Sixteen prompts of 512 tokens and more in one step: enough tiles for the prompt attention's blocks of eight waves (bfloat16)."""
    a = S.mixer(32, 8, 16, 24, 8, base=100.0, v_mix=True)
    b = S.mixer(32, 8, 16, 24, 8, base=100.0, v_mix=True, window=100, keep_first=70, softcap=20.0)
    cfg = S.config(80, 64, [(a, S.dense(48)), (b, S.dense(48)), (a, None)])
    w = S.weights(cfg, seed=3, sharp=1.5)
    eng = Engine(Model.from_dir(S.write_folder(str(tmp_path_factory.mktemp("sizudra_blocks")), cfg, w), dtype="bfloat16"), max_tokens=64 * 200, max_slots=16)
    reqs = [S.tokens(512 + 3 * i, cfg["vocab"], 60 + i) for i in range(16)]
    slots = [eng.open() for _ in reqs]
    got = eng.step([(s, t, [0, 255, len(t) - 2, len(t) - 1]) for s, t in zip(slots, reqs)])
    for i, t in enumerate(reqs):
        want = S.plain_logits(cfg, w, t)[[0, 255, len(t) - 2, len(t) - 1]]
        S.close(got[4 * i:4 * i + 4], want, "bfloat16", "request %d" % i, spare=0)
    for s in slots:
        eng.close(s)
