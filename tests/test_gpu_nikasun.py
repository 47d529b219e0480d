"""The Nikasun decoder through the library against the plain implementation (plain_nikasun.py):
each mechanism alone as a part, then whole models through Engine.step and generate() with every
way of cutting and batching, on configurations made here."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import nikasun_common as N
import plain_nikasun as plain
from tq_kv_amd import Engine, GenerationParams, Model, generate
from tq_kv_amd.cache import Cache
from tq_kv_amd.engine.context import StepContext
from tq_kv_amd.parts import BuildEnv, PartSpec

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda")
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
TOL = {"float32": dict(atol=2e-5, rtol=2e-5), "bfloat16": dict(atol=3e-2, rtol=3e-2)}
ROOT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..")
DTYPES = ["float32", "bfloat16"]


@pytest.fixture(autouse=True)
def _seeded():
    torch.manual_seed(1234)


def load(part, tensors, dtype):
    part.load({k: v.to(DT[dtype]).to(DEV) for k, v in tensors.items()})
    return {k: v.to(DT[dtype]).float() for k, v in tensors.items()}


def rand_weights(part, seed, gain=None):
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, s in part.tensors().items():
        if len(s.shape) == 2:
            out[name] = torch.randn(*s.shape, generator=g) * (gain or {}).get(name, 1.0) / s.shape[1] ** 0.5
        else:
            out[name] = (1.0 if s.init == "one_plus_normal" else 0.0) + 0.1 * torch.randn(*s.shape, generator=g)
    return out


# ---- each mechanism alone ------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
def test_norm_with_weight_around_zero(dtype):
    env = BuildEnv(DEV, DT[dtype])
    norm = env.build("norm", PartSpec("rms_norm", {"size": 150, "eps": 1e-3, "unit_offset": True, "tensor": ""}))
    assert list(norm.tensors()) == [""]
    w = load(norm, rand_weights(norm, 1), dtype)
    x = (3.0 * torch.randn(7, 150)).to(DT[dtype])
    torch.testing.assert_close(norm.forward(x.to(DEV)).float().cpu(), plain.offset_norm(x.float(), w[""], 1e-3), **TOL[dtype])
    h = torch.randn(7, 150, device=DEV)
    want = plain.offset_norm(h.cpu() + x.float(), w[""], 1e-3)
    torch.testing.assert_close(norm.add_norm(h, x.to(DEV)).float().cpu(), want, **TOL[dtype])
    # a weight of zero leaves x over its root mean square: the stored weight is an offset from one
    load(norm, {"": torch.zeros(150)}, dtype)
    torch.testing.assert_close(norm.forward(x.to(DEV)).float().cpu(), plain.rms(x.float(), 1e-3), **TOL[dtype])


GATES = {"relu": lambda g, u: torch.relu(g) * u, "silu": lambda g, u: g * torch.sigmoid(g) * u,
         "gelu_tanh": lambda g, u: plain.gelu_tanh(g) * u}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows", [1, 9, 40, 200])          # the few-row kernels, the mid-sized ones, the library
@pytest.mark.parametrize("gate", ["relu", "silu", "gelu_tanh", "clamped"])
def test_gated_feed_forward(dtype, rows, gate):
    env = BuildEnv(DEV, DT[dtype])
    params = {"hidden": 96, "inter": 72, "gate": gate, "names": {"gate": "a", "up": "b", "down": "c"}}
    if gate == "clamped":
        params.update(limit=0.8, alpha=1.702)
    ff = env.build("feed_forward", PartSpec("gated", params))
    assert sorted(ff.tensors()) == ["a", "b", "c"]
    w = load(ff, rand_weights(ff, 2, {"a": 2.0, "b": 2.0}), dtype)
    x = torch.randn(rows, 96).to(DT[dtype])
    low = DT[dtype]
    if gate == "clamped":
        want = plain.clamped_expert(x.float(), {"gate": w["a"], "up": w["b"], "down": w["c"]}, "", 0.8, low)
        g = plain.product(x.float(), w["a"], low)
        assert (g > 0.8).any() and (plain.product(x.float(), w["b"], low).abs() > 0.8).any()          # the limits bite
    else:
        g, u = plain.product(x.float(), w["a"], low), plain.product(x.float(), w["b"], low)
        want = plain.product(plain.rnd(GATES[gate](g, u), low), w["c"], low)
    torch.testing.assert_close(ff.forward(x.to(DEV), None).float().cpu(), want, **TOL[dtype])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("experts,top,shared", [(6, 2, True), (1, 1, False), (5, 5, False), (70, 3, True)])
@pytest.mark.parametrize("rows", [1, 11, 150, 700])         # tiles of 16, 32 and 64 rows, one and many an expert
def test_routed_experts(dtype, experts, top, shared, rows):
    env = BuildEnv(DEV, DT[dtype])
    hidden, inter = 80, 24
    sh = PartSpec("gated", {"hidden": hidden, "inter": 40, "gate": "clamped", "limit": 2.0, "alpha": 1.702,
                            "names": {"gate": "gate", "up": "up", "down": "down"}}) if shared else None
    ff = env.build("feed_forward", PartSpec("routed_experts", {"hidden": hidden, "inter": inter, "n_experts": experts, "top": top,
                                                               "router_scale": 1.75, "gate": "clamped", "limit": 1.0, "alpha": 1.702,
                                                               "shared": sh}))
    assert ff.graph_safe
    gain = {n: 1.5 for n in ff.tensors() if n.endswith("gate") or n.endswith("up")}
    gain["router"] = 4.0
    w = load(ff, rand_weights(ff, 3, gain), dtype)
    # inputs whose router's choice does not hang on rounding: the first `rows` such of four times as many
    cand = torch.randn(4 * rows + 8, hidden).to(DT[dtype]).float()
    zc = (cand @ w["router"].T).sort(-1, descending=True).values
    keep = torch.ones(cand.shape[0], dtype=torch.bool) if top == experts else (zc[:, top - 1] - zc[:, top]) > 0.1
    x = cand[keep][:rows]
    assert x.shape[0] == rows
    mlp = {"router": {"experts": experts, "top": top, "scale": 1.75}, "expert": {"ff": inter, "limit": 1.0},
           "shared": {"ff": 40, "limit": 2.0} if shared else None}
    want = plain.moe_ff(x, w, "", mlp, DT[dtype])
    got = ff.forward(x.to(DT[dtype]).to(DEV), None).float().cpu()
    # rows whose router's choice hangs on less than rounding are left out (there are none in float32)
    z = (x @ w["router"].T).sort(-1, descending=True).values
    sure = torch.ones(rows, dtype=torch.bool) if top == experts else (z[:, top - 1] - z[:, top]) > (1e-5 if dtype == "float32" else 0.05)
    assert sure.float().mean() > 0.5
    torch.testing.assert_close(got[sure], want[sure], **TOL[dtype])


def test_router_weights_are_scores_times_scale_not_renormalised():
    """One expert gives a constant, the others nothing: the output is that expert's score times the scale."""
    env = BuildEnv(DEV, torch.float32)
    hidden, inter, experts = 32, 8, 4
    ff = env.build("feed_forward", PartSpec("routed_experts", {"hidden": hidden, "inter": inter, "n_experts": experts, "top": 2,
                                                               "router_scale": 3.0, "gate": "clamped", "limit": 5.0, "alpha": 1.702,
                                                               "shared": None}))
    w = {n: torch.zeros(*s.shape) for n, s in ff.tensors().items()}
    w["router"] = torch.randn(experts, hidden)
    x = torch.randn(6, hidden)
    load(ff, w, "float32")
    assert ff.forward(x.to(DEV), None).abs().max().item() == 0.0
    # expert 2: gate = up = 0 except that its down product reads y = g sigmoid(1.702 g) (u + 1) of a gate that is x[0]
    w["e2.gate"][0, 0] = 1.0
    w["e2.down"][:, 0] = 1.0
    load(ff, w, "float32")
    s = torch.softmax(x @ w["router"].T, -1)
    chosen = s.topk(2, -1).indices
    g = x[:, 0].clamp(max=5.0)
    want = torch.where((chosen == 2).any(-1), s[:, 2] * 3.0 * g * torch.sigmoid(1.702 * g), torch.zeros(6))
    got = ff.forward(x.to(DEV), None).cpu()
    torch.testing.assert_close(got, want[:, None].expand(6, hidden), atol=1e-5, rtol=1e-5)


def step_ctx(cache, items):
    sizes = [(s, len(t)) for s, t in items]
    cache.reserve(sizes)
    return StepContext([(s, cache.length(s), t) for s, t in items], [[] for _ in items], cache, DEV), sizes


def latent_spec(m, hidden, eps, own=True, cache_window=None):
    pos = PartSpec("rotary", {"theta": m["rot"]["base"], "rot_dim": m["rot"]["dims"], "max_positions": 512, "style": "halves"})
    return PartSpec("latent_attention", {"hidden": hidden, "n_heads": m["heads"], "head_dim": m["dim"], "rot_dim": m["rot_dim"],
                                         "value_dim": m["vdim"], "q_rank": m["q_rank"], "kv_rank": m["kv_rank"], "scale": m["scale"],
                                         "eps": eps, "window": m["mask"]["size"], "cache_window": cache_window or m["mask"]["size"],
                                         "own_kv": own, "gate": True, "position": pos})


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(5, 24, 8, 40, 48, 56, 23), (1, 8, 2, 8, 16, 8, 1), (3, 10, 6, 14, 20, 18, 130), (2, 64, 32, 64, 96, 128, 64),
                                   (4, 16, 8, 16, 32, 24, 65), (2, 32, 64, 32, 64, 256, 70), (18, 32, 64, 32, 64, 512, 70),
                                   (1, 32, 128, 32, 64, 512, 33)])         # the last three: the kernels' builds for larger latents
def test_latent_attention_part(dtype, shape):
    """Two sequences in shared steps: one in two portions and then token by token, across a page border and past
    its window; the other whole.  A second mixer reads the first one's cache with a window of its own."""
    hidden, eps = 88, 1e-5
    m = N.mixer(*shape, base=40.0)
    m2 = dict(m, mask={"size": shape[6] + 11}, kv_from=0)
    env = BuildEnv(DEV, DT[dtype])
    att = env.build("mixer", latent_spec(m, hidden, eps, cache_window=shape[6] + 11))
    reader = env.build("mixer", latent_spec(m2, hidden, eps, own=False))
    assert att.cache_need() == reader.cache_need() and att.graph_safe
    assert "dkv" in att.tensors() and "dkv" not in reader.tensors()
    gain = {"uq": 2.0, "uk": 2.0, "g": 2.0}
    w, w2 = load(att, rand_weights(att, 4, gain), dtype), load(reader, rand_weights(reader, 5, gain), dtype)
    cache = Cache([att.cache_need(), reader.cache_need()], [None, 0], 64 * 16, 4, DT[dtype], DEV)
    xs = [torch.randn(n, hidden).to(DT[dtype]) for n in (150, 40)]
    slots = [cache.acquire(), cache.acquire()]
    plan = [[(0, 0, 100), (1, 0, 40)], [(0, 100, 126)]] + [[(0, t, t + 1)] for t in range(126, 150)]
    got, got2 = [[], []], [[], []]
    for step in plan:
        ctx, sizes = step_ctx(cache, [(slots[i], [0] * (b - a)) for i, a, b in step])
        x = torch.cat([xs[i][a:b] for i, a, b in step]).to(DEV)
        y, y2 = att.forward(x, ctx, cache.entry(0)), reader.forward(x, ctx, cache.entry(1))
        cache.commit(sizes)
        off = 0
        for i, a, b in step:
            got[i].append(y[off:off + b - a])
            got2[i].append(y2[off:off + b - a])
            off += b - a
    low = DT[dtype]
    for i in range(2):
        pos = torch.arange(xs[i].shape[0])
        kv = plain.latent_kv(xs[i].float(), w, "", m, eps, pos, low)
        # (rows against the outputs' own spread: sharpened scores carry bfloat16 rounding further than an absolute allowance fits)
        N.close(torch.cat(got[i]), plain.latent_attention(xs[i].float(), w, "", m, eps, pos, kv, low), dtype, "own cache, sequence %d" % i, spare=0)
        N.close(torch.cat(got2[i]), plain.latent_attention(xs[i].float(), w2, "", m2, eps, pos, kv, low), dtype, "read cache, sequence %d" % i, spare=0)


# ---- whole models ----------------------------------------------------------------------------------------
_MODELS = {}


def model(name, tmp_path_factory, sharp=1.0):
    key = (name, sharp)
    if key not in _MODELS:
        cfg = {"mixed": N.config_mixed, "ones": N.config_ones, "odd": N.config_odd, "single": lambda: N.config_single(21),
               "single64": lambda: N.config_single(64)}[name]()
        w = N.weights(cfg, seed=11 + len(name), sharp=sharp)
        folder = N.write_folder(str(tmp_path_factory.mktemp("nikasun_%s" % name)), cfg, w)
        _MODELS[key] = (cfg, w, folder, {})
    return _MODELS[key]


def engine(name, dtype, tmp_path_factory, sharp=1.0, max_tokens=4096, slots=8):
    cfg, w, folder, engines = model(name, tmp_path_factory, sharp)
    if dtype not in engines:
        engines[dtype] = Engine(Model.from_dir(folder, dtype=dtype), max_tokens=max_tokens, max_slots=slots)
    return cfg, w, engines[dtype]


def run_cut(eng, toks, cuts, want_all=True):
    """One request alone, its tokens in portions that end at `cuts`; the logits of every position."""
    s = eng.open()
    out, a = [], 0
    for b in list(cuts) + [len(toks)]:
        if b > a:
            out.append(eng.step([(s, toks[a:b], list(range(b - a)))]))
            a = b
    eng.close(s)
    return torch.cat(out)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,sharp", [("mixed", 1.0), ("mixed", 2.0), ("ones", 1.0), ("odd", 2.0)])
def test_whole_prompts_and_every_cut(name, sharp, dtype, tmp_path_factory):
    cfg, w, eng = engine(name, dtype, tmp_path_factory, sharp)
    assert eng.model.spec.architecture == "Nikasun" and eng.model.graph_safe
    toks = N.tokens(200, cfg["vocab"], 5)
    want = N.plain_logits(cfg, w, toks)
    whole = run_cut(eng, toks, [])
    N.close(whole, want, dtype, "whole")
    N.close(whole[:3], want[:3], dtype, "the first tokens", spare=0)
    for cuts in ([64], [63, 65], [1, 3, 128, 130], [150, 152, 154] + list(range(155, 200)), list(range(2, 200, 2)), list(range(1, 200))):
        got = run_cut(eng, toks, cuts)
        N.close(got, want, dtype, "cuts %s" % cuts[:4])
        if dtype == "float32":          # no sum depends on the cut
            assert torch.equal(got, whole), "float32 logits depend on the cut %s" % cuts[:4]


@pytest.mark.parametrize("dtype", DTYPES)
def test_batches_of_unequal_requests_and_reused_slots(dtype, tmp_path_factory):
    cfg, w, eng = engine("mixed", dtype, tmp_path_factory, 2.0, max_tokens=64 * 12, slots=4)
    reqs = [N.tokens(n, cfg["vocab"], 30 + n) for n in (130, 7, 66, 1, 95, 64, 20)]
    want = [N.plain_logits(cfg, w, t) for t in reqs]
    alone = [run_cut(eng, t, []) for t in reqs]
    # three batches one after the other in a cache that only holds them because ended requests give pages and slots
    # back; what they leave behind is overwritten with NaN as soon as nobody holds it
    for batch in ([0, 1, 2, 3], [4, 5, 6, 1], [2, 0, 4]):
        heads = {i: max(1, len(reqs[i]) - 3 - 5 * k) for k, i in enumerate(batch)}
        slots = {i: eng.open() for i in batch}
        poison(eng)
        got = eng.step([(slots[i], reqs[i][:heads[i]], list(range(heads[i]))) for i in batch])
        off = 0
        for i in batch:
            N.close(got[off:off + heads[i]], want[i][:heads[i]], dtype, "prompt of %d in a batch" % i)
            if dtype == "float32":
                assert torch.equal(got[off:off + heads[i]], alone[i][:heads[i]])
            off += heads[i]
        pos, live = dict(heads), [i for i in batch if heads[i] < len(reqs[i])]
        for i in batch:
            if i not in live:
                eng.close(slots[i])
        while live:
            got = eng.step([(slots[i], [reqs[i][pos[i]]], [0]) for i in live])
            for k, i in enumerate(live):
                N.close(got[k:k + 1], want[i][pos[i]:pos[i] + 1], dtype, "request %d decoded at %d" % (i, pos[i]), spare=1.0)
                if dtype == "float32":
                    assert torch.equal(got[k], alone[i][pos[i]])
                pos[i] += 1
            for i in live:
                if pos[i] == len(reqs[i]):
                    eng.close(slots[i])
                    poison(eng)
            live = [i for i in live if pos[i] < len(reqs[i])]


def poison(eng):
    """NaN into every page that no sequence holds: nothing may read them."""
    for g in eng.cache.kv_groups:
        held = {p for pages in g.pages.values() for p in pages if p >= 0}
        free = [p for p in range(g.pool.n) if p not in held]
        if free:
            g.keys[:, torch.tensor(free, device=g.keys.device)] = float("nan")
            g.values[:, torch.tensor(free, device=g.keys.device)] = float("nan")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,window", [("single", 21), ("single64", 64)])
def test_the_window_edge_in_prompts_and_in_decoding(name, window, dtype, tmp_path_factory):
    """One layer: the logits at position i depend on the token at i - window + 1 (the last one seen), as much as the
    plain implementation says, and not at all on the token at i - window."""
    cfg, w, eng = engine(name, dtype, tmp_path_factory, 2.0)
    n = 3 * window + 17
    base = N.tokens(n, cfg["vocab"], 77)
    for i in (window, window + 1, 63, 64, 65, 2 * window + 5, n - 1):
        if i - window < 0:
            continue
        inside, outside = list(base), list(base)
        inside[i - window + 1] = (base[i - window + 1] + 1) % cfg["vocab"]
        outside[i - window] = (base[i - window] + 1) % cfg["vocab"]
        want = {k: N.plain_logits(cfg, w, t[:i + 1])[i] for k, t in (("base", base), ("inside", inside))}
        moved = N.row_errors(want["inside"][None], want["base"][None]).item()
        assert moved > 1e-3                                                                     # the inside token matters
        for cut in (i + 1, i, max(1, i - window // 2)):        # position i in a prompt, decoded alone, decoded after others
            got = {k: run_cut(eng, t[:i + 1], range(cut, i + 1))[i] for k, t in (("base", base), ("inside", inside), ("outside", outside))}
            assert torch.equal(got["outside"], got["base"]), "the token just outside the window reaches position %d (cut %d)" % (i, cut)
            N.close(got["base"][None], want["base"][None], dtype, "position %d" % i, spare=0)
            N.close(got["inside"][None], want["inside"][None], dtype, "position %d, inside token changed" % i, spare=0)
            seen = N.row_errors(got["inside"][None], got["base"][None]).item()
            noise = 0.0 if dtype == "float32" else 0.02          # what bfloat16 rounding alone moves a row by
            assert seen > 0 and 0.5 * moved - noise < seen < 2.0 * moved + noise, "the token just inside the window moves position %d by %.3g, it should by %.3g" % (i, seen, moved)


@pytest.mark.parametrize("dtype", DTYPES)
def test_far_keys_among_hundreds(dtype, tmp_path_factory):
    """A window of 130 positions over 3 pages: the farthest key that the last query still sees matters as much as the
    plain implementation says, in a prompt's portion and in decoding."""
    cfg, w, eng = engine("odd", dtype, tmp_path_factory, 2.0)
    toks = N.tokens(330, cfg["vocab"], 9)
    want = N.plain_logits(cfg, w, toks)
    cuts = [300] + list(range(301, 330))
    got = run_cut(eng, toks, cuts)
    N.close(got, want, dtype, "long windows")
    changed = list(toks)
    changed[329 - 129] = (toks[329 - 129] + 1) % cfg["vocab"]
    want2 = N.plain_logits(cfg, w, changed)
    moved = N.row_errors(want2[329:], want[329:]).item()
    assert moved > 1e-3
    for c in (cuts, [200]):
        seen = N.row_errors(run_cut(eng, changed, c)[329:], run_cut(eng, toks, c)[329:]).item()
        noise = 0.0 if dtype == "float32" else 0.02
        assert seen > 0 and 0.5 * moved - noise < seen < 2.0 * moved + noise


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_long_prompt_in_one_step_and_in_two(dtype, tmp_path_factory):
    """Several hundred tokens in a step: the products per head and per expert run over many of their largest tiles."""
    cfg, w, eng = engine("mixed", dtype, tmp_path_factory, 1.0)
    toks = N.tokens(530, cfg["vocab"], 321)
    want = N.plain_logits(cfg, w, toks)
    whole = run_cut(eng, toks, [])
    N.close(whole, want, dtype, "530 tokens in one step")
    two = run_cut(eng, toks, [270])
    N.close(two, want, dtype, "530 tokens in two steps")
    if dtype == "float32":
        assert torch.equal(two, whole)


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding(dtype, tmp_path_factory):
    cfg, w, eng = engine("mixed", dtype, tmp_path_factory, 1.0)
    toks = N.tokens(5 + 260, cfg["vocab"], 123)
    N.close(run_cut(eng, toks, range(5, len(toks))), N.plain_logits(cfg, w, toks), dtype, "260 tokens one by one")


def test_greedy_generation_through_the_loop(tmp_path_factory):
    cfg, w, eng = engine("mixed", "float32", tmp_path_factory, 1.0)
    prompts = [N.tokens(n, cfg["vocab"], 50 + n) for n in (1, 9, 30, 70)]
    out = generate(eng, prompts, GenerationParams(max_tokens=12, temperature=0.0, repeat_penalty=1.0))
    for p, o in zip(prompts, out):
        assert o == plain.generate_greedy(N.as_float(w), cfg, p, 12)
    _, _, eng16 = engine("mixed", "bfloat16", tmp_path_factory, 1.0)
    out16 = generate(eng16, prompts, GenerationParams(max_tokens=12, temperature=0.0, repeat_penalty=1.0))
    for p, o in zip(prompts, out16):
        ref = N.plain_logits(cfg, w, p + o)
        for i, tok in enumerate(o):
            row = ref[len(p) - 1 + i]
            assert row[tok] >= row.max() - 0.25 * row.std().item()


@pytest.mark.parametrize("dtype", DTYPES)
def test_trace_replay_of_a_folder(dtype, tmp_path_factory, tmp_path):
    cfg, w, folder, _ = model("mixed", tmp_path_factory, 1.0)
    out = str(tmp_path / "out")
    proc = subprocess.Popen([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out", out,
                             "--max-tokens", "300"], stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    reqs = {"a": N.tokens(90, cfg["vocab"], 1), "b": N.tokens(33, cfg["vocab"], 2)}
    want = {k: N.plain_logits(cfg, w, t) for k, t in reqs.items()}

    def step(n, entries, end=()):
        proc.stdin.write(json.dumps({"step": n, "entries": [{"id": i, "tokens": t, "want": wnt} for i, t, wnt in entries], "end": list(end)}) + "\n")
        proc.stdin.flush()
        assert proc.stdout.readline().strip() == "done %d" % n
        path = os.path.join(out, "%d.f32" % n)
        return torch.from_numpy(np.fromfile(path, dtype="<f4")).view(-1, cfg["vocab"]) if os.path.exists(path) else None

    got = step(0, [("a", reqs["a"][:80], [0, 79]), ("b", reqs["b"][:30], [29])])
    N.close(got, torch.stack([want["a"][0], want["a"][79], want["b"][29]]), dtype, "prompts")
    for t in range(3):
        got = step(1 + t, [("a", [reqs["a"][80 + t]], [0]), ("b", [reqs["b"][30 + t]], [0])], end=["b"] if t == 2 else [])
        N.close(got, torch.stack([want["a"][80 + t], want["b"][30 + t]]), dtype, "decoding", spare=1.0)
    assert step(4, [("a", reqs["a"][83:], [])], end=["a"]) is None
    proc.stdin.close()
    assert proc.wait(timeout=60) == 0
