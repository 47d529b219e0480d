"""Nikasun without a GPU: its configuration keys and their errors, the ModelSpec they become, steps and
generation of a model in host memory on the null device, and the plain implementation pinned by closed forms."""
import copy
import math

import pytest
import torch

import nikasun_common as N
import plain_nikasun as plain
from tq_kv_amd import Engine, GenerationParams, Model, generate
from tq_kv_amd.cache import PAGE
from tq_kv_amd.config import ConfigError, config_from_dict, known_architectures
from tq_kv_amd.config.registry import spec_from_dict


def test_the_architecture_is_known_by_its_name():
    assert "Nikasun" in known_architectures()
    name, typed = config_from_dict(N.config_mixed())
    assert name == "Nikasun"
    assert config_from_dict(typed.to_dict())[1] == typed and typed.layers[3].mixer.kv_from == 0          # round trip through config.json
    typed = typed.to_typed()
    assert (typed["vocab"], typed["width"], typed["norm_eps"], typed["embedding_scale"]) == (331, 96, 3e-6, 7.5)
    assert [l["mixer"]["kv_from"] for l in typed["layers"]] == [None, None, None, 0, 2]
    assert [None if l["mlp"] is None else l["mlp"]["kind"] for l in typed["layers"]] == ["moe", None, "dense", "moe", "dense"]
    assert typed["layers"][0]["mlp"]["shared"] == {"ff": 56, "limit": 2.5} and typed["layers"][3]["mlp"]["shared"] is None


def test_the_spec_names_tensors_order_and_windows():
    spec = spec_from_dict(N.config_mixed())
    assert [(r.layer, r.cache_of) for r in spec.order] == [(0, None), (1, None), (2, None), (3, 0), (4, 2)]
    assert spec.embedding_name == "embed" and spec.head_name is None and spec.final_norm_prefix == "final.norm"
    mixers = [l.block.params["mixer"].params for l in spec.layers]
    assert [m["window"] for m in mixers] == [23, 70, 70, 37, 9]
    assert [m["cache_window"] for m in mixers] == [37, 70, 70, 37, 70]          # an owner keeps what its readers need
    assert [m["own_kv"] for m in mixers] == [True, True, True, False, False]
    assert spec.layers[1].block.params["feed_forward"] is None and spec.layers[1].block.params["ff_norm"] is None
    model = Model(spec, dtype="float32", device="cpu")
    names = set(model.tensor_specs())
    assert {"embed", "final.norm", "l0.norm1", "l0.norm2", "l0.mix.dkv", "l0.mlp.router", "l0.mlp.e5.down", "l0.mlp.shared.up",
            "l2.mlp.gate", "l3.mix.uk", "l3.mlp.e3.gate"} <= names
    assert not {"l1.norm2", "l3.mix.dkv", "l3.mix.dkv.norm", "l3.mlp.shared.gate", "l0.mlp.e6.gate"} & names
    assert model.tensor_specs()["l3.mix.uq"].shape == (5 * 32, 48) and model.tensor_specs()["l0.mix.dkv"].shape == (56 + 8, 96)


@pytest.mark.parametrize("path,value,word", [
    (("width",), None, "width"), (("vocab",), "many", "vocab"), (("norm",), None, "norm"), (("embedding", "scale"), None, "scale"),
    (("layers",), [], "layers"), (("layers", 0, "type"), "convolution", "convolution"), (("layers", 0, "mixer", "heads"), 0, "heads"),
    (("layers", 0, "mixer", "kv_rank"), None, "kv_rank"), (("layers", 0, "mixer", "rot", "dims"), 7, "dims"),
    (("layers", 0, "mixer", "mask", "size"), 0, "size"), (("layers", 3, "mixer", "kv_from"), 3, "kv_from"),
    (("layers", 4, "mixer", "kv_from"), 3, "kv_from"), (("layers", 3, "mixer", "kv_rank"), 64, "kv_rank"),
    (("layers", 0, "mlp", "kind"), "sparse", "sparse"), (("layers", 0, "mlp", "router", "top"), 7, "top"),
    (("layers", 0, "mlp", "expert", "limit"), None, "limit"), (("layers", 2, "mlp", "ff"), -3, "ff")])
def test_what_is_missing_or_wrong_is_named(path, value, word):
    raw = copy.deepcopy(N.config_mixed())
    at = raw
    for key in path[:-1]:
        at = at[key]
    if value is None:
        del at[path[-1]]
    else:
        at[path[-1]] = value
    with pytest.raises(ConfigError, match=word):
        config_from_dict(raw)


@pytest.mark.parametrize("make", [N.config_mixed, N.config_ones, N.config_odd])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_steps_and_generation_on_the_null_device(make, dtype):
    cfg = make()
    model = Model.random(cfg, seed=3, dtype=dtype, device="cpu")
    assert not model.on_gpu and model.graph_safe
    engine = Engine(model, max_tokens=6 * PAGE, max_slots=4)
    free0 = [g.pool.n_free for g in engine.cache.kv_groups]
    a, b = engine.open(), engine.open()
    out = engine.step([(a, N.tokens(150, cfg["vocab"], 1), [0, 149]), (b, N.tokens(3, cfg["vocab"], 2), [2])])
    assert tuple(out.shape) == (3, cfg["vocab"])
    for step in range(3):
        engine.step([(a, [step], [0]), (b, [step], [0])])
    assert (engine.length(a), engine.length(b)) == (153, 6)
    engine.close(a), engine.close(b)
    assert [g.pool.n_free for g in engine.cache.kv_groups] == free0
    engine.cache.check()
    got = generate(engine, [N.tokens(n, cfg["vocab"], n) for n in (4, 1, 20)], GenerationParams(max_tokens=3, temperature=0.0, repeat_penalty=1.0),
                   eos_ids=(), max_batch=2)
    assert got == [[0] * 3] * 3
    engine.cache.check()


def test_windowed_layers_give_pages_back_and_shared_caches_are_one():
    cfg = N.config_mixed()
    engine = Engine(Model.random(cfg, seed=1, dtype="float32", device="cpu"), max_tokens=16 * PAGE, max_slots=2)
    # three runs keep a cache (two of them alike), two read one: two groups, three runs' worth of pages
    assert sorted(len(g.runs) for g in engine.cache.kv_groups) == [1, 2]
    s = engine.open()
    engine.step([(s, N.tokens(500, cfg["vocab"], 1), [])])
    for g in engine.cache.kv_groups:
        held = [p for p in g.pages[s] if p >= 0]
        assert len(held) <= (g.need.window + PAGE - 1) // PAGE + 1          # what left the window went back
    engine.close(s)


# ---- the plain implementation, pinned ------------------------------------------------------------------------
def test_plain_norms():
    x = torch.tensor([[3.0, -4.0, 0.0, 0.0]])
    torch.testing.assert_close(plain.rms(x, 0.0), x / 2.5)
    torch.testing.assert_close(plain.offset_norm(x, torch.zeros(4), 0.0), x / 2.5)           # a stored zero multiplies by one
    torch.testing.assert_close(plain.plain_norm(x, torch.zeros(4), 0.0), torch.zeros(1, 4))   # here it multiplies by zero
    assert abs(plain.rms(torch.zeros(1, 4), 0.25)).max() == 0 and plain.rms(torch.ones(1, 4), 3.0)[0, 0].item() == 0.5  # eps inside the root


def test_plain_rotation_pairs_halves_and_keeps_the_rest():
    v = torch.tensor([[1.0, 2.0, 3.0, 4.0, 9.0, 8.0]])
    out = plain.rotate(v.repeat(3, 1), torch.tensor([0, 1, 5]), base=100.0, dims=4)
    torch.testing.assert_close(out[0], v[0])
    f = [1.0, 100.0 ** -0.5]
    for row, p in ((1, 1.0), (2, 5.0)):
        for i in range(2):
            a = p * f[i]
            assert out[row, i].item() == pytest.approx(v[0, i] * math.cos(a) - v[0, i + 2] * math.sin(a), abs=1e-6)
            assert out[row, i + 2].item() == pytest.approx(v[0, i + 2] * math.cos(a) + v[0, i] * math.sin(a), abs=1e-6)
    assert out[:, 4:].tolist() == [[9.0, 8.0]] * 3
    # scores of rotated vectors depend on the distance alone
    q, k = torch.randn(1, 8), torch.randn(1, 8)
    s = [(plain.rotate(q, torch.tensor([p]), 50.0, 8) * plain.rotate(k, torch.tensor([p - 3]), 50.0, 8)).sum().item() for p in (3, 40)]
    assert s[0] == pytest.approx(s[1], abs=1e-4)


def test_plain_window_and_softmax():
    m = plain.window_mask(5, 2)
    assert m.int().tolist() == [[1, 0, 0, 0, 0], [1, 1, 0, 0, 0], [0, 1, 1, 0, 0], [0, 0, 1, 1, 0], [0, 0, 0, 1, 1]]
    p = plain.softmax_rows(torch.zeros(5, 5), m)
    assert p[0].tolist() == [1, 0, 0, 0, 0] and p[4].tolist() == [0, 0, 0, 0.5, 0.5]


def test_plain_gates_and_router():
    w = {"gate": torch.tensor([[1.0]]), "up": torch.tensor([[1.0]]), "down": torch.tensor([[1.0]])}
    y = plain.clamped_expert(torch.tensor([[5.0], [-5.0], [0.5]]), w, "", 2.0, torch.float32).flatten().tolist()
    s = lambda g: g / (1 + math.exp(-1.702 * g))
    assert y[0] == pytest.approx(s(2.0) * 3.0, rel=1e-6)        # gate cut from above, up cut to the limit, plus one
    assert y[1] == pytest.approx(s(-5.0) * -1.0, rel=1e-5)      # the gate is not cut from below, up is
    assert y[2] == pytest.approx(s(0.5) * 1.5, rel=1e-6)
    assert plain.dense_ff(torch.tensor([[-2.0], [3.0]]), w, "", torch.float32).flatten().tolist() == [0.0, 9.0]
    idx, wt = plain.route(torch.eye(3), torch.tensor([[2.0, 0, 0], [1.0, 3.0, 0], [0, 0, 0], [0.5, 0, 1.0]]), 2, 10.0, torch.float32)
    z = torch.tensor([2.0, 1.0, 0.0, 0.5])
    assert idx[0].tolist() == [0, 1] and wt[0].tolist() == pytest.approx((10.0 * torch.softmax(z, 0)[:2]).tolist())
    assert wt[0].sum().item() < 10.0                            # not renormalised
    assert plain.gelu_tanh(torch.tensor(1.0)).item() == pytest.approx(0.841192, abs=1e-5)


def test_plain_layers_that_share_a_cache_and_layers_without_feed_forward():
    cfg = N.config_mixed()
    w = N.as_float(N.weights(cfg, 1))
    toks = N.tokens(50, cfg["vocab"], 1)
    base = plain.forward(w, cfg, toks)
    # the reading layer has no key-value projection: giving it the owner's changes nothing; the owner's matters to both
    assert "l3.mix.dkv" not in w
    w2 = dict(w)
    w2["l0.mix.dkv"] = w["l0.mix.dkv"] * 1.5
    assert not torch.allclose(plain.forward(w2, cfg, toks), base)
    assert "l1.norm2" not in w and base.shape == (50, cfg["vocab"]) and torch.isfinite(base).all()
    # causal
    torch.testing.assert_close(plain.forward(w, cfg, toks[:20]), base[:20], atol=1e-5, rtol=1e-5)


def test_more_windows_than_cache_groups_share_the_largest():
    """Twenty layers with windows of their own: caches of equal row size then keep the largest window, each layer still
    sees its own."""
    cfg = N.config(64, 32, [(N.mixer(2, 8, 8, 8, 16, 24, 10 + 3 * i), N.dense(16)) for i in range(20)])
    spec = spec_from_dict(cfg)
    mixers = [l.block.params["mixer"].params for l in spec.layers]
    assert {m["cache_window"] for m in mixers} == {67} and [m["window"] for m in mixers] == [10 + 3 * i for i in range(20)]
    engine = Engine(Model.random(cfg, seed=0, dtype="float32", device="cpu"), max_tokens=10 * PAGE, max_slots=2)
    assert len(engine.cache.kv_groups) == 1
    # with few windows every cache keeps its own
    few = N.config(64, 32, [(N.mixer(2, 8, 8, 8, 16, 24, w), None) for w in (5, 70, 5)])
    assert [l.block.params["mixer"].params["cache_window"] for l in spec_from_dict(few).layers] == [5, 70, 5]
