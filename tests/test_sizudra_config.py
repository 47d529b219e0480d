"""Sizudra without a GPU: its configuration keys and their errors, the ModelSpec they become, steps and generation of a
model in host memory on the null device, and the plain implementation pinned by closed forms."""
import copy
import math

import pytest
import torch

import plain_sizudra as plain
import sizudra_common as S
from tq_kv_amd import Engine, GenerationParams, Model, generate
from tq_kv_amd.cache import PAGE
from tq_kv_amd.config import ConfigError, config_from_dict, known_architectures
from tq_kv_amd.config.registry import spec_from_dict


def test_the_architecture_is_known_by_its_name():
    assert "Sizudra" in known_architectures()
    name, typed = config_from_dict(S.config_mixed())
    assert name == "Sizudra"
    assert config_from_dict(typed.to_dict())[1] == typed                # round trip through config.json
    t = typed.to_typed()
    assert (t["vocab"], t["width"], t["norm_eps"]) == (331, 96, 3e-6)
    assert (t["bigram_buckets"], t["bigram_mul_prev"], t["bigram_mul_cur"]) == (97, 31, 5)
    assert [l["type"] for l in t["layers"]] == ["attention", "attention_2", "attention", "attention", "attention_2"]
    assert [l["mixer"]["window"] for l in t["layers"]] == [None, 23, None, None, 70]
    assert [l["mixer"]["keep_first"] for l in t["layers"]] == [0, 5, 0, 0, 0]
    assert [l["mixer"]["v_mix"] for l in t["layers"]] == [False, True, False, True, True]
    assert [None if l["mlp"] is None else l["mlp"]["kind"] for l in t["layers"]] == ["dense", "moe", None, "dense", "moe"]
    assert t["layers"][1]["mlp"]["shared_ff"] == 56 and t["layers"][4]["mlp"]["shared_ff"] is None


def test_the_spec_names_tensors_parts_and_needs():
    spec = spec_from_dict(S.config_mixed())
    assert [(r.layer, r.cache_of) for r in spec.order] == [(i, None) for i in range(5)]
    assert spec.embedding_name == "embed" and spec.head_name == "head" and spec.final_norm_prefix == "final.norm"
    assert spec.stream_position.kind == "pair_hash" and spec.stream_position_prefix == "bigram"
    assert all(l.block.kind == "output_norm" for l in spec.layers)
    mixers = [l.block.params["mixer"].params for l in spec.layers]
    assert [m["value_mix"] for m in mixers] == ["none", "source", "none", "mixed", "mixed"]         # the first that mixes is the source
    assert [m["sink"] for m in mixers] == [False, True, False, False, True]
    assert [m["cap"] for m in mixers] == [None, 6.0, None, None, 30.0]
    assert spec.layers[2].block.params["feed_forward"] is None and spec.layers[2].block.params["ff_out_norm"] is None
    ff = spec.layers[1].block.params["feed_forward"].params
    assert (ff["gated"], ff["normalize"], ff["gate"], ff["shared_gate"]) == (False, "chosen", "relu2", "shared.sg")
    model = Model(spec, dtype="float32", device="cpu")
    names = set(model.tensor_specs())
    assert {"embed", "bigram", "head", "final.norm", "l0.norm1", "l0.norm2", "l1.mix.q.norm", "l1.mix.sink", "l1.mix.vmix", "l3.mix.vmix",
            "l1.mlp.router", "l1.mlp.e5.down", "l1.mlp.shared.sg", "l0.mlp.gate", "l4.mlp.e3.up"} <= names
    assert not {"l2.norm2", "l0.mix.vmix", "l0.mix.sink", "l3.mix.sink", "l1.mlp.e0.gate", "l4.mlp.shared.up", "l4.mlp.shared.sg", "l1.mlp.e6.up"} & names
    specs = model.tensor_specs()
    assert specs["l1.mix.v"].shape == (3 * 40, 96) and specs["l1.mix.o"].shape == (96, 6 * 40) and specs["bigram"].shape == (98, 96)
    assert specs["l1.mix.vmix"].shape == () and specs["l1.mix.sink"].shape == (6,)
    # the cache: keys and values of different sizes, the window with its kept positions, and the previous token as a state
    needs = model.needs
    assert len(needs) == 6 and needs[5].shape == (1,) and needs[5].dtype == "int32"
    assert (needs[1].n_kv_heads, needs[1].head_dim, needs[1].value_dim, needs[1].window, needs[1].keep_first) == (3, 24, 40, 23, 5)
    assert (needs[0].window, needs[0].keep_first) == (None, 0)


@pytest.mark.parametrize("path,value,word", [
    (("width",), None, "width"), (("vocab",), "many", "vocab"), (("norm",), None, "norm"), (("embedding", "bigram", "buckets"), 0, "buckets"),
    (("embedding", "bigram"), None, "bigram"), (("layers",), [], "layers"), (("layers", 0, "type"), "convolution", "convolution"),
    (("layers", 0, "mixer", "heads"), 0, "heads"), (("layers", 0, "mixer", "kv_heads"), 3, "kv_heads"), (("layers", 0, "mixer", "vdim"), None, "vdim"),
    (("layers", 0, "mixer", "rot", "dims"), 7, "dims"), (("layers", 1, "mixer", "mask", "size"), 0, "size"), (("layers", 1, "mixer", "softcap"), None, "softcap"),
    (("layers", 1, "mixer", "mask"), None, "mask"), (("layers", 3, "mixer", "vdim"), 32, "v_mix"),
    (("layers", 1, "mlp", "kind"), "sparse", "sparse"), (("layers", 1, "mlp", "router", "top"), 7, "top"),
    (("layers", 1, "mlp", "expert", "ff"), None, "ff"), (("layers", 0, "mlp", "ff"), -3, "ff")])
def test_what_is_missing_or_wrong_is_named(path, value, word):
    raw = copy.deepcopy(S.config_mixed())
    at = raw
    for key in path[:-1]:
        at = at[key]
    if value is None:
        del at[path[-1]]
    else:
        at[path[-1]] = value
    with pytest.raises(ConfigError, match=word):
        config_from_dict(raw)


@pytest.mark.parametrize("make", [S.config_mixed, S.config_ones, S.config_odd])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_steps_and_generation_on_the_null_device(make, dtype):
    cfg = make()
    model = Model.random(cfg, seed=3, dtype=dtype, device="cpu")
    assert not model.on_gpu and model.graph_safe
    engine = Engine(model, max_tokens=6 * PAGE, max_slots=4)
    free0 = [g.pool.n_free for g in engine.cache.kv_groups]
    a, b = engine.open(), engine.open()
    out = engine.step([(a, S.tokens(150, cfg["vocab"], 1), [0, 149]), (b, S.tokens(3, cfg["vocab"], 2), [2])])
    assert tuple(out.shape) == (3, cfg["vocab"])
    for step in range(3):
        engine.step([(a, [step], [0]), (b, [step], [0])])
    assert (engine.length(a), engine.length(b)) == (153, 6)
    # a window gives the pages between the kept first positions and itself back; nothing else does
    for g in engine.cache.kv_groups:
        pages = g.pages[a]
        if g.need.window is None:
            assert all(p >= 0 for p in pages)
        else:
            first_needed = max(0, 153 + 1 - g.need.window) // PAGE
            kept = -(-g.need.keep_first // PAGE)
            assert [p >= 0 for p in pages] == [i < kept or i >= first_needed for i in range(len(pages))]
    engine.close(a), engine.close(b)
    assert [g.pool.n_free for g in engine.cache.kv_groups] == free0
    engine.cache.check()
    got = generate(engine, [S.tokens(n, cfg["vocab"], 10 + n) for n in (5, 1, 17, 70)], GenerationParams(max_tokens=4, temperature=0.0, repeat_penalty=1.0),
                   eos_ids=(), max_batch=3)
    assert got == [[0] * 4] * 4
    assert [g.pool.n_free for g in engine.cache.kv_groups] == free0


# ---- the plain implementation, pinned by closed forms ----------------------------------------------------
def test_plain_embedding_hashes_the_pair_and_marks_the_first_token():
    table, big = torch.arange(10.0)[:, None] * torch.ones(1, 2), 100.0 * torch.arange(6.0)[:, None] * torch.ones(1, 2)
    x = plain.embed(torch.tensor([3, 4, 9]), table, big, 5, 2, 3)
    # rows: the last (5) for the first token, (3*2 + 4*3) % 5 = 3, (4*2 + 9*3) % 5 = 0
    assert x[:, 0].tolist() == [3 + 500.0, 4 + 300.0, 9 + 0.0]


def test_plain_mask_keeps_the_window_and_the_first_positions():
    m = plain.visible(9, 3, 2)
    assert m[8].tolist() == [True, True, False, False, False, False, True, True, True]
    assert m[2].tolist() == [True, True, True] + [False] * 6 and plain.visible(4)[3].all() and not plain.visible(4)[1, 2]


def test_plain_softmax_with_a_sink_and_a_cap():
    q, k, v = torch.zeros(1, 1, 4), torch.zeros(1, 1, 4), torch.ones(1, 1, 2)
    out = plain.attend(q, k, v, plain.visible(1), 1.0, sink=torch.tensor([0.0]))
    assert torch.allclose(out, torch.full((1, 1, 2), 0.5))              # one key of score 0 and a sink of 0 share the weight
    q = torch.tensor([[[10.0, 0.0]]]).expand(2, 1, 2)
    k = torch.tensor([[[0.0, 0.0]], [[10.0, 0.0]]])
    v = torch.tensor([[[1.0]], [[0.0]]])
    capped = plain.attend(q, k, v, plain.visible(2), 1.0, softcap=2.0)[1, 0, 0].item()
    assert abs(capped - 1.0 / (1.0 + math.exp(2.0 * math.tanh(50.0)))) < 1e-6      # scores 0 and 100 become 0 and 2 tanh(50)


def test_plain_rotation_turns_the_first_elements_only():
    v = torch.tensor([[[1.0, 0.0, 5.0, 7.0]]]).expand(3, 1, 4)
    r = plain.rotate(v, torch.arange(3), 1.0, 2)                        # base 1: the angle is the position
    assert torch.allclose(r[2, 0], torch.tensor([math.cos(2.0), math.sin(2.0), 5.0, 7.0]))


def test_plain_router_renormalises_over_the_chosen():
    idx, wt = plain.route(torch.tensor([[1.0, 0.0]]), torch.tensor([[2.0, 0.0], [0.0, 1.0], [1.0, 0.0], [-1.0, 0.0]]), 2, torch.float32)
    assert idx.tolist() == [[0, 2]] and torch.allclose(wt, torch.softmax(torch.tensor([[2.0, 1.0]]), -1))


def test_more_windows_than_the_cache_has_groups_keep_every_page():
    a = [(S.mixer(2, 1, 8, 8, 4, window=3 + i, keep_first=1), None) for i in range(20)]
    spec = spec_from_dict(S.config(50, 16, a))
    assert all(l.block.params["mixer"].params["cache_keeps_all"] for l in spec.layers)
    model = Model(spec, dtype="float32", device="cpu")
    assert len({(n.window, n.keep_first) for n in model.needs[:20]}) == 1 and model.needs[0].window is None
    few = spec_from_dict(S.config(50, 16, a[:5]))
    assert not any(l.block.params["mixer"].params["cache_keeps_all"] for l in few.layers)
    assert [n.window for n in Model(few, dtype="float32", device="cpu").needs[:5]] == [3, 4, 5, 6, 7]
