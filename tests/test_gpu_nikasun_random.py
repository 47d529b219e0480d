"""Nikasun configurations drawn at random from a seed (sizes, head counts, layer order, windows, constants, which
layers read whose cache, which feed-forward), each against the plain implementation in float32 and bfloat16: a
whole prompt, the same prompt in two portions and single tokens, and two requests of unequal lengths in one batch."""
import random

import pytest
import torch

import nikasun_common as N
from tq_kv_amd import Engine, Model

pytestmark = pytest.mark.gpu


def draw(seed):
    r = random.Random(seed)
    width = r.choice([48, 64, 96, 160, 200, 256])
    kinds = []
    n_layers = r.randint(1, 5)
    layers, owners = [], []
    for l in range(n_layers):
        reads = owners and r.random() < 0.4
        if reads:
            src = r.choice(owners)
            m = dict(layers[src][0])
            m.pop("kv_from", None)
            heads, dim, vdim, q_rank = r.choice([1, 2, 4, 7, 16, 20]), r.choice([8, 16, 32, 40]), r.choice([8, 16, 24, 64]), r.choice([16, 24, 64])
            m.update(heads=heads, dim=dim, vdim=vdim, q_rank=q_rank, mask={"size": r.choice([1, 5, 31, 64, 65, 200])},
                     scale=r.uniform(0.5, 1.5) / (dim + m["rot_dim"]) ** 0.5, kv_from=src)
        else:
            rot = r.choice([2, 8, 16, 32])
            m = N.mixer(r.choice([1, 3, 4, 6, 16, 18]), r.choice([8, 16, 32, 64]), rot, r.choice([8, 16, 32, 64]), r.choice([16, 32, 48, 128]),
                        r.choice([8, 24, 32, 64, 128, 256]) if rot % 8 == 0 else r.choice([6, 14, 30]), r.choice([1, 7, 32, 63, 64, 100, 300]),
                        base=r.choice([10.0, 500.0, 10000.0, 1e6]), scale=None)
            m["scale"] *= r.uniform(0.5, 1.5)
            owners.append(l)
        kind = r.choice(["dense", "moe", "moe", "none"])
        if kind == "dense":
            f = N.dense(r.choice([24, 64, 100, 256]))
        elif kind == "moe":
            experts = r.choice([1, 2, 4, 8, 16, 33])
            f = N.moe(experts, r.randint(1, min(experts, 4)), r.uniform(0.5, 3.0), r.choice([8, 16, 40, 64]), r.uniform(0.5, 4.0),
                      shared=(r.choice([8, 32, 72]), r.uniform(0.5, 4.0)) if r.random() < 0.6 else None)
        else:
            f = None
        kinds.append(kind)
        layers.append((m, f))
    return N.config(r.choice([64, 101, 256, 500]), width, layers, eps=r.choice([1e-6, 1e-5, 1e-3]), embedding_scale=r.uniform(0.5, 2.0) * width ** 0.5)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(16))
def test_random_configuration(seed, dtype, tmp_path):
    cfg = draw(1000 + seed)
    w = N.weights(cfg, seed, sharp=1.5)
    eng = Engine(Model.from_dir(N.write_folder(str(tmp_path), cfg, w), dtype=dtype), max_tokens=64 * 24, max_slots=4)
    a, b = N.tokens(150 + 7 * seed, cfg["vocab"], seed), N.tokens(40 + seed, cfg["vocab"], 100 + seed)
    want_a, want_b = N.plain_logits(cfg, w, a), N.plain_logits(cfg, w, b)
    s = eng.open()
    whole = eng.step([(s, a, list(range(len(a))))])
    eng.close(s)
    N.close(whole, want_a, dtype, "whole", spare=0.04)
    # two portions, then single tokens, with the second request alongside from its first token to its end
    sa, sb = eng.open(), eng.open()
    cut1, cut2 = 70 + seed, len(a) - 20
    got_a = [eng.step([(sa, a[:cut1], list(range(cut1)))])]
    both = eng.step([(sa, a[cut1:cut2], list(range(cut2 - cut1))), (sb, b[:-10], list(range(len(b) - 10)))])
    got_a.append(both[:cut2 - cut1])
    got_b = [both[cut2 - cut1:]]
    for i in range(20):
        items = [(sa, [a[cut2 + i]], [0])]
        if i < 10:
            items.append((sb, [b[len(b) - 10 + i]], [0]))
        out = eng.step(items)
        got_a.append(out[:1])
        if i < 10:
            got_b.append(out[1:])
        if i == 9:
            eng.close(sb)
    eng.close(sa)
    N.close(torch.cat(got_a), want_a, dtype, "portions and single tokens", spare=0.04)
    N.close(torch.cat(got_b), want_b, dtype, "the request alongside", spare=0.04)
    if dtype == "float32":
        assert torch.equal(torch.cat(got_a), whole)
