"""Sizudra configurations drawn at random from a seed (sizes, head counts and groups, key and value sizes, how much of a head is
rotated, layer order, windows and kept positions, caps, which layers mix values, which feed-forward, buckets and multipliers), each
against the plain implementation in float32 and bfloat16: a whole prompt, the same prompt in two portions and single tokens, and two
requests of unequal lengths in one batch."""
import random

import pytest
import torch

import sizudra_common as S
from tq_kv_amd import Engine, Model

pytestmark = pytest.mark.gpu


def draw(seed):
    r = random.Random(seed)
    width = r.choice([48, 64, 96, 160, 200, 256])
    n_layers = r.randint(1, 5)
    # the layers that mix values share kv heads and value size
    mix_kv, mix_dv = r.choice([1, 2, 3, 4]), r.choice([8, 16, 24, 40, 64, 72, 128])
    layers = []
    for l in range(n_layers):
        mixes = r.random() < 0.6
        kv = mix_kv if mixes else r.choice([1, 2, 4, 5])
        heads = kv * r.choice([1, 1, 2, 3, 4, 5, 8])
        dim = r.choice([8, 16, 24, 32, 40, 48, 64, 80, 96, 128, 12, 20])
        vdim = mix_dv if mixes else r.choice([8, 12, 16, 32, 48, 64, 96, 136])
        rot = r.choice([0, 2, dim // 2 // 2 * 2, dim // 4 * 2 if dim >= 8 else 2, dim])
        second = r.random() < 0.5
        m = S.mixer(heads, kv, dim, vdim, rot, base=r.choice([10.0, 500.0, 10000.0, 1e6]), v_mix=mixes,
                    window=r.choice([1, 7, 32, 63, 64, 65, 100, 300]) if second else None, keep_first=r.choice([0, 0, 1, 4, 63, 64, 70, 130]),
                    softcap=r.choice([2.0, 8.0, 30.0, 50.0]))
        m["scale"] *= r.uniform(0.5, 1.5)
        kind = r.choice(["dense", "moe", "moe", "none"])
        if kind == "dense":
            f = S.dense(r.choice([24, 64, 100, 256]))
        elif kind == "moe":
            experts = r.choice([1, 2, 4, 8, 16, 33])
            f = S.moe(experts, r.randint(1, min(experts, 4)), r.choice([8, 16, 40, 64]), shared=r.choice([8, 32, 72]) if r.random() < 0.6 else None)
        else:
            f = None
        layers.append((m, f))
    return S.config(r.choice([64, 101, 256, 500]), width, layers, eps=r.choice([1e-6, 1e-5, 1e-3]),
                    bigram=(r.choice([1, 7, 64, 1021]), r.choice([0, 1, 31, 1000003]), r.choice([1, 17, 65537])))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(20))
def test_random_configuration(seed, dtype, tmp_path):
    cfg = draw(2000 + seed)
    w = S.weights(cfg, seed, sharp=1.5)
    eng = Engine(Model.from_dir(S.write_folder(str(tmp_path), cfg, w), dtype=dtype), max_tokens=64 * 24, max_slots=4)
    a, b = S.tokens(150 + 7 * seed, cfg["vocab"], seed), S.tokens(40 + seed, cfg["vocab"], 100 + seed)
    want_a, want_b = S.plain_logits(cfg, w, a), S.plain_logits(cfg, w, b)
    # bfloat16: rows one of whose routers chooses by less than rounding reaches are left out (float32 compares every row)
    keep_a = S.sure_rows(cfg, w, a) if dtype == "bfloat16" else torch.ones(len(a), dtype=torch.bool)
    keep_b = S.sure_rows(cfg, w, b) if dtype == "bfloat16" else torch.ones(len(b), dtype=torch.bool)
    assert keep_a.float().mean() > 0.3
    s = eng.open()
    whole = eng.step([(s, a, list(range(len(a))))])
    eng.close(s)
    S.close_typical(whole[keep_a], want_a[keep_a], dtype, "whole")
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
    S.close_typical(torch.cat(got_a)[keep_a], want_a[keep_a], dtype, "portions and single tokens")
    S.close_typical(torch.cat(got_b)[keep_b], want_b[keep_b], dtype, "the request alongside")
    if dtype == "float32":
        assert torch.equal(torch.cat(got_a), whole)
