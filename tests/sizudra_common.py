"""Shared by the Sizudra tests: small configurations made here, random weights of a sensible size, model folders
written with the safetensors package, and how logits are compared."""
import json
import math
import os

import torch
from safetensors.torch import save_file

import plain_sizudra as plain


def mixer(heads, kv_heads, dim, vdim, rot_dims, base=10000.0, scale=None, v_mix=False, window=None, keep_first=0, softcap=None):
    """window given: a layer of the second kind (score cap, window with kept first positions, sink)."""
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "rot": {"base": base, "dims": rot_dims},
         "scale": scale if scale is not None else 1.0 / math.sqrt(dim)}
    if v_mix:
        m["v_mix"] = True
    if window is not None:
        m["mask"] = {"size": window, "keep_first": keep_first}
        m["softcap"] = softcap if softcap is not None else 20.0
    return m


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, shared=None):
    m = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if shared is not None:
        m["shared"] = {"ff": shared}
    return m


def config(vocab, width, layers, eps=1e-5, bigram=(251, 7, 13)):
    return {"architecture": "Sizudra", "vocab": vocab, "width": width, "norm": {"eps": eps},
            "embedding": {"bigram": {"buckets": bigram[0], "mul_prev": bigram[1], "mul_cur": bigram[2]}},
            "layers": [{"type": "attention_2" if "mask" in m else "attention", "mixer": m, "mlp": f} for m, f in layers]}


# Sizes chosen away from each other: 6 heads in 3 groups with values larger than keys, a layer of one group whose heads are
# rotated whole and that takes no part in the value mixing, a layer without a feed-forward, windows that are no multiple of
# anything, kept first positions, experts with and without a shared one, all experts chosen in one layer.
def config_mixed():
    a = mixer(6, 3, 24, 40, 16, base=5000.0, v_mix=True, window=23, keep_first=5, softcap=6.0)
    b = mixer(4, 1, 32, 16, 32, base=300.0)
    c = mixer(3, 3, 16, 40, 8, base=5000.0, v_mix=True)
    d = mixer(6, 3, 24, 40, 0, v_mix=True, window=70, keep_first=0, softcap=30.0)
    return config(331, 96, [(b, dense(72)), (a, moe(6, 2, 40, shared=56)), (b, None), (c, dense(136)), (d, moe(4, 4, 24))], eps=3e-6, bigram=(97, 31, 5))


# The smallest of everything: one head, one expert of which one is chosen, a window of one position that keeps the first
# one, two rotated elements, one bucket.
def config_ones():
    a = mixer(1, 1, 8, 8, 2, base=2.0, v_mix=True, window=1, keep_first=1, softcap=1.0)
    b = mixer(1, 1, 8, 8, 2, base=2.0, v_mix=True)
    return config(67, 32, [(a, moe(1, 1, 16)), (b, dense(16))], eps=1e-4, bigram=(1, 1, 1))


# Sizes that are no multiples of 8, a window and kept first positions beyond a page of the cache.
def config_odd():
    a = mixer(3, 3, 10, 14, 6, base=777.0, v_mix=True, window=130, keep_first=67, softcap=9.0)
    b = mixer(6, 3, 12, 14, 12, base=777.0, v_mix=True)
    return config(101, 52, [(b, dense(44)), (a, moe(5, 3, 12, shared=20)), (b, moe(3, 1, 20, shared=12))], eps=1e-5, bigram=(50, 101, 3))


# One layer and nothing else mixes tokens (the pair embedding aside, which reaches one token on): a token outside the
# window and the kept positions cannot reach the logits at all.
def config_single(window, keep_first, width=64, plain_attention=False):
    m = mixer(4, 2, 16, 24, 8, base=50.0) if plain_attention else mixer(4, 2, 16, 24, 8, base=50.0, window=window, keep_first=keep_first, softcap=15.0)
    return config(97, width, [(m, dense(48))], bigram=(61, 3, 11))


def weights(cfg, seed, sharp=1.0, store=torch.bfloat16):
    """name -> tensor of the store dtype.  Products keep the size of what they read (std 1/sqrt(inputs)); the routers are
    made decisive; sharp > 1 scales the heads' norm weights up so that attention picks out single keys."""
    g = torch.Generator().manual_seed(seed)

    def lin(o, i, gain=1.0):
        return (torch.randn(o, i, generator=g) * gain / math.sqrt(i)).to(store)

    def vec(n, around, spread=0.1):
        return (around + spread * torch.randn(n, generator=g)).to(store)

    D = cfg["width"]
    big = cfg["embedding"]["bigram"]
    w = {"embed": lin(cfg["vocab"], D, math.sqrt(D)), "bigram": lin(big["buckets"] + 1, D, 0.7 * math.sqrt(D)), "head": lin(cfg["vocab"], D),
         "final.norm": vec(D, 1.0)}
    for i, layer in enumerate(cfg["layers"]):
        p, m, f = "l%d." % i, layer["mixer"], layer["mlp"]
        H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        w[p + "norm1"] = vec(D, 1.0)
        w[p + "mix.q"] = lin(H * d, D)
        w[p + "mix.k"] = lin(G * d, D)
        w[p + "mix.v"] = lin(G * dv, D)
        w[p + "mix.o"] = lin(D, H * dv)
        w[p + "mix.q.norm"] = vec(d, sharp)
        w[p + "mix.k.norm"] = vec(d, sharp)
        if m.get("v_mix"):
            w[p + "mix.vmix"] = (0.25 + 0.5 * torch.rand((), generator=g)).to(store)
        if "mask" in m:
            w[p + "mix.sink"] = vec(H, 0.5, 1.0)
        if f is None:
            continue
        w[p + "norm2"] = vec(D, 1.0)
        if f["kind"] == "dense":
            for n, (o, k) in {"gate": (f["ff"], D), "up": (f["ff"], D), "down": (D, f["ff"])}.items():
                w[p + "mlp." + n] = lin(o, k)
            continue
        w[p + "mlp.router"] = lin(f["router"]["experts"], D, 3.0)
        units = [("e%d." % e, f["expert"]["ff"]) for e in range(f["router"]["experts"])]
        if f.get("shared"):
            units.append(("shared.", f["shared"]["ff"]))
            w[p + "mlp.shared.sg"] = lin(1, D, 2.0)
        for name, ff in units:
            w[p + "mlp." + name + "up"] = lin(ff, D, 1.5)
            w[p + "mlp." + name + "down"] = lin(D, ff)
    return w


def write_folder(path, cfg, w):
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in w.items()}, os.path.join(path, "model.safetensors"))
    return str(path)


def as_float(w):
    return {k: v.to(torch.float32) for k, v in w.items()}


def tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def row_errors(got, want):
    """Per row: root mean square of the difference (means taken off), over the spread of the wanted logits."""
    got, want = got.float().cpu(), want.float().cpu()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / want.std().clamp_min(1e-6)


def close(got, want, dtype, what="", spare=0.03):
    """float32: every row within 1e-4 of the spread.  bfloat16: every row within 0.15 of it (whole models with sharpened
    heads and experts stay below 0.13 on every path; a mixer alone, which is where the matrix-core kernels are held to
    the plain attention, stays below 0.01), but for a few (`spare` of them, at least one) where the rounding of the
    router's input may have chosen another expert than the float32 computation does; those stay within 1.5 of the spread."""
    assert got.shape == want.shape, "%s: shapes %s and %s" % (what, tuple(got.shape), tuple(want.shape))
    e = row_errors(got.reshape(-1, got.shape[-1]), want.reshape(-1, want.shape[-1]))
    assert torch.isfinite(e).all(), "%s: logits are not finite" % what
    if dtype == "float32":
        assert e.max().item() <= 1e-4, "%s: row error %.3g" % (what, e.max().item())
        return
    over = (e > 0.15).sum().item()
    assert over <= max(1, int(spare * e.numel())) and e.max().item() < 1.5, "%s: %d of %d rows over, worst %.3g" % (what, over, e.numel(), e.max().item())


def close_typical(got, want, dtype, what=""):
    """For models drawn at random, some of them small and with several layers of experts, where bfloat16 rounding moves a router's
    choice now and then and the moved token is seen by later ones: float32 as `close`; bfloat16 by the typical row (the median within
    0.08 of the spread, no more than an eighth of the rows beyond 0.15, none beyond 1.5).  A fault of structure (a head read from the
    wrong group, a window one off, a sink left out) moves every row."""
    if dtype == "float32":
        return close(got, want, dtype, what)
    assert got.shape == want.shape, "%s: shapes %s and %s" % (what, tuple(got.shape), tuple(want.shape))
    e = row_errors(got.reshape(-1, got.shape[-1]), want.reshape(-1, want.shape[-1]))
    assert torch.isfinite(e).all(), "%s: logits are not finite" % what
    over = (e > 0.15).float().mean().item()
    assert e.median().item() <= 0.08 and over <= 0.125 and e.max().item() < 1.5, "%s: median %.3g, %.3g of the rows over, worst %.3g" % (
        what, e.median().item(), over, e.max().item())


def plain_logits(cfg, w, toks, low=torch.float32):
    return plain.forward(cfg, as_float(w), toks, low)


def sure_rows(cfg, w, toks, least=0.1):
    """Which rows' routers all choose by a margin that rounding to bfloat16 does not reach (in units of the logits' spread)."""
    margins = []
    plain.forward(cfg, as_float(w), toks, margins=margins)
    sure = torch.ones(len(toks), dtype=torch.bool)
    for m in margins:
        sure &= m > least
    return sure
