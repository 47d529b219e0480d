"""Shared by the Nikasun tests: small configurations made here, random weights of a sensible
size, model folders written with the safetensors package, and how logits are compared."""
import json
import math
import os

import torch
from safetensors.torch import save_file

import plain_nikasun as plain


def mixer(heads, dim, rot_dim, vdim, q_rank, kv_rank, window, base=10000.0, scale=None, kv_from=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
         "rot": {"base": base, "dims": rot_dim}, "mask": {"size": window},
         "scale": scale if scale is not None else 1.0 / math.sqrt(dim + rot_dim)}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, scale, ff, limit, shared=None):
    m = {"kind": "moe", "router": {"experts": experts, "top": top, "scale": scale}, "expert": {"ff": ff, "limit": limit}}
    if shared is not None:
        m["shared"] = {"ff": shared[0], "limit": shared[1]}
    return m


def config(vocab, width, layers, eps=1e-5, embedding_scale=None):
    return {"architecture": "Nikasun", "vocab": vocab, "width": width, "norm": {"eps": eps},
            "embedding": {"scale": embedding_scale if embedding_scale is not None else math.sqrt(width)},
            "layers": [{"type": "latent_attention", "mixer": m, "mlp": f} for m, f in layers]}


# Sizes chosen away from each other and from powers of two where the design allows: 5 heads, value size unlike the
# key size, latents of different sizes, a window that is no multiple of anything, layers in mixed order, a layer
# without a feed-forward, a layer that reads the cache of a layer two before it with a larger window than the owner's.
def config_mixed():
    a = mixer(5, 24, 8, 40, 48, 56, 23, base=5000.0)
    b = mixer(5, 24, 8, 40, 48, 56, 37, base=5000.0, kv_from=0)
    c = mixer(3, 32, 16, 16, 64, 32, 70, base=300.0)
    d = mixer(3, 32, 16, 16, 64, 32, 9, base=300.0, kv_from=2)
    return config(331, 96, [(a, moe(6, 2, 1.5, 40, 1.25, shared=(56, 2.5))), (c, None), (c | {}, dense(136)), (b, moe(4, 4, 0.7, 24, 3.0)),
                            (d, dense(72))], eps=3e-6, embedding_scale=7.5)


# The smallest of everything: one head, one expert of which one is chosen, a window of one position, rotated part of
# two values, no shared expert.
def config_ones():
    a = mixer(1, 8, 2, 8, 16, 8, 1, base=2.0)
    b = mixer(1, 8, 2, 8, 16, 8, 3, base=2.0, kv_from=0)
    return config(67, 32, [(a, moe(1, 1, 1.0, 16, 1.0)), (b, dense(16))], eps=1e-4, embedding_scale=1.0)


# Sizes that are no multiples of 8: nothing may rest on alignment.
def config_odd():
    a = mixer(3, 10, 6, 14, 20, 18, 130, base=777.0)
    return config(101, 52, [(a, dense(44)), (a, moe(5, 3, 2.0, 12, 0.75, shared=(20, 1.0)))], eps=1e-5, embedding_scale=3.0)


# One layer and nothing else mixes tokens: a token outside the window cannot reach the logits at all.
def config_single(window, width=64):
    return config(97, width, [(mixer(2, 16, 8, 16, 32, 24, window, base=50.0), dense(48))], embedding_scale=4.0)


def weights(cfg, seed, sharp=1.0, store=torch.bfloat16):
    """name -> tensor of the store dtype.  Products keep the size of what they read (std 1/sqrt(inputs)); the
    routers are made decisive; sharp > 1 scales queries up so that attention picks out single keys."""
    g = torch.Generator().manual_seed(seed)

    def lin(o, i, gain=1.0):
        return (torch.randn(o, i, generator=g) * gain / math.sqrt(i)).to(store)

    def vec(n, around):
        return (around + 0.1 * torch.randn(n, generator=g)).to(store)

    D = cfg["width"]
    w = {"embed": (torch.randn(cfg["vocab"], D, generator=g) / math.sqrt(D)).to(store), "final.norm": vec(D, 0.0)}
    for i, layer in enumerate(cfg["layers"]):
        p, m, f = "l%d." % i, layer["mixer"], layer["mlp"]
        H, dn, dr, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
        w[p + "norm1"] = vec(D, 0.0)
        w[p + "mix.dq"] = lin(m["q_rank"], D)
        w[p + "mix.dq.norm"] = vec(m["q_rank"], 1.0)
        w[p + "mix.uq"] = lin(H * (dn + dr), m["q_rank"], sharp)
        if m.get("kv_from") is None:
            w[p + "mix.dkv"] = lin(m["kv_rank"] + dr, D)
            w[p + "mix.dkv.norm"] = vec(m["kv_rank"], 1.0)
        w[p + "mix.uk"] = lin(H * dn, m["kv_rank"], sharp)
        w[p + "mix.uv"] = lin(H * dv, m["kv_rank"])
        w[p + "mix.g"] = lin(H, D, 2.0)
        w[p + "mix.o"] = lin(D, H * dv)
        if f is None:
            continue
        w[p + "norm2"] = vec(D, 0.0)
        if f["kind"] == "dense":
            for n, (o, k) in {"gate": (f["ff"], D), "up": (f["ff"], D), "down": (D, f["ff"])}.items():
                w[p + "mlp." + n] = lin(o, k)
            continue
        w[p + "mlp.router"] = lin(f["router"]["experts"], D, 3.0)
        units = [("e%d." % e, f["expert"]["ff"]) for e in range(f["router"]["experts"])]
        if f.get("shared"):
            units.append(("shared.", f["shared"]["ff"]))
        for name, ff in units:
            w[p + "mlp." + name + "gate"] = lin(ff, D, 1.5)
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


def close(got, want, dtype, what="", spare=0.02):
    """float32: every row within 1e-4 of the spread (sharpened models carry rounding further than plain ones).
    bfloat16: every row within 0.1 of it, but for a few (`spare` of them, at least one) where the rounding of the router's input may have chosen another expert than the float32
    computation does; those stay within 1.5 of the spread."""
    assert got.shape == want.shape, "%s: shapes %s and %s" % (what, tuple(got.shape), tuple(want.shape))
    e = row_errors(got.reshape(-1, got.shape[-1]), want.reshape(-1, want.shape[-1]))
    assert torch.isfinite(e).all(), "%s: logits are not finite" % what
    if dtype == "float32":
        assert e.max().item() <= 1e-4, "%s: row error %.3g" % (what, e.max().item())
        return
    over = (e > 0.1).sum().item()
    assert over <= max(1, int(spare * e.numel())) and e.max().item() < 1.5, "%s: %d of %d rows over, worst %.3g" % (what, over, e.numel(), e.max().item())


def plain_logits(cfg, w, toks, low=torch.float32):
    return plain.forward(as_float(w), cfg, toks, low)
