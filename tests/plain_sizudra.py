"""A plain, slow implementation of the Sizudra decoder, one function per mechanism.

Whole sequences, float32 (or a low dtype for products and activations), no cache, no batching.
It shares no code with the library; the GPU tests compare the library with it.

Notation: T tokens, D the model's width, H query heads in G groups, d the size of a head's query
and key, dv of its value, r the number of rotated elements.

    x_0    = E[t_i] + B[(a t_{i-1} + b t_i) mod n]            (B[n] for a sequence's first token)
    x      = x + norm1(mix(x));   x = x + norm2(ff(x))       (ff may be absent; the parts read x itself)
    norm(y) = y / sqrt(mean(y^2) + eps) * w
    logits = W_head norm_final(x)

A weight dict maps the checkpoint's tensor names to float32 tensors (the bfloat16 values exactly).
`low` names the dtype the products and their activations are rounded to (float32: nothing is).
"""
import math

import torch

F32 = torch.float32


def rnd(x, low):
    return x if low == F32 else x.to(low).to(F32)


def product(x, w, low):
    """x W^T with operands of the low dtype and float32 sums, the result rounded to the low dtype."""
    return rnd(rnd(x, low) @ w.T, low)


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def embed(tokens, table, bigram, buckets, mul_prev, mul_cur):
    """Token rows plus the row of the hashed pair (previous token, token); the first token takes the table's last row."""
    x = table[tokens].clone()
    for i, t in enumerate(tokens.tolist()):
        row = buckets if i == 0 else (int(tokens[i - 1]) * mul_prev + t * mul_cur) % buckets
        x[i] += bigram[row]
    return x


def rotate(v, positions, base, dims):
    """Rotary positions on the first `dims` elements of the last axis of v [T, heads, d]; element i goes with
    element i + dims/2; the rest pass unchanged."""
    if dims == 0:
        return v
    half = dims // 2
    i = torch.arange(half, dtype=F32)
    freq = torch.pow(torch.tensor(float(base), dtype=F32), -2.0 * i / dims)
    ang = positions.to(F32)[:, None] * freq[None, :]
    cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    a, b = v[..., :half], v[..., half:dims]
    return torch.cat([a * cos - b * sin, b * cos + a * sin, v[..., dims:]], dim=-1)


def visible(T, window=None, keep_first=0):
    """[T, T] bool: query i sees key j if j <= i and (i - j < window or j < keep_first)."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    ok = j <= i
    if window is not None:
        ok = ok & ((i - j < window) | (j < keep_first))
    return ok


def attend(q, k, v, mask, scale, softcap=None, sink=None):
    """q [T, H, d], k [T, G, d], v [T, G, dv] -> [T, H, dv].  Scores in float32; an optional cap c tanh(s / c);
    an optional sink per head that adds exp(sink) to the softmax's denominator and nothing else."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[-1], dtype=F32)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        if softcap is not None:
            s = softcap * torch.tanh(s / softcap)
        s = s.masked_fill(~mask, float("-inf"))
        m = s.max(-1, keepdim=True).values
        if sink is not None:
            m = torch.maximum(m, sink[h].reshape(1, 1))
        e = torch.exp(s - m)
        den = e.sum(-1, keepdim=True)
        if sink is not None:
            den = den + torch.exp(sink[h] - m)
        out[:, h] = (e / den) @ v[:, g]
    return out


def mixer(x, w, p, m, eps, positions, low, carried):
    """One attention mixer.  m: the layer's mixer configuration; p: the tensors' prefix; carried: what layers hand on
    (the first value-mixing layer's values)."""
    T = x.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = product(x, w[p + "q"], low).reshape(T, H, d)
    k = product(x, w[p + "k"], low).reshape(T, G, d)
    v = product(x, w[p + "v"], low).reshape(T, G, dv)
    q = rms_norm(q, w[p + "q.norm"], eps)
    k = rms_norm(k, w[p + "k.norm"], eps)
    q = rotate(q, positions, m["rot"]["base"], m["rot"]["dims"])
    k = rotate(k, positions, m["rot"]["base"], m["rot"]["dims"])
    if m.get("v_mix"):
        if "v_first" in carried:
            lam = w[p + "vmix"].reshape(())
            v = (1.0 - lam) * v + lam * carried["v_first"]
        else:
            carried["v_first"] = v
    q, k, v = rnd(q, low), rnd(k, low), rnd(v, low)
    mask_cfg = m.get("mask")
    mask = visible(T, mask_cfg["size"], mask_cfg.get("keep_first", 0)) if mask_cfg else visible(T)
    o = attend(q, k, v, mask, m["scale"], m.get("softcap"), w.get(p + "sink"))
    return product(o.reshape(T, H * dv), w[p + "o"], low)


def dense_ff(x, w, p, low):
    g = product(x, w[p + "gate"], low)
    u = product(x, w[p + "up"], low)
    return product(gelu_tanh(g) * u, w[p + "down"], low)


def expert(x, w, p, low):
    """down(relu(up x)^2)"""
    u = product(x, w[p + "up"], low)
    return product(torch.relu(u) ** 2, w[p + "down"], low)


def route(x, w_router, top, low, margins=None):
    """The `top` experts with the largest logits (float32), and the softmax over those logits alone.  margins (a list, optional) gets,
    per token, how far the last chosen logit lies above the first one left out, in units of the logits' spread (inf where all are chosen)."""
    z = rnd(x, low) @ w_router.T
    val, idx = torch.topk(z, top, dim=-1)
    if margins is not None:
        if top < z.shape[-1]:
            ordered = z.sort(-1, descending=True).values
            margins.append((ordered[:, top - 1] - ordered[:, top]) / z.std(-1).clamp_min(1e-6))
        else:
            margins.append(torch.full((z.shape[0],), float("inf")))
    return idx, torch.softmax(val, dim=-1)


def moe_ff(x, w, p, f, low, margins=None):
    idx, wt = route(x, w[p + "router"], f["router"]["top"], low, margins)
    out = torch.zeros_like(x)
    for t in range(x.shape[0]):
        for c in range(idx.shape[1]):
            out[t] += wt[t, c] * expert(x[t:t + 1], w, p + "e%d." % int(idx[t, c]), low)[0]
    if f.get("shared"):
        gate = torch.sigmoid(rnd(x, low) @ w[p + "shared.sg"].T)          # [T, 1]
        out = out + gate * expert(x, w, p + "shared.", low)
    return out


def forward(cfg, w, tokens, low=F32, layers_out=None, margins=None):
    """Logits [T, vocab] of one sequence from its first token.  margins: see route (one entry per layer of experts)."""
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    eps = cfg["norm"]["eps"]
    big = cfg["embedding"]["bigram"]
    x = embed(tokens, w["embed"], w["bigram"], big["buckets"], big["mul_prev"], big["mul_cur"])
    positions = torch.arange(tokens.shape[0])
    carried = {}
    for i, layer in enumerate(cfg["layers"]):
        p = "l%d." % i
        x = x + rms_norm(mixer(x, w, p + "mix.", layer["mixer"], eps, positions, low, carried), w[p + "norm1"], eps)
        f = layer.get("mlp")
        if f:
            y = dense_ff(x, w, p + "mlp.", low) if f["kind"] == "dense" else moe_ff(x, w, p + "mlp.", f, low, margins)
            x = x + rms_norm(y, w[p + "norm2"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return rnd(rms_norm(x, w["final.norm"], eps), low) @ w["head"].T
