"""A plain, slow implementation of the Nikasun decoder, one function per mechanism.

Whole sequences, float32 (or any torch dtype for the products), no cache, no batching: every
function takes what it needs and returns what it computes.  It shares no code with the library;
the GPU tests compare the library with it.

Notation: T tokens, D the model's width, H heads, dn / dr the unrotated and rotated sizes of a
head's query and key, dv a head's value size, rq / rk the sizes of the query and key-value latents.

    x_0      = E[token] * s_e
    x        = x + mix(norm1(x));   x = x + ff(norm2(x))        (ff may be absent)
    norm(x)  = x / sqrt(mean(x^2) + eps) * (1 + w)
    logits   = E norm_final(x)

A weight dict maps the checkpoint's tensor names to float32 tensors (the bfloat16 values exactly).
`low` names the dtype the products and activations are rounded to (float32: nothing is rounded).
"""
import math

import torch

F32 = torch.float32


def rnd(x, low):
    """Round to the low dtype and come back to float32 (float32: the identity)."""
    return x if low == F32 else x.to(low).to(F32)


def product(x, w, low):
    """x W^T with operands of the low dtype and float32 sums, the result rounded to the low dtype."""
    return rnd(rnd(x, low) @ w.T, low)


def rms(x, eps):
    """x divided by its root mean square, eps inside the root."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def offset_norm(x, w, eps):
    """The layers' norm: the weight is stored around zero."""
    return rms(x, eps) * (1.0 + w)


def plain_norm(x, w, eps):
    """The latents' norm: the weight is used as it is."""
    return rms(x, eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rotate(v, positions, base, dims):
    """Rotary positions on the first `dims` elements of the last axis of v [T, ..., d]; element i is
    paired with element i + dims/2; the rest pass unchanged."""
    half = dims // 2
    i = torch.arange(half, dtype=F32)
    freq = torch.pow(torch.tensor(float(base), dtype=F32), -2.0 * i / dims)
    ang = positions.to(F32)[:, None] * freq[None, :]                    # [T, half]
    shape = [v.shape[0]] + [1] * (v.dim() - 2) + [half]
    cos, sin = torch.cos(ang).reshape(shape), torch.sin(ang).reshape(shape)
    a, b = v[..., :half], v[..., half:dims]
    return torch.cat([a * cos - b * sin, b * cos + a * sin, v[..., dims:]], dim=-1)


def window_mask(T, size):
    """visible[i, j]: 0 <= i - j < size."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    return (i - j >= 0) & (i - j < size)


def softmax_rows(scores, visible):
    s = torch.where(visible, scores, torch.full_like(scores, float("-inf")))
    s = s - s.max(-1, keepdim=True).values
    e = torch.exp(s)
    return e / e.sum(-1, keepdim=True)


def latent_kv(h, w, prefix, m, eps, positions, low):
    """What a layer with a key-value projection of its own leaves for itself and for the layers that
    read it: the normed latent [T, rk] and the rotated key part [T, dr] that all heads share."""
    rk, dr = m["kv_rank"], m["rot_dim"]
    both = product(h, w[prefix + "dkv"], low)
    c = rnd(plain_norm(both[:, :rk], w[prefix + "dkv.norm"], eps), low)
    k_rot = rnd(rotate(both[:, rk:rk + dr], positions, m["rot"]["base"], m["rot"]["dims"]), low)
    return c, k_rot


def latent_attention(h, w, prefix, m, eps, positions, kv, low):
    """The mixer.  kv: (latent, rotated key part) of this layer or of the layer it reads."""
    H, dn, dr, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    T = h.shape[0]
    c, k_rot = kv
    cq = rnd(plain_norm(product(h, w[prefix + "dq"], low), w[prefix + "dq.norm"], eps), low)
    q = product(cq, w[prefix + "uq"], low).reshape(T, H, dn + dr)
    q_plain = q[..., :dn]
    q_rot = rnd(rotate(q[..., dn:], positions, m["rot"]["base"], m["rot"]["dims"]), low)
    k_plain = product(c, w[prefix + "uk"], low).reshape(T, H, dn)
    v = product(c, w[prefix + "uv"], low).reshape(T, H, dv)
    scores = torch.einsum("ihd,jhd->hij", q_plain, k_plain) + torch.einsum("ihd,jd->hij", q_rot, k_rot)
    p = softmax_rows(scores * m["scale"], window_mask(T, m["mask"]["size"])[None])
    out = rnd(torch.einsum("hij,jhd->ihd", p, v), low)
    gate = torch.sigmoid(rnd(h, low) @ w[prefix + "g"].T)                      # [T, H]
    out = rnd(out * gate[:, :, None], low).reshape(T, H * dv)
    return product(out, w[prefix + "o"], low)


def dense_ff(h, w, prefix, low):
    g = product(h, w[prefix + "gate"], low)
    u = product(h, w[prefix + "up"], low)
    return product(rnd(torch.relu(g) * u, low), w[prefix + "down"], low)


def clamped_expert(h, w, prefix, limit, low):
    """One expert (or the shared one): the gate is cut from above, the up part from both sides."""
    g = torch.clamp(product(h, w[prefix + "gate"], low), max=limit)
    u = torch.clamp(product(h, w[prefix + "up"], low), -limit, limit)
    y = g * torch.sigmoid(1.702 * g) * (u + 1.0)
    return product(rnd(y, low), w[prefix + "down"], low)


def route(h, w_router, top, scale, low):
    """Chosen experts [T, top] and their weights: softmax over all experts, the largest `top`, times
    the scale, not renormalised."""
    z = rnd(h, low) @ w_router.T
    s = torch.softmax(z, dim=-1)
    val, idx = torch.topk(s, top, dim=-1)
    return idx, val * scale


def moe_ff(h, w, prefix, mlp, low):
    r = mlp["router"]
    idx, wt = route(h, w[prefix + "router"], r["top"], r["scale"], low)
    out = torch.zeros_like(h)
    for e in range(r["experts"]):
        hit = idx == e                                                       # [T, top]
        rows = hit.any(-1).nonzero().flatten()
        if rows.numel() == 0:
            continue
        y = clamped_expert(h[rows], w, prefix + "e%d." % e, mlp["expert"]["limit"], low)
        out[rows] += y * (wt[rows] * hit[rows]).sum(-1, keepdim=True)
    if mlp.get("shared"):
        out = out + clamped_expert(h, w, prefix + "shared.", mlp["shared"]["limit"], low)
    return rnd(out, low)


def forward(w, cfg, tokens, low=F32, keep_layers=False):
    """Logits [T, vocab] of one whole sequence (and, on request, the stream after every layer)."""
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(tokens.shape[0])
    eps = cfg["norm"]["eps"]
    x = w["embed"][tokens] * torch.tensor(cfg["embedding"]["scale"], dtype=F32)
    kept, streams = {}, []
    for i, layer in enumerate(cfg["layers"]):
        p = "l%d." % i
        m = layer["mixer"]
        assert layer["type"] == "latent_attention"
        h = rnd(offset_norm(x, w[p + "norm1"], eps), low)
        if m.get("kv_from") is None:
            kept[i] = latent_kv(h, w, p + "mix.", m, eps, positions, low)
            kv = kept[i]
        else:
            kv = kept[m["kv_from"]]
        x = x + latent_attention(h, w, p + "mix.", m, eps, positions, kv, low)
        mlp = layer.get("mlp")
        if mlp is not None:
            h = rnd(offset_norm(x, w[p + "norm2"], eps), low)
            x = x + (dense_ff(h, w, p + "mlp.", low) if mlp["kind"] == "dense" else moe_ff(h, w, p + "mlp.", mlp, low))
        streams.append(x.clone())
    logits = rnd(offset_norm(x, w["final.norm"], eps), low) @ w["embed"].T
    return (logits, torch.stack(streams)) if keep_layers else logits


def generate_greedy(w, cfg, prompt, n_new, low=F32):
    tokens = list(prompt)
    for _ in range(n_new):
        tokens.append(int(forward(w, cfg, tokens, low)[-1].argmax()))
    return tokens[len(prompt):]
