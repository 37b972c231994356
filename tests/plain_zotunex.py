"""A plain, slow rendition of the Zotunex design on one whole sequence: no cache, no batch, one function per
mechanism, written from the design's equations with torch tensor arithmetic only. It shares no code with the
package and is what the package's parts, kernels and engine are tested against.

A model is `(cfg, w)`: `cfg` the dictionary of its config.json, `w` a dictionary of tensors by checkpoint name.
Everything is computed in the dtype of `w`'s tensors after `widen` (float64 by default).

Notation: T tokens, D the model's width, H query heads, G key/value heads, n the unrotated (or whole) query/key
size of a head, r its rotated size, v its value size, R the size of the key/value latent.
"""
import math

import torch


def widen(w, dtype=torch.float64):
    return {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in w.items()}


# ---------------------------------------------------------------- norms and activations

def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def scalar_norm(x, g, eps):
    """The norm of a layer: unit root mean square, then one number for all coordinates."""
    return unit_rms(x, eps) * g


def sigmoid(z):
    return 1.0 / (1.0 + torch.exp(-z))


def squared_relu(z):
    return torch.clamp(z, min=0.0) ** 2


# ---------------------------------------------------------------- rotary positions

def frequencies(rot):
    """f_i = base^(-2i / dims) for i < dims / 2, each divided by `scaling.factor` where the mixer names one."""
    dims = rot["dims"]
    factor = (rot.get("scaling") or {}).get("factor", 1.0)
    return torch.tensor([rot["base"] ** (-2.0 * i / dims) / factor for i in range(dims // 2)], dtype=torch.float64)


def turn(u, v, angle):
    """The pair (u, v) turned by `angle`."""
    c, s = torch.cos(angle), torch.sin(angle)
    return u * c - v * s, v * c + u * s


def rotate_neighbours(x, positions, rot):
    """x `[T, heads, size]`: of the first `dims` elements of every head, element 2i and element 2i + 1 are a pair,
    turned by position * f_i; what lies beyond `dims` passes."""
    dims = rot["dims"]
    angle = (positions.to(torch.float64)[:, None] * frequencies(rot)[None, :]).to(x.dtype)[:, None, :]
    out = x.clone()
    out[..., 0:dims:2], out[..., 1:dims:2] = turn(x[..., 0:dims:2], x[..., 1:dims:2], angle)
    return out


def rotate_halves(x, positions, rot):
    """x `[T, heads, size]`: of the first `dims` elements of every head, element i and element i + dims / 2 are a
    pair, turned by position * f_i; what lies beyond `dims` passes."""
    dims = rot["dims"]
    half = dims // 2
    angle = (positions.to(torch.float64)[:, None] * frequencies(rot)[None, :]).to(x.dtype)[:, None, :]
    out = x.clone()
    out[..., :half], out[..., half:dims] = turn(x[..., :half], x[..., half:dims], angle)
    return out


# ---------------------------------------------------------------- softmax over the keys a query may see

def causal_weights(scores, sink=None):
    """scores `[H, T, T]` (query i, key j): the softmax over j <= i, query by query. `sink` `[H]`: the denominator
    also holds exp(sink) of the head, once: a term that stands for no token and adds nothing to the sum of values."""
    heads, t, _ = scores.shape
    out = torch.zeros_like(scores)
    for i in range(t):
        s = scores[:, i, :i + 1]
        top = s.max(dim=-1, keepdim=True).values
        if sink is not None:
            top = torch.maximum(top, sink[:, None])
        e = torch.exp(s - top)
        denom = e.sum(-1, keepdim=True)
        if sink is not None:
            denom = denom + torch.exp(sink[:, None] - top)
        out[:, i, :i + 1] = e / denom
    return out


def weights_over(scores, seen, sink=None):
    """The same for queries that are a part of their sequence: scores `[H, I, J]`, `seen` `[I, J]` true where query
    i may see key j."""
    out = torch.zeros_like(scores)
    for i in range(scores.shape[1]):
        js = torch.nonzero(seen[i])[:, 0]
        s = scores[:, i, js]
        top = s.max(dim=-1, keepdim=True).values
        if sink is not None:
            top = torch.maximum(top, sink[:, None])
        e = torch.exp(s - top)
        denom = e.sum(-1, keepdim=True)
        if sink is not None:
            denom = denom + torch.exp(sink[:, None] - top)
        out[:, i, js] = e / denom
    return out


# ---------------------------------------------------------------- the two mixers

def attention(m, w, p, h, eps):
    """Softmax attention whose values are the keys as projected: `m` the mixer's entry of the configuration, `w`
    the tensors, `p` the mixer's prefix, `h` `[T, D]`."""
    t = h.shape[0]
    heads, groups, n = m["heads"], m.get("kv_heads", m["heads"]), m["dim"]
    positions = torch.arange(t)
    q = (h @ w[p + "q"].T).view(t, heads, n)
    k = (h @ w[p + "k"].T).view(t, groups, n)
    values = k                                           # before the norm and the turn; there is no other projection
    q = unit_rms(q, eps) * w[p + "q.norm"]
    k = unit_rms(k, eps) * w[p + "k.norm"]
    if m.get("rot"):
        q, k = rotate_neighbours(q, positions, m["rot"]), rotate_neighbours(k, positions, m["rot"])
    per = heads // groups
    out = torch.zeros(t, heads, n, dtype=h.dtype)
    gate = sigmoid(h @ w[p + "g"].T)                     # [T, H]: one number a head
    for head in range(heads):
        g = head // per
        scores = (q[:, head] @ k[:, g].T) * m["scale"] * w[p + "temp"][head]
        weights = causal_weights(scores[None])[0]
        out[:, head] = (weights @ values[:, g]) * gate[:, head:head + 1]
    return out.reshape(t, heads * n) @ w[p + "o"].T


def latent_attention(m, w, p, h, eps):
    """Attention over keys and values made from one small vector a token, with a sink in the softmax."""
    t = h.shape[0]
    heads, n, r, v, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    positions = torch.arange(t)
    q = (h @ w[p + "q"].T).view(t, heads, n + r)
    q_plain, q_rot = q[..., :n], rotate_halves(q[..., n:], positions, m["rot"])
    down = h @ w[p + "dkv"].T
    c = unit_rms(down[:, :rank], eps) * w[p + "dkv.norm"]
    k_rot = rotate_halves(down[:, None, rank:], positions, m["rot"])[:, 0]        # one for all heads
    k_plain = (c @ w[p + "uk"].T).view(t, heads, n)
    values = (c @ w[p + "uv"].T).view(t, heads, v)
    scores = (torch.einsum("ihd,jhd->hij", q_plain, k_plain) + torch.einsum("ihd,jd->hij", q_rot, k_rot)) * m["scale"]
    weights = causal_weights(scores, w[p + "sink"])
    out = torch.einsum("hij,jhd->ihd", weights, values)
    out = out * sigmoid(h @ w[p + "g"].T)[:, :, None]
    return out.reshape(t, heads * v) @ w[p + "o"].T


# ---------------------------------------------------------------- feed-forward

def dense(w, p, h):
    return squared_relu(h @ w[p + "up"].T) @ w[p + "down"].T


def clamped_expert(w, p, h, limit):
    """g = min(W_gate h, limit), u = clamp(W_up h, -limit, limit); W_down (g sigmoid(1.702 g) (u + 1))."""
    g = torch.clamp(h @ w[p + "gate"].T, max=limit)
    u = torch.clamp(h @ w[p + "up"].T, min=-limit, max=limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ w[p + "down"].T


def route(z, correction, top, scale):
    """z `[T, E]` router logits: scores sigmoid(z); the `top` experts with the largest score + correction (the lower
    number where two are equal); their weights are the scores without the correction, times `scale`."""
    s = sigmoid(z)
    chosen = torch.sort(s + correction, dim=-1, descending=True, stable=True).indices[:, :top]
    return chosen, torch.gather(s, 1, chosen) * scale


def mixture(mlp, w, p, h):
    router = mlp["router"]
    chosen, weights = route(h @ w[p + "router"].T, w[p + "correction"], router["top"], router["scale"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for c in range(router["top"]):
            e = int(chosen[t, c])
            out[t] += weights[t, c] * clamped_expert(w, f"{p}e{e}.", h[t:t + 1], mlp["expert"]["limit"])[0]
    if mlp.get("shared"):
        out = out + clamped_expert(w, p + "shared.", h, mlp["shared"]["limit"])
    return out


# ---------------------------------------------------------------- the model

def forward(cfg, w, tokens, return_layers=False):
    """Logits `[T, vocab]` of one sequence; with `return_layers` also the stream after every layer."""
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)] * (cfg.get("embedding") or {}).get("scale", 1.0)
    after = []
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = scalar_norm(x, w[p + "norm1"], eps)
        mix = attention if layer["type"] == "attention" else latent_attention
        x = x + mix(layer["mixer"], w, p + "mix.", h, eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            h = scalar_norm(x, w[p + "norm2"], eps)
            x = x + (dense(w, p + "mlp.", h) if mlp["kind"] == "dense" else mixture(mlp, w, p + "mlp.", h))
        after.append(x)
    logits = scalar_norm(x, w["final.norm"], eps) @ w["head"].T
    return (logits, after) if return_layers else logits
