"""A plain, slow implementation of the Tadolix design: whole sequences, no cache, float64, one function a
mechanism, every recurrence token by token. It shares no code with the engine; the tests hold the engine to it.

Notation: T tokens, D the model's width; a weight `W [out, in]` is applied as `x @ W.T`; `w` maps tensor names to
float64 tensors (`widen`); `raw` is the configuration as config.json holds it.
"""
import math

import torch

F64 = torch.float64


def widen(w):
    return {k: v.to(F64) for k, v in w.items()}


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z / (1.0 + torch.exp(-z))


def unit_rms(x, eps):
    """x over its root mean square along the last axis, eps inside the root."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def offset_norm(x, weight, eps):
    """The norm whose weight is stored around zero."""
    return unit_rms(x, eps) * (1.0 + weight)


def sinusoid(T, width, base=10000.0):
    """[T, width]: sin(p base^(-2i / width)) at element 2i, the cosine at 2i + 1."""
    out = torch.zeros(T, width, dtype=F64)
    for p in range(T):
        for i in range(width // 2):
            angle = p * base ** (-2.0 * i / width)
            out[p, 2 * i], out[p, 2 * i + 1] = math.sin(angle), math.cos(angle)
    return out


def embed(raw, w, tokens):
    x = w["embed"][torch.tensor(tokens)] * (raw.get("embedding") or {}).get("scale", 1.0)
    return x + sinusoid(len(tokens), raw["width"])


def causal_conv(h, weight):
    """conv(h)_t = sum_j weight[:, j] h_(t - taps + 1 + j), nothing before the sequence's start."""
    T, taps = h.shape[0], weight.shape[1]
    out = torch.zeros_like(h)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] += weight[:, j] * h[s]
    return out


def bucket(n, rows, far):
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + math.floor(math.log(n / half) / math.log(far / half) * (rows - half)))


def chunk_attention(m, w, p, h, eps, only=None, weights=None):
    """The left half of a pair: softmax attention inside chunks, unit-norm queries and keys, capped scores, a bias
    by distance, an output gate. Returns what the output matrix gives, `[T, D]`. `only`: the queries to work out
    (the other rows stay zero before the gate); `weights`: a dict that gets the softmax weights by (head, query)."""
    T = h.shape[0]
    H, G, n, v = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m["vdim"]
    q = unit_rms((h @ w[p + "q"].T).view(T, H, n), eps)
    k = unit_rms((h @ w[p + "k"].T).view(T, G, n), eps)
    val = (h @ w[p + "v"].T).view(T, G, v)
    rel = w[p + "rel"]
    size = (m.get("mask") or {}).get("size")
    cap = m.get("softcap")
    out = torch.zeros(T, H, v, dtype=F64)
    for head in range(H):
        g = head // (H // G)
        for i in (range(T) if only is None else only):
            first = (i // size) * size if size else 0
            s = torch.stack([q[i, head] @ k[j, g] for j in range(first, i + 1)]) * m.get("scale", n ** -0.5)
            if cap:
                s = cap * torch.tanh(s / cap)
            s = s + torch.stack([rel[bucket(i - j, rel.shape[0], m["bias_max"]), head] for j in range(first, i + 1)])
            a = torch.softmax(s, 0)
            if weights is not None:
                weights[(head, i)] = (first, a)
            out[i, head] = (a[:, None] * val[first:i + 1, g]).sum(0)
    gate = torch.sigmoid(h @ w[p + "g"].T)
    return (out.reshape(T, H * v) * gate) @ w[p + "o"].T


def min_gru(w, p, h):
    """The right half of a pair: S_t = (1 - z) S_(t-1) + z c, token by token from S = 0."""
    z = torch.sigmoid(h @ w[p + "z"].T + w[p + "z.b"])
    u = h @ w[p + "x"].T + w[p + "x.b"]
    c = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    s = torch.zeros(z.shape[1], dtype=F64)
    states = []
    for t in range(h.shape[0]):
        s = (1.0 - z[t]) * s + z[t] * c[t]
        states.append(s)
    return (torch.stack(states) * silu(h @ w[p + "g"].T)) @ w[p + "o"].T


def rglru(m, w, p, h):
    """Griffin's recurrent block: S_t = a S_(t-1) + sqrt(1 - a^2) i u, token by token from S = 0."""
    T = h.shape[0]
    y = gelu_tanh(h @ w[p + "y"].T + w[p + "y.b"])
    u = causal_conv(h @ w[p + "x"].T + w[p + "x.b"], w[p + "conv"]) + w[p + "conv.b"]
    blocks = m["blocks"]
    each = m["width"] // blocks
    r, i = torch.zeros_like(u), torch.zeros_like(u)
    for b in range(blocks):
        part = u[:, b * each:(b + 1) * each]
        r[:, b * each:(b + 1) * each] = torch.sigmoid(part @ w[p + "ra"][b].T + w[p + "ra.b"][b])
        i[:, b * each:(b + 1) * each] = torch.sigmoid(part @ w[p + "ri"][b].T + w[p + "ri.b"][b])
    a = torch.exp(-8.0 * r * torch.log1p(torch.exp(w[p + "lam"])))
    s = torch.zeros(m["width"], dtype=F64)
    states = []
    for t in range(T):
        s = a[t] * s + torch.sqrt(1.0 - a[t] ** 2) * i[t] * u[t]
        states.append(s)
    return (torch.stack(states) * y) @ w[p + "o"].T


def gated_mlp(w, p, h):
    return (gelu_tanh(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def mixer(layer, w, p, h, eps):
    m = layer["mixer"]
    if layer["type"] == "parallel":
        return (m.get("left_scale", 1.0) * chunk_attention(m["left"], w, p + "left.", h, eps)
                + m.get("right_scale", 1.0) * min_gru(w, p + "right.", h))
    return rglru(m, w, p, h)


def run_order(raw):
    n = len(raw["layers"])
    loop = raw.get("loop")
    if not loop:
        return list(range(n))
    return list(range(loop["start"])) + list(range(loop["start"], loop["stop"])) * loop["times"] + list(range(loop["stop"], n))


def hyper(copies, y, mix, out):
    """All copies at once from the old ones: x_b <- sum_a mix[a, b] x_a + out[b] y."""
    return [sum(mix[a, b] * copies[a] for a in range(len(copies))) + out[b] * y for b in range(len(copies))]


def forward(raw, w, tokens, after_each=None):
    """Logits `[T, vocab]` of a whole sequence. `after_each`: a list that gets the sum of the copies after every
    run of a layer."""
    eps = raw["norm"]["eps"]
    x = embed(raw, w, tokens)
    streams = raw.get("streams")
    copies = [x.clone() for _ in range(streams or 1)]
    taps = (raw.get("canon") or {}).get("taps", 0)
    for li in run_order(raw):
        layer, p = raw["layers"][li], f"l{li}."
        for which, sub in ((1, "mixer"), (2, "mlp")):
            if sub == "mlp" and layer.get("mlp") is None:
                continue
            hc = f"{p}hc{which}."
            u = sum(w[hc + "in"][a] * copies[a] for a in range(streams)) if streams else copies[0]
            h = offset_norm(u, w[f"{p}norm{which}"], eps)
            if sub == "mixer":
                if taps:
                    h = h + causal_conv(h, w[p + "canon1"])
                y = mixer(layer, w, p + "mix.", h, eps)
            else:
                y = gated_mlp(w, p + "mlp.", h)
            copies = hyper(copies, y, w[hc + "mix"], w[hc + "out"]) if streams else [copies[0] + y]
        if after_each is not None:
            after_each.append(sum(copies))
    return offset_norm(sum(copies), w["final.norm"], eps) @ w["head"].T
