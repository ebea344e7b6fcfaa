"""Dupidra, plainly: NumPy with float64 sums, whole sequences, no cache, no batches, one function per mechanism.

It shares no code with the package.  A model is a configuration dictionary (as in config.json) and a dictionary of
float32 arrays by tensor name; `forward` returns the logits of every position.  Matrices are stored [outputs, inputs].

    layer:       x <- LN1(alpha x + mixer(x));  x <- LN2(alpha x + ff(x))         (the second only with a feed-forward)
    layer norm:  (x - mean) / sqrt(mean of squared deviations + eps) * w + b
    rms:         x / sqrt(mean(x^2) + eps)
"""

from __future__ import annotations

import math

import numpy as np


def f64(a):
    return np.asarray(a, dtype=np.float64)


def linear(x, w, name, bias=False):
    y = f64(x) @ f64(w[name]).T
    return y + f64(w[name + ".b"]) if bias else y


def layer_norm(x, w, name, eps):
    x = f64(x)
    centred = x - x.mean(-1, keepdims=True)
    return centred / np.sqrt((centred ** 2).mean(-1, keepdims=True) + eps) * f64(w[name]) + f64(w[name + ".b"])


def rms(x, eps):
    x = f64(x)
    return x / np.sqrt((x ** 2).mean(-1, keepdims=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-f64(z)))


def gelu_tanh(z):
    z = f64(z)
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rotate_halves(x, positions, dims, base):
    """x [T, heads, d]: dimension i < dims/2 of every head is paired with i + dims/2 and the pair (u, v) at position p
    becomes (u cos a - v sin a, v cos a + u sin a), a = p * base^(-2i/dims); dimensions from `dims` on pass.  The angle
    is a float32 product, as positions and angles are 32-bit numbers in this design."""
    if not dims:
        return f64(x)
    x = f64(x)
    half = dims // 2
    freq = np.array([base ** (-2.0 * i / dims) for i in range(half)], dtype=np.float32)
    angle = f64(np.asarray(positions, dtype=np.float32)[:, None] * freq[None, :])[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return np.concatenate([u * np.cos(angle) - v * np.sin(angle), v * np.cos(angle) + u * np.sin(angle), x[..., dims:]], axis=-1)


def visible(t_len, kind=None, size=0):
    """[query, key] booleans: key j <= query i, and with kind "chunk" floor(i / size) == floor(j / size), with kind
    "window" i - j < size."""
    i, j = np.arange(t_len)[:, None], np.arange(t_len)[None, :]
    seen = j <= i
    if kind == "chunk":
        seen &= (i // size) == (j // size)
    elif kind == "window":
        seen &= (i - j) < size
    return seen


def softmax_attention(q, k, v, scale, seen):
    """q [T, H, d], k [T, G, d], v [T, G, e]; query head h reads key/value head h // (H / G)."""
    t_len, heads = q.shape[0], q.shape[1]
    per = heads // k.shape[1]
    out = np.zeros((t_len, heads, v.shape[2]))
    for h in range(heads):
        scores = (f64(q[:, h]) @ f64(k[:, h // per]).T) * scale
        scores = np.where(seen, scores, -np.inf)
        weights = np.exp(scores - scores.max(-1, keepdims=True))
        weights /= weights.sum(-1, keepdims=True)
        out[:, h] = weights @ f64(v[:, h // per])
    return out


def gated_attention(h, w, p, m, eps):
    """Biased projections, every head of q and k normed with one weight of its size, the rotation of the first rot.dims
    dimensions, keys within the query's chunk, a sigmoid gate from the same input on the joined heads."""
    t_len = h.shape[0]
    heads, groups, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = linear(h, w, p + "q", True).reshape(t_len, heads, dim)
    k = linear(h, w, p + "k", True).reshape(t_len, groups, dim)
    v = linear(h, w, p + "v", True).reshape(t_len, groups, vdim)
    q, k = rms(q, eps) * f64(w[p + "q.norm"]), rms(k, eps) * f64(w[p + "k.norm"])
    rot = m.get("rot")
    if rot:
        q, k = (rotate_halves(x, np.arange(t_len), rot["dims"], rot["base"]) for x in (q, k))
    seen = visible(t_len, "chunk", m["mask"]["size"]) if m.get("mask") else visible(t_len)
    out = softmax_attention(q, k, v, m["scale"], seen).reshape(t_len, heads * vdim)
    return linear(out * sigmoid(linear(h, w, p + "g")), w, p + "o")


def latent_attention(h, w, p, m, eps):
    """Keys and values of every head come from one normed latent per position; the last mask.size positions are seen."""
    t_len = h.shape[0]
    heads, dim, vdim = m["heads"], m["dim"], m["vdim"]
    q = linear(h, w, p + "q").reshape(t_len, heads, dim)
    latent = rms(linear(h, w, p + "dkv"), eps) * f64(w[p + "dkv.norm"])
    k = linear(latent, w, p + "uk").reshape(t_len, heads, dim)
    v = linear(latent, w, p + "uv").reshape(t_len, heads, vdim)
    seen = visible(t_len, "window", m["mask"]["size"]) if m.get("mask") else visible(t_len)
    out = softmax_attention(q, k, v, m["scale"], seen).reshape(t_len, heads * vdim)
    return linear(out * sigmoid(linear(h, w, p + "g")), w, p + "o")


def log_sigmoid(z):
    z = f64(z)
    return np.minimum(z, 0.0) - np.log1p(np.exp(-np.abs(z)))


def matrix_memory(h, w, p, m, eps, state=None):
    """The mLSTM recurrence, token by token.  Returns the mixer's output and the state (S, n, m) after the last token."""
    t_len = h.shape[0]
    heads, dim, vdim, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = linear(h, w, p + "q").reshape(t_len, heads, dim) / math.sqrt(dim)
    k = linear(h, w, p + "k").reshape(t_len, heads, dim)
    v = linear(h, w, p + "v").reshape(t_len, heads, vdim)
    gate_in = cap * np.tanh(linear(h, w, p + "i", True) / cap)
    gate_forget = log_sigmoid(cap * np.tanh(linear(h, w, p + "f", True) / cap))
    if state is None:
        state = (np.zeros((heads, dim, vdim)), np.zeros((heads, dim)), np.zeros(heads))
    memory, norm, top = (f64(part).copy() for part in state)
    out = np.zeros((t_len, heads, vdim))
    for t in range(t_len):
        new_top = np.maximum(gate_forget[t] + top, gate_in[t])
        keep, take = np.exp(gate_forget[t] + top - new_top), np.exp(gate_in[t] - new_top)
        memory = keep[:, None, None] * memory + take[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        norm = keep[:, None] * norm + take[:, None] * k[t]
        top = new_top
        under = np.maximum(np.abs((norm * q[t]).sum(-1)), np.exp(-top)) + 1e-6
        out[t] = np.einsum("hde,hd->he", memory, q[t]) / under[:, None]
    out = rms(out, eps).reshape(t_len, heads * vdim) * f64(w[p + "norm"])
    return linear(out * sigmoid(linear(h, w, p + "g")), w, p + "o"), (memory, norm, top)


def route(h, w, p, top):
    """The `top` experts with the largest softmax scores (ties to the lower index), their scores divided by their sum."""
    scores = f64(np.asarray(linear(h, w, p + "router"), dtype=np.float32))
    scores = np.exp(scores - scores.max(-1, keepdims=True))
    scores /= scores.sum(-1, keepdims=True)
    chosen = np.argsort(-scores, axis=-1, kind="stable")[:, :top]
    picked = np.take_along_axis(scores, chosen, axis=-1)
    return chosen, picked / (picked.sum(-1, keepdims=True) + 1e-20)


def clamped_expert(h, w, p, limit):
    gate = np.minimum(linear(h, w, p + "gate"), limit)
    up = np.clip(linear(h, w, p + "up"), -limit, limit)
    return linear(gate * sigmoid(1.702 * gate) * (up + 1.0), w, p + "down")


def feed_forward(h, w, p, mlp):
    if mlp["kind"] == "dense":
        return linear(gelu_tanh(linear(h, w, p + "up")), w, p + "down")
    chosen, shares = route(h, w, p, mlp["router"]["top"])
    out = np.zeros((h.shape[0], w[p + "e0.down"].shape[0]))
    for e in range(mlp["router"]["experts"]):
        share = ((chosen == e) * shares).sum(-1)
        rows = np.nonzero(share)[0]
        if len(rows):
            out[rows] += share[rows, None] * clamped_expert(f64(h)[rows], w, f"{p}e{e}.", mlp["expert"]["limit"])
    return out


MIXERS = {"attention": gated_attention, "latent_attention": latent_attention,
          "mlstm": lambda h, w, p, m, eps: matrix_memory(h, w, p, m, eps)[0]}


def owner(config, index):
    """The layer whose tensors layer `index` runs."""
    seen = set()
    while "weights_of" in config["layers"][index] and config["layers"][index]["weights_of"] != index:
        assert index not in seen
        seen.add(index)
        index = config["layers"][index]["weights_of"]
    return index


def residual_after_layers(config, w, tokens):
    """The residual after every layer [layers, T, width]."""
    eps, alpha = config["norm"]["eps"], config.get("postln_alpha", 1.0)
    x = f64(w["embed"])[np.asarray(tokens)]
    after = []
    for index, layer in enumerate(config["layers"]):
        p = f"l{owner(config, index)}."
        x = layer_norm(alpha * x + MIXERS[layer["type"]](x, w, p + "mix.", layer["mixer"], eps), w, p + "norm1", eps)
        if layer.get("mlp"):
            x = layer_norm(alpha * x + feed_forward(x, w, p + "mlp.", layer["mlp"]), w, p + "norm2", eps)
        after.append(x)
    return np.stack(after)


def forward(config, w, tokens):
    """Logits of every position [T, vocab], float32."""
    x = residual_after_layers(config, w, tokens)[-1]
    return (layer_norm(x, w, "final.norm", config["norm"]["eps"]) @ f64(w["embed"]).T).astype(np.float32)


def greedy(config, w, prompt, n_new):
    tokens = list(prompt)
    for _ in range(n_new):
        tokens.append(int(np.argmax(forward(config, w, tokens)[-1])))
    return tokens[len(prompt):]
