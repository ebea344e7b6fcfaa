"""A plain, slow implementation of the Vepelix decoder in NumPy: whole sequences, no cache, no batches, one
function per mechanism, float64 sums.  It shares no code with the package and is the oracle of the tests.

The design in this file's notation (T tokens, width D):
  embedding            x = E[token];  x0 = x is kept
  layer                x <- x + ls1 * M(n1(x));  x <- x + ls2 * F(n2(x))  (F may be absent)
  norm                 n(x) = x / sqrt(mean(x^2) + eps) * (1 + w)
  loop                 layers start..stop-1 run `times` times in a row, every pass with memory of its own; ahead of
                       every pass but the first x <- x + x0
  latent attention     cq = rms(Wdq h) * w_q;  q = Wuq cq = per head [q_c (dim) | q_r (rot)];  Wdkv h = [c_raw | k_r];
                       c = rms(c_raw) * w_c;  s_ij = (q_c,i . (Wuk c_j) + R_i q_r,i . R_j k_r,j) * scale  for j <= i;
                       p_ij = exp(s_ij) / (exp(sink_h) + sum_j exp(s_ij));  o_i = sigmoid(Wg h)_h sum_j p_ij (Wuv c_j);
                       out = Wo concat_h o
  parallel mixer       a_left * window attention(h) + a_right * gated linear attention(h)
  window attention     q, k normed per head (rms * w), turned, s_ij = q_i . k_j * scale for 0 <= i - j < window, softmax
  gated linear attn.   S_t = diag(alpha_t) S_(t-1) + k_t v_t^T,  o_t = S_t^T (q_t / sqrt(dim)),
                       alpha = sigmoid(Wa2 Wa1 h + b)^(1/tau);  out = Wo (rms(o_t per head) * w * silu(Wg h))
  rotation R_p         neighbours (2i, 2i+1) of the first `dims` dimensions turned by p * f_i, f_i stretched for long
                       contexts (below), cosine and sine times 0.1 ln(factor) + 1
  dense feed-forward   g = min(Wg h, L), u = clamp(Wu h, -L, L);  Wd (g sigmoid(1.702 g) (u + 1))
  experts              s = sigmoid(Wr h); the `top` largest; out = sum_e E_e(s_e h) + E_shared(h),
                       E(h) = Wd (silu(Wg h) * (Wu h))
  output               logits = H n_final(x)
"""

from __future__ import annotations

import json
import math
import os

import numpy as np

F32 = np.float32
F64 = np.float64


def load(folder):
    """(config dictionary, {name: float32 array}) of a model folder."""
    import torch
    from safetensors import safe_open

    with open(os.path.join(folder, "config.json")) as handle:
        config = json.load(handle)
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as handle:
        weights = {name: handle.get_tensor(name).to(torch.float32).numpy() for name in handle.keys()}
    return config, weights


def linear(x, w):
    return np.asarray(x, F64) @ np.asarray(w, F64).T


def rms(x, eps):
    x = np.asarray(x, F64)
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)


def one_plus_norm(x, w, eps):
    return rms(x, eps) * (1.0 + np.asarray(w, F64))


def weight_norm(x, w, eps):
    return rms(x, eps) * np.asarray(w, F64)


def sigmoid(x):
    return 1.0 / (1.0 + np.exp(-np.asarray(x, F64)))


def silu(x):
    x = np.asarray(x, F64)
    return x * sigmoid(x)


def stretched_frequencies(rot):
    """(frequencies [dims / 2], factor on cosine and sine) of a rotation block {base, dims, scaling?}."""
    dims, base = int(rot["dims"]), float(rot["base"])
    plain = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)], F64)
    scaling = rot.get("scaling")
    if not scaling:
        return plain, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def turns_to_dimension(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    low = max(math.floor(turns_to_dimension(float(scaling["fast"]))), 0)
    high = min(math.ceil(turns_to_dimension(float(scaling["slow"]))), dims - 1)
    ramp = np.clip((np.arange(dims // 2, dtype=F64) - low) / max(high - low, 0.001), 0.0, 1.0)
    return plain / factor * ramp + plain * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def turn_neighbours(x, positions, rot):
    """x [T, ..., n]: dimensions 2i and 2i + 1 (i < dims / 2) turned by position * f_i; the rest passes."""
    frequencies, magnitude = stretched_frequencies(rot)
    dims = int(rot["dims"])
    angles = np.asarray(positions, F64)[:, None] * frequencies[None, :]
    shape = (len(positions),) + (1,) * (x.ndim - 2) + (dims // 2,)
    cos, sin = (np.cos(angles) * magnitude).reshape(shape), (np.sin(angles) * magnitude).reshape(shape)
    out = np.asarray(x, F64).copy()
    u, v = out[..., 0:dims:2].copy(), out[..., 1:dims:2].copy()
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


def softmax_rows(scores, visible, sink=None):
    """Softmax over the visible keys of every row; `sink` adds exp(sink) to every row's denominator."""
    masked = np.where(visible, scores, -np.inf)
    top = masked.max(axis=-1, keepdims=True)
    if sink is not None:
        top = np.maximum(top, sink)
    e = np.where(visible, np.exp(masked - top), 0.0)
    total = e.sum(axis=-1, keepdims=True)
    if sink is not None:
        total = total + np.exp(sink - top)
    return e / total


def latent_attention(h, w, prefix, sizes, eps, first_position=0):
    heads, dim, rot_dim, vdim, rank = sizes["heads"], sizes["dim"], sizes["rot_dim"], sizes["vdim"], sizes["kv_rank"]
    t_len = h.shape[0]
    positions = np.arange(first_position, first_position + t_len)
    query_latent = weight_norm(linear(h, w[prefix + "dq"]), w[prefix + "dq.norm"], eps)
    q = linear(query_latent, w[prefix + "uq"]).reshape(t_len, heads, dim + rot_dim)
    q_plain, q_turned = q[..., :dim], turn_neighbours(q[..., dim:], positions, sizes["rot"])
    down = linear(h, w[prefix + "dkv"])
    latent = weight_norm(down[:, :rank], w[prefix + "dkv.norm"], eps)
    k_turned = turn_neighbours(down[:, rank:], positions, sizes["rot"])
    k_plain = linear(latent, w[prefix + "uk"]).reshape(t_len, heads, dim)
    values = linear(latent, w[prefix + "uv"]).reshape(t_len, heads, vdim)
    gate = sigmoid(linear(h, w[prefix + "g"]))                      # [T, heads]
    sinks = np.asarray(w[prefix + "sink"], F64)
    visible = np.tril(np.ones((t_len, t_len), bool))
    out = np.zeros((t_len, heads, vdim), F64)
    for head in range(heads):
        scores = (q_plain[:, head] @ k_plain[:, head].T + q_turned[:, head] @ k_turned.T) * sizes["scale"]
        out[:, head] = softmax_rows(scores, visible, sink=sinks[head]) @ values[:, head] * gate[:, head:head + 1]
    return linear(out.reshape(t_len, heads * vdim), w[prefix + "o"])


def window_attention(h, w, prefix, sizes, eps, first_position=0):
    heads, groups, dim, vdim = sizes["heads"], sizes["kv_heads"], sizes["dim"], sizes["vdim"]
    t_len = h.shape[0]
    positions = np.arange(first_position, first_position + t_len)
    q = weight_norm(linear(h, w[prefix + "q"]).reshape(t_len, heads, dim), w[prefix + "q.norm"], eps)
    k = weight_norm(linear(h, w[prefix + "k"]).reshape(t_len, groups, dim), w[prefix + "k.norm"], eps)
    v = linear(h, w[prefix + "v"]).reshape(t_len, groups, vdim)
    if sizes.get("rot"):
        q, k = turn_neighbours(q, positions, sizes["rot"]), turn_neighbours(k, positions, sizes["rot"])
    distance = positions[:, None] - positions[None, :]
    visible = distance >= 0
    if sizes.get("mask"):
        visible &= distance < int(sizes["mask"]["size"])
    out = np.zeros((t_len, heads, vdim), F64)
    for head in range(heads):
        group = head // (heads // groups)
        out[:, head] = softmax_rows(q[:, head] @ k[:, group].T * sizes["scale"], visible) @ v[:, group]
    return linear(out.reshape(t_len, heads * vdim), w[prefix + "o"])


def gated_linear_attention(h, w, prefix, sizes, eps, state=None):
    """-> (output [T, D], state [heads, dim, vdim] after the last token)."""
    heads, dim, vdim, tau = sizes["heads"], sizes["dim"], sizes["vdim"], float(sizes["tau"])
    t_len = h.shape[0]
    q = linear(h, w[prefix + "q"]).reshape(t_len, heads, dim) * dim ** -0.5
    k = linear(h, w[prefix + "k"]).reshape(t_len, heads, dim)
    v = linear(h, w[prefix + "v"]).reshape(t_len, heads, vdim)
    z = linear(linear(h, w[prefix + "a1"]), w[prefix + "a2"]) + np.asarray(w[prefix + "a2.b"], F64)
    alpha = (sigmoid(z) ** (1.0 / tau)).reshape(t_len, heads, dim)
    s = np.zeros((heads, dim, vdim), F64) if state is None else np.asarray(state, F64).copy()
    o = np.zeros((t_len, heads, vdim), F64)
    for t in range(t_len):
        s = alpha[t][:, :, None] * s + k[t][:, :, None] * v[t][:, None, :]
        o[t] = np.einsum("hdv,hd->hv", s, q[t])
    normed = weight_norm(o, w[prefix + "norm"], eps).reshape(t_len, heads * vdim)
    return linear(normed * silu(linear(h, w[prefix + "g"])), w[prefix + "o"]), s


def parallel_mixer(h, w, prefix, sizes, eps):
    left = window_attention(h, w, prefix + "left.", sizes["left"], eps)
    right, _ = gated_linear_attention(h, w, prefix + "right.", sizes["right"], eps)
    return float(sizes["left_scale"]) * left + float(sizes["right_scale"]) * right


def clamped_feed_forward(h, w, prefix, limit):
    g = np.minimum(linear(h, w[prefix + "gate"]), limit)
    u = np.clip(linear(h, w[prefix + "up"]), -limit, limit)
    return linear(g * sigmoid(1.702 * g) * (u + 1.0), w[prefix + "down"])


def silu_expert(h, w, prefix):
    return linear(silu(linear(h, w[prefix + "gate"])) * linear(h, w[prefix + "up"]), w[prefix + "down"])


def route(h, w, prefix, top):
    """-> (chosen [T, top] by falling score, ties to the lower index; their scores)."""
    scores = sigmoid(linear(h, w[prefix + "router"]))
    chosen = np.argsort(-scores, axis=-1, kind="stable")[:, :top]
    return chosen, np.take_along_axis(scores, chosen, axis=-1)


def experts(h, w, prefix, sizes):
    chosen, scores = route(h, w, prefix, int(sizes["router"]["top"]))
    out = np.zeros((h.shape[0], w[prefix + "e0.down"].shape[0]), F64)
    for t in range(h.shape[0]):
        for e, s in zip(chosen[t], scores[t]):
            out[t] += silu_expert(s * np.asarray(h[t:t + 1], F64), w, f"{prefix}e{e}.")[0]
    if sizes.get("shared"):
        out += silu_expert(h, w, prefix + "shared.")
    return out


def run_order(config):
    n = len(config["layers"])
    loop = config.get("loop") or {"start": 0, "stop": 0, "times": 1}
    order = [(i, False) for i in range(loop["start"])]
    for turn in range(loop["times"]):
        order += [(i, turn > 0 and i == loop["start"]) for i in range(loop["start"], loop["stop"])]
    return order + [(i, False) for i in range(loop["stop"], n)]


def forward(config, w, tokens, residuals=None):
    """Logits [T, vocab] (float64) of a whole sequence; `residuals`: a list that gets x after every layer run."""
    eps = float(config["norm"]["eps"])
    x = np.asarray(w["embed"], F64)[np.asarray(tokens)]
    first = x.copy()
    for index, entering in run_order(config):
        layer, prefix = config["layers"][index], f"l{index}."
        if entering:
            x = x + first
        h = one_plus_norm(x, w[prefix + "norm1"], eps)
        if layer["type"] == "latent_attention":
            y = latent_attention(h, w, prefix + "mix.", layer["mixer"], eps)
        elif layer["type"] == "parallel":
            y = parallel_mixer(h, w, prefix + "mix.", layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        x = x + y * np.asarray(w[prefix + "ls1"], F64)
        mlp = layer.get("mlp")
        if mlp:
            h = one_plus_norm(x, w[prefix + "norm2"], eps)
            if mlp["kind"] == "dense":
                y = clamped_feed_forward(h, w, prefix + "mlp.", float(mlp["limit"]))
            else:
                y = experts(h, w, prefix + "mlp.", mlp)
            x = x + y * np.asarray(w[prefix + "ls2"], F64)
        if residuals is not None:
            residuals.append(x.copy())
    return linear(one_plus_norm(x, w["final.norm"], eps), w["head"])


def greedy(config, w, prompt, n_new):
    """The tokens that greedy decoding appends (ties to the lowest id), each from a whole forward of what stands so far."""
    tokens, made = list(prompt), []
    for _ in range(n_new):
        made.append(int(np.argmax(forward(config, w, tokens)[-1])))
        tokens.append(made[-1])
    return made
