"""Small Vepelix configurations and random weights for the tests: the tensor list is derived here from the configuration
alone (not from the package's manifest), the weights are drawn so that every mechanism moves the logits (norm weights away
from zero, channel scales away from one, sinks of the scores' size, decays spread between short and long memory), and
model folders are written with the package's safetensors writer."""

from __future__ import annotations

import json
import os

import numpy as np
import torch


def rotation(dims, base, stretch=None):
    rot = {"base": base, "dims": dims}
    if stretch:
        rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), stretch))
    return rot


def latent(heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, base=10000.0, stretch=None, mlp=None):
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank, "scale": scale,
                      "rot": rotation(rot_dim, base, stretch)}, "mlp": mlp}


def parallel(heads, kv_heads, dim, vdim, scale, window, r_heads, r_dim, r_vdim, tau, rank, left_scale=1.0, right_scale=1.0,
             dims=None, base=10000.0, stretch=None, mlp=None):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window:
        left["mask"] = {"size": window}
    if dims:
        left["rot"] = rotation(dims, base, stretch)
    return {"type": "parallel", "mixer": {"left": left, "left_scale": left_scale, "right_scale": right_scale,
                                          "right": {"heads": r_heads, "dim": r_dim, "vdim": r_vdim, "tau": tau, "decay_rank": rank}},
            "mlp": mlp}


def dense(ff, limit):
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe(experts, top, ff, shared=None):
    mlp = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if shared:
        mlp["shared"] = {"ff": shared}
    return mlp


STRETCH = (4.0, 64, 16.0, 1.0)
# Both mixers, all three feed-forwards, a loop over the two middle layers; three experts a row and none shared in one layer;
# the window attention turns half a head, keys and values of different sizes (96 against 40: the padded head is the key's).
MIXED = {
    "architecture": "Vepelix", "vocab": 97, "width": 64, "norm": {"eps": 1e-5}, "loop": {"start": 1, "stop": 3, "times": 2},
    "layers": [latent(3, 16, 16, 24, 48, 40, 0.3, base=500.0, stretch=STRETCH, mlp=dense(80, 1.2)),
               parallel(4, 2, 96, 40, 0.12, 70, 2, 16, 24, 8.0, 8, 1.3, 0.8, dims=48, base=1000.0, stretch=(6.0, 128, 20.0, 1.0),
                        mlp=moe(6, 3, 32)),
               latent(2, 24, 8, 16, 56, 24, 0.25, mlp=moe(4, 1, 40, shared=48)),
               parallel(2, 2, 32, 32, 0.2, 0, 3, 8, 8, 2.0, 4, 0.7, 1.1, dims=32, base=100.0)],
}
# No loop; one head everywhere; a window of one page and one; no rotation beside the gated linear attention; a layer without
# a feed-forward; one expert of which one is used.
PLAIN = {
    "architecture": "Vepelix", "vocab": 131, "width": 96, "norm": {"eps": 1e-6},
    "layers": [parallel(1, 1, 64, 64, 0.15, 65, 1, 32, 40, 12.0, 16, 1.0, 1.0, mlp=dense(128, 7.0)),
               latent(1, 8, 4, 40, 28, 12, 0.6, base=100.0),
               latent(4, 32, 32, 32, 96, 64, 0.2, base=20000.0, stretch=(2.0, 32, 8.0, 2.0), mlp=moe(1, 1, 64, shared=32))],
}
# A loop that starts at the first layer and runs three times over both kinds; sizes that are no multiples of 8; as many
# experts a row as there are.
ODD = {
    "architecture": "Vepelix", "vocab": 53, "width": 36, "norm": {"eps": 1e-5}, "loop": {"start": 0, "stop": 2, "times": 3},
    "layers": [parallel(3, 1, 12, 20, 0.3, 9, 2, 5, 7, 3.0, 3, 0.5, 1.5, dims=6, base=50.0, mlp=moe(3, 3, 20, shared=12)),
               latent(5, 6, 2, 10, 14, 9, 0.4, base=10.0, mlp=dense(50, 0.8)),
               latent(2, 20, 12, 12, 20, 30, 0.3, base=1000.0, stretch=(16.0, 16, 4.0, 0.5))],
}
# A loop that runs once and one that is empty in another copy; a cached head of 256 (the matrix-core attention's largest).
WIDE = {
    "architecture": "Vepelix", "vocab": 211, "width": 128, "norm": {"eps": 1e-6}, "loop": {"start": 1, "stop": 2, "times": 1},
    "layers": [latent(4, 32, 64, 32, 192, 96, 0.15, base=250000.0, stretch=(16.0, 256, 24.0, 2.0), mlp=moe(8, 2, 64, shared=64)),
               parallel(8, 2, 64, 128, 0.125, 130, 4, 32, 64, 10.0, 16, 0.9, 1.3, dims=64, base=250000.0, stretch=(16.0, 256, 24.0, 2.0),
                        mlp=moe(8, 2, 64)),
               latent(8, 16, 16, 16, 48, 32, 0.2, mlp=dense(192, 1.5))],
}
CONFIGS = {"mixed": MIXED, "plain": PLAIN, "odd": ODD, "wide": WIDE}
GAIN = {}


def tensor_shapes(config):
    """{name: shape} of a configuration's checkpoint."""
    width = config["width"]
    shapes = {"embed": (config["vocab"], width), "final.norm": (width,), "head": (config["vocab"], width)}

    def feed_forward(p, ff):
        shapes.update({p + "gate": (ff, width), p + "up": (ff, width), p + "down": (width, ff)})

    for index, layer in enumerate(config["layers"]):
        p, m = f"l{index}.", layer["mixer"]
        for q in [1] + ([2] if layer["mlp"] else []):
            shapes[f"{p}norm{q}"] = (width,)
            shapes[f"{p}ls{q}"] = (width,)
        if layer["type"] == "latent_attention":
            shapes.update({p + "mix.dq": (m["q_rank"], width), p + "mix.dq.norm": (m["q_rank"],),
                           p + "mix.uq": (m["heads"] * (m["dim"] + m["rot_dim"]), m["q_rank"]),
                           p + "mix.dkv": (m["kv_rank"] + m["rot_dim"], width), p + "mix.dkv.norm": (m["kv_rank"],),
                           p + "mix.uk": (m["heads"] * m["dim"], m["kv_rank"]), p + "mix.uv": (m["heads"] * m["vdim"], m["kv_rank"]),
                           p + "mix.sink": (m["heads"],), p + "mix.g": (m["heads"], width), p + "mix.o": (width, m["heads"] * m["vdim"])})
        else:
            a, b = m["left"], m["right"]
            shapes.update({p + "mix.left.q": (a["heads"] * a["dim"], width), p + "mix.left.k": (a["kv_heads"] * a["dim"], width),
                           p + "mix.left.v": (a["kv_heads"] * a["vdim"], width), p + "mix.left.q.norm": (a["dim"],),
                           p + "mix.left.k.norm": (a["dim"],), p + "mix.left.o": (width, a["heads"] * a["vdim"])})
            keys, values = b["heads"] * b["dim"], b["heads"] * b["vdim"]
            shapes.update({p + "mix.right.q": (keys, width), p + "mix.right.k": (keys, width), p + "mix.right.v": (values, width),
                           p + "mix.right.g": (values, width), p + "mix.right.o": (width, values), p + "mix.right.norm": (b["vdim"],),
                           p + "mix.right.a1": (b["decay_rank"], width), p + "mix.right.a2": (keys, b["decay_rank"]),
                           p + "mix.right.a2.b": (keys,)})
        mlp = layer["mlp"]
        if mlp and mlp["kind"] == "dense":
            feed_forward(p + "mlp.", mlp["ff"])
        elif mlp:
            shapes[p + "mlp.router"] = (mlp["router"]["experts"], width)
            for e in range(mlp["router"]["experts"]):
                feed_forward(f"{p}mlp.e{e}.", mlp["expert"]["ff"])
            if mlp.get("shared"):
                feed_forward(p + "mlp.shared.", mlp["shared"]["ff"])
    return shapes


def random_weights(config, seed, gain=1.0):
    """float32 arrays that are exact in bfloat16.  Matrices N(0, gain / sqrt(inputs)); router matrices four times that, so
    that scores spread and few choices are close calls; zero-centred norm weights N(0, 0.3); plain norm weights and channel
    scales 1 + N(0, 0.3); sinks N(0, 1); the decays' biases spread over -1 .. 5 (memories of a few to hundreds of tokens)."""
    rng = np.random.default_rng(seed)
    out = {}
    for name, shape in tensor_shapes(config).items():
        last = name.split(".")[-1]
        if name == "embed":
            values = rng.standard_normal(shape)
        elif last == "router":
            values = rng.standard_normal(shape) * 4.0 / np.sqrt(shape[1])
        elif len(shape) == 2:
            values = rng.standard_normal(shape) * gain / np.sqrt(shape[1])
        elif last in ("norm1", "norm2") or name == "final.norm":
            values = 0.3 * rng.standard_normal(shape)
        elif last == "sink":
            values = rng.standard_normal(shape)
        elif last == "b":
            values = rng.uniform(-1.0, 5.0, shape)
        else:       # plain norm weights and channel scales
            values = 1.0 + 0.3 * rng.standard_normal(shape)
        out[name] = torch.from_numpy(values.astype(np.float32)).to(torch.bfloat16).to(torch.float32).numpy()
    return out


def write_model(folder, config, weights):
    from beholdd.weights import write_safetensors

    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as handle:
        json.dump(config, handle)
    write_safetensors(os.path.join(folder, "model.safetensors"),
                      {name: torch.from_numpy(np.ascontiguousarray(value)).to(torch.bfloat16) for name, value in weights.items()})
    return str(folder)


def drawn_config(seed):
    """A configuration whose every size, count, constant and layer order is drawn."""
    rng = np.random.default_rng(seed)
    pick = lambda *values: values[int(rng.integers(len(values)))]
    width = int(pick(24, 40, 52, 64, 72, 96, 130))
    n_layers = int(rng.integers(1, 5))

    def feed_forward():
        kind = pick("none", "dense", "moe", "moe")
        if kind == "none":
            return None
        if kind == "dense":
            return dense(int(pick(36, 64, 100)), float(pick(0.5, 1.5, 7.0)))
        experts = int(pick(1, 2, 5, 8))
        return moe(experts, int(rng.integers(1, min(experts, 3) + 1)), int(pick(8, 20, 32, 64)), shared=int(pick(0, 16, 40)))

    def stretch():
        return pick(None, (float(pick(2.0, 6.0, 32.0)), int(pick(16, 64, 256)), float(pick(4.0, 24.0)), float(pick(0.5, 1.0))))

    layers = []
    for _ in range(n_layers):
        if rng.random() < 0.5:
            rot_dim = int(pick(2, 4, 8, 16, 24))
            layers.append(latent(int(pick(1, 2, 3, 6)), int(pick(4, 8, 20, 32)), rot_dim, int(pick(4, 12, 16, 36)),
                                 int(pick(8, 24, 30, 40, 56, 112)), int(pick(8, 20, 32, 64)), float(pick(0.1, 0.2, 0.35)),
                                 base=float(pick(100.0, 10000.0, 300000.0)), stretch=stretch(), mlp=feed_forward()))
        else:
            kv_heads = int(pick(1, 2, 3))
            dim = int(pick(8, 12, 32, 64, 96))
            dims = int(pick(0, *[d for d in (2, 8, 12, 32, 64, 96) if d <= dim]))
            layers.append(parallel(kv_heads * int(pick(1, 2, 4)), kv_heads, dim, int(pick(8, 20, 32, 64, 100)), float(pick(0.1, 0.2, 0.3)),
                                   int(pick(0, 1, 3, 64, 65, 100)), int(pick(1, 2, 5)), int(pick(4, 12, 16, 33, 64)),
                                   int(pick(4, 10, 16, 40, 72)), float(pick(1.0, 4.0, 12.0)), int(pick(1, 4, 7, 16)),
                                   float(pick(0.5, 1.0, 1.2)), float(pick(0.5, 1.0, 1.1)), dims=dims,
                                   base=float(pick(100.0, 10000.0, 1e6)), stretch=stretch() if dims else None, mlp=feed_forward()))
    config = {"architecture": "Vepelix", "vocab": int(pick(37, 64, 150, 301)), "width": width,
              "norm": {"eps": float(pick(1e-6, 1e-5, 1e-3))}, "layers": layers}
    if rng.random() < 0.8:
        start = int(rng.integers(0, n_layers + 1))
        config["loop"] = {"start": start, "stop": int(rng.integers(start, n_layers + 1)), "times": int(pick(1, 2, 3))}
    return config
