"""Small Dupidra configurations and random weights for the tests: the tensor list is derived here from the configuration
alone (not from the package's manifest), the weights are drawn so that every mechanism moves the logits (norm weights and
biases away from one and zero, projection biases of order one, gates that neither forget everything nor nothing, a router
whose choices vary), and model folders are written with the package's safetensors writer."""

from __future__ import annotations

import json
import os

import numpy as np
import torch


def attention(heads, kv_heads, dim, vdim, scale, chunk=None, rot_dims=None, base=10000.0, mlp=None, weights_of=None):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if chunk:
        mixer["mask"] = {"size": chunk}
    if rot_dims:
        mixer["rot"] = {"base": base, "dims": rot_dims}
    return _layer("attention", mixer, mlp, weights_of)


def latent(heads, dim, vdim, kv_rank, scale, window=None, mlp=None, weights_of=None):
    mixer = {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale}
    if window:
        mixer["mask"] = {"size": window}
    return _layer("latent_attention", mixer, mlp, weights_of)


def mlstm(heads, dim, vdim, gate_cap, mlp=None, weights_of=None):
    return _layer("mlstm", {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": gate_cap}, mlp, weights_of)


def _layer(kind, mixer, mlp, weights_of):
    layer = {"type": kind, "mixer": mixer, "mlp": mlp}
    if weights_of is not None:
        layer["weights_of"] = weights_of
    return layer


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, limit):
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff, "limit": limit}}


def borrowed(layers, index, owner):
    """A copy of layer `owner`'s entry that runs its tensors."""
    return dict(json.loads(json.dumps(layers[owner])), weights_of=owner)


def _with_borrowers(config, pairs):
    for index, owner in pairs:
        config["layers"].insert(index, borrowed(config["layers"], index, owner))
    return config


# All three mixers and both feed-forwards; keys of 24 and values of 40 under one cached head of 64; a rotation over half a
# head; chunks and a window that are no divisors of a page; three query heads a key/value head; layers that run
# another layer's tensors (one of each kind of memory); a layer without a feed-forward.
MIXED = _with_borrowers({
    "architecture": "Dupidra", "vocab": 97, "width": 64, "postln_alpha": 1.7, "norm": {"eps": 1e-5},
    "layers": [mlstm(3, 8, 20, 9.0, mlp=dense(80)),
               attention(6, 2, 24, 40, 0.2, chunk=20, rot_dims=12, base=500.0, mlp=moe(5, 2, 24, 1.2)),
               latent(3, 16, 12, 32, 0.3, window=27, mlp=moe(4, 1, 40, 3.0)),
               attention(2, 2, 16, 48, 0.3, chunk=50, mlp=None)],
}, [(4, 1), (5, 0), (6, 2)])
# Values that usual sizes make equal or one: one head everywhere, alpha 1, no mask, no rotation, one expert, keys as wide as
# values, a latent as wide as a head, a gate cap of 1, one layer.
PLAIN = {
    "architecture": "Dupidra", "vocab": 131, "width": 96, "postln_alpha": 1.0, "norm": {"eps": 1e-6},
    "layers": [attention(1, 1, 32, 32, 0.18, mlp=moe(1, 1, 64, 2.0)),
               latent(1, 32, 32, 32, 0.2, mlp=dense(96)),
               mlstm(1, 16, 16, 1.0, mlp=None)],
}
# Edges: chunks of exactly a page, of one position (a query sees itself alone) and of more than two pages; windows of one,
# of a page and one more than a page; the rotation over a whole head; heads that the matrix-core kernels take (64, 128) and
# a cached latent of 96; eight query heads on one key/value head; a head of the recurrence wider than a wave.
EDGES = _with_borrowers({
    "architecture": "Dupidra", "vocab": 53, "width": 72, "postln_alpha": 3.0, "norm": {"eps": 1e-3},
    "layers": [attention(8, 1, 64, 64, 0.125, chunk=64, rot_dims=64, base=1e6, mlp=dense(40)),
               latent(4, 24, 32, 96, 0.2, window=64, mlp=moe(6, 3, 24, 1.5)),
               attention(2, 2, 12, 20, 0.4, chunk=1, rot_dims=4, mlp=None),
               latent(2, 8, 8, 20, 0.35, window=1, mlp=None),
               mlstm(2, 80, 70, 15.0, mlp=moe(2, 2, 36, 0.7)),
               attention(4, 2, 128, 32, 0.09, chunk=150, rot_dims=32, base=100.0, mlp=None),
               latent(5, 16, 16, 64, 0.25, window=65, mlp=None)],
}, [(7, 4)])
# Deeper, with every layer borrowing from the first of its kind, in another order.
DEEP = _with_borrowers({
    "architecture": "Dupidra", "vocab": 211, "width": 128, "postln_alpha": 2.0, "norm": {"eps": 1e-5},
    "layers": [latent(8, 16, 16, 48, 0.25, window=40, mlp=moe(8, 2, 64, 2.0)),
               mlstm(4, 32, 32, 12.0, mlp=moe(8, 4, 32, 1.0)),
               attention(8, 2, 32, 32, 0.18, chunk=33, rot_dims=8, base=1000.0, mlp=dense(200))],
}, [(3, 1), (4, 0), (5, 2), (6, 1)])
# Sizes that are multiples of nothing: a width of 100, heads of 6, 10, 5 and 7 dimensions, a latent of 50, feed-forwards of 10
# and 30, a vocabulary of 101, seven experts of which three are used; a borrower that stands ahead of its owner.
ODD = {
    "architecture": "Dupidra", "vocab": 101, "width": 100, "postln_alpha": 2.25, "norm": {"eps": 1e-4},
    "layers": [attention(3, 1, 6, 10, 0.4, chunk=37, rot_dims=2, base=300.0, mlp=moe(7, 3, 10, 0.9)),
               latent(5, 10, 6, 50, 0.3, window=45, mlp=dense(30)),
               mlstm(3, 5, 7, 4.0, mlp=moe(3, 2, 18, 2.0))],
}
ODD["layers"].insert(0, borrowed(ODD["layers"], 0, 2))      # runs the memory's tensors, which are then layer 3's
ODD["layers"][0]["weights_of"] = 3
# The same layers with a residual that weighs little beside the sublayers (with matrices of twice the usual size): the
# logits come from the embedding table too, so a model whose residual dominates predicts its last token over and over,
# and greedy continuations would say nothing.
GENERATING = dict(json.loads(json.dumps(MIXED)), postln_alpha=0.4)
GENERATING_GAIN = 2.0
CONFIGS = {"mixed": MIXED, "plain": PLAIN, "edges": EDGES, "deep": DEEP, "odd": ODD}


def tensor_shapes(config):
    """{name: shape} of a configuration's checkpoint: only layers with tensors of their own have any."""
    width, vocab = config["width"], config["vocab"]
    shapes = {"embed": (vocab, width), "final.norm": (width,), "final.norm.b": (width,)}
    for index, layer in enumerate(config["layers"]):
        if layer.get("weights_of", index) != index:
            continue
        p, m = f"l{index}.", layer["mixer"]
        for q in (1, 2) if layer["mlp"] else (1,):
            shapes[f"{p}norm{q}"] = (width,)
            shapes[f"{p}norm{q}.b"] = (width,)
        if layer["type"] == "attention":
            q_width, k_width, v_width = m["heads"] * m["dim"], m["kv_heads"] * m["dim"], m["kv_heads"] * m["vdim"]
            shapes.update({p + "mix.q": (q_width, width), p + "mix.q.b": (q_width,), p + "mix.k": (k_width, width),
                           p + "mix.k.b": (k_width,), p + "mix.v": (v_width, width), p + "mix.v.b": (v_width,),
                           p + "mix.q.norm": (m["dim"],), p + "mix.k.norm": (m["dim"],),
                           p + "mix.g": (m["heads"] * m["vdim"], width), p + "mix.o": (width, m["heads"] * m["vdim"])})
        elif layer["type"] == "latent_attention":
            shapes.update({p + "mix.q": (m["heads"] * m["dim"], width), p + "mix.dkv": (m["kv_rank"], width),
                           p + "mix.dkv.norm": (m["kv_rank"],), p + "mix.uk": (m["heads"] * m["dim"], m["kv_rank"]),
                           p + "mix.uv": (m["heads"] * m["vdim"], m["kv_rank"]), p + "mix.g": (m["heads"] * m["vdim"], width),
                           p + "mix.o": (width, m["heads"] * m["vdim"])})
        else:
            key, value = m["heads"] * m["dim"], m["heads"] * m["vdim"]
            shapes.update({p + "mix.q": (key, width), p + "mix.k": (key, width), p + "mix.v": (value, width), p + "mix.g": (value, width),
                           p + "mix.o": (width, value), p + "mix.norm": (value,), p + "mix.i": (m["heads"], width),
                           p + "mix.i.b": (m["heads"],), p + "mix.f": (m["heads"], width), p + "mix.f.b": (m["heads"],)})
        mlp = layer["mlp"]
        if mlp and mlp["kind"] == "dense":
            shapes.update({p + "mlp.up": (mlp["ff"], width), p + "mlp.down": (width, mlp["ff"])})
        elif mlp:
            shapes[p + "mlp.router"] = (mlp["router"]["experts"], width)
            for e in range(mlp["router"]["experts"]):
                ff = mlp["expert"]["ff"]
                shapes.update({f"{p}mlp.e{e}.gate": (ff, width), f"{p}mlp.e{e}.up": (ff, width), f"{p}mlp.e{e}.down": (width, ff)})
    return shapes


def random_weights(config, seed, gain=1.0):
    """float32 arrays that are exact in bfloat16.  Matrices N(0, gain / sqrt(inputs)), so that activations stay of order
    one; norm weights 1 + N(0, 0.3) with biases N(0, 0.3); projection biases N(0, 0.5); the input gates' matrices and
    biases of order one and the forget gates' biases in [0.5, 4], so that the memory neither empties nor stands still and
    the running maximum moves; router matrices four times the others, so that the choice varies from token to token."""
    rng = np.random.default_rng(seed)
    out = {}
    for name, shape in tensor_shapes(config).items():
        parts = name.split(".")
        last = parts[-1]
        if name == "embed":
            values = rng.standard_normal(shape)
        elif last == "router":
            values = rng.standard_normal(shape) * 4.0 / np.sqrt(shape[1])
        elif last in ("i", "f") and len(shape) == 2:
            values = rng.standard_normal(shape) * 3.0 / np.sqrt(shape[1])
        elif len(shape) == 2:
            values = rng.standard_normal(shape) * gain / np.sqrt(shape[1])
        elif name.endswith(".f.b"):
            values = rng.uniform(0.5, 4.0, shape)
        elif name.endswith(".i.b"):
            values = rng.standard_normal(shape)
        elif last == "b" and parts[-2] in ("q", "k", "v"):
            values = 0.5 * rng.standard_normal(shape)
        elif last == "b":
            values = 0.3 * rng.standard_normal(shape)
        else:       # norm weights
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
    """A configuration whose every size, count, constant and layer order is drawn: widths and head sizes that are no
    multiples of 8 among them, key and value sizes that differ, chunks and windows around and beyond a page, with and
    without rotation and masks, layers that borrow another layer's tensors (earlier or later in the list)."""
    rng = np.random.default_rng(seed)
    pick = lambda *values: values[int(rng.integers(len(values)))]
    width = int(pick(24, 40, 52, 64, 72, 96, 130))
    layers = []
    for _ in range(int(rng.integers(1, 5))):
        mlp = None
        roll = rng.random()
        if roll < 0.5:
            experts = int(pick(1, 2, 4, 7, 12))
            mlp = moe(experts, int(rng.integers(1, min(experts, 4) + 1)), int(pick(12, 32, 50)), float(pick(0.5, 1.5, 7.0)))
        elif roll < 0.8:
            mlp = dense(int(pick(20, 64, 100)))
        kind = pick("attention", "latent_attention", "mlstm")
        if kind == "attention":
            kv_heads = int(pick(1, 2, 3))
            dim = int(pick(4, 8, 20, 32, 48, 64))
            turned = int(pick(*[d for d in (0, 2, 4, 8, 20, 32, 64) if d <= dim]))
            layers.append(attention(kv_heads * int(pick(1, 2, 4)), kv_heads, dim, int(pick(4, 12, 16, 36, 64)), float(pick(0.1, 0.2, 0.35)),
                                    chunk=int(pick(0, 1, 7, 32, 64, 65, 100, 200)), rot_dims=turned,
                                    base=float(pick(100.0, 10000.0, 500000.0)), mlp=mlp))
        elif kind == "latent_attention":
            layers.append(latent(int(pick(1, 2, 3, 6)), int(pick(4, 12, 16, 32)), int(pick(4, 8, 20, 32)), int(pick(8, 20, 32, 64, 96)),
                                 float(pick(0.1, 0.2, 0.35)), window=int(pick(0, 1, 5, 63, 64, 65, 130)), mlp=mlp))
        else:
            layers.append(mlstm(int(pick(1, 2, 3, 5)), int(pick(4, 8, 12, 16, 40)), int(pick(4, 8, 15, 16, 33, 48)),
                                float(pick(1.0, 8.0, 15.0)), mlp=mlp))
    config = {"architecture": "Dupidra", "vocab": int(pick(37, 64, 150, 301)), "width": width,
              "postln_alpha": float(pick(1.0, 1.5, 2.5, 4.0)), "norm": {"eps": float(pick(1e-6, 1e-5, 1e-3))}, "layers": layers}
    for _ in range(int(rng.integers(0, 3))):
        owner = int(rng.integers(len(layers)))
        if layers[owner].get("weights_of", owner) != owner:
            continue
        at = int(rng.integers(0, len(layers) + 1))
        layers.insert(at, None)
        owner_now = owner + 1 if at <= owner else owner
        for other in layers:      # the owners that moved down by one
            if other is not None and "weights_of" in other and other["weights_of"] >= at:
                other["weights_of"] += 1
        layers[at] = borrowed(layers, at, owner_now)
    return config
