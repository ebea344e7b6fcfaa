"""Dupidra: the typed configuration read from config.json.

A config.json of this design lists its layers one by one, each with the kind of its mixer ("attention": grouped
softmax attention with biases, per-head query and key norms, a rotation over part of a head, keys seen chunk by chunk
and a gate on the heads; "latent_attention": softmax attention over a cached latent within a sliding window, gated the
same way; "mlstm": a matrix memory with exponential gates kept as a recurrent state), the mixer's sizes and constants,
and its feed-forward (dense with a tanh-form GELU, routed experts, or none).  A layer may say `weights_of: j`: it then
has no tensors of its own and runs layer j's, with memory of its own.  Every layer is norm-after-sum:
x <- norm(alpha x + sublayer(x)) with `postln_alpha`.  Every size and constant comes from the file or from a tensor's
shape; a block that the file does not have stands for a mechanism the model does not have (no `mask`: every earlier
key is seen; no `rot`: no rotation).  The file gives no longest position: a sequence may be as long as the cache it
runs in.
"""

from __future__ import annotations

from dataclasses import dataclass

from .base import ConfigError, ConfigReader, LayerKinds


@dataclass(frozen=True)
class GatedAttentionSizes:
    heads: int
    kv_heads: int
    dim: int              # query/key dimensions of a head
    vdim: int             # value dimensions of a head
    scale: float
    rot_dims: int         # how many of a head's first dimensions the rotation turns, i with i + rot_dims/2 (0: none)
    rot_base: float
    chunk: int            # keys are seen within the query's chunk of that many positions, counted from 0 (0: all earlier keys)


@dataclass(frozen=True)
class WindowedLatentSizes:
    heads: int
    dim: int
    vdim: int
    kv_rank: int
    scale: float
    window: int           # the last `window` positions are seen, the query's own among them (0: all)
    # what the latent attention part reads beside these: no rotated part, a gate on the heads
    rot_dim: int = 0
    rot_dims: int = 0
    rot_base: float = 1.0
    gate: bool = True


@dataclass(frozen=True)
class MatrixMemorySizes:
    heads: int
    dim: int
    vdim: int
    gate_cap: float


@dataclass(frozen=True)
class DenseSizes:
    ff: int


@dataclass(frozen=True)
class ExpertSizes:
    ff: int
    limit: float


@dataclass(frozen=True)
class RoutedSizes:
    experts: int
    top: int
    expert: ExpertSizes
    shared: ExpertSizes | None = None     # this design has no shared expert and no bias on the router
    router_bias: bool = False


@dataclass(frozen=True)
class DupidraLayer:
    kind: str             # "attention", "latent_attention" or "mlstm"
    mixer: object
    mlp: object           # DenseSizes, RoutedSizes or None
    weights_of: int       # the layer whose tensors this one runs (its own index where it has its own)


MIXER_KINDS = {"attention": "gated_attention", "latent_attention": "latent_attention", "mlstm": "mlstm"}


@dataclass(frozen=True)
class DupidraConfig:
    architecture: str
    vocab: int
    hidden: int
    layers: tuple
    rms_eps: float        # the one eps of every norm of the model
    postln_alpha: float

    max_position = None   # the file sets no limit: the cache's capacity is the limit
    tie_word_embeddings = True

    @property
    def n_layers(self) -> int:
        return len(self.layers)

    def layer_kinds(self) -> list:
        """One entry per layer; None for a layer that runs another layer's parts."""
        kinds = []
        for index, layer in enumerate(self.layers):
            if layer.weights_of != index:
                kinds.append(None)
                continue
            feed_forward = "none" if layer.mlp is None else ("gelu_tanh" if isinstance(layer.mlp, DenseSizes) else "routed_experts")
            kinds.append(LayerKinds(mixer=MIXER_KINDS[layer.kind], feed_forward=feed_forward, norm="layernorm", block="post_norm"))
        return kinds

    def schedule(self) -> list:
        """(layer whose parts run, cache entry): every layer of the file is a run with memory of its own."""
        return [(layer.weights_of, run) for run, layer in enumerate(self.layers)]

    # ---- reading ----
    @classmethod
    def from_dict(cls, data: dict, origin: str = "config.json") -> "DupidraConfig":
        r = ConfigReader(data, origin)
        architecture = r.string("architecture") if r.has("architecture") else str((data.get("architectures") or ["Dupidra"])[0])
        vocab = r.integer("vocab", minimum=1)
        hidden = r.integer("width", minimum=1)
        rms_eps = _block(r, "norm", origin).number("eps")
        if rms_eps <= 0.0:
            raise ConfigError(f"{origin}: norm.eps must be positive, got {rms_eps}")
        alpha = r.number("postln_alpha") if r.has("postln_alpha") else 1.0
        listed = r.raw("layers")
        if not isinstance(listed, list) or not listed:
            raise ConfigError(f"{origin}: 'layers' must be a list with at least one layer")
        layers = [cls._layer(item, index, len(listed), f"{origin}: layers[{index}]") for index, item in enumerate(listed)]
        for index, layer in enumerate(layers):
            owner, seen = layer.weights_of, {index}
            while layers[owner].weights_of != owner:          # a layer that borrows from a borrower runs the first owner's
                if owner in seen:
                    raise ConfigError(f"{origin}: layers[{index}]: 'weights_of' leads in a circle")
                seen.add(owner)
                owner = layers[owner].weights_of
            if owner != index:
                theirs = layers[owner]
                # (the feed-forward is the owner's too: an entry that leaves it out runs the owner's, one that names another is wrong)
                if (theirs.kind, theirs.mixer) != (layer.kind, layer.mixer) or (layer.mlp is not None and layer.mlp != theirs.mlp):
                    raise ConfigError(f"{origin}: layers[{index}] runs the tensors of layers[{owner}] but has other sizes")
                layers[index] = DupidraLayer(theirs.kind, theirs.mixer, theirs.mlp, owner)
        return cls(architecture=architecture, vocab=vocab, hidden=hidden, layers=tuple(layers), rms_eps=rms_eps, postln_alpha=alpha)

    @staticmethod
    def _layer(item, index: int, count: int, origin: str) -> DupidraLayer:
        r = ConfigReader(item, origin)
        kind = r.string("type")
        m = _block(r, "mixer", origin)
        if kind == "attention":
            heads, kv_heads = m.integer("heads", minimum=1), m.integer("kv_heads", minimum=1)
            if heads % kv_heads:
                raise ConfigError(f"{origin}: {heads} query heads do not group evenly into {kv_heads} kv_heads")
            dim = m.integer("dim", minimum=1)
            rot_dims, base = 0, 1.0
            if m.has("rot"):
                rot = _block(m, "rot", origin + ": mixer")
                rot_dims = rot.integer("dims", minimum=0, maximum=dim)
                if rot_dims % 2:
                    raise ConfigError(f"{origin}: mixer.rot.dims turns pairs of dimensions, got {rot_dims}")
                base = rot.number("base")
                if base <= 0.0:
                    raise ConfigError(f"{origin}: mixer.rot.base must be positive, got {base}")
            mixer = GatedAttentionSizes(heads=heads, kv_heads=kv_heads, dim=dim, vdim=m.integer("vdim", minimum=1),
                                        scale=m.number("scale"), rot_dims=rot_dims, rot_base=base, chunk=_mask(m, origin))
        elif kind == "latent_attention":
            mixer = WindowedLatentSizes(heads=m.integer("heads", minimum=1), dim=m.integer("dim", minimum=1),
                                        vdim=m.integer("vdim", minimum=1), kv_rank=m.integer("kv_rank", minimum=1),
                                        scale=m.number("scale"), window=_mask(m, origin))
        elif kind == "mlstm":
            cap = m.number("gate_cap")
            if cap <= 0.0:
                raise ConfigError(f"{origin}: mixer.gate_cap must be positive, got {cap}")
            mixer = MatrixMemorySizes(heads=m.integer("heads", minimum=1), dim=m.integer("dim", minimum=1),
                                      vdim=m.integer("vdim", minimum=1), gate_cap=cap)
        else:
            raise ConfigError(f"{origin}: layer type {kind!r} is not implemented; only {sorted(MIXER_KINDS)}")
        mlp = None
        if r.has("mlp"):
            block = _block(r, "mlp", origin)
            form = block.string("kind")
            if form == "dense":
                mlp = DenseSizes(ff=block.integer("ff", minimum=1))
            elif form == "moe":
                router = _block(block, "router", origin + ": mlp")
                experts = router.integer("experts", minimum=1)
                expert = _block(block, "expert", origin + ": mlp")
                limit = expert.number("limit")
                if limit <= 0.0:
                    raise ConfigError(f"{origin}: mlp.expert.limit must be positive, got {limit}")
                mlp = RoutedSizes(experts=experts, top=router.integer("top", minimum=1, maximum=min(experts, 32)),
                                  expert=ExpertSizes(ff=expert.integer("ff", minimum=1), limit=limit))
            else:
                raise ConfigError(f"{origin}: mlp.kind {form!r} is not implemented; only 'dense' and 'moe'")
        weights_of = index
        if r.has("weights_of"):
            weights_of = r.integer("weights_of", minimum=0, maximum=count - 1)
        return DupidraLayer(kind=kind, mixer=mixer, mlp=mlp, weights_of=weights_of)


def _mask(mixer: ConfigReader, origin: str) -> int:
    if not mixer.has("mask"):
        return 0
    return _block(mixer, "mask", origin + ": mixer").integer("size", minimum=1)


def _block(reader: ConfigReader, key: str, origin: str) -> ConfigReader:
    value = reader.raw(key)
    if not isinstance(value, dict):
        raise ConfigError(f"{origin}: {key!r} must be an object")
    return ConfigReader(value, f"{origin}: {key}")
