"""Vepelix: the typed configuration read from config.json.

A config.json of this design lists its layers one by one, each with the kind of its mixer ("latent_attention" or
"parallel"), the mixer's sizes and constants, and its feed-forward ("dense", "moe" or none); a `loop` runs a stretch of the
layers several times in a row, every pass with memory of its own, and every pass but the first is entered with the
embedding's output added to the residual.  Every size and constant comes from the file or from a tensor's shape; a key that
a formula needs and the file does not give is an error.  The file gives no longest position: a sequence may be as long as
the cache it runs in.  Sizes that only a tensor's shape gives (the rank of the decays' low-rank projection) are read from
the checkpoint's header by the loader and handed in as `shapes`.
"""

from __future__ import annotations

from dataclasses import dataclass

from .base import ConfigError, ConfigReader, LayerKinds


@dataclass(frozen=True)
class VepelixLatentSizes:
    heads: int
    dim: int              # unrotated query/key dimensions of a head
    rot_dim: int          # rotated query/key dimensions of a head (the key's are shared by all heads)
    vdim: int
    kv_rank: int          # the latent that is cached
    q_rank: int           # the latent that the queries are made from
    rot_dims: int
    rot_base: float
    rot_stretch: tuple | None      # (factor, original, fast, slow) or None
    scale: float
    gate: str = "head"    # one sigmoid gate a head
    sinks: bool = True
    neighbours: bool = True


@dataclass(frozen=True)
class VepelixWindowSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    rot_dims: int         # 0: no rotation
    rot_base: float
    rot_stretch: tuple | None
    scale: float
    window: int           # 0: every earlier key


@dataclass(frozen=True)
class VepelixLinearSizes:
    heads: int
    dim: int
    vdim: int
    tau: float
    decay_rank: int       # rows of the decays' first matrix; from that tensor's shape


@dataclass(frozen=True)
class VepelixParallelSizes:
    left: VepelixWindowSizes
    right: VepelixLinearSizes
    left_scale: float
    right_scale: float


@dataclass(frozen=True)
class VepelixDense:
    ff: int
    limit: float


@dataclass(frozen=True)
class VepelixExperts:
    experts: int
    top: int
    expert_ff: int
    shared_ff: int        # 0: no shared expert


@dataclass(frozen=True)
class VepelixLayer:
    kind: str             # "latent_attention" or "parallel"
    mixer: object
    mlp: object           # VepelixDense, VepelixExperts or None


MIXER_KINDS = {"latent_attention": "latent_attention", "parallel": "parallel_attention_gla"}


def _block(reader: ConfigReader, key: str, origin: str) -> ConfigReader:
    value = reader.raw(key)
    if not isinstance(value, dict):
        raise ConfigError(f"{origin}: {key!r} must be an object")
    return ConfigReader(value, f"{origin}: {key}")


def _rotation(mixer: ConfigReader, origin: str, most: int):
    """(dims, base, stretch) of a mixer's `rot` block; (0, 1.0, None) without one."""
    if not mixer.has("rot"):
        return 0, 1.0, None
    rot = _block(mixer, "rot", origin)
    dims = rot.integer("dims", minimum=2, maximum=most)
    if dims % 2:
        raise ConfigError(f"{origin}: rot.dims must be even, got {dims}")
    base = rot.number("base")
    if base <= 0.0:
        raise ConfigError(f"{origin}: rot.base must be positive, got {base}")
    stretch = None
    if rot.has("scaling"):
        scaling = _block(rot, "scaling", origin + ": rot")
        stretch = (scaling.number("factor"), scaling.number("original"), scaling.number("fast"), scaling.number("slow"))
        if min(stretch) <= 0.0 or base == 1.0:
            raise ConfigError(f"{origin}: rot.scaling needs a positive factor, length and turn counts, got {stretch}")
    return dims, base, stretch


@dataclass(frozen=True)
class VepelixConfig:
    architecture: str
    vocab: int
    hidden: int
    layers: tuple
    loop_start: int
    loop_stop: int
    loop_times: int
    rms_eps: float

    max_position = None   # the file sets no limit: the cache's capacity is the limit
    tie_word_embeddings = False
    streams = 0           # one plain residual

    @property
    def n_layers(self) -> int:
        return len(self.layers)

    @property
    def has_loop(self) -> bool:
        return self.loop_times > 1 and self.loop_stop > self.loop_start

    def layer_kinds(self) -> list:
        def feed_forward(layer):
            if layer.mlp is None:
                return "none"
            return "clamped_glu" if isinstance(layer.mlp, VepelixDense) else "routed_silu_experts"

        return [LayerKinds(mixer=MIXER_KINDS[layer.kind], feed_forward=feed_forward(layer), norm="rmsnorm_zero_centred",
                           block="stream_mixing") for layer in self.layers]

    def run_order(self) -> list:
        """Layer indices in the order in which they run: the looped stretch `loop_times` times in a row."""
        order = list(range(self.loop_start))
        order += list(range(self.loop_start, self.loop_stop)) * self.loop_times
        return order + list(range(self.loop_stop, self.n_layers))

    def schedule(self) -> list:
        """(layer index, cache entry index): every run of a layer has an entry of its own."""
        return [(layer, run) for run, layer in enumerate(self.run_order())]

    def pass_starts(self) -> list:
        """The runs (indices into the schedule) that open a pass of the loop after the first."""
        length = self.loop_stop - self.loop_start
        if length <= 0:
            return []
        return [self.loop_start + n * length for n in range(1, self.loop_times)]

    # ---- reading ----
    needs_shapes = True      # from_dict takes the checkpoint's tensor shapes (name -> shape) as `shapes`

    @classmethod
    def from_dict(cls, data: dict, origin: str = "config.json", shapes: dict | None = None) -> "VepelixConfig":
        r = ConfigReader(data, origin)
        architecture = r.string("architecture") if r.has("architecture") else str((data.get("architectures") or ["Vepelix"])[0])
        vocab = r.integer("vocab", minimum=1)
        hidden = r.integer("width", minimum=1)
        rms_eps = _block(r, "norm", origin).number("eps")
        if rms_eps <= 0.0:
            raise ConfigError(f"{origin}: norm.eps must be positive, got {rms_eps}")
        listed = r.raw("layers")
        if not isinstance(listed, list) or not listed:
            raise ConfigError(f"{origin}: 'layers' must be a list with at least one layer")
        layers = tuple(cls._layer(item, f"{origin}: layers[{index}]", index, shapes) for index, item in enumerate(listed))
        start, stop, times = 0, 0, 1
        if r.has("loop"):
            loop = _block(r, "loop", origin)
            start = loop.integer("start", minimum=0, maximum=len(layers))
            stop = loop.integer("stop", minimum=start, maximum=len(layers))
            times = loop.integer("times", minimum=1, maximum=1 << 16)
        return cls(architecture=architecture, vocab=vocab, hidden=hidden, layers=layers, loop_start=start, loop_stop=stop,
                   loop_times=times, rms_eps=rms_eps)

    @staticmethod
    def _layer(item, origin: str, index: int, shapes) -> VepelixLayer:
        r = ConfigReader(item, origin)
        kind = r.string("type")
        m = _block(r, "mixer", origin)
        if kind == "latent_attention":
            rot_dim = m.integer("rot_dim", minimum=2)
            dims, base, stretch = _rotation(m, origin + ": mixer", rot_dim)
            if dims != rot_dim:
                raise ConfigError(f"{origin}: the rotation turns the whole rotated part: rot.dims {dims} is not rot_dim {rot_dim}")
            mixer = VepelixLatentSizes(heads=m.integer("heads", minimum=1), dim=m.integer("dim", minimum=1), rot_dim=rot_dim,
                                       vdim=m.integer("vdim", minimum=1), kv_rank=m.integer("kv_rank", minimum=1),
                                       q_rank=m.integer("q_rank", minimum=1), rot_dims=dims, rot_base=base, rot_stretch=stretch,
                                       scale=m.number("scale"))
        elif kind == "parallel":
            left, right = _block(m, "left", origin + ": mixer"), _block(m, "right", origin + ": mixer")
            heads, kv_heads, dim = left.integer("heads", minimum=1), left.integer("kv_heads", minimum=1), left.integer("dim", minimum=1)
            if heads % kv_heads:
                raise ConfigError(f"{origin}: {heads} query heads do not group evenly into {kv_heads} key/value heads")
            dims, base, stretch = _rotation(left, origin + ": mixer: left", dim)
            window = 0
            if left.has("mask"):
                window = _block(left, "mask", origin + ": mixer: left").integer("size", minimum=1)
            attention = VepelixWindowSizes(heads=heads, kv_heads=kv_heads, dim=dim, vdim=left.integer("vdim", minimum=1), rot_dims=dims,
                                           rot_base=base, rot_stretch=stretch, scale=left.number("scale"), window=window)
            tau = right.number("tau")
            if tau <= 0.0:
                raise ConfigError(f"{origin}: mixer.right.tau must be positive, got {tau}")
            name = f"l{index}.mix.right.a1"
            if shapes is not None and name in shapes and len(shapes[name]) == 2:
                decay_rank = int(shapes[name][0])
            elif right.has("decay_rank"):      # a configuration without a checkpoint (random weights) says it itself
                decay_rank = right.integer("decay_rank", minimum=1)
            else:
                raise ConfigError(f"{origin}: the rank of the decays' projection is the first size of tensor {name!r} (or "
                                  "mixer.right.decay_rank where there is no checkpoint); neither was given")
            linear = VepelixLinearSizes(heads=right.integer("heads", minimum=1), dim=right.integer("dim", minimum=1),
                                        vdim=right.integer("vdim", minimum=1), tau=tau, decay_rank=decay_rank)
            mixer = VepelixParallelSizes(left=attention, right=linear, left_scale=m.number("left_scale"), right_scale=m.number("right_scale"))
        else:
            raise ConfigError(f"{origin}: layer type {kind!r} is not implemented; only {sorted(MIXER_KINDS)}")
        mlp = None
        if r.has("mlp"):
            f = _block(r, "mlp", origin)
            form = f.string("kind")
            if form == "dense":
                limit = f.number("limit")
                if limit <= 0.0:
                    raise ConfigError(f"{origin}: mlp.limit must be positive, got {limit}")
                mlp = VepelixDense(ff=f.integer("ff", minimum=1), limit=limit)
            elif form == "moe":
                router = _block(f, "router", origin + ": mlp")
                experts = router.integer("experts", minimum=1)
                top = router.integer("top", minimum=1)
                if top > experts:
                    raise ConfigError(f"{origin}: mlp.router.top {top} is more than the {experts} experts")
                shared_ff = _block(f, "shared", origin + ": mlp").integer("ff", minimum=1) if f.has("shared") else 0
                mlp = VepelixExperts(experts=experts, top=top, expert_ff=_block(f, "expert", origin + ": mlp").integer("ff", minimum=1),
                                     shared_ff=shared_ff)
            else:
                raise ConfigError(f"{origin}: mlp.kind {form!r} is not implemented; only 'dense' and 'moe'")
        return VepelixLayer(kind=kind, mixer=mixer, mlp=mlp)
