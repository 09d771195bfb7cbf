"""Pudorax: the typed configuration read from config.json.

A config.json of this design lists its layers one by one, each with the kind of its mixer ("attention": softmax
attention behind short convolutions, with a gate on its heads; "mamba2": a state-space recurrence), the mixer's
sizes and constants, and its feed-forward (routed experts, or none).  A `loop` runs a stretch of the layers several
times in a row, every pass with memory of its own and entered through a matrix that also reads the embedding;
`token_side` gives every layer a second, small input from the token itself; `embedding.scale` multiplies the
embedding and `logit_softcap` bounds the logits.  Every size and constant comes from the file or from a tensor's
shape; a block that the file does not have stands for a mechanism the model does not have.  The file gives no longest
position: a sequence may be as long as the cache it runs in.
"""

from __future__ import annotations

from dataclasses import dataclass

from .base import ConfigError, ConfigReader, LayerKinds


@dataclass(frozen=True)
class ConvAttentionSizes:
    heads: int
    kv_heads: int
    dim: int              # query/key dimensions of a head
    vdim: int             # value dimensions of a head
    conv: int             # taps of the short convolution on q, k and v (0: none)
    rot_dims: int         # how many of a head's first dimensions the rotation turns, in neighbouring pairs
    rot_base: float
    scale: float


@dataclass(frozen=True)
class StateSpaceSizes:
    heads: int
    vdim: int
    state: int            # N: rows of a head's state
    groups: int           # heads that share one B and C
    norm_groups: int      # parts of a row that the norm behind the recurrence norms apart
    conv: int


@dataclass(frozen=True)
class GatedExpertSizes:
    ff: int
    limit: float


@dataclass(frozen=True)
class RoutedExpertsSizes:
    experts: int
    top: int
    expert: GatedExpertSizes
    shared: GatedExpertSizes | None


@dataclass(frozen=True)
class PudoraxLayer:
    kind: str             # "attention" or "mamba2"
    mixer: object
    mlp: RoutedExpertsSizes | None


MIXER_KINDS = {"attention": "conv_gated_attention", "mamba2": "state_space_scan"}


@dataclass(frozen=True)
class PudoraxConfig:
    architecture: str
    vocab: int
    hidden: int
    layers: tuple
    loop_start: int
    loop_stop: int
    loop_times: int
    has_loop: bool
    rms_eps: float        # the one eps of every norm of the model
    embedding_scale: float
    logit_softcap: float  # 0: none
    token_side_dim: int   # 0: no per-layer token input

    max_position = None   # the file sets no limit: the cache's capacity is the limit
    tie_word_embeddings = False

    @property
    def n_layers(self) -> int:
        return len(self.layers)

    def layer_kinds(self) -> list:
        return [LayerKinds(mixer=MIXER_KINDS[layer.kind], feed_forward="routed_experts" if layer.mlp else "none",
                           norm="layernorm", block="pre_norm_token_side") for layer in self.layers]

    def run_order(self) -> list:
        """Layer indices in the order in which they run: the looped stretch `loop_times` times in a row."""
        order = list(range(self.loop_start))
        order += list(range(self.loop_start, self.loop_stop)) * self.loop_times
        return order + list(range(self.loop_stop, self.n_layers))

    def schedule(self) -> list:
        """(layer index, cache entry index): every run of a layer has an entry of its own."""
        return [(layer, run) for run, layer in enumerate(self.run_order())]

    def pass_starts(self) -> list:
        """The runs (indices into the schedule) that open a pass of the loop."""
        length = self.loop_stop - self.loop_start
        if not self.has_loop or length <= 0:
            return []
        return [self.loop_start + n * length for n in range(self.loop_times)]

    # ---- reading ----
    @classmethod
    def from_dict(cls, data: dict, origin: str = "config.json") -> "PudoraxConfig":
        r = ConfigReader(data, origin)
        architecture = r.string("architecture") if r.has("architecture") else str((data.get("architectures") or ["Pudorax"])[0])
        vocab = r.integer("vocab", minimum=1)
        hidden = r.integer("width", minimum=1)
        rms_eps = _block(r, "norm", origin).number("eps")
        if rms_eps <= 0.0:
            raise ConfigError(f"{origin}: norm.eps must be positive, got {rms_eps}")
        embedding_scale = _block(r, "embedding", origin).number("scale") if r.has("embedding") else 1.0
        softcap = r.number("logit_softcap") if r.has("logit_softcap") else 0.0
        if softcap < 0.0:
            raise ConfigError(f"{origin}: logit_softcap must be positive, got {softcap}")
        side = _block(r, "token_side", origin).integer("dim", minimum=1) if r.has("token_side") else 0
        listed = r.raw("layers")
        if not isinstance(listed, list) or not listed:
            raise ConfigError(f"{origin}: 'layers' must be a list with at least one layer")
        layers = tuple(cls._layer(item, f"{origin}: layers[{index}]") for index, item in enumerate(listed))
        start, stop, times = 0, 0, 1
        if r.has("loop"):
            loop = _block(r, "loop", origin)
            start = loop.integer("start", minimum=0, maximum=len(layers))
            stop = loop.integer("stop", minimum=start, maximum=len(layers))
            times = loop.integer("times", minimum=1, maximum=1 << 16)
        return cls(architecture=architecture, vocab=vocab, hidden=hidden, layers=layers, loop_start=start, loop_stop=stop,
                   loop_times=times, has_loop=r.has("loop"), rms_eps=rms_eps, embedding_scale=embedding_scale,
                   logit_softcap=softcap, token_side_dim=side)

    @staticmethod
    def _layer(item, origin: str) -> PudoraxLayer:
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
                if rot_dims % 2 or (rot_dims and dim % 2):
                    raise ConfigError(f"{origin}: mixer.rot.dims turns pairs of a head's {dim} dimensions, got {rot_dims}")
                base = rot.number("base")
                if base <= 0.0:
                    raise ConfigError(f"{origin}: mixer.rot.base must be positive, got {base}")
            mixer = ConvAttentionSizes(heads=heads, kv_heads=kv_heads, dim=dim, vdim=m.integer("vdim", minimum=1),
                                       conv=m.integer("conv", minimum=1, maximum=16) if m.has("conv") else 0,
                                       rot_dims=rot_dims, rot_base=base, scale=m.number("scale"))
        elif kind == "mamba2":
            heads, groups = m.integer("heads", minimum=1), m.integer("groups", minimum=1)
            if heads % groups:
                raise ConfigError(f"{origin}: {heads} heads do not fall into {groups} groups evenly")
            vdim = m.integer("vdim", minimum=1, maximum=256)
            norm_groups = m.integer("norm_groups", minimum=1) if m.has("norm_groups") else 1
            if (heads * vdim) % norm_groups:
                raise ConfigError(f"{origin}: {heads * vdim} inner channels do not fall into {norm_groups} norm_groups evenly")
            mixer = StateSpaceSizes(heads=heads, vdim=vdim, state=m.integer("state", minimum=1), groups=groups,
                                    norm_groups=norm_groups, conv=m.integer("conv", minimum=1, maximum=16))
        else:
            raise ConfigError(f"{origin}: layer type {kind!r} is not implemented; only {sorted(MIXER_KINDS)}")
        mlp = None
        if r.has("mlp"):
            block = _block(r, "mlp", origin)
            if block.string("kind") != "moe":
                raise ConfigError(f"{origin}: mlp.kind {block.string('kind')!r} is not implemented; only 'moe'")
            router = _block(block, "router", origin + ": mlp")
            experts = router.integer("experts", minimum=1)
            mlp = RoutedExpertsSizes(experts=experts, top=router.integer("top", minimum=1, maximum=min(experts, 32)),
                                     expert=_expert(block, "expert", origin), shared=_expert(block, "shared", origin) if block.has("shared") else None)
        return PudoraxLayer(kind=kind, mixer=mixer, mlp=mlp)


def _expert(reader: ConfigReader, key: str, origin: str) -> GatedExpertSizes:
    block = _block(reader, key, origin + ": mlp")
    limit = block.number("limit")
    if limit <= 0.0:
        raise ConfigError(f"{origin}: mlp.{key}.limit must be positive, got {limit}")
    return GatedExpertSizes(ff=block.integer("ff", minimum=1), limit=limit)


def _block(reader: ConfigReader, key: str, origin: str) -> ConfigReader:
    value = reader.raw(key)
    if not isinstance(value, dict):
        raise ConfigError(f"{origin}: {key!r} must be an object")
    return ConfigReader(value, f"{origin}: {key}")
