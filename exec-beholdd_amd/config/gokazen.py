"""Gokazen: the typed configuration read from config.json.

A config.json of this design lists its layers one by one, each with the kind of its mixer ("lightning" or
"latent_attention"), the mixer's sizes and constants, and its feed-forward (or none); a `loop` runs a stretch
of the layers several times in a row, every pass with memory of its own; `streams` residual streams are joined
by learned hyper-connections.  Every size and constant comes from the file or from a tensor's shape; a key that
a formula needs and the file does not give is an error.  The file gives no longest position: a sequence may be as
long as the cache it runs in.
"""

from __future__ import annotations

from dataclasses import dataclass

from .base import ConfigError, ConfigReader, LayerKinds


@dataclass(frozen=True)
class LightningSizes:
    heads: int
    dim: int
    vdim: int
    decay: tuple          # one factor per head


@dataclass(frozen=True)
class LatentAttentionSizes:
    heads: int
    dim: int              # unrotated query/key dimensions of a head
    rot_dim: int          # rotated query/key dimensions of a head (the key's are shared by all heads)
    vdim: int
    kv_rank: int          # the latent that is cached
    rot_dims: int         # how many of the rot_dim dimensions the rotation turns
    rot_base: float
    scale: float


@dataclass(frozen=True)
class GokazenLayer:
    kind: str             # "lightning" or "latent_attention"
    mixer: object         # LightningSizes or LatentAttentionSizes
    ff: int               # the dense feed-forward's inner width, 0 for a layer without one


MIXER_KINDS = {"lightning": "lightning_attention", "latent_attention": "latent_attention"}


@dataclass(frozen=True)
class GokazenConfig:
    architecture: str
    vocab: int
    hidden: int
    layers: tuple
    loop_start: int
    loop_stop: int
    loop_times: int
    streams: int          # residual streams joined by hyper-connections; 0: one plain residual
    rms_eps: float
    logit_scale: float

    max_position = None   # the file sets no limit: the cache's capacity is the limit
    tie_word_embeddings = False

    @property
    def n_layers(self) -> int:
        return len(self.layers)

    def layer_kinds(self) -> list:
        return [LayerKinds(mixer=MIXER_KINDS[layer.kind], feed_forward="squared_relu" if layer.ff else "none",
                           norm="rmsnorm_zero_centred", block="stream_mixing") for layer in self.layers]

    def run_order(self) -> list:
        """Layer indices in the order in which they run: the looped stretch `loop_times` times in a row."""
        order = list(range(self.loop_start))
        order += list(range(self.loop_start, self.loop_stop)) * self.loop_times
        return order + list(range(self.loop_stop, self.n_layers))

    def schedule(self) -> list:
        """(layer index, cache entry index): every run of a layer has an entry of its own."""
        return [(layer, run) for run, layer in enumerate(self.run_order())]

    # ---- reading ----
    @classmethod
    def from_dict(cls, data: dict, origin: str = "config.json") -> "GokazenConfig":
        r = ConfigReader(data, origin)
        architecture = r.string("architecture") if r.has("architecture") else str((data.get("architectures") or ["Gokazen"])[0])
        vocab = r.integer("vocab", minimum=1)
        hidden = r.integer("width", minimum=1)
        norm = _block(r, "norm", origin)
        rms_eps = norm.number("eps")
        if rms_eps <= 0.0:
            raise ConfigError(f"{origin}: norm.eps must be positive, got {rms_eps}")
        logit_scale = r.number("logit_scale")
        streams = r.integer("streams", minimum=1, maximum=64) if r.has("streams") else 0
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
                   loop_times=times, streams=streams, rms_eps=rms_eps, logit_scale=logit_scale)

    @staticmethod
    def _layer(item, origin: str) -> GokazenLayer:
        r = ConfigReader(item, origin)
        kind = r.string("type")
        m = _block(r, "mixer", origin)
        if kind == "lightning":
            heads = m.integer("heads", minimum=1)
            decay = m.raw("decay")
            if (not isinstance(decay, list) or len(decay) != heads
                    or any(isinstance(d, bool) or not isinstance(d, (int, float)) for d in decay)):
                raise ConfigError(f"{origin}: mixer.decay must list one number for each of the {heads} heads")
            mixer = LightningSizes(heads=heads, dim=m.integer("dim", minimum=1), vdim=m.integer("vdim", minimum=1),
                                   decay=tuple(float(d) for d in decay))
        elif kind == "latent_attention":
            rot = _block(m, "rot", origin + ": mixer")
            rot_dim = m.integer("rot_dim", minimum=2)
            rot_dims = rot.integer("dims", minimum=2, maximum=rot_dim)
            if rot_dims % 2:
                raise ConfigError(f"{origin}: mixer.rot.dims must be even, got {rot_dims}")
            base = rot.number("base")
            if base <= 0.0:
                raise ConfigError(f"{origin}: mixer.rot.base must be positive, got {base}")
            mixer = LatentAttentionSizes(heads=m.integer("heads", minimum=1), dim=m.integer("dim", minimum=1),
                                         rot_dim=rot_dim, vdim=m.integer("vdim", minimum=1),
                                         kv_rank=m.integer("kv_rank", minimum=1), rot_dims=rot_dims, rot_base=base,
                                         scale=m.number("scale"))
        else:
            raise ConfigError(f"{origin}: layer type {kind!r} is not implemented; only {sorted(MIXER_KINDS)}")
        ff = 0
        if r.has("mlp"):
            mlp = _block(r, "mlp", origin)
            if mlp.string("kind") != "dense":
                raise ConfigError(f"{origin}: mlp.kind {mlp.string('kind')!r} is not implemented; only 'dense'")
            ff = mlp.integer("ff", minimum=1)
        return GokazenLayer(kind=kind, mixer=mixer, ff=ff)


def _block(reader: ConfigReader, key: str, origin: str) -> ConfigReader:
    value = reader.raw(key)
    if not isinstance(value, dict):
        raise ConfigError(f"{origin}: {key!r} must be an object")
    return ConfigReader(value, f"{origin}: {key}")
