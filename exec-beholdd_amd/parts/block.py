"""The arrangement of parts in a layer.

Pre-norm residual block: h = h + Mixer(Norm(h)); h = h + FeedForward(Norm(h))
(crates/beholdd-model/src/qwen3moe/forward.rs:1022-1414).  The residual `hidden` is float32
and is updated in place; the mixer and the feed-forward add into it.
"""

from __future__ import annotations

from .base import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, graph_rows_allowed


class PreNormBlock:
    """`feed_forward` (with its norm) may be None: a layer of a mixer alone.  `after`: parts that run once the layer's
    sublayers have, each `forward(ctx, hidden)` on the residual (a second input from the token, say)."""

    def __init__(self, mixer_norm, mixer, feed_forward_norm, feed_forward, after=()):
        self.mixer_norm, self.mixer = mixer_norm, mixer
        self.feed_forward_norm, self.feed_forward = feed_forward_norm, feed_forward
        self.after = [part for part in after if part is not None]

    def parts(self):
        sublayer = [self.feed_forward_norm, self.feed_forward] if self.feed_forward is not None else []
        return [self.mixer_norm, self.mixer, *sublayer, *self.after]

    @property
    def graph_safe(self):
        return all(getattr(part, "graph_safe", False) for part in self.parts())

    @property
    def graph_safe_rows(self):
        return graph_rows_allowed(self.parts())

    def tensor_specs(self):
        return [spec for part in self.parts() for spec in part.tensor_specs()]

    def load(self, get):
        for part in self.parts():
            part.load(get)

    def prepare(self, kernels):
        for part in self.parts():
            if hasattr(part, "prepare"):
                part.prepare(kernels)

    def working_bytes(self, step) -> int:
        """Everything the four parts allocate, as if nothing were freed before the layer ends."""
        total = sum(part.working_bytes(step) for part in self.after if hasattr(part, "working_bytes"))
        for norm, consumer in ((self.mixer_norm, self.mixer), (self.feed_forward_norm, self.feed_forward)):
            if consumer is None:
                continue
            if hasattr(norm, "working_bytes"):
                total += norm.working_bytes(step)
            if hasattr(consumer, "working_bytes"):
                total += consumer.working_bytes(step)
        return total

    def unaccounted_parts(self) -> list:
        return [type(part).__name__ for part in self.parts() if not hasattr(part, "working_bytes")]

    def cache_need(self):
        return self.mixer.cache_need()

    @staticmethod
    def _joined(producer, norm, consumer):
        """The request to hand `producer` so that its last product prepares `norm` for `consumer`, or None."""
        if (getattr(producer, "prepares_next_norm", False) and getattr(consumer, "takes_prepared_input", False)
                and hasattr(norm, "request")):
            reader = PreNormBlock._reader(norm, consumer)
            return norm.request(reader) if reader is not None else norm.request()
        return None

    @staticmethod
    def _reader(norm, consumer):
        """The product of `consumer` that alone reads what `norm` writes, if both parts say so."""
        return getattr(consumer, "input_reader", None) if getattr(norm, "serves_reader", False) else None

    @staticmethod
    def _normed(ctx, norm, consumer, hidden):
        reader = PreNormBlock._reader(norm, consumer)
        return norm.forward(ctx, hidden, reader=reader) if reader is not None else norm.forward(ctx, hidden)

    def entry_request(self, producer):
        """What the part that runs before this block (`producer`) may prepare of this block's first norm."""
        return self._joined(producer, self.mixer_norm, self.mixer)

    def forward(self, ctx, hidden, cache, prepared=None, next_block=None):
        """One layer.  `prepared`: the mixer's input if the block before has prepared it already;
        `next_block`: the block that runs after this one, whose first norm this block's feed-forward
        may prepare.  Returns that prepared input, or None."""
        x = prepared if prepared is not None else self._normed(ctx, self.mixer_norm, self.mixer, hidden)
        if self.feed_forward is None or self.after:
            return self._plain(ctx, x, hidden, cache)
        request = self._joined(self.mixer, self.feed_forward_norm, self.feed_forward)
        if request is not None:
            x = self.mixer.forward(ctx, x, hidden, cache, then_norm=request)
        else:
            self.mixer.forward(ctx, x, hidden, cache)
            x = None
        if x is None:
            x = self._normed(ctx, self.feed_forward_norm, self.feed_forward, hidden)
        request = next_block.entry_request(self.feed_forward) if hasattr(next_block, "entry_request") else None
        if request is not None:
            return self.feed_forward.forward(ctx, x, hidden, then_norm=request)
        self.feed_forward.forward(ctx, x, hidden)
        return None

    def _plain(self, ctx, x, hidden, cache):
        """The layer without norms that ride on products across its end: what follows the feed-forward reads the finished
        residual."""
        self.mixer.forward(ctx, x, hidden, cache)
        if self.feed_forward is not None:
            self.feed_forward.forward(ctx, self._normed(ctx, self.feed_forward_norm, self.feed_forward, hidden), hidden)
        for part in self.after:
            part.forward(ctx, hidden)
        return None


@BLOCKS.register("pre_norm_token_side")
def _build_pre_norm_token_side(config, layer_index, prefix, kinds, shared):
    """Tensor names: <prefix>norm1 / norm2 (with the norm's own suffixes), <prefix>side.gate / .proj / .norm where the model
    has a token side table (`shared["token_side_table"]`)."""
    from .token_side import TokenSideInput

    norm = NORMS.get(kinds.norm)
    feed_forward = FEED_FORWARDS.get(kinds.feed_forward)(config, layer_index, prefix, shared)
    table = shared.get("token_side_table")
    side = TokenSideInput(config.hidden, table.dim, layer_index, table, config.rms_eps, prefix + "side.") if table is not None else None
    return PreNormBlock(
        norm(config, config.hidden, prefix + "norm1", shared), MIXERS.get(kinds.mixer)(config, layer_index, prefix, shared),
        norm(config, config.hidden, prefix + "norm2", shared) if feed_forward is not None else None, feed_forward, after=[side])


@BLOCKS.register("pre_norm")
def _build_pre_norm(config, layer_index, prefix, kinds, shared):
    norm = NORMS.get(kinds.norm)
    return PreNormBlock(
        norm(config, config.hidden, prefix + "input_layernorm.weight", shared),
        MIXERS.get(kinds.mixer)(config, layer_index, prefix, shared),
        norm(config, config.hidden, prefix + "post_attention_layernorm.weight", shared),
        FEED_FORWARDS.get(kinds.feed_forward)(config, layer_index, prefix, shared))
