"""Layers over several residual streams (hyper-connections), with a per-channel scale on every sublayer's result.

The residual of a token is `streams` vectors X_1 .. X_S instead of one, all equal to the embedding at the start.
A sublayer F with its norm reads one weighted sum of them and its result goes back into all of them:

    u = sum_s take[s] X_s;   y = scale * F(norm(u));   X_t <- sum_s mix[s, t] X_s + give[t] * y   (all t at once)

`take` [S], `give` [S] and `mix` [S, S] (indexed [from, to]) are tensors of the layer, `scale` [width] multiplies
the sublayer's result channel by channel ("layer scale").  With one stream and no such tensors this is the plain
pre-norm residual X <- X + scale * F(norm(X)).  The model's output is the sum of the streams, which the final norm
forms (`ZeroCentredRMSNorm` reads [n, S, width] with every stream taken once).

All of it is float32: the streams, their sums and the update.  The streams lie [rows, S, width]; two kernels do the
work, `streams_rmsnorm` (sum, statistic and norm in one pass) and `streams_update`, and where another sublayer of
this make follows (in this block or the next) one kernel does the update and that sublayer's norm together.  A sublayer that can write its
result instead of adding it (`writes_fresh`) gets an empty matrix; any other registered mixer or feed-forward gets a
zeroed one to add into, so the block takes every part the pre-norm block takes.
"""

from __future__ import annotations

import torch

from ..weights.binder import TensorSpec
from .base import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, graph_rows_allowed


class StreamsResidual:
    """Opens the residual: the embedding's rows [n, width] become [n, streams, width], every stream a copy."""
    graph_safe = True
    graph_safe_rows = None

    def __init__(self, streams: int, width: int):
        self.streams, self.width = max(int(streams), 1), int(width)

    def tensor_specs(self):
        return []

    def load(self, get):
        pass

    def working_bytes(self, step) -> int:
        return step.matrix(step.rows, self.streams * self.width, 4)

    def open(self, ctx, hidden):
        if self.streams == 1:
            return hidden.view(hidden.shape[0], 1, self.width)
        out = ctx.new_f32(hidden.shape[0], self.streams, self.width)
        ctx.kernels.streams_open(hidden, out)
        return out


class StreamConnection:
    """The tensors that join one sublayer to the streams: `take`, `give`, `mix` (absent for a plain residual) and
    the per-channel `scale` of the sublayer's result (optional)."""

    def __init__(self, streams: int, width: int, prefix: str | None, scale_name: str | None):
        self.streams, self.width, self.prefix, self.scale_name = int(streams), int(width), prefix, scale_name
        self.take = self.give = self.mix = self.scale = None

    def tensor_specs(self):
        specs = []
        if self.prefix is not None:
            specs += [TensorSpec(self.prefix + "in", (self.streams,), "norm"), TensorSpec(self.prefix + "out", (self.streams,), "norm"),
                      TensorSpec(self.prefix + "mix", (self.streams, self.streams), "identity")]
        if self.scale_name is not None:
            specs.append(TensorSpec(self.scale_name, (self.width,), "norm"))
        return specs

    def load(self, get):
        if self.prefix is not None:
            self.take = get(self.prefix + "in").to(torch.float32).contiguous()
            self.give = get(self.prefix + "out").to(torch.float32).contiguous()
            self.mix = get(self.prefix + "mix").to(torch.float32).contiguous()
        if self.scale_name is not None:
            self.scale = get(self.scale_name).to(torch.float32).contiguous()


class StreamMixingBlock:
    """norm -> mixer -> back into the streams; then, if the layer has one, norm -> feed-forward -> back into the streams."""

    def __init__(self, streams: int, width: int, mixer_norm, mixer, mixer_connection, feed_forward_norm=None,
                 feed_forward=None, feed_forward_connection=None):
        self.streams, self.width = max(int(streams), 1), int(width)
        self.mixer_norm, self.mixer, self.mixer_connection = mixer_norm, mixer, mixer_connection
        self.feed_forward_norm, self.feed_forward, self.feed_forward_connection = feed_forward_norm, feed_forward, feed_forward_connection

    def parts(self):
        found = [self.mixer_norm, self.mixer, self.mixer_connection]
        if self.feed_forward is not None:
            found += [self.feed_forward_norm, self.feed_forward, self.feed_forward_connection]
        return found

    def _computing(self):
        return [part for part in self.parts() if not isinstance(part, StreamConnection)]

    @property
    def graph_safe(self):
        return all(getattr(part, "graph_safe", False) for part in self._computing())

    @property
    def graph_safe_rows(self):
        return graph_rows_allowed(self._computing())

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
        total = 2 * step.matrix(step.rows, self.width, 4)           # a sublayer's result, kept apart from the streams
        for part in self._computing():
            if hasattr(part, "working_bytes"):
                total += part.working_bytes(step)
        return total

    def unaccounted_parts(self) -> list:
        return [type(part).__name__ for part in self._computing() if not hasattr(part, "working_bytes")]

    def cache_need(self):
        return self.mixer.cache_need()

    def _read(self, ctx, hidden, norm, part, connection):
        reader = getattr(part, "input_reader", None) if getattr(norm, "serves_reader", False) else None
        if getattr(norm, "reads_streams", False):
            return norm.forward(ctx, hidden, reader=reader, take=connection.take)
        if self.streams == 1 and connection.take is None:       # any other norm reads the one plain residual
            plain = hidden.view(hidden.shape[0], self.width)
            return norm.forward(ctx, plain, reader=reader) if reader is not None else norm.forward(ctx, plain)
        raise TypeError(f"{type(norm).__name__} cannot read a weighted sum of residual streams")

    def _run(self, ctx, hidden, x, part, *cache):
        result = ctx.new_f32(hidden.shape[0], self.width)
        if getattr(part, "writes_fresh", False):
            part.forward(ctx, x, result, *cache, fresh=True)
        else:
            result.zero_()
            part.forward(ctx, x, result, *cache)
        return result

    @staticmethod
    def _write(ctx, hidden, result, connection, then=None):
        """The sublayer's result into the streams; `then` = (norm, part, connection) of the sublayer that runs next, whose
        input the same kernel writes where norm and kernels offer it.  Returns that input, or None."""
        if then is not None:
            norm, part, following = then
            fused = getattr(norm, "update_then_forward", None)
            if fused is not None:
                reader = getattr(part, "input_reader", None) if getattr(norm, "serves_reader", False) else None
                x = fused(ctx, hidden, result, connection.mix, connection.give, connection.scale, reader=reader, take=following.take)
                if x is not None:
                    return x
        ctx.kernels.streams_update(hidden, result, connection.mix, connection.give, connection.scale)
        return None

    def entry(self):
        """What the block before needs to prepare this block's first input: (norm, mixer, connection)."""
        return (self.mixer_norm, self.mixer, self.mixer_connection)

    def forward(self, ctx, hidden, cache, prepared=None, next_block=None):
        """`hidden` [rows, streams, width] float32, updated in place.  `prepared`: the mixer's input, if the block before
        wrote it with its last update; returns the next block's, if this block could write it."""
        following = next_block.entry() if isinstance(next_block, StreamMixingBlock) and next_block.streams == self.streams else None
        x = prepared if prepared is not None else self._read(ctx, hidden, self.mixer_norm, self.mixer, self.mixer_connection)
        result = self._run(ctx, hidden, x, self.mixer, cache)
        if self.feed_forward is None:
            return self._write(ctx, hidden, result, self.mixer_connection, following)
        inner = (self.feed_forward_norm, self.feed_forward, self.feed_forward_connection)
        x = self._write(ctx, hidden, result, self.mixer_connection, inner)
        if x is None:
            x = self._read(ctx, hidden, *inner)
        result = self._run(ctx, hidden, x, self.feed_forward)
        return self._write(ctx, hidden, result, self.feed_forward_connection, following)


@BLOCKS.register("stream_mixing")
def _build_stream_mixing(config, layer_index, prefix, kinds, shared):
    """Tensor names: <prefix>norm1/norm2, <prefix>ls1/ls2, <prefix>hc1./hc2. (in, out, mix); `config.streams` 0 means
    one plain residual without the hc tensors."""
    streams = int(getattr(config, "streams", 0))
    norm = NORMS.get(kinds.norm)

    def connection(q):
        return StreamConnection(max(streams, 1), config.hidden, f"{prefix}hc{q}." if streams else None, f"{prefix}ls{q}")

    feed_forward = FEED_FORWARDS.get(kinds.feed_forward)(config, layer_index, prefix, shared)
    return StreamMixingBlock(
        streams, config.hidden, norm(config, config.hidden, prefix + "norm1", shared),
        MIXERS.get(kinds.mixer)(config, layer_index, prefix, shared), connection(1),
        norm(config, config.hidden, prefix + "norm2", shared) if feed_forward is not None else None,
        feed_forward, connection(2) if feed_forward is not None else None)
