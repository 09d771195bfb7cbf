"""Softmax attention behind short convolutions, with queries and keys normed over the whole projection and a gate on
the heads' outputs.

    q, k, v = conv(Wq x), conv(Wk x), conv(Wv x)      a causal convolution over time on every channel, `taps` long
    q <- rms(q over all heads' channels together) * wq;  k likewise      (before the rotation)
    dimensions 2i, 2i+1 (i < turned / 2) of every head of q and k turned by position * base^(-2i/turned)
    causal softmax of q.k * scale; query head h reads key/value head h // (heads / kv_heads)
    out = Wo (heads * sigmoid(Wg x))

The four projections are one stacked product [q | k | v | g].  Per sequence the layer keeps paged keys and values and,
beside them, the last taps - 1 projected rows (before the convolution) as a fixed-size float32 state.  Keys have
`dim` dimensions a head and values `vdim`; both are cached as heads of one padded size (zeros beyond), which the paged
attention kernels take as it is.  Norm statistics, angles and the softmax are float32; the convolution is summed in
float32 and normed without being rounded in between.  Every size and constant is a constructor parameter.
"""

from __future__ import annotations

import torch

from ..weights.binder import TensorSpec
from .base import MIXERS, CacheNeed
from .linear import Linear
from .rope import RotaryFrequencies


def padded_head(dim: int, vdim: int) -> int:
    """The one head size under which keys of `dim` and values of `vdim` are cached: the larger of the two, rounded up
    to the matrix-core attention kernels' step of 32 where they take it (up to 256), and to an even size beyond."""
    size = max(int(dim), int(vdim))
    if -(-size // 32) * 32 <= 256:
        size = -(-size // 32) * 32
    return size + size % 2      # the kernel that writes the heads takes their dimensions in pairs


class ConvGatedAttention:
    graph_safe = True
    graph_safe_rows = None

    def __init__(self, hidden: int, n_heads: int, n_kv_heads: int, dim: int, vdim: int, taps: int, turned: int, base: float,
                 scale: float, norm_eps: float, prefix: str):
        """`taps` 0: no convolution (and no convolution tensors); `turned` 0: no rotation."""
        if n_heads % n_kv_heads:
            raise ValueError(f"{n_heads} query heads do not group evenly into {n_kv_heads} kv heads")
        self.hidden, self.n_heads, self.n_kv_heads, self.dim, self.vdim = int(hidden), int(n_heads), int(n_kv_heads), int(dim), int(vdim)
        self.taps, self.turned, self.scale, self.norm_eps, self.prefix = int(taps), int(turned), float(scale), float(norm_eps), prefix
        self.q_width, self.k_width, self.v_width = self.n_heads * self.dim, self.n_kv_heads * self.dim, self.n_kv_heads * self.vdim
        self.conv_width = self.q_width + self.k_width + self.v_width
        self.gate_width = self.n_heads * self.vdim
        self.pad = padded_head(dim, vdim)
        self.rotation = RotaryFrequencies(self.turned, base) if self.turned else None
        self.proj = Linear(hidden, [self.q_width, self.k_width, self.v_width, self.gate_width],
                           [prefix + "q", prefix + "k", prefix + "v", prefix + "g"])
        self.out = Linear(self.gate_width, hidden, prefix + "o")
        self.q_norm = self.k_norm = self.conv_weight = None

    @property
    def input_reader(self):
        return self.proj.reader()

    def tensor_specs(self):
        specs = self.proj.tensor_specs() + self.out.tensor_specs() + [
            TensorSpec(self.prefix + "q.norm", (self.q_width,), "norm"), TensorSpec(self.prefix + "k.norm", (self.k_width,), "norm")]
        for name, width in (("q", self.q_width), ("k", self.k_width), ("v", self.v_width)):
            if self.taps:
                specs.append(TensorSpec(f"{self.prefix}{name}.conv", (width, self.taps), "linear"))
        return specs

    def load(self, get):
        self.proj.load(get)
        self.out.load(get)
        self.q_norm = get(self.prefix + "q.norm").to(torch.float32).contiguous()
        self.k_norm = get(self.prefix + "k.norm").to(torch.float32).contiguous()
        if self.taps:
            self.conv_weight = torch.cat([get(f"{self.prefix}{name}.conv").to(torch.float32) for name in ("q", "k", "v")], dim=0).contiguous()
        else:
            self.conv_weight = torch.ones((self.conv_width, 1), dtype=torch.float32, device=self.q_norm.device)

    def prepare(self, kernels):
        self.proj.prepare(kernels)
        self.out.prepare(kernels)

    def cache_need(self):
        state = ((self.taps - 1) * self.conv_width,) if self.taps > 1 else ()
        return CacheNeed(kind="kv", kv_heads=self.n_kv_heads, head_dim=self.pad, state_shape=state, state_dtype=torch.float32)

    def working_bytes(self, step) -> int:
        total = self.proj.working_bytes(step, step.rows)
        total += step.matrix(step.rows, self.conv_width, 4)                      # the convolution's result
        total += 2 * step.matrix(step.rows, self.n_heads * self.pad)             # queries, attended
        total += step.matrix(step.rows, self.gate_width, reader=self.out.reader_for_plan(step.act_size))
        if step.sizes is not None:
            total += step.sizes.attention_working_bytes(step.rows, step.seqs, step.max_rows_per_seq, self.n_heads, self.n_kv_heads,
                                                        self.pad, step.max_position, step.act_size)
        return total + self.out.working_bytes(step, step.rows, accumulate=True)

    def forward(self, ctx, x, hidden, cache, then_norm=None):
        k = ctx.kernels
        n = ctx.n_rows
        proj = self.proj.forward(ctx, x)
        state = cache.state if self.taps > 1 else None
        q = ctx.new_activations(n, self.n_heads * self.pad)
        freq = self.rotation.frequencies(ctx.device) if self.rotation is not None else None
        in_one = getattr(k, "conv_norm_rope_write", None)      # convolution, norm, rotation and cache write in one launch
        if in_one is not None:
            in_one(proj, 0, self.conv_weight if self.taps else None, state, 0, ctx.seq_start, ctx.seq_slot, self.q_norm, self.k_norm,
                   self.norm_eps, freq, self.turned, ctx.positions, ctx.row_seq, q, cache.k_pages, cache.v_pages, cache.page_table,
                   self.n_heads, self.n_kv_heads, self.dim, self.vdim, self.pad, cache.writes)
        else:
            conv = ctx.new_f32(n, self.conv_width)
            k.short_conv(proj, 0, self.conv_weight, None, state, 0, ctx.row_seq, ctx.seq_start, ctx.seq_slot, conv)
            k.whole_norm_rope_write(conv, self.q_norm, self.k_norm, self.norm_eps, freq, self.turned, ctx.positions, ctx.row_seq, q,
                                    cache.k_pages, cache.v_pages, cache.page_table, self.n_heads, self.n_kv_heads, self.dim, self.vdim,
                                    self.pad, cache.writes)
        if state is not None and cache.writes:      # after every reader of the old state
            k.short_conv_state(proj, 0, self.conv_width, self.taps, state, 0, ctx.seq_start, ctx.seq_slot)
        attended = ctx.new_activations(n, self.n_heads * self.pad)
        k.attention(q, attended, cache.k_pages, cache.v_pages, cache.page_table, ctx.row_seq, ctx.positions, self.n_heads,
                    self.n_kv_heads, self.pad, self.scale, 0, layout=ctx)
        gated = ctx.new_activations(n, self.gate_width, reader=self.out.reader())
        k.gate_heads(attended, self.pad, proj, self.conv_width, gated, self.n_heads, self.vdim)
        self.out.forward(ctx, gated, out=hidden, accumulate=True)
        return None


@MIXERS.register("conv_gated_attention")
def _build_conv_gated_attention(config, layer_index, prefix, shared):
    sizes = config.layers[layer_index].mixer
    return ConvGatedAttention(config.hidden, sizes.heads, sizes.kv_heads, sizes.dim, sizes.vdim, sizes.conv, sizes.rot_dims,
                              sizes.rot_base, sizes.scale, config.rms_eps, prefix + "mix.")
