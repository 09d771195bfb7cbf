"""A selective state-space mixer with a scalar decay per head, kept as a recurrent state.

    [z | x | B | C | dt] = Win h          z, x: heads * vdim;  B, C: groups * N;  dt: heads
    (x, B, C) <- silu(conv(x, B, C) + bias)             one causal convolution over time on every channel, `taps` long
    dt <- softplus(dt + dt_bias)                        no clamp
    S_t = exp(-exp(A_log_h) dt) S_(t-1) + dt B_t x_t^T  S [N, vdim] per (sequence, head), zero at the start; head h reads
    y_t = S_t^T C_t + D_h x_t                           group h // (heads / groups)
    out = Wo (rms(y * silu(z), in `norm_groups` equal parts of a row) * w)

Per sequence the layer keeps one float32 region: the heads' states, then the last taps - 1 rows of (x, B, C) as they
were projected.  The step sizes, decays, the state, both products of the recurrence and the norm are float32; the
projection and the convolution's inputs have the engine's activation type.  One kernel walks a sequence's rows of the
step in order, so prompts, portions and decode steps are one code path.  Every size is a constructor parameter.
"""

from __future__ import annotations

import torch

from ..weights.binder import TensorSpec
from .base import MIXERS, CacheNeed
from .linear import Linear


class StateSpaceScan:
    graph_safe = True
    graph_safe_rows = None

    def __init__(self, hidden: int, n_heads: int, vdim: int, n_state: int, n_groups: int, norm_groups: int, taps: int,
                 norm_eps: float, prefix: str):
        if n_heads % n_groups:
            raise ValueError(f"{n_heads} heads do not fall into {n_groups} groups evenly")
        if (n_heads * vdim) % norm_groups:
            raise ValueError(f"{n_heads * vdim} channels do not fall into {norm_groups} parts evenly")
        self.hidden, self.n_heads, self.vdim, self.n_state, self.n_groups = int(hidden), int(n_heads), int(vdim), int(n_state), int(n_groups)
        self.norm_groups, self.taps, self.norm_eps, self.prefix = int(norm_groups), int(taps), float(norm_eps), prefix
        self.inner = self.n_heads * self.vdim
        self.conv_width = self.inner + 2 * self.n_groups * self.n_state
        self.dt_first = self.inner + self.conv_width
        self.proj = Linear(hidden, self.inner + self.conv_width + self.n_heads, prefix + "in")
        self.out = Linear(self.inner, hidden, prefix + "o")
        self.state_floats = self.n_heads * self.n_state * self.vdim
        self.conv_weight = self.conv_bias = self.dt_bias = self.a_log = self.d_skip = self.norm_weight = None

    @property
    def input_reader(self):
        return self.proj.reader()

    def tensor_specs(self):
        return self.proj.tensor_specs() + self.out.tensor_specs() + [
            TensorSpec(self.prefix + "conv", (self.conv_width, self.taps), "linear"),
            TensorSpec(self.prefix + "conv.b", (self.conv_width,), "linear"),
            TensorSpec(self.prefix + "dt_bias", (self.n_heads,), "linear"), TensorSpec(self.prefix + "A_log", (self.n_heads,), "linear"),
            TensorSpec(self.prefix + "D", (self.n_heads,), "norm"), TensorSpec(self.prefix + "norm", (self.inner,), "norm")]

    def load(self, get):
        self.proj.load(get)
        self.out.load(get)
        f32 = lambda name: get(self.prefix + name).to(torch.float32).contiguous()
        self.conv_weight, self.conv_bias = f32("conv"), f32("conv.b")
        self.dt_bias, self.a_log, self.d_skip, self.norm_weight = f32("dt_bias"), f32("A_log"), f32("D"), f32("norm")

    def prepare(self, kernels):
        self.proj.prepare(kernels)
        self.out.prepare(kernels)

    def cache_need(self):
        return CacheNeed(kind="state", state_shape=(self.state_floats + (self.taps - 1) * self.conv_width,), state_dtype=torch.float32)

    def working_bytes(self, step) -> int:
        chunks = 0
        if step.sizes is not None and hasattr(step.sizes, "ssm_chunk_bytes"):
            chunks = step.sizes.ssm_chunk_bytes(step.seqs, step.rows, step.max_rows_per_seq, self.n_heads, self.vdim, self.n_state)
        return (chunks + self.proj.working_bytes(step, step.rows) + step.matrix(step.rows, self.conv_width, 4) + step.matrix(step.rows, self.inner, 4)
                + step.matrix(step.rows, self.inner, reader=self.out.reader_for_plan(step.act_size))
                + self.out.working_bytes(step, step.rows, accumulate=True))

    def forward(self, ctx, x, hidden, cache, then_norm=None):
        k = ctx.kernels
        n = ctx.n_rows
        proj = self.proj.forward(ctx, x)
        xbc = ctx.new_f32(n, self.conv_width)
        k.short_conv(proj, self.inner, self.conv_weight, self.conv_bias, cache.state, self.state_floats, ctx.row_seq, ctx.seq_start,
                     ctx.seq_slot, xbc, silu=True)
        if self.taps > 1:
            k.short_conv_state(proj, self.inner, self.conv_width, self.taps, cache.state, self.state_floats, ctx.seq_start, ctx.seq_slot)
        y = ctx.new_f32(n, self.inner)
        k.ssm_scan(xbc, proj, self.dt_first, self.dt_bias, self.a_log, self.d_skip, cache.state, 0, ctx.seq_start, ctx.seq_slot, y,
                   self.n_heads, self.vdim, self.n_state, self.n_groups, max_rows_per_seq=ctx.max_rows_per_seq)
        normed = ctx.new_activations(n, self.inner, reader=self.out.reader())
        k.gated_group_rmsnorm(y, proj, 0, self.norm_weight, self.norm_eps, normed, self.norm_groups)
        self.out.forward(ctx, normed, out=hidden, accumulate=True)
        return None


@MIXERS.register("state_space_scan")
def _build_state_space_scan(config, layer_index, prefix, shared):
    sizes = config.layers[layer_index].mixer
    return StateSpaceScan(config.hidden, sizes.heads, sizes.vdim, sizes.state, sizes.groups, sizes.norm_groups, sizes.conv,
                          config.rms_eps, prefix + "mix.")
