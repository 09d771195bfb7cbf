"""Linear attention with a per-head decay ("lightning attention"), kept as a recurrent state.

    q = silu(Wq x), k = silu(Wk x)   heads x dim;     v = silu(Wv x)   heads x vdim
    S_t = decay_h * S_(t-1) + k_t v_t^T               a [dim, vdim] matrix per (sequence, head), zero at the start
    o_t = S_t^T q_t                                   no other scale
    out = Wo ( rms(o_t over all heads together) * w_norm * sigmoid(Wg x) )

The four projections are one stacked product.  The state is a fixed-size float32 region of the cache (kind
"state"): a step continues from what the sequence's slot holds, whatever the step's cut, and a slot starts at
zero.  State, decay and both products of the recurrence are float32; the projections and their activations have
the engine's activation type.  One kernel walks a sequence's rows of the step in order with the state in
registers (`lightning_scan`, prompts and decode steps alike), one norms and gates (`gated_rmsnorm`).
Every size and the decays are constructor parameters.
"""

from __future__ import annotations

import torch

from ..weights.binder import TensorSpec
from .base import MIXERS, CacheNeed
from .linear import Linear


class LightningAttention:
    graph_safe = True      # forward reads only the step's device tensors
    graph_safe_rows = None
    writes_fresh = True    # forward(..., fresh=True) writes its result instead of adding it

    def __init__(self, hidden: int, n_heads: int, dim: int, vdim: int, decay, norm_eps: float, prefix: str):
        if len(decay) != n_heads:
            raise ValueError(f"{len(decay)} decay factors for {n_heads} heads")
        self.hidden, self.n_heads, self.dim, self.vdim = int(hidden), int(n_heads), int(dim), int(vdim)
        self.decay_values, self.norm_eps, self.prefix = [float(d) for d in decay], float(norm_eps), prefix
        key_width, value_width = self.n_heads * self.dim, self.n_heads * self.vdim
        self.q_off, self.k_off, self.v_off, self.g_off = 0, key_width, 2 * key_width, 2 * key_width + value_width
        self.proj = Linear(hidden, [key_width, key_width, value_width, value_width],
                           [prefix + "q", prefix + "k", prefix + "v", prefix + "g"])
        self.out = Linear(value_width, hidden, prefix + "o")
        self.norm_weight = self.decay = None

    @property
    def input_reader(self):
        return self.proj.reader()

    def tensor_specs(self):
        return self.proj.tensor_specs() + self.out.tensor_specs() + [
            TensorSpec(self.prefix + "norm", (self.n_heads * self.vdim,), "norm")]

    def load(self, get):
        self.proj.load(get)
        self.out.load(get)
        self.norm_weight = get(self.prefix + "norm").to(torch.float32).contiguous()
        self.decay = torch.tensor(self.decay_values, dtype=torch.float32, device=self.norm_weight.device)

    def prepare(self, kernels):
        self.proj.prepare(kernels)
        self.out.prepare(kernels)

    def cache_need(self):
        return CacheNeed(kind="state", state_shape=(self.n_heads, self.dim, self.vdim), state_dtype=torch.float32)

    def working_bytes(self, step) -> int:
        width = self.n_heads * self.vdim
        chunks = 0
        if step.sizes is not None and hasattr(step.sizes, "lightning_chunk_bytes"):
            chunks = step.sizes.lightning_chunk_bytes(step.seqs, step.rows, step.max_rows_per_seq, self.n_heads, self.dim, self.vdim)
        return (chunks + self.proj.working_bytes(step, step.rows) + step.matrix(step.rows, width, 4)
                + step.matrix(step.rows, width, reader=self.out.reader_for_plan(step.act_size))
                + self.out.working_bytes(step, step.rows, accumulate=True))

    def forward(self, ctx, x, hidden, cache, then_norm=None, fresh=False):
        k = ctx.kernels
        width = self.n_heads * self.vdim
        proj = self.proj.forward(ctx, x)
        mixed = ctx.new_f32(ctx.n_rows, width)
        k.lightning_scan(proj, self.q_off, self.k_off, self.v_off, cache.state, self.decay, ctx.seq_start, ctx.seq_slot,
                         mixed, self.n_heads, self.dim, self.vdim, max_rows_per_seq=ctx.max_rows_per_seq)
        gated = ctx.new_activations(ctx.n_rows, width, reader=self.out.reader())
        k.gated_rmsnorm(mixed, proj, self.g_off, self.norm_weight, self.norm_eps, gated)
        self.out.forward(ctx, gated, out=hidden, accumulate=not fresh)
        return None


@MIXERS.register("lightning_attention")
def _build_lightning_attention(config, layer_index, prefix, shared):
    sizes = config.layers[layer_index].mixer
    return LightningAttention(config.hidden, sizes.heads, sizes.dim, sizes.vdim, sizes.decay, config.rms_eps, prefix + "mix.")
