"""Pudorax: a decoder whose layers mix tokens either by softmax attention behind short convolutions (queries and keys
normed over the whole projection, a partial rotation in neighbouring pairs, a gate on the heads) or by a state-space
recurrence with a scalar decay per head; routed experts with a shared one as feed-forward (a layer may have none);
layer norms with a bias; a second, small input from the token itself after every layer; a stretch of layers that runs
several times in a row with the same weights, every pass with memory of its own and entered through a matrix that also
reads the embedding; a scaled embedding and capped logits.

Tensor names and shapes (D width, V vocab, per layer N):
  embed [V, D]; final.norm, final.norm.b [D]; head [V, D]; loop.in [D, 2 D] with a loop; side.embed [V, layers * dim]
  lN.norm1, lN.norm1.b, lN.norm2, lN.norm2.b [D]; lN.side.gate [dim, D], lN.side.proj [D, dim], lN.side.norm [D]
  attention:  lN.mix.q [heads * dim, D], .k [kv_heads * dim, D], .v [kv_heads * vdim, D], .g [heads * vdim, D],
              .q.norm, .k.norm (over the whole projection), .q.conv / .k.conv / .v.conv [channels, taps], .o [D, heads * vdim]
  mamba2:     lN.mix.in [2 inner + 2 groups * state + heads, D], .conv [inner + 2 groups * state, taps], .conv.b,
              .dt_bias, .A_log, .D [heads], .norm [inner], .o [D, inner]            (inner = heads * vdim)
  experts:    lN.mlp.router [experts, D], .router.b, lN.mlp.eK.gate / .up [ff, D], .down [D, ff], lN.mlp.shared.*
"""

from __future__ import annotations

from ..config.pudorax import PudoraxConfig
from ..parts.embedding import CappedLMHead, ScaledEmbedding
from ..parts.token_side import LoopInput, TokenSideTable
from ..registry import register_architecture
from .decoder import build_decoder


def build_pudorax(config: PudoraxConfig):
    def shared_parts(c):
        if not c.token_side_dim:
            return {}
        return {"token_side_table": TokenSideTable(c.vocab, c.n_layers, c.token_side_dim, "side.embed")}

    return build_decoder(
        config, position_encoding="none", layer_prefix="l{}.", final_norm_name="final.norm", final_norm_kind="layernorm",
        make_embedding=lambda c: ScaledEmbedding(c.vocab, c.hidden, "embed", c.embedding_scale),
        make_head=lambda c, embedding: CappedLMHead(c.vocab, c.hidden, "head", c.logit_softcap),
        make_shared=shared_parts, make_pass_input=lambda c: LoopInput(c.hidden, "loop.in") if c.has_loop else None)


register_architecture("Pudorax", PudoraxConfig, build_pudorax)
