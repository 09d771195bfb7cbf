"""Gokazen: a decoder whose layers mix tokens either by linear attention with a decay, kept as a recurrent state,
or by softmax attention over a cached latent; dense squared-ReLU feed-forwards (a layer may have none); RMSNorms
whose weights are stored around zero; a per-channel scale on every sublayer's result; several residual streams
joined by hyper-connections; a stretch of layers that runs several times in a row with the same weights, every
pass with memory of its own; logits times a constant.

Tensor names and shapes (D width, V vocab, S streams, per layer N):
  embed [V, D]; final.norm [D]; head [V, D]
  lN.norm1, lN.norm2 [D]; lN.ls1, lN.ls2 [D]; lN.hc1.in / .out [S], lN.hc1.mix [S, S] (and hc2) when there are streams
  lightning:         lN.mix.q / .k [heads * dim, D], .v / .g [heads * vdim, D], .norm [heads * vdim], .o [D, heads * vdim]
  latent attention:  lN.mix.q [heads * (dim + rot_dim), D], .dkv [kv_rank + rot_dim, D], .dkv.norm [kv_rank],
                     .uk [heads * dim, kv_rank], .uv [heads * vdim, kv_rank], .o [D, heads * vdim]
  feed-forward:      lN.mlp.up [ff, D], lN.mlp.down [D, ff]
"""

from __future__ import annotations

from ..config.gokazen import GokazenConfig
from ..parts.embedding import ScaledLMHead
from ..parts.streams import StreamsResidual
from ..registry import register_architecture
from .decoder import build_decoder


def build_gokazen(config: GokazenConfig):
    return build_decoder(
        config, position_encoding="none", layer_prefix="l{}.", embedding_name="embed", final_norm_name="final.norm",
        head_name="head", final_norm_kind="rmsnorm_zero_centred",
        make_head=lambda c, embedding: ScaledLMHead(c.vocab, c.hidden, "head", c.logit_scale),
        make_residual=lambda c: StreamsResidual(c.streams, c.hidden))


register_architecture("Gokazen", GokazenConfig, build_gokazen)
