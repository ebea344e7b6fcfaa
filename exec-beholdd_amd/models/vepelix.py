"""Vepelix: a decoder whose layers mix tokens either by softmax attention over a cached latent (queries through a latent
of their own, a rotated key part shared by all heads, a learned sink in every head's softmax sum, one sigmoid gate a head)
or by two mixers side by side, windowed grouped attention with normed heads beside gated linear attention kept as a
recurrent state; rotations in neighbouring pairs, stretched for long contexts; feed-forwards that are dense with a clamped
gated activation, or routed experts weighed by sigmoid scores on their inputs with a shared expert, or absent; RMSNorms
whose weights are stored around zero; a per-channel scale on every sublayer's result; a stretch of layers that runs several
times in a row with the same weights, every pass with memory of its own and every pass but the first entered with the
embedding's output added to the residual.

Tensor names and shapes (D width, V vocab, per layer N):
  embed [V, D]; final.norm [D]; head [V, D]
  lN.norm1, lN.norm2 [D]; lN.ls1, lN.ls2 [D]
  latent attention:  lN.mix.dq [q_rank, D], .dq.norm [q_rank], .uq [heads * (dim + rot_dim), q_rank], .dkv [kv_rank + rot_dim, D],
                     .dkv.norm [kv_rank], .uk [heads * dim, kv_rank], .uv [heads * vdim, kv_rank], .sink [heads], .g [heads, D],
                     .o [D, heads * vdim]
  parallel:          lN.mix.left.q [heads * dim, D], .k [kv_heads * dim, D], .v [kv_heads * vdim, D], .q.norm / .k.norm [dim],
                     .o [D, heads * vdim];  lN.mix.right.q / .k [heads * dim, D], .v / .g [heads * vdim, D], .a1 [rank, D],
                     .a2 [heads * dim, rank], .a2.b [heads * dim], .norm [vdim], .o [D, heads * vdim]
  dense:             lN.mlp.gate / .up [ff, D], .down [D, ff]
  experts:           lN.mlp.router [experts, D], lN.mlp.eK.gate / .up [ff, D], .down [D, ff], lN.mlp.shared.gate / .up / .down
"""

from __future__ import annotations

from ..config.vepelix import VepelixConfig
from ..parts.streams import StreamsResidual
from ..parts.token_side import EmbeddingAgain
from ..registry import register_architecture
from .decoder import build_decoder


def build_vepelix(config: VepelixConfig):
    return build_decoder(
        config, position_encoding="none", layer_prefix="l{}.", embedding_name="embed", final_norm_name="final.norm",
        head_name="head", final_norm_kind="rmsnorm_zero_centred",
        make_residual=lambda c: StreamsResidual(1, c.hidden),      # one plain residual, in the stream block's form
        make_pass_input=lambda c: EmbeddingAgain(c.hidden) if c.pass_starts() else None)


register_architecture("Vepelix", VepelixConfig, build_vepelix)
