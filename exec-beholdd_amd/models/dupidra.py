"""Dupidra: a decoder whose layers mix tokens by grouped softmax attention within chunks (biased projections, per-head
query and key norms, a rotation over part of a head, gated heads), by softmax attention over a cached latent within a
sliding window (gated the same way), or by a matrix memory with exponential gates kept as a recurrent state; dense
GELU feed-forwards or routed experts (a layer may have none); layer norms with a bias that stand behind the sums,
x <- norm(alpha x + sublayer(x)); layers that run another layer's tensors with memory of their own; logits from the
embedding table.

Tensor names and shapes (D width, V vocab, per layer N that has tensors of its own):
  embed [V, D] (also the head); final.norm, final.norm.b [D]
  lN.norm1, lN.norm1.b [D], and lN.norm2, lN.norm2.b where the layer has a feed-forward
  attention:         lN.mix.q [heads * dim, D], .k [kv_heads * dim, D], .v [kv_heads * vdim, D] with .q.b / .k.b / .v.b,
                     .q.norm, .k.norm [dim], .g [heads * vdim, D], .o [D, heads * vdim]
  latent attention:  lN.mix.q [heads * dim, D], .dkv [kv_rank, D], .dkv.norm [kv_rank], .uk [heads * dim, kv_rank],
                     .uv [heads * vdim, kv_rank], .g [heads * vdim, D], .o [D, heads * vdim]
  mlstm:             lN.mix.q / .k [heads * dim, D], .v / .g [heads * vdim, D], .i / .f [heads, D] with .i.b / .f.b [heads],
                     .norm [heads * vdim], .o [D, heads * vdim]
  dense:             lN.mlp.up [ff, D], lN.mlp.down [D, ff]
  experts:           lN.mlp.router [experts, D], lN.mlp.eK.gate / .up [ff, D], .down [D, ff]
"""

from __future__ import annotations

from ..config.dupidra import DupidraConfig
from ..registry import register_architecture
from .decoder import build_decoder


def build_dupidra(config: DupidraConfig):
    return build_decoder(config, position_encoding="none", layer_prefix="l{}.", embedding_name="embed",
                         final_norm_name="final.norm", final_norm_kind="layernorm")


register_architecture("Dupidra", DupidraConfig, build_dupidra)
