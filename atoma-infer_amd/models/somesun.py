"""The Somesun decoder put together from parts.

Every layer is a sandwich block (a norm before and behind each sublayer) around two mixers that run side by side
on the same input, attention with values tied to its keys (chunked mask, a sink per head) and a gated delta rule,
and, where the layer has one, a feed-forward of routed experts.  Tensor names are the checkpoint's own: ``embed``,
``l<i>.norm1`` / ``norm1b`` / ``norm2`` / ``norm2b``, ``l<i>.mix.left.*``, ``l<i>.mix.right.*``, ``l<i>.mlp.*``,
``final.norm``, ``head``.
"""
from __future__ import annotations

from ..config.registry import register_architecture
from ..config.somesun import SomesunConfig
from ..parts.base import make_part
from ..parts.embedding import OutputHead, TokenEmbedding
from .spec import ModelSpec


def build_somesun(cfg: SomesunConfig) -> ModelSpec:
    w, eps = cfg.width, cfg.norm_eps
    norm = lambda name: make_part("norm", "rmsnorm", width=w, eps=eps, name=name)
    layers = []
    for i, layer in enumerate(cfg.layers):
        l, r = layer.mixer.left, layer.mixer.right
        left = make_part("mixer", "tied_value_attention", width=w, num_heads=l.heads, num_kv_heads=l.kv_heads,
                         head_size=l.dim, scale=l.scale, norm_eps=eps, rotary_base=l.rot.base, rotary_dim=l.rot.dims,
                         chunk=l.mask.size, sink=True)
        right = make_part("mixer", "gated_delta_rule", width=w, heads=r.heads, kv_heads=r.kv_heads, dim=r.dim,
                          vdim=r.vdim, taps=r.conv, norm_eps=eps, decay_rank=r.decay_rank, gate_rank=r.gate_rank)
        mixer = make_part("mixer", "parallel", branches=[left, right],
                          scales=[layer.mixer.left_scale, layer.mixer.right_scale], names=["left", "right"])
        ffn = None
        if layer.mlp is not None:
            ffn = make_part("feed_forward", "routed_experts", width=w, intermediate=layer.mlp.ff,
                            experts=layer.mlp.experts, top=layer.mlp.top)
        norms = (norm("norm1"), norm("norm1b"), norm("norm2") if ffn else None, norm("norm2b") if ffn else None)
        layers.append((f"l{i}", make_part("block", "sandwich", norms=norms, mixer=mixer, feed_forward=ffn)))
    # a layer without a feed-forward may still carry the two norms of one in its checkpoint
    ignorable = tuple(rf"l{i}\.norm2b?" for i, layer in enumerate(cfg.layers) if layer.mlp is None)
    return ModelSpec(width=w, vocab_size=cfg.vocab, max_positions=cfg.max_positions,
                     embedding=("", TokenEmbedding(cfg.vocab, w, name="embed")), layers=layers,
                     final_norm=("", norm("final.norm")), head=("", OutputHead(w, cfg.vocab, name="head")),
                     ignorable=ignorable)


for _name in SomesunConfig.architectures:
    register_architecture(_name, SomesunConfig, build_somesun, replace=True)
