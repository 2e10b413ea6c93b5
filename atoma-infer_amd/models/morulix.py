"""The Morulix decoder put together from parts.

Every layer is a side-by-side block: one norm (weight stored around zero), whose output the mixer and, where the layer
has one, a dense SwiGLU feed-forward both read, their outputs added to the stream together.  The mixer is, layer by
layer, windowed attention with rotated heads (``attention``), attention over one cached latent vector per token
(``latent_attention``) or a state-space recurrence (``mamba2``).  A run of layers may be gone through several times
with the same weights, each pass with a cache or state of its own and begun by a map of the stream and the
embedding's rows (``loop``).  Tensor names are the checkpoint's own: ``embed``, ``loop.in``, ``loop.step``,
``l<i>.norm1``, ``l<i>.mix.*``, ``l<i>.mlp.gate`` / ``up`` / ``down``, ``final.norm``, ``head``.
"""
from __future__ import annotations

from ..config.morulix import AttentionMixer, LatentMixer, MorulixConfig, StateSpaceMixer
from ..config.registry import register_architecture
from ..parts.base import make_part
from ..parts.embedding import OutputHead, TokenEmbedding
from .spec import LayerCall, ModelSpec


def _mixer(m, width: int, eps: float, max_positions: int):
    if isinstance(m, AttentionMixer):
        position = None
        if m.rot is not None and m.rot.dims > 0:
            sc = m.rot.scaling
            scaling = None if sc is None else {"factor": sc.factor, "low_freq_factor": sc.low, "high_freq_factor": sc.high,
                                               "original_max_position_embeddings": sc.original}
            position = make_part("position", "rotary", head_size=m.dim, theta=m.rot.base, max_positions=max_positions,
                                 scaling=scaling, rotary_dim=m.rot.dims, precise=True)
        return make_part("mixer", "attention", width=width, num_heads=m.heads, num_kv_heads=m.kv_heads, head_size=m.dim,
                         value_size=m.vdim, position=position, window=m.mask.size if m.mask is not None else None,
                         scale=m.scale, names=("q", "k", "v", "o"))
    if isinstance(m, LatentMixer):
        return make_part("mixer", "latent_attention", width=width, num_heads=m.heads, head_size=m.dim,
                         value_size=m.vdim, rank=m.kv_rank, scale=m.scale, norm_eps=eps)
    if isinstance(m, StateSpaceMixer):
        return make_part("mixer", "state_space_duality", width=width, heads=m.heads, groups=m.groups, vdim=m.vdim,
                         state=m.state, taps=m.conv, norm_groups=m.norm_groups, norm_eps=eps)
    raise TypeError(f"no part for mixer {m!r}")


def build_morulix(cfg: MorulixConfig) -> ModelSpec:
    w, eps = cfg.width, cfg.norm_eps
    norm = lambda name: make_part("norm", "rmsnorm", width=w, eps=eps, name=name, offset=1.0)
    layers = []
    for i, layer in enumerate(cfg.layers):
        ffn = None
        if layer.mlp is not None:
            ffn = make_part("feed_forward", "swiglu", width=w, intermediate=layer.mlp.ff, names=("gate", "up", "down"))
        layers.append((f"l{i}", make_part("block", "side_by_side", norm1=norm("norm1"),
                                          mixer=_mixer(layer.mixer, w, eps, cfg.max_positions), feed_forward=ffn)))
    n = len(layers)
    order = [LayerCall(i) for i in range(n)]
    if cfg.loop is not None:
        entry = n
        layers.append(("loop", make_part("block", "loop_entry", width=w, times=cfg.loop.times)))
        lo, hi = cfg.loop.start, cfg.loop.stop
        order = [LayerCall(i) for i in range(lo)]
        for _ in range(cfg.loop.times):
            order += [LayerCall(entry)] + [LayerCall(i) for i in range(lo, hi)]
        order += [LayerCall(i) for i in range(hi, n)]
    return ModelSpec(width=w, vocab_size=cfg.vocab, max_positions=cfg.max_positions,
                     embedding=("", TokenEmbedding(cfg.vocab, w, name="embed")), layers=layers,
                     final_norm=("", norm("final.norm")), head=("", OutputHead(w, cfg.vocab, name="head")),
                     run_order=order)


for _name in MorulixConfig.architectures:
    register_architecture(_name, MorulixConfig, build_morulix, replace=True)
