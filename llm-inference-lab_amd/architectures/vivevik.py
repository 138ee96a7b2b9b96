"""Vivevik as data: configuration -> ``ModelSpec``.

A stack of layers of two kinds, each ``x += norm1(mixer(x))`` then (where the layer has one)
``x += norm2(feed_forward(x))`` with layer norms on the sublayers' outputs: a gated linear
attention mixer with a recurrent state, or grouped-query attention through a sliding window
that keeps the first positions and has a sink term, whose keys and values may be those of an
earlier layer.  The head is the embedding table behind a last layer norm.

Tensor names: ``embed``, ``final.norm``, and per layer ``l<i>.norm1``, ``l<i>.norm2``,
``l<i>.mix.<role>``, ``l<i>.mlp.up`` / ``.down``.
"""
from __future__ import annotations

import dataclasses

from ..config.registry import register_architecture
from ..config.spec import BlockSpec, ModelSpec, PartSpec, ScheduleEntry
from ..config.vivevik import VivevikConfig


def build_vivevik_spec(cfg: VivevikConfig) -> ModelSpec:
    w = cfg.width
    norm = lambda name: PartSpec("layernorm", params=dict(size=w, eps=cfg.norm_eps), tensors=dict(weight=name))
    blocks, schedule = [], []
    for i, l in enumerate(cfg.layers):
        p = f"l{i}."
        if l.type == "gla":
            mixer = PartSpec(
                "gated_linear_attention",
                params=dict(hidden_size=w, num_heads=l.heads, key_dim=l.dim, value_dim=l.vdim, decay_rank=l.rank,
                            tau=l.tau, norm_eps=cfg.norm_eps),
                tensors=dict(q_weight=p + "mix.q", k_weight=p + "mix.k", v_weight=p + "mix.v",
                             gate_weight=p + "mix.g", o_weight=p + "mix.o", out_norm=p + "mix.norm",
                             decay_down=p + "mix.a1", decay_up=p + "mix.a2", decay_bias=p + "mix.a2.b"))
        else:
            own = l.kv_from is None
            names = dict(q_weight=p + "mix.q", o_weight=p + "mix.o", q_norm=p + "mix.q.norm", sink=p + "mix.sink")
            if own:
                names.update(k_weight=p + "mix.k", v_weight=p + "mix.v", k_norm=p + "mix.k.norm")
            mixer = PartSpec(
                "windowed_sink_attention",
                params=dict(hidden_size=w, num_heads=l.heads, num_kv_heads=l.kv_heads, key_dim=l.dim,
                            value_dim=l.vdim, scale=l.scale, window=l.window, keep_first=l.keep_first, sink=True,
                            qk_norm="whole", norm_eps=cfg.norm_eps, own_kv=own),
                tensors=names)
        parts = dict(mixer=mixer, norm1=norm(p + "norm1"))
        if l.mlp is not None:
            parts.update(
                feed_forward=PartSpec("dense", params=dict(hidden_size=w, intermediate_size=l.mlp.ff,
                                                           activation="relu2"),
                                      tensors=dict(up_weight=p + "mlp.up", down_weight=p + "mlp.down")),
                norm2=norm(p + "norm2"))
        blocks.append(BlockSpec("sublayer_norm", parts=parts, params=dict(hidden_size=w)))
        schedule.append(ScheduleEntry(i, cache_of=l.kv_from if l.type == "attention" else None))
    sizes = dict(vocab_size=cfg.vocab, hidden_size=w)
    spec = ModelSpec(
        architecture=VivevikConfig.ARCHITECTURE, vocab_size=cfg.vocab, hidden_size=w,
        max_positions=VivevikConfig.MAX_POSITIONS,
        embedding=PartSpec("token_embedding", params=sizes, tensors=dict(weight="embed")),
        blocks=tuple(blocks), schedule=tuple(schedule), final_norm=norm("final.norm"),
        head=PartSpec("linear_head", params=sizes, tensors=dict(weight="embed")),
        eos_token_ids=tuple(cfg.eos_token_ids))
    spec.validate()
    return spec


def vivevik_random_init(cfg: VivevikConfig, expected, seed: int, dtype):
    """Random-weights mode: a size that the configuration leaves to the tensors' shapes takes
    the configuration class's default."""
    from ..weights.random_init import random_tensors
    rank = VivevikConfig.DEFAULT_DECAY_RANK
    filled = {name: dataclasses.replace(s, shape=tuple(rank if d is None else d for d in s.shape))
              for name, s in expected.items()}
    return random_tensors(filled, seed, dtype)


register_architecture(VivevikConfig.ARCHITECTURE, VivevikConfig, build_vivevik_spec, random_init=vivevik_random_init,
                      replace=True)
