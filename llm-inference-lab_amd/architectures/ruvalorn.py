"""Ruvalorn as data: configuration -> ``ModelSpec``.

A stack of pre-norm layers ``x += mixer(norm1(x)); x += feed_forward(norm2(x))`` whose norms are
RMS norms with a weight stored around zero (scale ``1 + w``).  The mixer is grouped-query
attention through a sliding window: queries and keys with biases, the values are the keys
before they are rotated, a rotation of the first channels of each head, one sigmoid gate per
head on the heads' outputs.  The feed-forward is a gated one (SiLU), a mixture of such experts
behind a router with grouped choice, identity outputs and a shared expert, or absent.  A run
of layers may be repeated with the same weights: every pass has caches of its own and starts
with a learned vector added to the stream.  The head is a matrix of its own behind a last norm.

Tensor names: ``embed``, ``head``, ``final.norm``, ``loop.step``, and per layer ``l<i>.norm1``,
``l<i>.norm2``, ``l<i>.mix.{q,q.b,k,k.b,g,o}``, ``l<i>.mlp.{gate,up,down}`` or
``l<i>.mlp.{router,correction,e<j>.gate,e<j>.up,e<j>.down,shared.gate,shared.up,shared.down}``.
"""
from __future__ import annotations

import dataclasses

from ..config.registry import register_architecture
from ..config.ruvalorn import RuvalornConfig
from ..config.spec import BlockSpec, ModelSpec, PartSpec, ScheduleEntry, StreamOffset


def _gated(prefix: str, width: int, ff: int) -> PartSpec:
    return PartSpec("swiglu", params=dict(hidden_size=width, intermediate_size=ff, activation="silu"),
                    tensors=dict(gate_weight=prefix + "gate", up_weight=prefix + "up", down_weight=prefix + "down"))


def build_ruvalorn_spec(cfg: RuvalornConfig) -> ModelSpec:
    w = cfg.width
    norm = lambda name: PartSpec("rmsnorm", params=dict(size=w, eps=cfg.norm_eps, weight_offset=1.0),
                                 tensors=dict(weight=name))
    blocks = []
    for i, l in enumerate(cfg.layers):
        p = f"l{i}."
        position = (PartSpec("rope", params=dict(dim=l.dim, rotary_dim=l.rot_dims, theta=l.rot_base))
                    if l.rot_dims else None)
        mixer = PartSpec(
            "gqa_attention",
            params=dict(hidden_size=w, num_heads=l.heads, num_kv_heads=l.kv_heads, head_dim=l.dim, qkv_bias=True,
                        out_bias=False, window=l.window, scale=l.scale, position=position, values_from_keys=True,
                        output_gate="sigmoid"),
            tensors=dict(q_weight=p + "mix.q", q_bias=p + "mix.q.b", k_weight=p + "mix.k", k_bias=p + "mix.k.b",
                         gate_weight=p + "mix.g", o_weight=p + "mix.o"))
        parts = dict(norm1=norm(p + "norm1"), mixer=mixer)
        f = l.mlp
        if f is not None and f.kind == "dense":
            parts.update(norm2=norm(p + "norm2"), feed_forward=_gated(p + "mlp.", w, f.ff))
        elif f is not None:
            r = f.router
            parts.update(norm2=norm(p + "norm2"), feed_forward=PartSpec(
                "routed_experts",
                params=dict(hidden_size=w, expert_size=f.ff, num_experts=r.experts, top=r.top, identity=r.identity,
                            scale=r.scale, groups=r.groups, groups_keep=r.groups_keep, correction=True,
                            shared=None if f.shared_ff is None else _gated(p + "mlp.shared.", w, f.shared_ff)),
                tensors=dict(router=p + "mlp.router", correction=p + "mlp.correction",
                             expert_gate=p + "mlp.e{}.gate", expert_up=p + "mlp.e{}.up",
                             expert_down=p + "mlp.e{}.down")))
        blocks.append(BlockSpec("prenorm", parts=parts, params=dict(hidden_size=w)))
    schedule = []
    first = cfg.loop.start if cfg.loop is not None else None
    for layer, turn in cfg.runs():
        # every run owns its cache; a pass of the repeated layers starts with its vector
        offset = (StreamOffset("loop.step", turn, cfg.loop.times)
                  if turn is not None and layer == first else None)
        schedule.append(ScheduleEntry(layer, offset=offset))
    sizes = dict(vocab_size=cfg.vocab, hidden_size=w)
    spec = ModelSpec(
        architecture=RuvalornConfig.ARCHITECTURE, vocab_size=cfg.vocab, hidden_size=w,
        max_positions=RuvalornConfig.MAX_POSITIONS,
        embedding=PartSpec("token_embedding", params=sizes, tensors=dict(weight="embed")),
        blocks=tuple(blocks), schedule=tuple(schedule), final_norm=norm("final.norm"),
        head=PartSpec("linear_head", params=sizes, tensors=dict(weight="head")),
        eos_token_ids=tuple(cfg.eos_token_ids))
    spec.validate()
    return spec


register_architecture(RuvalornConfig.ARCHITECTURE, RuvalornConfig, build_ruvalorn_spec, replace=True)
