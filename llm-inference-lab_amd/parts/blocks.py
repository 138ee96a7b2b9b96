"""Arrangements of parts in a layer, the embedding and the output head."""
from __future__ import annotations

from typing import Dict

import torch

from ..config.spec import PartSpec
from ..weights.loader import TensorSpec, MATRIX
from .base import Block, Part, NormedInput
from .registry import register_part, build_part


class PreNormBlock(Block):
    """``x += mixer(norm1(x)); x += feed_forward(norm2(x))``; the sums are taken
    in float32 on the float32 residual stream.

    Arrangement: rust/engine/src/runner/model/qwen2/engine.rs:1065-1122 (layer
    loop), 1140-1147 and 1234-1241 (norm before each sublayer)."""

    def __init__(self, hidden_size: int, norm1: PartSpec, mixer: PartSpec, norm2: PartSpec = None,
                 feed_forward: PartSpec = None, tensors: Dict[str, str] = None):
        super().__init__(tensors)
        if (feed_forward is None) != (norm2 is None):
            raise ValueError("a feed-forward and its norm come together")
        self.hidden_size = int(hidden_size)
        self.norm1 = build_part("norm", norm1)
        self.mixer = build_part("mixer", mixer)
        # (a layer may be its mixer alone)
        self.norm2 = build_part("norm", norm2) if norm2 is not None else None
        self.feed_forward = build_part("feed_forward", feed_forward) if feed_forward is not None else None

    def parts(self):
        return [p for p in (self.norm1, self.mixer, self.norm2, self.feed_forward) if p is not None]

    def mixer_part(self):
        return self.mixer

    def tensor_specs(self):
        specs = {}
        for p in self.parts():
            specs.update(p.tensor_specs())
        return specs

    def bind(self, tensors, ops, dtype):
        super().bind(tensors, ops, dtype)
        for p in self.parts():
            p.bind(tensors, ops, dtype)

    def forward(self, residual, ctx, entry):
        h = NormedInput(self.norm1, residual, ctx, "block.normed", self.dtype)
        self.mixer.forward(h if self.mixer.takes_normed_input else h.tensor(), residual, ctx, entry)
        if self.feed_forward is None:
            return
        h = NormedInput(self.norm2, residual, ctx, "block.normed", self.dtype)
        self.feed_forward.forward(h if self.feed_forward.takes_normed_input else h.tensor(),
                                  residual, ctx)

    def weight_bytes(self):
        return sum(p.weight_bytes() for p in self.parts())


class SublayerNormBlock(Block):
    """``x += norm1(mixer(x)); x += norm2(feed_forward(x))``: the sublayers read the stream
    itself and each norm acts on its sublayer's OUTPUT, before the sum.  A block without a
    feed-forward has the first half only.  The stream and both sums are float32; the
    sublayers' products read the stream rounded to the compute dtype.

    A part that ``writes_output`` writes its float32 result into a scratch buffer
    (``forward_into``); any other part (made for blocks that add the sublayer's result
    straight into the stream) is handed a zeroed buffer in the stream's place."""

    def __init__(self, hidden_size: int, mixer: PartSpec, norm1: PartSpec, feed_forward: PartSpec = None,
                 norm2: PartSpec = None, tensors: Dict[str, str] = None):
        super().__init__(tensors)
        if (feed_forward is None) != (norm2 is None):
            raise ValueError("a feed-forward and its norm come together")
        self.hidden_size = int(hidden_size)
        self.mixer = build_part("mixer", mixer)
        self.norm1 = build_part("norm", norm1)
        self.feed_forward = build_part("feed_forward", feed_forward) if feed_forward is not None else None
        self.norm2 = build_part("norm", norm2) if norm2 is not None else None
        for n in (self.norm1, self.norm2):
            if n is not None and not hasattr(n, "add_into"):
                raise ValueError(f"{type(n).__name__} cannot norm a sublayer's output into the stream (no add_into)")

    def parts(self):
        return [p for p in (self.mixer, self.norm1, self.feed_forward, self.norm2) if p is not None]

    def mixer_part(self):
        return self.mixer

    def tensor_specs(self):
        specs = {}
        for p in self.parts():
            specs.update(p.tensor_specs())
        return specs

    def bind(self, tensors, ops, dtype):
        super().bind(tensors, ops, dtype)
        for p in self.parts():
            p.bind(tensors, ops, dtype)

    def _fold(self, residual, ctx):
        pending = getattr(ctx, "pending", None)
        if pending is not None:          # (sums another kind of block left in pieces)
            self.ops.add_pending(residual, pending)
            ctx.pending = None

    NOTE = "sublayer_norm.copy"      # in the step's notes: the run whose last sum left the stream's copy behind

    def _input(self, residual, ctx, entry):
        """The stream as the sublayers' products read it: the stream itself in float32, else its
        rounded copy, which the run just before this one has left behind if it was of this kind."""
        if self.dtype == torch.float32:
            return residual
        h = ctx.scratch("block.stream_copy", tuple(residual.shape), self.dtype)
        memo = getattr(ctx, "memo", None)
        if memo is not None and memo.pop(self.NOTE, None) == entry.index - 1:
            return h
        self.ops.activation(residual, h, "cast")
        return h

    def _sublayer(self, part, h, residual, ctx, *entry):
        y = ctx.scratch("block.sublayer_out", tuple(residual.shape), torch.float32)
        if part.writes_output:
            part.forward_into(h, y, ctx, *entry)
        else:
            self.ops.activation(y, y, "zero")
            part.forward(h, y, ctx, *entry)
            self._fold(y, ctx)
        return y

    def forward(self, residual, ctx, entry):
        self._fold(residual, ctx)
        h = self._input(residual, ctx, entry)
        # every sum's new rows go to the next reader of the stream in the same pass
        copy = h if self.dtype != torch.float32 else None
        y = self._sublayer(self.mixer, h, residual, ctx, entry)
        self.norm1.add_into(y, residual, copy)
        if self.feed_forward is not None:
            y = self._sublayer(self.feed_forward, h, residual, ctx)
            self.norm2.add_into(y, residual, copy)
        memo = getattr(ctx, "memo", None)
        if memo is not None and copy is not None:
            memo[self.NOTE] = entry.index

    def weight_bytes(self):
        return sum(p.weight_bytes() for p in self.parts())


class TokenEmbedding(Part):
    """``x[r] = table[id_r]`` into the float32 residual stream
    (rust/engine/src/runner/model/qwen2/kernels.rs:46-57)."""

    def __init__(self, vocab_size: int, hidden_size: int, tensors: Dict[str, str]):
        super().__init__(tensors)
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.table = None

    def tensor_specs(self):
        return {self.tensor_names["weight"]: TensorSpec((self.vocab_size, self.hidden_size), MATRIX)}

    def bind(self, tensors, ops, dtype):
        super().bind(tensors, ops, dtype)
        ops.check_product_sizes(self.hidden_size, dtype, "embedding (hidden size)")
        # in the order the product kernels read, so that a tied output head shares it
        self.table = ops.prepare_weight(tensors[self.tensor_names["weight"]], shared=True)

    def forward(self, ids, out, ctx=None):
        """``ctx``: the step's batch description, for embeddings that need more than the
        ids (positions, say); this one does not."""
        self.ops.embed(self.table, ids, out)

    def weight_bytes(self):
        return 0     # a step reads one row per token, not the table


class LinearHead(Part):
    """``logits = h W^T`` in float32; ``W`` is the embedding table when the
    names coincide (tied), as in rust/engine/src/runner/model/qwen2/engine.rs:299-303
    and 1312-1319."""

    def __init__(self, vocab_size: int, hidden_size: int, tensors: Dict[str, str]):
        super().__init__(tensors)
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.weight = None

    def tensor_specs(self):
        return {self.tensor_names["weight"]: TensorSpec((self.vocab_size, self.hidden_size), MATRIX)}

    def bind(self, tensors, ops, dtype):
        super().bind(tensors, ops, dtype)
        ops.check_product_sizes(self.hidden_size, dtype, "output head (hidden size)")
        self.weight = ops.prepare_weight(tensors[self.tensor_names["weight"]], shared=True)

    takes_normed_input = True

    def forward(self, h, out):
        fuse = (isinstance(h, NormedInput) and self.ops.can_fuse(out.shape[0], self.dtype, self.hidden_size, out.shape[1])
                and not self.ops.pieces_too_large_to_read_per_block(getattr(h.ctx, "pending", None)))
        rms = h.rms(accept_pending=True) if fuse else None
        if rms is not None:
            # the last reader of the stream: pieces still owed to it are added on the fly
            pending = getattr(h.ctx, "pending", None)
            self.ops.fused_norm_logits(rms[0], rms[1], rms[2], rms[3], self.weight, out, pending=pending)
            h.ctx.pending = None
        else:
            if isinstance(h, NormedInput):
                h = h.tensor()
            self.ops.linear_logits(h, self.weight, out)

    def weight_bytes(self):
        return self.weight.numel() * self.weight.element_size()


register_part("block", "prenorm", PreNormBlock)
register_part("block", "sublayer_norm", SublayerNormBlock)
register_part("embedding", "token_embedding", TokenEmbedding)
register_part("head", "linear_head", LinearHead)
