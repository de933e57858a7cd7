"""Parts that act on the embedded rows or on the logits, outside the blocks.

A model names them in ``ModelSpec.after_embed`` / ``.on_logits``. One that keeps something
per sequence between steps offers ``cache_need()`` and is then run as
``run(t, ctx, cache, layer)``; the others as ``run(t, ctx)``.
"""
from __future__ import annotations

import torch

from .. import kernels
from ..cache.storage import StateNeed
from ..weights.loader import Param
from .base import Part, PartError, register_part


class PairHashEmbed(Part):
    """x_t += table[(previous token * mul_prev + token * mul_cur) mod buckets]; a sequence's
    first token takes the table's extra last row. The previous token of a sequence's first
    token in a step is the last token of its step before, kept as one int32 per sequence."""
    graph_safe = True

    def __init__(self, spec, dtype, device):
        if spec.buckets < 1 or spec.mul_prev < 0 or spec.mul_cur < 0:
            raise PartError(f"pair embedding: buckets {spec.buckets}, multipliers {spec.mul_prev}, "
                            f"{spec.mul_cur}")
        self.spec = spec

    def params(self):
        return {"table": Param((self.spec.buckets + 1, self.spec.hidden), "matrix")}

    def cache_need(self):
        return StateNeed((), torch.int32)

    def run(self, x, ctx, cache, layer):
        s = self.spec
        kernels.pair_embed_add(x, self.w["table"], ctx.tokens, cache.layer_state(layer), ctx.cu_q,
                               ctx.pos0, ctx.slots, s.buckets, s.mul_prev, s.mul_cur)
        return x


class LogitScale(Part):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        self.scale = float(spec.scale)

    def run(self, logits, ctx):
        if self.scale != 1.0:
            kernels.scale_(logits, self.scale)
        return logits


register_part("pair_hash_embed", PairHashEmbed)
register_part("logit_scale", LogitScale)


class EmbedScale(Part):
    """The embedded rows times a constant."""
    graph_safe = True

    def __init__(self, spec, dtype, device):
        self.scale = float(spec.scale)

    def run(self, x, ctx):
        if self.scale != 1.0:
            kernels.scale_(x, self.scale)
        return x


class TokenSideTable(Part):
    """Gathers the step's rows of a second table indexed by token, as float32, into
    ``ctx.shared[TokenSideTable.KEY]`` [nt, width]; the blocks' token-side parts read their
    own columns of it."""
    graph_safe = True
    KEY = "token_side.rows"

    def __init__(self, spec, dtype, device):
        if spec.vocab < 1 or spec.width < 1:
            raise PartError(f"token side table of {spec.vocab} x {spec.width}")
        self.spec = spec

    def params(self):
        return {"table": Param((self.spec.vocab, self.spec.width), "matrix")}

    def run(self, x, ctx):
        rows = ctx.ws.take(self.KEY, (ctx.nt, self.spec.width), torch.float32)
        ctx.shared[self.KEY] = kernels.embed(self.w["table"], ctx.tokens, rows)
        return x


class Chain(Part):
    """Parts around the blocks run one after another."""

    def __init__(self, spec, dtype, device):
        from .base import build_part
        self.parts = [build_part(s, dtype, device) for s in spec.parts]
        if any(getattr(p, "cache_need", None) is not None for p in self.parts):
            raise PartError("parts of a chain keep nothing between steps")

    @property
    def graph_safe(self):
        return all(getattr(p, "graph_safe", False) for p in self.parts)

    def children(self):
        return {str(i): p for i, p in enumerate(self.parts)}

    def run(self, t, ctx):
        for p in self.parts:
            p.run(t, ctx)
        return t


register_part("embed_scale", EmbedScale)
register_part("token_side_table", TokenSideTable)
register_part("chain", Chain)
