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
