"""Blocks whose sublayers' results are normed before they join the residual stream.

``SandwichBlock``: x += s1 * norm1b(mixer(norm1(x))); x += s2 * norm2b(ffn(norm2(x))), s1 and s2
learned vectors, then an optional ``TokenSide`` part. Each add runs in ONE kernel that norms
the sublayer's float32 result, scales it, adds it to the float32 stream and, in the same pass
over the row, applies the stream's NEXT norm (norm2 of this block, norm1 of the block that
follows), so the stream is read and written once per sublayer.

``TokenSide``: x += rms_norm(P (gelu_tanh(G x) * e)) * w with e the block's own columns of the
step's side-table rows (``parts.embedding.TokenSideTable``).
"""
from __future__ import annotations

import torch

from .. import kernels
from ..weights.loader import Param
from .base import Part, PartError, build_part, register_part, span
from .embedding import TokenSideTable
from .linear import linear, linear_delta


class TokenSide(Part):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        if spec.dim < 1 or spec.offset < 0:
            raise PartError(f"token side input of {spec.dim} columns at {spec.offset}")
        self.spec, self.dtype = spec, dtype

    def params(self):
        s = self.spec
        return {"gate.weight": Param((s.dim, s.hidden), "matrix"),
                "proj.weight": Param((s.hidden, s.dim), "matrix"),
                "norm.weight": Param((s.hidden,), "vector", init="around_one")}

    def run(self, x, xcast, ctx, next_norm=None, out=None):
        """x: the float32 stream, updated in place; xcast: the same rows in the engine's type.
        next_norm / out: the norm that reads the stream next and where its rows go."""
        s, nt = self.spec, x.shape[0]
        rows = ctx.shared.get(TokenSideTable.KEY)
        if rows is None or rows.shape[1] < s.offset + s.dim:
            raise PartError("the token side input needs the step's side-table rows "
                            f"(columns {s.offset}..{s.offset + s.dim})")
        g = linear(xcast, self.w["gate.weight"], ctx.ws.take("side.gate", (nt, s.dim), self.dtype))
        kernels.activation(g, g, "gelu_tanh", side=rows[:, s.offset:s.offset + s.dim])
        y = linear(g, self.w["proj.weight"], ctx.ws.take("side.y", (nt, s.hidden), torch.float32))
        kernels.postnorm_add(x, y, self.w["norm.weight"], float(s.eps),
                             next_weight=None if next_norm is None else next_norm.gain(),
                             next_eps=0.0 if next_norm is None else next_norm.eps, out=out)


register_part("token_side", TokenSide)


class SandwichBlock(Part):
    folds_norms = True      # ``run`` is told which block follows, and applies that block's first norm

    def __init__(self, spec, dtype, device):
        self.spec, self.dtype, self.hidden = spec, dtype, spec.hidden
        self.norm1 = build_part(spec.norm1, dtype, device)
        self.mixer = build_part(spec.mixer, dtype, device)
        self.norm1b = build_part(spec.norm1b, dtype, device)
        self.ffn = build_part(spec.ffn, dtype, device) if spec.ffn is not None else None
        self.norm2 = build_part(spec.norm2, dtype, device) if self.ffn is not None else None
        self.norm2b = build_part(spec.norm2b, dtype, device) if self.ffn is not None else None
        self.side = build_part(spec.side, dtype, device) if spec.side is not None else None
        for n in (self.norm1, self.norm1b, self.norm2, self.norm2b):
            if n is not None and not (hasattr(n, "gain") and hasattr(n, "eps")):
                raise PartError("the norms of a sandwich block are RMS norms with a gain per coordinate")

    def children(self):
        c = {"norm1": self.norm1, "mixer": self.mixer, "norm1b": self.norm1b}
        if self.ffn is not None:
            c.update(norm2=self.norm2, ffn=self.ffn, norm2b=self.norm2b)
        if self.side is not None:
            c["side"] = self.side
        return c

    def params(self):
        if not self.spec.layer_scale:
            return {}
        p = {"ls1": Param((self.hidden,), "vector", init="around_one")}
        if self.ffn is not None:
            p["ls2"] = Param((self.hidden,), "vector", init="around_one")
        return p

    def bind(self, tensors):
        super().bind(tensors)
        self._scaled = {}

    def _post_weight(self, which):
        """The output norm's gain times the layer scale, one vector (made at first use, when
        the children are bound as well)."""
        w = self._scaled.get(which)
        if w is None:
            w = getattr(self, "norm" + which + "b").gain()
            if self.spec.layer_scale:
                w = (w * self.w["ls" + which]).contiguous()
            self._scaled[which] = w
        return w

    def cache_need(self):
        return self.mixer.cache_need()

    def step_planner(self):
        f = getattr(self.mixer, "step_planner", None)
        return f() if f is not None else None

    @property
    def graph_safe(self) -> bool:
        return all(getattr(p, "graph_safe", False) for p in self.children().values())

    def entry_norm(self):
        """The norm that reads the stream first: the block in front applies it in its last add."""
        return self.norm1

    def run(self, x, pending, ctx, cache, layer, writes_cache=True, after=None):
        """pending: (delta, bias) still to be added before norm1, (None, None), or "normed":
        the block in front has already left norm1's rows in the shared buffer."""
        h = ctx.ws.take("block.h", x.shape, self.dtype)
        if pending != "normed":
            with span(ctx, "norm"):
                self.norm1.run(x, h, pending[0], pending[1])
        with span(ctx, "mixer"):
            delta, bias = self.mixer.run(h, ctx, cache, layer, writes_cache)
        if bias is not None:
            raise PartError("a sandwich block's sublayers return no bias rows")
        # what follows the last add of this block: the next block's first norm, when it offers it
        follow = getattr(after, "entry_norm", None)
        follow = follow() if follow is not None else None
        last = self.side if self.side is not None else "ffn" if self.ffn is not None else "mixer"
        xcast = ctx.ws.take("block.xcast", x.shape, self.dtype) if self.side is not None else None

        def add(which, delta, nxt, is_last):
            with span(ctx, "norm"):
                kernels.postnorm_add(
                    x, delta, self._post_weight(which), float(getattr(self, "norm" + which + "b").eps),
                    xcast=xcast if (self.side is not None and is_last) else None,
                    next_weight=None if nxt is None else nxt.gain(),
                    next_eps=0.0 if nxt is None else nxt.eps, out=None if nxt is None else h)

        if self.ffn is None:
            add("1", delta, follow if last == "mixer" else None, True)
        else:
            add("1", delta, self.norm2, False)
            with span(ctx, "ffn"):
                delta, bias = self.ffn.run(h, ctx)
            if bias is not None:
                raise PartError("a sandwich block's sublayers return no bias rows")
            add("2", delta, follow if last == "ffn" else None, True)
        if self.side is not None:
            with span(ctx, "side"):
                self.side.run(x, xcast, ctx, next_norm=follow, out=None if follow is None else h)
        return "normed" if follow is not None else (None, None)


register_part("sandwich", SandwichBlock)
