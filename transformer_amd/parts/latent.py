"""Attention over one cached latent row per token (``LatentAttentionSpec``).

The cache layer holds, per token, the normed latent c [kv_rank] and the rotated key part
[rope_dim] that all heads share: one "kv head" of keys only. The heads' key and value maps are
applied to the queries and to the attention's result instead of to the cached rows:

    qa_h = [Uk_h^T q_h(unrotated) | rotated q_h]      score = qa_h . [c | shared part] * scale
    out_h = Uv_h (sum_j p_j c_j) * sigmoid(g_h . h)

so a step reads kv_rank + rope_dim numbers per cached token whatever the number of heads, and
nothing is expanded per cached token. The first product of a step joins the query latent's
map, the key/value latent's map and the heads' gates.
"""
from __future__ import annotations

import torch

from .. import kernels
from ..cache.storage import KVNeed
from ..config.spec import PositionSpec
from ..weights.loader import Param
from .base import Part, PartError, build_part, register_part
from .linear import linear, linear_delta


class LatentAttention(Part):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        s = spec
        if min(s.num_heads, s.nope_dim + s.rope_dim, s.value_dim, s.q_rank, s.kv_rank) < 1 or s.rope_dim < 0 \
                or s.nope_dim < 0:
            raise PartError(f"latent attention: heads {s.num_heads} of {s.nope_dim} + {s.rope_dim} / "
                            f"{s.value_dim}, ranks {s.q_rank} / {s.kv_rank}")
        if s.rot_dims % 2 or not 0 <= s.rot_dims <= s.rope_dim:
            raise PartError(f"{s.rot_dims} rotated coordinates do not fit a part of {s.rope_dim}")
        if s.kv_rank > kernels.LATENT_MAX_RANK or s.rope_dim > kernels.LATENT_MAX_RANK:
            raise PartError(f"latent attention takes latents and rotated parts up to {kernels.LATENT_MAX_RANK}, "
                            f"not {s.kv_rank} / {s.rope_dim}")
        for w in (s.window, s.cache_window):
            if w is not None and w < 1:
                raise PartError(f"attention window must be >= 1, got {w}")
        if s.cache_window is not None and (s.window is None or s.window > s.cache_window):
            raise PartError(f"a window of {s.window} reads past the {s.cache_window} tokens its cache keeps")
        self.spec, self.dtype = s, dtype
        self.H, self.dn, self.dr, self.dv = s.num_heads, s.nope_dim, s.rope_dim, s.value_dim
        self.kv_off = s.q_rank
        self.gate_off = s.q_rank + (s.kv_rank + s.rope_dim if s.own_kv else 0)
        self.width = self.gate_off + (self.H if s.gated else 0)
        self.row = kernels.latent_row_width(s.kv_rank, s.rope_dim, dtype)      # a cached row, a wide query
        self.rotary = None
        if s.rot_dims:
            self.rotary = build_part(PositionSpec(head_dim=s.rot_dims, theta=s.rot_base, style="interleaved"),
                                     dtype, device)

    def params(self):
        s = self.spec
        p = {"in.weight": Param((self.width, s.hidden), "matrix"),     # query latent, kv latent + shared key part, gates
             "q_norm.weight": Param((s.q_rank,), "vector", init="around_one"),
             "uq.weight": Param((self.H * (self.dn + self.dr), s.q_rank), "matrix"),
             "uk.weight": Param((self.H * self.dn, s.kv_rank), "matrix"),
             "uv.weight": Param((self.H * self.dv, s.kv_rank), "matrix"),
             "out.weight": Param((s.hidden, self.H * self.dv), "matrix")}
        if s.own_kv:
            p["kv_norm.weight"] = Param((s.kv_rank,), "vector", init="around_one")
        return p

    def cache_need(self):
        s = self.spec
        return KVNeed(1, self.row, s.cache_window, 0)

    def bind(self, tensors):
        super().bind(tensors)
        s = self.spec
        # per head: Uk as [kv_rank, nope_dim] (the product's "weight" form) and Uv as it is
        self.uk_t = tensors["uk.weight"].view(self.H, self.dn, s.kv_rank).transpose(1, 2).contiguous() \
            if self.dn else None
        self.uv = tensors["uv.weight"].view(self.H, self.dv, s.kv_rank)

    def _per_head(self, a, w, out):
        """out[:, h] = a[:, h] @ w[h].T for views a [nt, H, K], w [H, N, K], out [nt, H, N]."""
        if a.dtype == torch.float32 or w.dtype == torch.float32:
            return kernels.gemm_simple_batched(a.transpose(0, 1), w, out.transpose(0, 1))
        torch.bmm(a.transpose(0, 1), w.transpose(1, 2), out=out.transpose(0, 1))
        return out

    def run(self, h, ctx, cache, layer, writes_cache=True):
        s, nt, H = self.spec, h.shape[0], self.H
        r, dr = s.kv_rank, self.dr
        if writes_cache != s.own_kv:
            raise PartError("a latent attention layer stores rows exactly when it forms them itself: "
                            "its schedule entry and its spec disagree")
        proj = linear(h, self.w["in.weight"], ctx.ws.take("latent.in", (nt, self.width), self.dtype))
        kc, _, group = cache.layer_kv(layer)
        meta = ctx.kv[group]
        angles = self.rotary.angles(ctx) if self.rotary is not None else None
        cq = ctx.ws.take("latent.cq", (nt, s.q_rank), self.dtype)
        kernels.latent_prepare(proj, s.q_rank, self.w["q_norm.weight"], cq, self.kv_off, r, dr, s.rot_dims,
                               self.w.get("kv_norm.weight"), float(s.eps), angles,
                               meta.dest if s.own_kv else None, kc if s.own_kv else None)
        q = linear(cq, self.w["uq.weight"], ctx.ws.take("latent.q", (nt, H * (self.dn + dr)), self.dtype))
        qa = ctx.ws.take("latent.qa", (nt, H, self.row), self.dtype)
        kernels.latent_query_rot(q, H, self.dn, dr, s.rot_dims, angles, qa, r)
        if self.dn:
            self._per_head(q.view(nt, H, self.dn + dr)[:, :, :self.dn], self.uk_t, qa[:, :, :r])
        else:
            qa[:, :, :r].zero_()
        ol = ctx.ws.take("latent.ol", (nt, H, r), self.dtype)
        shares = kernels.latent_key_shares(ctx.batch, ctx.max_qlen, H, r, self.row, ctx.max_kv_len, s.window)
        kernels.latent_attention(qa, ol, kc, meta.block_table, ctx.cu_q, ctx.pos0, ctx.max_qlen, r, dr,
                                 float(s.scale), s.window,
                                 gate=proj[:, self.gate_off:] if s.gated else None, shares=shares)
        o = ctx.ws.take("latent.o", (nt, H, self.dv), self.dtype)
        self._per_head(ol, self.uv, o)
        return linear_delta(o.view(nt, H * self.dv), self.w["out.weight"], ctx.ws, "latent.delta"), None


register_part("latent_attention", LatentAttention)
