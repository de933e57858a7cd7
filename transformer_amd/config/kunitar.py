"""Typed configuration of the Kunitar decoder, read from its own config.json.

A Kunitar model is a list of layers. Each has one of two mixers (attention over a cached
latent with a sliding window and an output gate per head, which may read the rows another
layer cached; a matrix-state recurrence with a bonus for the current token and token-shifted
inputs) and an optional feed-forward (dense, or routed to the top experts by sigmoid scores,
with a gated shared expert). Every sublayer's result is normed and scaled per channel before
it joins the residual stream; after the feed-forward a small per-layer input derived from the
token itself is added; the embedding is scaled and doubles as the output matrix.

Keys: ``architecture``, ``vocab``, ``width``, ``norm.eps``, ``embedding.scale``,
``token_side.dim`` (absent: no per-layer token input), ``layers[i].{type, mixer, mlp}``. A
layer's ``mixer`` holds, by type: latent_attention: heads, dim, rot_dim, vdim, q_rank, kv_rank,
scale, rot.{base, dims}, mask.size (absent: no window), kv_from (absent: rows of its own);
wkv: heads, dim (the width of the decay's low-rank input is a tensor's shape:
``complete_from_file`` reads it; a configuration made by hand may give it as ``decay_rank``).
``mlp``: null, {kind: "dense", ff} or {kind: "moe", router.{experts, top}, expert.ff,
shared.ff (absent: no shared expert)}.
"""
from __future__ import annotations

import dataclasses
from dataclasses import dataclass, field
from typing import Optional, Tuple

from .spec import (BonusRecurrenceSpec, ChainSpec, ConfigError, EmbedScaleSpec, LatentAttentionSpec,
                   MLPSpec, ModelSpec, NormSpec, RoutedMLPSpec, RunSpec, SandwichBlockSpec,
                   TokenSideSpec, TokenSideTableSpec)
from .vametar import _get

LAYER_TYPES = ("latent_attention", "wkv")
# fixed by the design: the dense feed-forward's activation, the experts', the router's scores
DENSE_ACTIVATION = "gelu"
EXPERT_ACTIVATION = "relu2"


@dataclass(frozen=True)
class KunitarLayer:
    type: str
    heads: int
    dim: int
    # feed-forward: None, "dense" or "moe"
    mlp: Optional[str] = None
    ff: int = 0                          # dense width, or an expert's
    experts: int = 0
    top: int = 0
    shared_ff: Optional[int] = None
    # latent attention
    rot_dim: int = 0
    vdim: int = 0
    q_rank: int = 0
    kv_rank: int = 0
    scale: float = 0.0
    rot_dims: int = 0
    rot_base: float = 10000.0
    window: Optional[int] = None
    kv_from: Optional[int] = None
    # wkv
    decay_rank: Optional[int] = None     # None until a weight file has said it

    @classmethod
    def from_dict(cls, d: dict, i: int) -> "KunitarLayer":
        where = f"layers[{i}]."
        typ = d.get("type") if isinstance(d, dict) else None
        if typ not in LAYER_TYPES:
            raise ConfigError(f"config key '{where}type' must be one of {LAYER_TYPES}, got {typ!r}")
        kw = {}
        mlp = d.get("mlp")
        if mlp is not None:
            kind = mlp.get("kind") if isinstance(mlp, dict) else None
            if kind == "dense":
                kw.update(mlp="dense", ff=_get(mlp, "ff", int, where + "mlp."))
            elif kind == "moe":
                r = mlp.get("router")
                shared = mlp.get("shared")
                kw.update(mlp="moe", ff=_get(mlp.get("expert"), "ff", int, where + "mlp.expert."),
                          experts=_get(r, "experts", int, where + "mlp.router."),
                          top=_get(r, "top", int, where + "mlp.router."),
                          shared_ff=None if shared is None else _get(shared, "ff", int, where + "mlp.shared."))
            else:
                raise ConfigError(f"config key '{where}mlp.kind' must be 'dense' or 'moe', got {kind!r}")
        m, w = d.get("mixer"), where + "mixer."
        if not isinstance(m, dict):
            raise ConfigError(f"config key '{where}mixer' is required")
        heads, dim = _get(m, "heads", int, w), _get(m, "dim", int, w)
        if typ == "wkv":
            return cls(type=typ, heads=heads, dim=dim, decay_rank=_get(m, "decay_rank", int, w, None), **kw)
        rot, mask = m.get("rot"), m.get("mask")
        rot_dim = _get(m, "rot_dim", int, w)
        return cls(type=typ, heads=heads, dim=dim, rot_dim=rot_dim, vdim=_get(m, "vdim", int, w, dim),
                   q_rank=_get(m, "q_rank", int, w), kv_rank=_get(m, "kv_rank", int, w),
                   scale=_get(m, "scale", float, w),
                   rot_dims=_get(rot, "dims", int, w + "rot.") if rot else 0,
                   rot_base=_get(rot, "base", float, w + "rot.") if rot else 10000.0,
                   window=_get(mask, "size", int, w + "mask.") if mask else None,
                   kv_from=_get(m, "kv_from", int, w, None), **kw)

    def to_dict(self) -> dict:
        if self.type == "wkv":
            m = {"heads": self.heads, "dim": self.dim}
            if self.decay_rank is not None:
                m["decay_rank"] = self.decay_rank
        else:
            m = {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim,
                 "q_rank": self.q_rank, "kv_rank": self.kv_rank, "scale": self.scale}
            if self.rot_dims:
                m["rot"] = {"base": self.rot_base, "dims": self.rot_dims}
            if self.window is not None:
                m["mask"] = {"size": self.window}
            if self.kv_from is not None:
                m["kv_from"] = self.kv_from
        if self.mlp is None:
            mlp = None
        elif self.mlp == "dense":
            mlp = {"kind": "dense", "ff": self.ff}
        else:
            mlp = {"kind": "moe", "router": {"experts": self.experts, "top": self.top}, "expert": {"ff": self.ff}}
            if self.shared_ff is not None:
                mlp["shared"] = {"ff": self.shared_ff}
        return {"type": self.type, "mixer": m, "mlp": mlp}


@dataclass(frozen=True)
class KunitarConfig:
    vocab: int
    width: int
    layers: Tuple[KunitarLayer, ...]
    eps: float
    embed_scale: float = 1.0
    side_dim: Optional[int] = None
    stop_ids: Tuple[int, ...] = field(default_factory=tuple)
    torch_dtype: Optional[str] = None
    tie_embeddings: Optional[bool] = True       # the embedding table is the output matrix
    architecture: str = "Kunitar"

    def __post_init__(self):
        if self.vocab <= 0 or self.width <= 0 or not self.layers:
            raise ConfigError("vocab, width and the number of layers must be positive")
        if self.side_dim is not None and self.side_dim <= 0:
            raise ConfigError(f"token_side.dim must be positive, got {self.side_dim}")
        for i, l in enumerate(self.layers):
            if l.heads <= 0 or l.dim <= 0:
                raise ConfigError(f"layers[{i}]: heads {l.heads} of {l.dim}")
            if l.mlp == "moe" and not 1 <= l.top <= l.experts:
                raise ConfigError(f"layers[{i}]: top {l.top} of {l.experts} experts")
            if l.type != "latent_attention":
                continue
            if l.rot_dims % 2 or l.rot_dims > l.rot_dim:
                raise ConfigError(f"layers[{i}]: rot.dims {l.rot_dims} must be even and at most rot_dim {l.rot_dim}")
            if l.q_rank <= 0 or l.kv_rank <= 0 or l.vdim <= 0 or l.rot_dim < 0:
                raise ConfigError(f"layers[{i}]: q_rank {l.q_rank}, kv_rank {l.kv_rank}, vdim {l.vdim}")
            if l.window is not None and l.window < 1:
                raise ConfigError(f"layers[{i}]: mask.size must be at least 1, got {l.window}")
            if l.kv_from is not None:
                j = l.kv_from
                if not 0 <= j < i or self.layers[j].type != "latent_attention" or self.layers[j].kv_from is not None:
                    raise ConfigError(f"layers[{i}]: kv_from {j} must name an earlier latent_attention layer "
                                      f"that caches rows of its own")
                o = self.layers[j]
                if (o.kv_rank, o.rot_dim, o.rot_dims, o.rot_base) != (l.kv_rank, l.rot_dim, l.rot_dims, l.rot_base):
                    raise ConfigError(f"layers[{i}]: kv_rank, rot_dim and rot must equal those of layer {j}, "
                                      f"whose rows it reads")

    # ------------------------------------------------------------- config.json
    @classmethod
    def from_dict(cls, d: dict) -> "KunitarConfig":
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config key 'layers' must be a list with at least one layer")
        eos = d.get("eos_token_id")
        stops = () if eos is None else (eos,) if isinstance(eos, int) else tuple(eos)
        dt = d.get("torch_dtype", d.get("dtype"))
        side = d.get("token_side")
        return cls(vocab=_get(d, "vocab", int, ""), width=_get(d, "width", int, ""),
                   layers=tuple(KunitarLayer.from_dict(l, i) for i, l in enumerate(layers)),
                   eps=_get(d.get("norm"), "eps", float, "norm."),
                   embed_scale=_get(d.get("embedding"), "scale", float, "embedding.", 1.0),
                   side_dim=None if side is None else _get(side, "dim", int, "token_side."),
                   stop_ids=stops, torch_dtype=dt[6:] if isinstance(dt, str) and dt.startswith("torch.") else dt)

    def to_dict(self) -> dict:
        d = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
             "norm": {"eps": self.eps}, "embedding": {"scale": self.embed_scale},
             "layers": [l.to_dict() for l in self.layers]}
        if self.side_dim is not None:
            d["token_side"] = {"dim": self.side_dim}
        if self.torch_dtype is not None:
            d["torch_dtype"] = self.torch_dtype
        if self.stop_ids:
            d["eos_token_id"] = list(self.stop_ids)
        return d

    def complete_from_file(self, file, name_of=lambda i: f"l{i}.mix.w1") -> "KunitarConfig":
        """Sizes that only a tensor's shape gives: the rank of each wkv layer's decay input."""
        layers = list(self.layers)
        for i, l in enumerate(layers):
            if l.type == "wkv" and name_of(i) in file:
                layers[i] = dataclasses.replace(l, decay_rank=int(file.shape(name_of(i))[0]))
        return dataclasses.replace(self, layers=tuple(layers))

    def default_engine_dtype(self) -> str:
        return "float32" if self.torch_dtype == "float32" else "bfloat16"

    def with_layers(self, n: int) -> "KunitarConfig":
        """The first n layers (a layer that reads the rows of a dropped layer cannot stay)."""
        return dataclasses.replace(self, layers=self.layers[:int(n)])

    def cache_window(self, i: int) -> Optional[int]:
        """The window that the rows cached by layer i are kept for: the widest among the layer
        itself and the layers that read its rows; None when one of them reads everything."""
        users = [self.layers[i]] + [l for l in self.layers if l.kv_from == i]
        if any(l.window is None for l in users):
            return None
        return max(l.window for l in users)

    # ------------------------------------------------------------ model layout
    def model_spec(self) -> ModelSpec:
        d = self.width
        norm = NormSpec(size=d, eps=self.eps)
        blocks, schedule = [], []
        for i, l in enumerate(self.layers):
            if l.type == "latent_attention":
                owner = i if l.kv_from is None else l.kv_from
                mixer = LatentAttentionSpec(
                    hidden=d, num_heads=l.heads, nope_dim=l.dim, rope_dim=l.rot_dim, value_dim=l.vdim,
                    q_rank=l.q_rank, kv_rank=l.kv_rank, scale=l.scale, eps=self.eps, rot_dims=l.rot_dims,
                    rot_base=l.rot_base, window=l.window, cache_window=self.cache_window(owner), gated=True,
                    own_kv=l.kv_from is None)
            else:
                if l.decay_rank is None:
                    raise ConfigError(f"layers[{i}]: the rank of the decay input is not known: load the "
                                      f"model from its folder, or give mixer.decay_rank")
                mixer = BonusRecurrenceSpec(hidden=d, num_heads=l.heads, head_dim=l.dim,
                                            decay_rank=l.decay_rank, eps=self.eps)
            if l.mlp is None:
                ffn = None
            elif l.mlp == "dense":
                ffn = MLPSpec(hidden=d, intermediate=l.ff, activation=DENSE_ACTIVATION)
            else:
                ffn = RoutedMLPSpec(hidden=d, experts=l.experts, top=l.top, intermediate=l.ff,
                                    activation=EXPERT_ACTIVATION, score="sigmoid", renormalize=False,
                                    weight_on="input", shared_intermediate=l.shared_ff, shared_gate=True)
            side = None if self.side_dim is None else \
                TokenSideSpec(hidden=d, dim=self.side_dim, offset=i * self.side_dim, eps=self.eps)
            blocks.append(SandwichBlockSpec(norm1=norm, mixer=mixer, norm1b=norm,
                                            norm2=norm if ffn else None, ffn=ffn,
                                            norm2b=norm if ffn else None, side=side, hidden=d,
                                            layer_scale=True))
            schedule.append(RunSpec(block=i, cache_of=l.kv_from))
        after = [EmbedScaleSpec(scale=self.embed_scale)] if self.embed_scale != 1.0 else []
        if self.side_dim is not None:
            after.append(TokenSideTableSpec(vocab=self.vocab, width=self.side_dim * len(self.layers)))
        spec = ModelSpec(
            vocab=self.vocab, hidden=d, blocks=tuple(blocks), schedule=tuple(schedule), final_norm=norm,
            tie_embeddings=True, max_position=None, stop_ids=self.stop_ids,
            after_embed=None if not after else after[0] if len(after) == 1 else ChainSpec(parts=tuple(after)))
        spec.validate()
        return spec
