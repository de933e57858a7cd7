"""Typed configuration of the Vametar decoder, read from its own config.json.

A Vametar model is a list of layers, each with one of three mixers (softmax attention with
normed q/k and narrow values, a gated diagonal recurrence, gated linear attention) and an
optional dense gated feed-forward; every sublayer is gated and scaled by ``residual_mult``, the
mixers read token-shifted rows, norms have one gain, the embedding adds a hashed row for the
pair (previous token, token) and the logits are scaled.

Keys: ``architecture``, ``vocab``, ``width``, ``norm.eps``, ``residual_mult``, ``logit_scale``,
``embedding.bigram.{buckets, mul_prev, mul_cur}``, ``layers[i].{type, mixer, mlp}``. A layer's
``mixer`` holds, by type: attention: heads, kv_heads, dim, vdim, scale, rot.{base, dims},
v_mix; rglru: width, blocks, conv; gla: heads, dim, vdim, tau (the width of its low-rank decay
input is a tensor's shape: ``complete_from_file`` reads it; a configuration made by hand may
give it as ``rank``). ``mlp``: null or {kind: "dense", ff}.
"""
from __future__ import annotations

import dataclasses
import math
from dataclasses import dataclass, field
from typing import Optional, Tuple

from .spec import (ConfigError, DiagonalRecurrenceSpec, GLUSpec, GatedBlockSpec,
                   GatedLinearAttentionSpec, LogitScaleSpec, ModelSpec, NormedAttentionSpec,
                   PairHashEmbedSpec, RunSpec, ScalarNormSpec)

LAYER_TYPES = ("attention", "rglru", "gla")
RGLRU_DECAY_SCALE = 8.0          # a = exp(-8 r softplus(lam)): fixed by the design


def _get(d, key, typ, where, default=dataclasses.MISSING):
    if not isinstance(d, dict) or key not in d or d[key] is None:
        if default is not dataclasses.MISSING:
            return default
        raise ConfigError(f"config key '{where}{key}' is required")
    v = d[key]
    if typ is int:
        if isinstance(v, bool) or not isinstance(v, int):
            raise ConfigError(f"config key '{where}{key}' must be an integer, got {v!r}")
    elif typ is float:
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"config key '{where}{key}' must be a number, got {v!r}")
        v = float(v)
    elif typ is bool:
        if not isinstance(v, bool):
            raise ConfigError(f"config key '{where}{key}' must be true or false, got {v!r}")
    return v


@dataclass(frozen=True)
class VametarLayer:
    type: str
    ff: Optional[int] = None            # None: no feed-forward
    # attention and gla
    heads: int = 0
    kv_heads: int = 0
    dim: int = 0
    vdim: int = 0
    # attention
    scale: float = 0.0
    rot_dims: int = 0
    rot_base: float = 10000.0
    v_mix: bool = False
    # gla
    tau: float = 1.0
    rank: Optional[int] = None          # None until a weight file has said it
    # rglru
    width: int = 0
    blocks: int = 0
    conv: int = 0

    @classmethod
    def from_dict(cls, d: dict, i: int) -> "VametarLayer":
        where = f"layers[{i}]."
        typ = d.get("type") if isinstance(d, dict) else None
        if typ not in LAYER_TYPES:
            raise ConfigError(f"config key '{where}type' must be one of {LAYER_TYPES}, got {typ!r}")
        mlp = d.get("mlp")
        ff = None
        if mlp is not None:
            kind = mlp.get("kind") if isinstance(mlp, dict) else None
            if kind != "dense":
                raise ConfigError(f"config key '{where}mlp.kind' must be 'dense', got {kind!r}")
            ff = _get(mlp, "ff", int, where + "mlp.")
        m, w = d.get("mixer"), where + "mixer."
        if not isinstance(m, dict):
            raise ConfigError(f"config key '{where}mixer' is required")
        if typ == "attention":
            heads = _get(m, "heads", int, w)
            rot = m.get("rot")
            dim = _get(m, "dim", int, w)
            return cls(type=typ, ff=ff, heads=heads, kv_heads=_get(m, "kv_heads", int, w, heads), dim=dim,
                       vdim=_get(m, "vdim", int, w, dim), scale=_get(m, "scale", float, w),
                       rot_dims=_get(rot, "dims", int, w + "rot.") if rot else 0,
                       rot_base=_get(rot, "base", float, w + "rot.") if rot else 10000.0,
                       v_mix=_get(m, "v_mix", bool, w, False))
        if typ == "gla":
            dim = _get(m, "dim", int, w)
            return cls(type=typ, ff=ff, heads=_get(m, "heads", int, w), dim=dim,
                       vdim=_get(m, "vdim", int, w, dim), tau=_get(m, "tau", float, w),
                       rank=_get(m, "rank", int, w, None))
        return cls(type=typ, ff=ff, width=_get(m, "width", int, w), blocks=_get(m, "blocks", int, w),
                   conv=_get(m, "conv", int, w))

    def to_dict(self) -> dict:
        if self.type == "attention":
            m = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
                 "scale": self.scale, "v_mix": self.v_mix}
            if self.rot_dims:
                m["rot"] = {"base": self.rot_base, "dims": self.rot_dims}
        elif self.type == "gla":
            m = {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "tau": self.tau}
            if self.rank is not None:
                m["rank"] = self.rank
        else:
            m = {"width": self.width, "blocks": self.blocks, "conv": self.conv}
        return {"type": self.type, "mixer": m,
                "mlp": None if self.ff is None else {"kind": "dense", "ff": self.ff}}


@dataclass(frozen=True)
class VametarConfig:
    vocab: int
    width: int
    layers: Tuple[VametarLayer, ...]
    eps: float
    residual_mult: float = 1.0
    logit_scale: float = 1.0
    buckets: int = 1
    mul_prev: int = 1
    mul_cur: int = 1
    stop_ids: Tuple[int, ...] = field(default_factory=tuple)
    torch_dtype: Optional[str] = None
    tie_embeddings: Optional[bool] = False      # the output matrix is a tensor of its own
    architecture: str = "Vametar"

    def __post_init__(self):
        if self.vocab <= 0 or self.width <= 0 or not self.layers:
            raise ConfigError("vocab, width and the number of layers must be positive")
        if self.buckets <= 0 or self.mul_prev < 0 or self.mul_cur < 0:
            raise ConfigError("embedding.bigram: buckets must be positive, multipliers not negative")
        for i, l in enumerate(self.layers):
            if l.type == "attention":
                if l.heads <= 0 or l.kv_heads <= 0 or l.heads % l.kv_heads:
                    raise ConfigError(f"layers[{i}]: {l.heads} heads do not divide into {l.kv_heads} kv heads")
                if l.rot_dims % 2 or l.rot_dims > l.dim:
                    raise ConfigError(f"layers[{i}]: rot.dims {l.rot_dims} must be even and at most dim {l.dim}")
            if l.type == "rglru" and (l.blocks <= 0 or l.width % l.blocks or l.conv < 1):
                raise ConfigError(f"layers[{i}]: width {l.width}, blocks {l.blocks}, conv {l.conv}")

    # ------------------------------------------------------------- config.json
    @classmethod
    def from_dict(cls, d: dict) -> "VametarConfig":
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config key 'layers' must be a list with at least one layer")
        bg = (d.get("embedding") or {}).get("bigram")
        if not isinstance(bg, dict):
            raise ConfigError("config key 'embedding.bigram' is required")
        eos = d.get("eos_token_id")
        stops = () if eos is None else (eos,) if isinstance(eos, int) else tuple(eos)
        dt = d.get("torch_dtype", d.get("dtype"))
        return cls(vocab=_get(d, "vocab", int, ""), width=_get(d, "width", int, ""),
                   layers=tuple(VametarLayer.from_dict(l, i) for i, l in enumerate(layers)),
                   eps=_get(d.get("norm"), "eps", float, "norm."),
                   residual_mult=_get(d, "residual_mult", float, "", 1.0),
                   logit_scale=_get(d, "logit_scale", float, "", 1.0),
                   buckets=_get(bg, "buckets", int, "embedding.bigram."),
                   mul_prev=_get(bg, "mul_prev", int, "embedding.bigram."),
                   mul_cur=_get(bg, "mul_cur", int, "embedding.bigram."),
                   stop_ids=stops, torch_dtype=dt[6:] if isinstance(dt, str) and dt.startswith("torch.") else dt)

    def to_dict(self) -> dict:
        d = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
             "norm": {"eps": self.eps}, "residual_mult": self.residual_mult,
             "logit_scale": self.logit_scale,
             "embedding": {"bigram": {"buckets": self.buckets, "mul_prev": self.mul_prev,
                                      "mul_cur": self.mul_cur}},
             "layers": [l.to_dict() for l in self.layers]}
        if self.torch_dtype is not None:
            d["torch_dtype"] = self.torch_dtype
        if self.stop_ids:
            d["eos_token_id"] = list(self.stop_ids)
        return d

    def complete_from_file(self, file, name_of=lambda i: f"l{i}.mix.a1") -> "VametarConfig":
        """Sizes that only a tensor's shape gives: the rank of each gla layer's decay input."""
        layers = list(self.layers)
        for i, l in enumerate(layers):
            if l.type == "gla" and name_of(i) in file:
                layers[i] = dataclasses.replace(l, rank=int(file.shape(name_of(i))[0]))
        return dataclasses.replace(self, layers=tuple(layers))

    def default_engine_dtype(self) -> str:
        return "float32" if self.torch_dtype == "float32" else "bfloat16"

    def with_layers(self, n: int) -> "VametarConfig":
        return dataclasses.replace(self, layers=self.layers[:int(n)])

    # ------------------------------------------------------------ model layout
    def model_spec(self) -> ModelSpec:
        d = self.width
        norm = ScalarNormSpec(size=d, eps=self.eps)
        blocks, seen_source = [], False
        for i, l in enumerate(self.layers):
            if l.type == "attention":
                role = None
                if l.v_mix:
                    role = "mix" if seen_source else "source"
                    seen_source = True
                mixer = NormedAttentionSpec(hidden=d, num_heads=l.heads, num_kv_heads=l.kv_heads,
                                            key_dim=l.dim, value_dim=l.vdim, scale=l.scale, eps=self.eps,
                                            qk_norm=True, rot_dims=l.rot_dims, rot_base=l.rot_base,
                                            value_mix=role)
            elif l.type == "rglru":
                mixer = DiagonalRecurrenceSpec(hidden=d, channels=l.width, blocks=l.blocks, taps=l.conv,
                                               decay_scale=RGLRU_DECAY_SCALE)
            else:
                if l.rank is None:
                    raise ConfigError(f"layers[{i}]: the rank of the decay input is not known: load the "
                                      f"model from its folder, or give mixer.rank")
                mixer = GatedLinearAttentionSpec(hidden=d, num_heads=l.heads, key_dim=l.dim,
                                                 value_dim=l.vdim, rank=l.rank, tau=l.tau, eps=self.eps)
            ffn = None if l.ff is None else GLUSpec(hidden=d, intermediate=l.ff, activation="gelu_tanh")
            blocks.append(GatedBlockSpec(norm1=norm, mixer=mixer, norm2=norm if ffn else None, ffn=ffn,
                                         hidden=d, mult=self.residual_mult, gated=True, token_shift=True))
        spec = ModelSpec(
            vocab=self.vocab, hidden=d, blocks=tuple(blocks),
            schedule=tuple(RunSpec(block=i) for i in range(len(blocks))), final_norm=norm,
            tie_embeddings=False, max_position=None, stop_ids=self.stop_ids,
            after_embed=PairHashEmbedSpec(hidden=d, buckets=self.buckets, mul_prev=self.mul_prev,
                                          mul_cur=self.mul_cur),
            on_logits=LogitScaleSpec(scale=self.logit_scale) if self.logit_scale != 1.0 else None)
        spec.validate()
        return spec
