"""The Vametar decoder as a registry entry: its configuration, its blocks and where its
parameters are found in a safetensors file.

File names: ``embed``, ``bigram``, ``head``, ``final.norm``, and per layer i ``l<i>.norm1``,
``l<i>.norm2``, ``l<i>.shift``, ``l<i>.rg1`` / ``.rg1.b`` / ``.rg2`` / ``.rg2.b`` (the
sublayers' gates), ``l<i>.mix.*`` (the mixer) and ``l<i>.mlp.{gate, up, down}``. Projections
that read the same rows are joined by rows into one matrix: q, k, v of attention; the y and x
branches of the recurrence (and the blocks of its two gates); q, k, v, g and the decay's
low-rank input of gated linear attention; gate and up of the feed-forward.
"""
from __future__ import annotations

from typing import Dict

from ..config.registry import Architecture, register_architecture
from ..config.spec import ConfigError
from ..config.vametar import VametarConfig
from ..weights.loader import Piece, Source


def _one(name, shape):
    return Source(options=((Piece(name, tuple(shape)),),))


def _join(*pieces):
    return Source(options=(tuple(Piece(n, tuple(s)) for n, s in pieces),))


def vametar_weight_sources(cfg: VametarConfig, file_format: str) -> Dict[str, Source]:
    if file_format != "safetensors":
        raise ValueError(f"Vametar weights come as safetensors, not {file_format!r}")
    d, V = cfg.width, cfg.vocab
    src = {"embed.weight": _one("embed", (V, d)), "head.weight": _one("head", (V, d)),
           "final_norm.weight": _one("final.norm", ()),
           "after_embed.table": _one("bigram", (cfg.buckets + 1, d))}
    for i, l in enumerate(cfg.layers):
        f, p = f"l{i}.", f"blocks.{i}."
        src[p + "norm1.weight"] = _one(f + "norm1", ())
        src[p + "shift"] = _one(f + "shift", (d,))
        src[p + "gate1.weight"], src[p + "gate1.bias"] = _one(f + "rg1", (d, d)), _one(f + "rg1.b", (d,))
        m, q = f + "mix.", p + "mixer."
        if l.type == "attention":
            H, G, dk, dv = l.heads, l.kv_heads, l.dim, l.vdim
            src[q + "qkv.weight"] = _join((m + "q", (H * dk, d)), (m + "k", (G * dk, d)), (m + "v", (G * dv, d)))
            src[q + "q_norm.weight"] = _one(m + "q.norm", (H * dk,))
            src[q + "k_norm.weight"] = _one(m + "k.norm", (G * dk,))
            if l.v_mix:
                src[q + "value_mix"] = _one(m + "vmix", ())
            src[q + "out.weight"] = _one(m + "o", (d, H * dv))
        elif l.type == "rglru":
            C, nb = l.width, l.blocks
            bs = C // nb
            src[q + "in.weight"] = _join((m + "y", (C, d)), (m + "x", (C, d)))
            src[q + "in.bias"] = _join((m + "y.b", (C,)), (m + "x.b", (C,)))
            src[q + "conv.weight"], src[q + "conv.bias"] = _one(m + "conv", (C, l.conv)), _one(m + "conv.b", (C,))
            src[q + "gates.weight"] = _join((m + "ra", (nb, bs, bs)), (m + "ri", (nb, bs, bs)))
            src[q + "gates.bias"] = _join((m + "ra.b", (nb, bs)), (m + "ri.b", (nb, bs)))
            src[q + "lam"] = _one(m + "lam", (C,))
            src[q + "out.weight"] = _one(m + "o", (d, C))
        else:
            H, dk, dv, r = l.heads, l.dim, l.vdim, l.rank
            if r is None:
                raise ConfigError(f"layers[{i}]: the rank of the decay input is not known")
            src[q + "in.weight"] = _join((m + "q", (H * dk, d)), (m + "k", (H * dk, d)), (m + "v", (H * dv, d)),
                                         (m + "g", (H * dv, d)), (m + "a1", (r, d)))
            src[q + "decay.weight"], src[q + "decay.bias"] = _one(m + "a2", (H * dk, r)), _one(m + "a2.b", (H * dk,))
            src[q + "norm.weight"] = _one(m + "norm", (dv,))
            src[q + "out.weight"] = _one(m + "o", (d, H * dv))
        if l.ff is not None:
            src[p + "norm2.weight"] = _one(f + "norm2", ())
            src[p + "gate2.weight"], src[p + "gate2.bias"] = _one(f + "rg2", (d, d)), _one(f + "rg2.b", (d,))
            src[p + "ffn.gate_up.weight"] = _join((f + "mlp.gate", (l.ff, d)), (f + "mlp.up", (l.ff, d)))
            src[p + "ffn.down.weight"] = _one(f + "mlp.down", (d, l.ff))
    return src


def _no_gguf(meta, rows=None):
    raise ConfigError("Vametar models are read from a folder with config.json and model.safetensors")


VAMETAR = Architecture(
    name="Vametar",
    config_from_dict=VametarConfig.from_dict,
    config_from_gguf=_no_gguf,
    model_spec=lambda cfg: cfg.model_spec(),
    weight_sources=vametar_weight_sources,
    complete_config=lambda cfg, file: cfg.complete_from_file(file),
)

register_architecture(VAMETAR, "vametar")
