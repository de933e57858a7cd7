"""The Kunitar decoder as a registry entry: its configuration, its blocks and where its
parameters are found in a safetensors file.

File names: ``embed`` (also the output matrix), ``side.embed``, ``final.norm``, and per layer i
``l<i>.norm1`` / ``.norm1b`` / ``.norm2`` / ``.norm2b``, ``l<i>.ls1`` / ``.ls2``, ``l<i>.mix.*``,
``l<i>.mlp.*`` and ``l<i>.side.{gate, proj, norm}``. Projections that read the same rows are
joined by rows into one matrix: the query latent, the key/value latent and the heads' gates of
latent attention; r, k, v, g of the recurrence (kept as four blocks of one tensor, each read
by its own shifted rows); the router and the shared expert's gate; all experts' up matrices,
and all their down matrices.
"""
from __future__ import annotations

from typing import Dict

from ..config.kunitar import KunitarConfig
from ..config.registry import Architecture, register_architecture
from ..config.spec import ConfigError
from ..weights.loader import Piece, Source


def _one(name, shape):
    return Source(options=((Piece(name, tuple(shape)),),))


def _join(*pieces):
    return Source(options=(tuple(Piece(n, tuple(s)) for n, s in pieces),))


def kunitar_weight_sources(cfg: KunitarConfig, file_format: str) -> Dict[str, Source]:
    if file_format != "safetensors":
        raise ValueError(f"Kunitar weights come as safetensors, not {file_format!r}")
    d, V = cfg.width, cfg.vocab
    src = {"embed.weight": _one("embed", (V, d)),
           "head.weight": Source(options=(), stand_in="embed.weight"),
           "final_norm.weight": _one("final.norm", (d,))}
    if cfg.side_dim is not None:
        name = "after_embed.1.table" if cfg.embed_scale != 1.0 else "after_embed.table"
        src[name] = _one("side.embed", (V, cfg.side_dim * len(cfg.layers)))
    for i, l in enumerate(cfg.layers):
        f, p = f"l{i}.", f"blocks.{i}."
        for n in ("norm1", "norm1b"):
            src[p + n + ".weight"] = _one(f + n, (d,))
        src[p + "ls1"] = _one(f + "ls1", (d,))
        m, q = f + "mix.", p + "mixer."
        if l.type == "latent_attention":
            H = l.heads
            pieces = [(m + "dq", (l.q_rank, d))]
            if l.kv_from is None:
                pieces.append((m + "dkv", (l.kv_rank + l.rot_dim, d)))
                src[q + "kv_norm.weight"] = _one(m + "dkv.norm", (l.kv_rank,))
            pieces.append((m + "g", (H, d)))
            src[q + "in.weight"] = _join(*pieces)
            src[q + "q_norm.weight"] = _one(m + "dq.norm", (l.q_rank,))
            src[q + "uq.weight"] = _one(m + "uq", (H * (l.dim + l.rot_dim), l.q_rank))
            src[q + "uk.weight"] = _one(m + "uk", (H * l.dim, l.kv_rank))
            src[q + "uv.weight"] = _one(m + "uv", (H * l.vdim, l.kv_rank))
            src[q + "out.weight"] = _one(m + "o", (d, H * l.vdim))
        else:
            n, r = l.heads * l.dim, l.decay_rank
            if r is None:
                raise ConfigError(f"layers[{i}]: the rank of the decay input is not known")
            src[q + "mu"] = _join(*[(m + "mu." + s, (d,)) for s in "rkvgw"])
            src[q + "rkvg.weight"] = _join(*[(m + s, (n, d)) for s in "rkvg"])
            src[q + "w1.weight"], src[q + "w2.weight"] = _one(m + "w1", (r, d)), _one(m + "w2", (n, r))
            src[q + "w0"], src[q + "bonus"] = _one(m + "w0", (n,)), _one(m + "u", (l.heads, l.dim))
            src[q + "norm.weight"] = _one(m + "norm", (n,))
            src[q + "out.weight"] = _one(m + "o", (d, n))
        if l.mlp is not None:
            for nme in ("norm2", "norm2b"):
                src[p + nme + ".weight"] = _one(f + nme, (d,))
            src[p + "ls2"] = _one(f + "ls2", (d,))
            g, q = f + "mlp.", p + "ffn."
            if l.mlp == "dense":
                src[q + "up.weight"], src[q + "down.weight"] = _one(g + "up", (l.ff, d)), _one(g + "down", (d, l.ff))
            else:
                E = l.experts
                router = [(g + "router", (E, d))]
                if l.shared_ff is not None:
                    router.append((g + "shared.sg", (1, d)))
                    src[q + "shared.up.weight"] = _one(g + "shared.up", (l.shared_ff, d))
                    src[q + "shared.down.weight"] = _one(g + "shared.down", (d, l.shared_ff))
                src[q + "router.weight"] = _join(*router)
                src[q + "experts.up.weight"] = _join(*[(f"{g}e{e}.up", (l.ff, d)) for e in range(E)])
                src[q + "experts.down.weight"] = _join(*[(f"{g}e{e}.down", (d, l.ff)) for e in range(E)])
        if cfg.side_dim is not None:
            s, q = f + "side.", p + "side."
            src[q + "gate.weight"] = _one(s + "gate", (cfg.side_dim, d))
            src[q + "proj.weight"] = _one(s + "proj", (d, cfg.side_dim))
            src[q + "norm.weight"] = _one(s + "norm", (d,))
    return src


def _no_gguf(meta, rows=None):
    raise ConfigError("Kunitar models are read from a folder with config.json and model.safetensors")


KUNITAR = Architecture(
    name="Kunitar",
    config_from_dict=KunitarConfig.from_dict,
    config_from_gguf=_no_gguf,
    model_spec=lambda cfg: cfg.model_spec(),
    weight_sources=kunitar_weight_sources,
    complete_config=lambda cfg, file: cfg.complete_from_file(file),
)

register_architecture(KUNITAR, "kunitar")
