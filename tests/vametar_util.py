"""Tiny Vametar configurations and helpers shared by the Vametar tests. Every size differs
between the configurations, few are powers of two, and the values that are easy to confuse
(query heads and kv heads, key and value widths, heads * value width and the model's width,
rotated coordinates and the head's width) are all different from one another."""
import functools
import tempfile

import numpy as np

import plain_vametar as P


def _att(heads, kv, dim, vdim, scale, rot=None, v_mix=False, ff=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "scale": scale, "v_mix": v_mix}
    if kv is not None:
        m["kv_heads"] = kv
    if rot is not None:
        m["rot"] = {"base": rot[0], "dims": rot[1]}
    return {"type": "attention", "mixer": m, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def _gla(heads, dim, vdim, tau, rank, ff=None):
    return {"type": "gla", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau, "rank": rank},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def _rec(width, blocks, conv, ff=None):
    return {"type": "rglru", "mixer": {"width": width, "blocks": blocks, "conv": conv},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


# attention first (so the values' source is the first layer), three layers that mix values,
# one attention layer without mixing, kv heads absent, no rotation in one layer
CFG_A = {
    "architecture": "Vametar", "vocab": 331, "width": 96, "norm": {"eps": 1e-5},
    "residual_mult": 0.5, "logit_scale": 1.5,
    "embedding": {"bigram": {"buckets": 97, "mul_prev": 13, "mul_cur": 5}},
    "layers": [
        _att(6, 3, 40, 24, 0.2, rot=(1000.0, 16), v_mix=True, ff=136),
        _gla(3, 20, 28, 8.0, 5),
        _rec(144, 3, 4, ff=72),
        _att(6, 3, 40, 24, 0.15, rot=(1000.0, 40), v_mix=True),
        _att(4, None, 24, 8, 0.3),
        _att(3, 1, 16, 72, 0.25, rot=(77.0, 8), v_mix=True, ff=40),
        _gla(2, 36, 12, 3.0, 9, ff=64),
    ],
}
# the corners: one block and one tap (no convolution memory at all), one head, a value width
# above the key width, multiplier and scale equal to one, a recurrence first and last
CFG_B = {
    "architecture": "Vametar", "vocab": 50, "width": 64, "norm": {"eps": 1e-6},
    "residual_mult": 1.0, "logit_scale": 1.0,
    "embedding": {"bigram": {"buckets": 7, "mul_prev": 3, "mul_cur": 1}},
    "layers": [
        _rec(48, 1, 1),
        _gla(1, 64, 16, 1.0, 2),
        _att(2, 2, 32, 80, 0.18, rot=(10000.0, 32), ff=100),
        _rec(80, 5, 2, ff=32),
    ],
}
# wide enough that products of 17 to 64 rows are cut along k into planes, and heads of 128
CFG_C = {
    "architecture": "Vametar", "vocab": 1200, "width": 1024, "norm": {"eps": 1e-5},
    "residual_mult": 0.8, "logit_scale": 0.7,
    "embedding": {"bigram": {"buckets": 509, "mul_prev": 101, "mul_cur": 3}},
    "layers": [
        _gla(4, 128, 64, 16.0, 16, ff=1536),
        _att(8, 2, 128, 64, 0.09, rot=(50000.0, 64), v_mix=True),
        _rec(1280, 4, 3),
        _att(8, 2, 128, 64, 0.09, rot=(50000.0, 64), v_mix=True, ff=1024),
    ],
}
# a width that is no multiple of four (rows of the matrices start off 16-byte boundaries), key
# widths the matrix-core kernels take with values as wide as the keys, narrower, and wider, and
# a head of 160 with six query heads per kv head
CFG_D = {
    "architecture": "Vametar", "vocab": 77, "width": 90, "norm": {"eps": 1e-5},
    "residual_mult": 1.3, "logit_scale": 0.5,
    "embedding": {"bigram": {"buckets": 3, "mul_prev": 1, "mul_cur": 2}},
    "layers": [
        _att(4, 1, 64, 64, 0.12, rot=(10000.0, 32), ff=50),
        _att(2, 2, 32, 16, 0.2, rot=(300.0, 32), v_mix=True),
        _gla(2, 24, 40, 2.0, 3),
        _att(6, 1, 160, 32, 0.08, rot=(10000.0, 160), v_mix=True, ff=33),
        _att(2, 2, 32, 48, 0.2),
        _rec(66, 3, 3),
    ],
}
CONFIGS = {"A": (CFG_A, 11), "B": (CFG_B, 12), "C": (CFG_C, 13), "D": (CFG_D, 14)}
STORAGE = {"float32": "F32", "bfloat16": "BF16"}
# largest allowed rms(engine - plain) / rms(plain) over a row of logits
TOL = {"float32": 2e-4, "bfloat16": 5e-2}

_keep = []


def _sharp(w):
    """Peaked attention: q and k are normed, so the gains of their norms set how sharp the
    softmax is. A fault in any single key then moves the logits visibly."""
    for n in w:
        if n.endswith("q.norm"):
            w[n] = w[n] * 5.0


def _slow_decay(w):
    """Recurrent state that forgets slowly, so that the first tokens still count at the end."""
    for n in w:
        if n.endswith("mix.lam"):
            w[n] = w[n] - 6.0
        if n.endswith("mix.a2.b"):
            w[n] = w[n] + 6.0


EDITS = {None: None, "sharp": _sharp, "slow": _slow_decay}


@functools.lru_cache(maxsize=None)
def folder(name, dtype, edit=None):
    cfg, seed = CONFIGS[name]
    d = tempfile.TemporaryDirectory(prefix=f"vm_{name}_{dtype}_")
    _keep.append(d)
    P.make_model_folder(d.name, cfg, seed, storage=STORAGE[dtype], edit=EDITS[edit])
    return d.name


@functools.lru_cache(maxsize=None)
def plain(name, dtype, edit=None):
    return P.PlainVametar(folder(name, dtype, edit))


@functools.lru_cache(maxsize=None)
def engine(name, dtype, edit=None):
    import transformer_amd as ta
    return ta.load_model(folder(name, dtype, edit), dtype, "cuda:0")


def tokens(name, n, seed):
    cfg, _ = CONFIGS[name]
    return [int(t) for t in np.random.default_rng(seed).integers(0, cfg["vocab"], n)]


@functools.lru_cache(maxsize=None)
def plain_logits(name, dtype, edit, toks):
    return plain(name, dtype, edit).forward(list(toks))


def row_error(got, want):
    """rms of the difference (mean taken off) over rms of the expected row, per row."""
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    d = got - want
    d = d - d.mean(axis=-1, keepdims=True)
    return np.sqrt((d ** 2).mean(axis=-1)) / np.sqrt((want ** 2).mean(axis=-1))


def run_cuts(model, cache, slot, toks, cuts):
    """Feeds ``toks`` into ``slot`` in portions of the given sizes (the rest one by one) and
    returns the logits of every position, [len(toks), vocab]."""
    from transformer_amd import Entry
    out, at = [], 0
    sizes = list(cuts)
    while at < len(toks):
        n = sizes.pop(0) if sizes else 1
        n = min(n, len(toks) - at)
        lg = model.step(cache, [Entry(slot, toks[at:at + n], list(range(n)))])
        out.append(lg.detach().cpu().numpy().copy())
        at += n
    return np.concatenate(out, 0)
