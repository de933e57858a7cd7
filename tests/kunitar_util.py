"""Tiny Kunitar configurations and helpers shared by the Kunitar tests. Sizes differ between the
configurations and from one another inside each (heads of the two mixers, unrotated, rotated
and value widths, the two latents' ranks, the windows of a layer and of the layer whose rows
it reads), few are powers of two, and the corners (one head, one expert, as many chosen as
there are, no window, no feed-forward, no token input, scale 1) each appear somewhere."""
import functools
import tempfile

import numpy as np

import plain_kunitar as P


def _lat(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, base, window=None, kv_from=None, mlp=None, dims=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
         "scale": scale, "rot": {"base": base, "dims": rot_dim if dims is None else dims}}
    if window is not None:
        m["mask"] = {"size": window}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def _wkv(heads, dim, rank, mlp=None):
    return {"type": "wkv", "mixer": {"heads": heads, "dim": dim, "decay_rank": rank}, "mlp": mlp}


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _moe(experts, top, ff, shared=None):
    m = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if shared is not None:
        m["shared"] = {"ff": shared}
    return m


# attention first; a layer that reads rows cached two layers before it through a WIDER window
# than the layer that cached them; a second source without a window and its reader with one;
# two and three chosen experts, all of them chosen, no shared expert, no feed-forward
CFG_A = {
    "architecture": "Kunitar", "vocab": 211, "width": 72, "norm": {"eps": 1e-5},
    "embedding": {"scale": 2.5}, "token_side": {"dim": 12},
    "layers": [
        _lat(3, 20, 8, 28, 40, 48, 0.2, 1000.0, window=33, mlp=_moe(5, 2, 24, shared=40)),
        _wkv(3, 24, 6, mlp=_dense(100)),
        _lat(2, 12, 8, 36, 24, 48, 0.25, 1000.0, window=70, kv_from=0),
        _wkv(2, 20, 3, mlp=_moe(3, 3, 16)),
        _lat(4, 10, 6, 14, 30, 26, 0.3, 77.0, mlp=_moe(7, 1, 20, shared=12)),
        _lat(1, 32, 6, 9, 17, 26, 0.2, 77.0, window=20, kv_from=4, mlp=_dense(50)),
    ],
}
# the corners: one head everywhere, one expert, no token input, embedding scale one, a window
# of one token (a token sees itself only), a recurrence first and last
CFG_B = {
    "architecture": "Kunitar", "vocab": 50, "width": 64, "norm": {"eps": 1e-6},
    "embedding": {"scale": 1.0},
    "layers": [
        _wkv(1, 64, 2),
        _lat(1, 16, 16, 16, 16, 16, 0.18, 10000.0, window=1, mlp=_moe(1, 1, 32, shared=8)),
        _lat(2, 8, 4, 40, 12, 20, 0.4, 300.0, window=64, mlp=_dense(32)),
        _wkv(4, 8, 5, mlp=_moe(4, 2, 8)),
    ],
}
# wide enough for the matrix cores' products and for partial planes; windows over page borders
CFG_C = {
    "architecture": "Kunitar", "vocab": 1200, "width": 1024, "norm": {"eps": 1e-5},
    "embedding": {"scale": 1.5}, "token_side": {"dim": 32},
    "layers": [
        _wkv(16, 64, 16, mlp=_moe(8, 2, 256, shared=512)),
        _lat(8, 64, 32, 64, 192, 128, 0.1, 50000.0, window=150, mlp=_dense(1536)),
        _lat(8, 64, 32, 96, 160, 128, 0.1, 50000.0, window=100, kv_from=1, mlp=_moe(6, 3, 128, shared=256)),
    ],
}
# a width that is no multiple of four, odd sizes everywhere, the rotation on part of the rotated part
CFG_D = {
    "architecture": "Kunitar", "vocab": 77, "width": 90, "norm": {"eps": 1e-5},
    "embedding": {"scale": 0.5}, "token_side": {"dim": 5},
    "layers": [
        _lat(5, 7, 6, 11, 13, 19, 0.3, 100.0, window=9, dims=4, mlp=_moe(9, 4, 10, shared=3)),
        _wkv(3, 14, 1, mlp=_dense(33)),
        _lat(2, 33, 2, 5, 21, 19, 0.2, 100.0, window=130, kv_from=0, dims=2),
    ],
}
# kv_from needs equal rot.dims: D's reader has rot_dim 2 where its source has 6, so give it the source's
CFG_D["layers"][2] = _lat(2, 33, 6, 5, 21, 19, 0.2, 100.0, window=130, kv_from=0, dims=4)
CONFIGS = {"A": (CFG_A, 21), "B": (CFG_B, 22), "C": (CFG_C, 23), "D": (CFG_D, 24)}
STORAGE = {"float32": "F32", "bfloat16": "BF16"}
# largest allowed rms(engine - plain) / rms(plain) over a row of logits
TOL = {"float32": 2e-4, "bfloat16": 1e-1}

_keep = []


def _sharp(w):
    """Peaked attention: larger queries make one key stand out, so a fault in any single key
    (a window that is one token off, a key of the wrong position) moves the logits visibly."""
    for n in w:
        if n.endswith("mix.uq"):
            w[n] = w[n] * 6.0


def _slow_decay(w):
    """Recurrent state that forgets slowly, so that the first tokens still count at the end."""
    for n in w:
        if n.endswith("mix.w0"):
            w[n] = w[n] - 5.0


EDITS = {None: None, "sharp": _sharp, "slow": _slow_decay}


@functools.lru_cache(maxsize=None)
def folder(name, dtype, edit=None):
    cfg, seed = CONFIGS[name]
    d = tempfile.TemporaryDirectory(prefix=f"ku_{name}_{dtype}_")
    _keep.append(d)
    P.make_model_folder(d.name, cfg, seed, storage=STORAGE[dtype], edit=EDITS[edit])
    return d.name


@functools.lru_cache(maxsize=None)
def plain(name, dtype, edit=None):
    return P.PlainKunitar(folder(name, dtype, edit))


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


class Routes:
    """Collects the experts that the engine's routed feed-forwards choose, step by step:
    ``with Routes(model) as r`` ... ``r.steps`` is a list of {layer: [tokens of the step, top]}.
    A bfloat16 engine decides a close call between two experts differently from the float64
    plain model now and then; the plain model is then told the engine's choice, checks that it
    was a close call indeed, and follows it (``plain_kunitar.moe``). Steps run eagerly meanwhile."""

    def __init__(self, model):
        self.model, self.steps = model, []

    def __enter__(self):
        self.steps.append({})
        self.model.dump = self._take
        return self

    def __exit__(self, *exc):
        self.model.dump = None
        return False

    def _take(self, name, t):
        if name.endswith(".experts"):
            self.steps[-1][int(name.split(".")[1])] = t.detach().cpu().numpy().copy()

    def next_step(self):
        self.steps.append({})

    def of_rows(self, rows_of_step):
        """{layer: [T, top]} of one sequence: rows_of_step[i] = slice of its rows in step i (or None)."""
        out = {}
        for step, rows in zip(self.steps, rows_of_step):
            if rows is None:
                continue
            for layer, chosen in step.items():
                out.setdefault(layer, []).append(chosen[rows])
        return {layer: np.concatenate(parts) for layer, parts in out.items()}


def run_cuts(model, cache, slot, toks, cuts, routes=False):
    """Feeds ``toks`` into ``slot`` in portions of the given sizes (the rest one by one) and
    returns the logits of every position, [len(toks), vocab]; with ``routes`` also the experts
    the engine chose, {layer: [len(toks), top]}."""
    from transformer_amd import Entry
    out, at = [], 0
    sizes = list(cuts)
    rec = Routes(model) if routes else None
    if rec is not None:
        rec.__enter__()
    try:
        while at < len(toks):
            n = sizes.pop(0) if sizes else 1
            n = min(n, len(toks) - at)
            lg = model.step(cache, [Entry(slot, toks[at:at + n], list(range(n)))])
            out.append(lg.detach().cpu().numpy().copy())
            at += n
            if rec is not None:
                rec.next_step()
    finally:
        if rec is not None:
            rec.__exit__()
    logits = np.concatenate(out, 0)
    if rec is None:
        return logits
    return logits, rec.of_rows([slice(None)] * len(rec.steps))


def check_against_plain(name, dtype, edit, toks, got, routes=None, what=""):
    """The engine's logits of a whole sequence against the plain model's. float32: the plain
    model's own routing, every row. bfloat16: the plain model follows the engine's choice of
    experts where that was a close call (and fails where it was not)."""
    toks = list(toks)[:len(got)]
    if dtype == "float32" or not routes:
        want = plain_logits(name, dtype, edit, tuple(toks))
    else:
        want = plain(name, dtype, edit).forward(list(toks), routes=routes)
    err = row_error(got, want[:len(got)]).max()
    assert err < TOL[dtype], f"{what}: {err}"
