"""Plain, slow Kunitar decoder: the oracle of the Kunitar tests.

Whole sequences, no cache, NumPy float64, one function per mechanism. It shares no code
with ``transformer_amd``: it reads config.json and the safetensors file itself (through the
test-suite's own reader) and states every formula once more.

Notation: T tokens, d the model's width, x the residual stream [T, d]. A weight ``W`` is
stored [out, in] and used as ``h @ W.T``.
"""
from __future__ import annotations

import json
import math
from pathlib import Path

import numpy as np

from plain_llama import read_safetensors, round_bf16  # noqa: F401  (the suite's own file code)
from plain_vametar import write_safetensors  # noqa: F401


# --------------------------------------------------------------------------
# small functions
# --------------------------------------------------------------------------
def sigmoid(z):
    z = np.asarray(z, dtype=np.float64)
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def gelu_tanh(z):
    z = np.asarray(z, dtype=np.float64)
    return 0.5 * z * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (z + 0.044715 * z ** 3)))


_erf = np.vectorize(math.erf, otypes=[np.float64])


def gelu_erf(z):
    z = np.asarray(z, dtype=np.float64)
    return 0.5 * z * (1.0 + _erf(z / np.sqrt(2.0)))


def relu_squared(z):
    return np.maximum(np.asarray(z, dtype=np.float64), 0.0) ** 2


def unit_rms(x, eps):
    x = np.asarray(x, dtype=np.float64)
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def rms_norm(x, weight, eps):
    return unit_rms(x, eps) * weight


# --------------------------------------------------------------------------
# mechanisms
# --------------------------------------------------------------------------
def rotate_pairs(t, positions, base, dims):
    """t: [T, heads, dh]. Coordinates (2i, 2i + 1), i < dims / 2, of every head turn by the
    angle position * base^(-2i/dims); coordinates from ``dims`` on stay."""
    out = np.array(t, dtype=np.float64)
    i = np.arange(dims // 2, dtype=np.float64)
    ang = np.asarray(positions, dtype=np.float64)[:, None] * base ** (-2.0 * i / dims)
    c, s = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    u, v = t[..., 0:dims:2], t[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def latent_kv(h, w, p, m, eps, positions):
    """What a latent-attention layer keeps per token: the normed latent [T, kv_rank] and the
    rotated key part [T, rot_dim] that all heads share."""
    r, dr = m["kv_rank"], m["rot_dim"]
    both = h @ w[p + "dkv"].T
    c = rms_norm(both[:, :r], w[p + "dkv.norm"], eps)
    rot = m["rot"]
    kr = rotate_pairs(both[:, None, r:r + dr], positions, rot["base"], rot["dims"])[:, 0]
    return c, kr


def latent_attention(h, w, p, m, eps, positions, kv):
    """kv = (latent, rotated key part) of this layer or of the layer it borrows from."""
    T = h.shape[0]
    H, dn, dr, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    c, kr = kv
    cq = rms_norm(h @ w[p + "dq"].T, w[p + "dq.norm"], eps)
    q = (cq @ w[p + "uq"].T).reshape(T, H, dn + dr)
    qn = q[..., :dn]
    rot = m["rot"]
    qr = rotate_pairs(q[..., dn:], positions, rot["base"], rot["dims"])
    kn = (c @ w[p + "uk"].T).reshape(T, H, dn)
    v = (c @ w[p + "uv"].T).reshape(T, H, dv)
    gate = sigmoid(h @ w[p + "g"].T)                         # [T, H]
    size = (m.get("mask") or {}).get("size")
    out = np.zeros((T, H, dv))
    for i in range(T):
        lo = 0 if size is None else max(0, i - size + 1)
        for hd in range(H):
            s = (kn[lo:i + 1, hd] @ qn[i, hd] + kr[lo:i + 1] @ qr[i, hd]) * m["scale"]
            e = np.exp(s - s.max())
            out[i, hd] = (e / e.sum()) @ v[lo:i + 1, hd]
    out = out * gate[:, :, None]
    return out.reshape(T, H * dv) @ w[p + "o"].T


def wkv_recurrence(r, k, v, decay, u, state=None):
    """Per head: o_t = (S + diag(u) k_t v_t^T)^T r_t, then S <- diag(decay_t) S + k_t v_t^T.
    r, k, v, decay: [T, H, n]; u: [H, n]. Returns (o [T, H, n], final S [H, n, n])."""
    T, H, n = r.shape
    S = np.zeros((H, n, n)) if state is None else np.array(state, dtype=np.float64)
    o = np.zeros((T, H, n))
    for t in range(T):
        for hd in range(H):
            kv = np.outer(k[t, hd], v[t, hd])
            o[t, hd] = (S[hd] + u[hd][:, None] * kv).T @ r[t, hd]
            S[hd] = decay[t, hd][:, None] * S[hd] + kv
    return o, S


def wkv_mixer(h, w, p, m, eps):
    T, d = h.shape
    H, n = m["heads"], m["dim"]
    prev = np.vstack([np.zeros((1, d)), h[:-1]])

    def mix(s):
        return h + (prev - h) * w[p + "mu." + s]

    r = (mix("r") @ w[p + "r"].T).reshape(T, H, n)
    k = (mix("k") @ w[p + "k"].T).reshape(T, H, n)
    v = (mix("v") @ w[p + "v"].T).reshape(T, H, n)
    gate = silu(mix("g") @ w[p + "g"].T)
    decay = np.exp(-np.exp(np.tanh(mix("w") @ w[p + "w1"].T) @ w[p + "w2"].T + w[p + "w0"]))
    o, _ = wkv_recurrence(r, k, v, decay.reshape(T, H, n), w[p + "u"])
    o = unit_rms(o, eps).reshape(T, H * n) * w[p + "norm"] * gate
    return o @ w[p + "o"].T


def dense_mlp(h, w, p, act=gelu_erf):
    return act(h @ w[p + "up"].T) @ w[p + "down"].T


def route(h, router, top):
    """(chosen experts [T, top], their weights [T, top]): the ``top`` largest sigmoid scores
    of every token, the scores themselves as weights."""
    s = sigmoid(h @ router.T)
    order = np.argsort(-s, axis=-1, kind="stable")[:, :top]
    return order, np.take_along_axis(s, order, axis=-1)


def moe(h, w, p, m, forced=None, slack=0.0):
    """forced [T, top]: experts that another implementation chose. Where they differ from this
    function's own choice they must be as good within ``slack`` (a close call that rounding
    decides); the function then goes on with them, so that one close call does not change
    everything behind it."""
    T = h.shape[0]
    chosen, weight = route(h, w[p + "router"], m["router"]["top"])
    if forced is not None:
        s = sigmoid(h @ w[p + "router"].T)
        forced = np.asarray(forced, dtype=np.int64)
        for t in range(T):
            if set(forced[t]) != set(chosen[t]):
                assert len(set(forced[t])) == len(forced[t]), f"token {t}: an expert chosen twice"
                assert s[t, forced[t]].min() >= weight[t].min() - slack, \
                    f"token {t}: experts {forced[t]} chosen, {chosen[t]} have the largest scores"
        chosen, weight = forced, np.take_along_axis(s, forced, axis=-1)
    out = np.zeros((T, w[p + "e0.down"].shape[0]))
    for t in range(T):
        for e, g in zip(chosen[t], weight[t]):
            out[t] += dense_mlp((g * h[t])[None], w, f"{p}e{int(e)}.", relu_squared)[0]
    if m.get("shared") is not None:
        out += dense_mlp(h, w, p + "shared.", relu_squared) * sigmoid(h @ w[p + "shared.sg"].T)
    return out


def token_side(x, tokens, w, layer, dim, eps):
    """What the layer's token input adds to the stream."""
    e = w["side.embed"][np.asarray(tokens), layer * dim:(layer + 1) * dim]
    y = (gelu_tanh(x @ w[f"l{layer}.side.gate"].T) * e) @ w[f"l{layer}.side.proj"].T
    return unit_rms(y, eps) * w[f"l{layer}.side.norm"]


# --------------------------------------------------------------------------
# the model
# --------------------------------------------------------------------------
class PlainKunitar:
    def __init__(self, folder=None, config=None, weights=None):
        if folder is not None:
            config = json.loads((Path(folder) / "config.json").read_text())
            weights = read_safetensors(Path(folder) / "model.safetensors")
        self.c, self.w = config, weights

    def forward(self, tokens, layers_out=None, routes=None, slack=0.03):
        """Logits [T, vocab] of a whole sequence from position 0. ``layers_out``: a list that
        receives the residual stream after every layer. ``routes``: {layer: experts [T, top]}
        chosen elsewhere (see ``moe``)."""
        c, w = self.c, self.w
        eps = c["norm"]["eps"]
        tokens = np.asarray(tokens, dtype=np.int64)
        positions = np.arange(len(tokens))
        x = w["embed"][tokens] * c["embedding"]["scale"]
        side = (c.get("token_side") or {}).get("dim")
        kept = {}
        for li, layer in enumerate(c["layers"]):
            L, mx = f"l{li}.", layer["mixer"]
            h = rms_norm(x, w[L + "norm1"], eps)
            if layer["type"] == "latent_attention":
                src = mx.get("kv_from")
                if src is None:
                    kept[li] = latent_kv(h, w, L + "mix.", mx, eps, positions)
                    src = li
                out = latent_attention(h, w, L + "mix.", mx, eps, positions, kept[src])
            elif layer["type"] == "wkv":
                out = wkv_mixer(h, w, L + "mix.", mx, eps)
            else:
                raise ValueError(f"layer {li}: unknown type {layer['type']!r}")
            x = x + rms_norm(out, w[L + "norm1b"], eps) * w[L + "ls1"]
            mlp = layer.get("mlp")
            if mlp is not None:
                h = rms_norm(x, w[L + "norm2"], eps)
                if mlp["kind"] == "dense":
                    f = dense_mlp(h, w, L + "mlp.")
                elif mlp["kind"] == "moe":
                    f = moe(h, w, L + "mlp.", mlp, None if routes is None else routes.get(li), slack)
                else:
                    raise ValueError(f"layer {li}: unknown feed-forward {mlp['kind']!r}")
                x = x + rms_norm(f, w[L + "norm2b"], eps) * w[L + "ls2"]
            if side:
                x = x + token_side(x, tokens, w, li, side, eps)
            if layers_out is not None:
                layers_out.append(x.copy())
        return rms_norm(x, w["final.norm"], eps) @ w["embed"].T


# --------------------------------------------------------------------------
# random models for the tests
# --------------------------------------------------------------------------
def tensor_shapes(c):
    """{tensor name: shape} of a configuration, in the file's own names."""
    d, V = c["width"], c["vocab"]
    s = {"embed": (V, d), "final.norm": (d,)}
    side = (c.get("token_side") or {}).get("dim")
    if side:
        s["side.embed"] = (V, side * len(c["layers"]))
    for li, layer in enumerate(c["layers"]):
        L, mx, M = f"l{li}.", layer["mixer"], f"l{li}.mix."
        for n in ("norm1", "norm1b", "ls1"):
            s[L + n] = (d,)
        if layer["type"] == "latent_attention":
            H, dn, dr, dv = mx["heads"], mx["dim"], mx["rot_dim"], mx["vdim"]
            s[M + "dq"], s[M + "dq.norm"] = (mx["q_rank"], d), (mx["q_rank"],)
            s[M + "uq"] = (H * (dn + dr), mx["q_rank"])
            if mx.get("kv_from") is None:
                s[M + "dkv"], s[M + "dkv.norm"] = (mx["kv_rank"] + dr, d), (mx["kv_rank"],)
            s[M + "uk"], s[M + "uv"] = (H * dn, mx["kv_rank"]), (H * dv, mx["kv_rank"])
            s[M + "g"], s[M + "o"] = (H, d), (d, H * dv)
        else:
            H, n, r = mx["heads"], mx["heads"] * mx["dim"], mx.get("decay_rank", 4)
            for nme in "rkvgw":
                s[M + "mu." + nme] = (d,)
            for nme in "rkvg":
                s[M + nme] = (n, d)
            s[M + "w1"], s[M + "w2"], s[M + "w0"] = (r, d), (n, r), (n,)
            s[M + "u"], s[M + "norm"], s[M + "o"] = (H, mx["dim"]), (n,), (d, n)
        mlp = layer.get("mlp")
        if mlp is not None:
            for n in ("norm2", "norm2b", "ls2"):
                s[L + n] = (d,)
            F = L + "mlp."
            if mlp["kind"] == "dense":
                s[F + "up"], s[F + "down"] = (mlp["ff"], d), (d, mlp["ff"])
            else:
                for e in range(mlp["router"]["experts"]):
                    s[f"{F}e{e}.up"], s[f"{F}e{e}.down"] = (mlp["expert"]["ff"], d), (d, mlp["expert"]["ff"])
                s[F + "router"] = (mlp["router"]["experts"], d)
                if mlp.get("shared") is not None:
                    ff = mlp["shared"]["ff"]
                    s[F + "shared.up"], s[F + "shared.down"], s[F + "shared.sg"] = (ff, d), (d, ff), (1, d)
        if side:
            s[L + "side.gate"], s[L + "side.proj"], s[L + "side.norm"] = (side, d), (d, side), (d,)
    return s


def random_weights(c, seed, edit=None):
    """float64 weights, already rounded to bfloat16 values so that a bfloat16 file holds them
    exactly. Matrices ~ N(0, 1/sqrt(in)); gains near 1; shift weights in (0, 1); decays between
    0.4 and 0.95 a step; router rows large enough that the chosen experts are no close call."""
    rng = np.random.default_rng(seed)
    w = {}
    for name, shape in tensor_shapes(c).items():
        last = name.rsplit(".", 1)[-1]
        if last in ("norm1", "norm2", "norm1b", "norm2b", "norm"):
            a = 1.0 + 0.2 * rng.standard_normal(shape)
        elif last in ("ls1", "ls2"):
            a = 0.7 + 0.2 * rng.standard_normal(shape)
        elif ".mu." in name:
            a = rng.uniform(0.1, 0.9, shape)
        elif last == "w0":
            a = rng.uniform(-3.0, 0.0, shape)
        elif last == "u":
            a = 0.5 * rng.standard_normal(shape)
        elif last == "router":
            a = 4.0 * rng.standard_normal(shape) / np.sqrt(shape[-1])
        elif name in ("embed", "side.embed"):
            a = rng.standard_normal(shape)
        else:
            a = rng.standard_normal(shape) / np.sqrt(shape[-1])
        w[name] = round_bf16(a)
    if edit is not None:
        edit(w)
        for n in w:
            w[n] = round_bf16(w[n].reshape(-1)).reshape(w[n].shape)
    return w


def make_model_folder(folder, c, seed, storage="BF16", edit=None):
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    w = random_weights(c, seed, edit)
    write_safetensors(folder / "model.safetensors", w, dtype=storage)
    cfg = json.loads(json.dumps(c))
    for layer in cfg["layers"]:                       # the file says it: a tensor's shape
        layer["mixer"].pop("decay_rank", None)
    (folder / "config.json").write_text(json.dumps(cfg, indent=1))
    return w
