"""Plain, slow Vametar decoder: the oracle of the Vametar tests.

Whole sequences, no cache, NumPy float64, one function per mechanism. It shares
no code with ``transformer_amd``: it reads config.json and the safetensors file
itself (through the reader of ``plain_llama``, which is the test-suite's own)
and states every formula once more.

Notation: T tokens, d the model's width, x the residual stream [T, d]. A weight
``W`` is stored [out, in] and used as ``h @ W.T``.
"""
from __future__ import annotations

import json
from pathlib import Path

import numpy as np

from plain_llama import read_safetensors, round_bf16  # noqa: F401  (the suite's own file code)


def write_safetensors(path, tensors: dict, dtype="BF16"):
    """name -> float ndarray (0-d included), stored as F32 or BF16."""
    import struct
    header, blobs, off = {}, [], 0
    for name, a in tensors.items():
        a = np.asarray(a, dtype=np.float64)
        flat = a.reshape(-1)
        if dtype == "F32":
            b = flat.astype("<f4").tobytes()
        elif dtype == "BF16":
            b = (round_bf16(flat).astype(np.float32).view(np.uint32) >> 16).astype("<u2").tobytes()
        else:
            raise ValueError(dtype)
        header[name] = {"dtype": dtype, "shape": list(a.shape), "data_offsets": [off, off + len(b)]}
        blobs.append(b)
        off += len(b)
    h = json.dumps(header, separators=(",", ":")).encode()
    h += b" " * ((8 - len(h) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(h)))
        f.write(h)
        for b in blobs:
            f.write(b)


# --------------------------------------------------------------------------
# small functions
# --------------------------------------------------------------------------
def sigmoid(z):
    z = np.asarray(z, dtype=np.float64)
    return 1.0 / (1.0 + np.exp(-z))


def softplus(z):
    z = np.asarray(z, dtype=np.float64)
    return np.logaddexp(0.0, z)


def silu(z):
    return z * sigmoid(z)


def gelu_tanh(z):
    z = np.asarray(z, dtype=np.float64)
    return 0.5 * z * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (z + 0.044715 * z ** 3)))


def unit_rms(x, eps):
    """x divided by sqrt(mean(x^2) + eps) over the last axis."""
    x = np.asarray(x, dtype=np.float64)
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


# --------------------------------------------------------------------------
# mechanisms
# --------------------------------------------------------------------------
def bigram_rows(tokens, buckets, mul_prev, mul_cur):
    """Row of the pair table for every token: a hash of (previous, current) into
    ``buckets`` rows; the first token of a sequence takes the extra last row."""
    rows = np.empty(len(tokens), dtype=np.int64)
    for t, tok in enumerate(tokens):
        rows[t] = buckets if t == 0 else (int(tokens[t - 1]) * mul_prev + int(tok) * mul_cur) % buckets
    return rows


def embed(tokens, table, pair_table, buckets, mul_prev, mul_cur):
    tokens = np.asarray(tokens, dtype=np.int64)
    return table[tokens] + pair_table[bigram_rows(tokens, buckets, mul_prev, mul_cur)]


def scalar_norm(x, g, eps):
    """RMS norm whose gain is one number for all coordinates."""
    return unit_rms(x, eps) * float(g)


def token_shift(h, mu):
    """h_t + (h_{t-1} - h_t) * mu, with h_{-1} = 0; h_{t-1} is the unshifted row."""
    prev = np.vstack([np.zeros((1, h.shape[1])), h[:-1]])
    return h + (prev - h) * mu


def residual_gate(h, w, b):
    return sigmoid(h @ w.T + b)


def rotate_partial(t, positions, base, dims):
    """t: [T, heads, dh]. The first ``dims`` coordinates of every head are rotated in pairs
    (i, i + dims/2) by the angle position * base^(-2i/dims); the others stay."""
    out = np.array(t, dtype=np.float64)
    half = dims // 2
    i = np.arange(half, dtype=np.float64)
    ang = np.asarray(positions, dtype=np.float64)[:, None] * base ** (-2.0 * i / dims)   # [T, half]
    c, s = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    u, v = t[..., :half], t[..., half:dims]
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


def softmax_attention(q, k, v, scale, window=None):
    """q [T, H, dk], k [T, G, dk], v [T, G, dv] -> [T, H, dv]; token i reads j <= i
    (and j > i - window where a window is given)."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        i, j = np.arange(T)[:, None], np.arange(T)[None, :]
        mask = j <= i
        if window is not None:
            mask &= j > i - window
        s = np.where(mask, s, -np.inf)
        s = s - s.max(axis=1, keepdims=True)
        p = np.exp(s)
        p /= p.sum(axis=1, keepdims=True)
        out[:, h] = p @ v[:, g]
    return out


def attention_mixer(h, w, p, m, eps, positions, v_first=None):
    """p: prefix of the layer's mixer tensors; m: its 'mixer' configuration. Returns
    (output [T, d], this layer's values [T, G*dv] before mixing)."""
    T = h.shape[0]
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    G = m.get("kv_heads", H)
    q, k, v = h @ w[p + "q"].T, h @ w[p + "k"].T, h @ w[p + "v"].T
    q = unit_rms(q, eps) * w[p + "q.norm"]          # over all heads at once
    k = unit_rms(k, eps) * w[p + "k.norm"]
    q, k = q.reshape(T, H, dk), k.reshape(T, G, dk)
    rot = m.get("rot")
    if rot:
        q = rotate_partial(q, positions, rot["base"], rot["dims"])
        k = rotate_partial(k, positions, rot["base"], rot["dims"])
    own_v = v
    if v_first is not None:
        lam = float(w[p + "vmix"])
        v = (1.0 - lam) * v + lam * v_first
    o = softmax_attention(q, k, v.reshape(T, G, dv), m["scale"])
    return o.reshape(T, H * dv) @ w[p + "o"].T, own_v


def causal_conv(x, taps, bias):
    """x [T, C]; taps [C, K], the last column weighs the current token; zeros before 0."""
    T, C = x.shape
    K = taps.shape[1]
    padded = np.vstack([np.zeros((K - 1, C)), x])
    out = np.tile(bias, (T, 1)).astype(np.float64)
    for j in range(K):
        out += padded[j:j + T] * taps[:, j]
    return out


def rglru_mixer(h, w, p, m):
    """Two branches of m['width'] channels; the second goes through a short causal
    convolution and a gated linear recurrence, per channel:
    a = exp(-8 r softplus(lam)), S_t = a S_{t-1} + sqrt(1 - a^2) (i u)."""
    T = h.shape[0]
    C, nb = m["width"], m["blocks"]
    y = gelu_tanh(h @ w[p + "y"].T + w[p + "y.b"])
    u = causal_conv(h @ w[p + "x"].T + w[p + "x.b"], w[p + "conv"], w[p + "conv.b"])
    ub = u.reshape(T, nb, C // nb)
    r = sigmoid(np.einsum("tbi,boi->tbo", ub, w[p + "ra"]) + w[p + "ra.b"]).reshape(T, C)
    i = sigmoid(np.einsum("tbi,boi->tbo", ub, w[p + "ri"]) + w[p + "ri.b"]).reshape(T, C)
    a = np.exp(-8.0 * r * softplus(w[p + "lam"]))
    S = np.zeros(C)
    out = np.empty((T, C))
    for t in range(T):
        S = a[t] * S + np.sqrt(1.0 - a[t] ** 2) * i[t] * u[t]
        out[t] = S
    return (out * y) @ w[p + "o"].T


def gla_mixer(h, w, p, m, eps):
    """Per head a matrix state S [dk, dv]: S_t = diag(alpha_t) S_{t-1} + k_t v_t^T,
    o_t = S_t^T q_t, alpha = sigmoid(z)^(1/tau) per key channel."""
    T = h.shape[0]
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T) * dk ** -0.5
    k = h @ w[p + "k"].T
    v = h @ w[p + "v"].T
    z = (h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "a2.b"]
    alpha = sigmoid(z) ** (1.0 / m["tau"])
    q, k, alpha, v = (t.reshape(T, H, -1) for t in (q, k, alpha, v))
    S = np.zeros((H, dk, dv))
    o = np.empty((T, H, dv))
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = np.einsum("hkv,hk->hv", S, q[t])
    o = unit_rms(o, eps) * w[p + "norm"]
    return (o.reshape(T, H * dv) * silu(h @ w[p + "g"].T)) @ w[p + "o"].T


def geglu(h, w, p):
    return (gelu_tanh(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


# --------------------------------------------------------------------------
# the model
# --------------------------------------------------------------------------
class PlainVametar:
    def __init__(self, folder=None, config=None, weights=None):
        if folder is not None:
            config = json.loads((Path(folder) / "config.json").read_text())
            weights = read_safetensors(Path(folder) / "model.safetensors")
        self.c, self.w = config, weights

    def forward(self, tokens, layers_out=None):
        """Logits [T, vocab] of a whole sequence from position 0. ``layers_out``: a list
        that receives the residual stream after every layer."""
        c, w = self.c, self.w
        eps, m = c["norm"]["eps"], c["residual_mult"]
        T = len(tokens)
        positions = np.arange(T)
        bg = c["embedding"]["bigram"]
        x = embed(tokens, w["embed"], w["bigram"], bg["buckets"], bg["mul_prev"], bg["mul_cur"])
        v_first = None
        for li, layer in enumerate(c["layers"]):
            L = f"l{li}."
            h = scalar_norm(x, w[L + "norm1"], eps)
            gate = residual_gate(h, w[L + "rg1"], w[L + "rg1.b"])
            hs = token_shift(h, w[L + "shift"])
            kind, mx = layer["type"], layer["mixer"]
            if kind == "attention":
                mixing = bool(mx.get("v_mix")) and v_first is not None
                out, own_v = attention_mixer(hs, w, L + "mix.", mx, eps, positions,
                                             v_first if mixing else None)
                if mx.get("v_mix") and v_first is None:
                    v_first = own_v
            elif kind == "rglru":
                out = rglru_mixer(hs, w, L + "mix.", mx)
            elif kind == "gla":
                out = gla_mixer(hs, w, L + "mix.", mx, eps)
            else:
                raise ValueError(f"layer {li}: unknown type {kind!r}")
            x = x + m * gate * out
            if layer.get("mlp") is not None:
                if layer["mlp"]["kind"] != "dense":
                    raise ValueError(f"layer {li}: unknown feed-forward {layer['mlp']['kind']!r}")
                h2 = scalar_norm(x, w[L + "norm2"], eps)
                gate2 = residual_gate(h2, w[L + "rg2"], w[L + "rg2.b"])
                x = x + m * gate2 * geglu(h2, w, L + "mlp.")
            if layers_out is not None:
                layers_out.append(x.copy())
        return (scalar_norm(x, w["final.norm"], eps) @ w["head"].T) * c["logit_scale"]


# --------------------------------------------------------------------------
# random models for the tests
# --------------------------------------------------------------------------
def tensor_shapes(c):
    """{tensor name: shape} of a configuration, in the file's own names."""
    d, V = c["width"], c["vocab"]
    s = {"embed": (V, d), "bigram": (c["embedding"]["bigram"]["buckets"] + 1, d),
         "final.norm": (), "head": (V, d)}
    for li, layer in enumerate(c["layers"]):
        L, mx = f"l{li}.", layer["mixer"]
        s[L + "norm1"] = ()
        s[L + "shift"] = (d,)
        s[L + "rg1"], s[L + "rg1.b"] = (d, d), (d,)
        M = L + "mix."
        if layer["type"] == "attention":
            H, G, dk, dv = mx["heads"], mx.get("kv_heads", mx["heads"]), mx["dim"], mx["vdim"]
            s[M + "q"], s[M + "k"], s[M + "v"] = (H * dk, d), (G * dk, d), (G * dv, d)
            s[M + "q.norm"], s[M + "k.norm"] = (H * dk,), (G * dk,)
            if mx.get("v_mix"):
                s[M + "vmix"] = ()
            s[M + "o"] = (d, H * dv)
        elif layer["type"] == "rglru":
            C, nb, K = mx["width"], mx["blocks"], mx["conv"]
            for n in ("y", "x"):
                s[M + n], s[M + n + ".b"] = (C, d), (C,)
            s[M + "conv"], s[M + "conv.b"] = (C, K), (C,)
            for n in ("ra", "ri"):
                s[M + n], s[M + n + ".b"] = (nb, C // nb, C // nb), (nb, C // nb)
            s[M + "lam"] = (C,)
            s[M + "o"] = (d, C)
        elif layer["type"] == "gla":
            H, dk, dv = mx["heads"], mx["dim"], mx["vdim"]
            r = mx.get("rank", 16)
            s[M + "q"], s[M + "k"] = (H * dk, d), (H * dk, d)
            s[M + "v"], s[M + "g"] = (H * dv, d), (H * dv, d)
            s[M + "o"] = (d, H * dv)
            s[M + "norm"] = (dv,)
            s[M + "a1"], s[M + "a2"], s[M + "a2.b"] = (r, d), (H * dk, r), (H * dk,)
        if layer.get("mlp") is not None:
            ff = layer["mlp"]["ff"]
            s[L + "norm2"] = ()
            s[L + "rg2"], s[L + "rg2.b"] = (d, d), (d,)
            s[L + "mlp.gate"], s[L + "mlp.up"], s[L + "mlp.down"] = (ff, d), (ff, d), (d, ff)
    return s


def random_weights(c, seed, edit=None):
    """float64 weights, already rounded to bfloat16 values so that a bfloat16 file holds them
    exactly. Matrices ~ N(0, 1/sqrt(in)); gains near 1; shifts and mixing weights in (0, 1)."""
    rng = np.random.default_rng(seed)
    w = {}
    for name, shape in tensor_shapes(c).items():
        last = name.rsplit(".", 1)[-1]
        if name.endswith(("norm1", "norm2", "final.norm")):
            a = 1.0 + 0.2 * rng.standard_normal(shape)
        elif last == "norm":                       # q.norm, k.norm, the per-head norm of gla
            a = 1.0 + 0.2 * rng.standard_normal(shape)
        elif last in ("shift", "vmix"):
            a = rng.uniform(0.1, 0.9, shape)
        elif last == "lam":
            a = rng.uniform(-2.0, 1.0, shape)
        elif last == "b":
            a = 0.3 * rng.standard_normal(shape)
        elif last == "conv":
            a = rng.standard_normal(shape) / np.sqrt(shape[-1])
        elif name in ("embed", "bigram"):
            a = rng.standard_normal(shape)
        else:
            a = rng.standard_normal(shape) / np.sqrt(shape[-1])
        w[name] = round_bf16(a) if np.ndim(a) else round_bf16(np.asarray(a).reshape(1)).reshape(())
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
    (folder / "config.json").write_text(json.dumps(c, indent=1))
    return w
