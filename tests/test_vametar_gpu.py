"""The Vametar decoder on the GPU against the plain implementation in ``plain_vametar``.

Each mechanism alone (its kernels against the plain function, with the state carried over a
cut), then the engine: whole prompts, portions, token-by-token decoding, unequal batches, slots
and pages used again, recorded steps, far and edge keys, greedy generation and the replayer."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_vametar as P
import vametar_util as U

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = ["float32", "bfloat16"]


def _t(a, dtype=torch.float32):
    return torch.tensor(np.asarray(a), dtype=dtype, device=DEV)


def _bf(a):
    from plain_llama import round_bf16
    return round_bf16(np.asarray(a, dtype=np.float64))


def _tables(lens):
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    return _t(cu, torch.int32)


def _atol(dtype):
    return 2e-5 if dtype == "float32" else 2e-2


def _rtol(dtype):
    """One rounding of a result to the storage type, relative."""
    return 1e-5 if dtype == "float32" else 2.0 ** -7


# ----------------------------------------------------------------------------- mechanisms alone
@pytest.mark.parametrize("dtype", DTYPES)
def test_token_shift_carries_the_last_row(dtype):
    from transformer_amd import kernels as K
    td = torch.float32 if dtype == "float32" else torch.bfloat16
    rng = np.random.default_rng(0)
    d, lens = 70, [5, 1, 3]
    mu = rng.uniform(0, 1, d)
    seqs = [_bf(rng.standard_normal((n, d))) for n in lens]
    want = [P.token_shift(s, mu) for s in seqs]
    state = torch.zeros(4, d, device=DEV)
    slots = _t([2, 0, 3], torch.int32)
    # first two rows of every sequence in one step, the rest in a second one
    for lo, hi in ((0, 2), (2, 9)):
        part = [s[lo:hi] for s in seqs]
        keep = [i for i, p in enumerate(part) if len(p)]
        h = _t(np.concatenate([part[i] for i in keep]), td)
        out = torch.empty_like(h)
        K.token_shift(h, out, _t(mu), state, _tables([len(part[i]) for i in keep]), slots[keep].contiguous())
        got, at = out.float().cpu().numpy(), 0
        for i in keep:
            n = len(part[i])
            np.testing.assert_allclose(got[at:at + n], want[i][lo:lo + n], atol=_atol(dtype))
            at += n
    np.testing.assert_allclose(state[2].cpu().numpy(), seqs[0][-1], atol=1e-6)


def test_pair_embedding_rows_and_state():
    from transformer_amd import kernels as K
    rng = np.random.default_rng(1)
    d, buckets, mp, mc = 24, 11, 7, 3
    table = rng.standard_normal((buckets + 1, d))
    seqs = [[4, 9, 9, 2, 30], [8], [1, 1]]
    want = [table[P.bigram_rows(s, buckets, mp, mc)] for s in seqs]
    last = torch.full((5,), 17, dtype=torch.int32, device=DEV)        # stale values of earlier owners
    slots = _t([4, 1, 0], torch.int32)
    for lo, hi in ((0, 1), (1, 9)):
        part = [s[lo:hi] for s in seqs]
        keep = [i for i, p in enumerate(part) if p]
        toks = _t(np.concatenate([part[i] for i in keep]), torch.int32)
        x = torch.zeros(toks.numel(), d, device=DEV)
        K.pair_embed_add(x, _t(table), toks, last, _tables([len(part[i]) for i in keep]),
                         _t([lo] * len(keep), torch.int32), slots[keep].contiguous(), buckets, mp, mc)
        got, at = x.cpu().numpy(), 0
        for i in keep:
            n = len(part[i])
            np.testing.assert_allclose(got[at:at + n], want[i][lo:lo + n], atol=1e-6)
            at += n
    assert last.tolist()[4] == 30 and last.tolist()[0] == 1 and last.tolist()[1] == 8


@pytest.mark.parametrize("dtype", DTYPES)
def test_gated_add_and_norm(dtype):
    from transformer_amd import kernels as K
    td = torch.float32 if dtype == "float32" else torch.bfloat16
    rng = np.random.default_rng(2)
    nt, d, mult, eps = 7, 100, 0.6, 1e-5
    x, delta = rng.standard_normal((nt, d)), rng.standard_normal((3, nt, d))
    gate, gb, db, w = (rng.standard_normal(s) for s in ((nt, d), (d,), (d,), (d,)))
    v = x + mult * P.sigmoid(gate + gb) * (delta.sum(0) + db)
    xt, out = _t(x), torch.empty(nt, d, dtype=td, device=DEV)
    pend = K.GatedDelta(_t(delta), _t(db), _t(gate), _t(gb), mult)
    rows = _t([5, 0], torch.int32)
    few = torch.empty(2, d, dtype=td, device=DEV)
    K.gated_add_rmsnorm(xt, _t(w), eps, few, pend, rows)              # gathers, leaves x alone
    np.testing.assert_allclose(xt.cpu().numpy(), x, atol=1e-6)
    np.testing.assert_allclose(few.float().cpu().numpy(), (P.unit_rms(v, eps) * w)[[5, 0]], atol=_atol(dtype))
    K.gated_add_rmsnorm(xt, _t(w), eps, out, pend)
    np.testing.assert_allclose(xt.cpu().numpy(), v, atol=1e-5)
    np.testing.assert_allclose(out.float().cpu().numpy(), P.unit_rms(v, eps) * w, atol=_atol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
def test_token_shift_on_the_norm_of_single_token_steps(dtype):
    """The norm's kernel takes the shift over when every sequence brings one token: the same
    rows and the same state as the norm followed by the shift's own kernel."""
    from transformer_amd import kernels as K
    td = torch.float32 if dtype == "float32" else torch.bfloat16
    rng = np.random.default_rng(9)
    nt, d, eps = 5, 72, 1e-5
    x, delta, gate = (rng.standard_normal((nt, d)) for _ in range(3))
    w, mu = 1 + 0.1 * rng.standard_normal(d), rng.uniform(0, 1, d)
    st = rng.standard_normal((7, d))
    slots, cu = _t([6, 0, 3, 2, 5], torch.int32), _tables([1] * nt)
    pend = lambda: K.GatedDelta(_t(delta), None, _t(gate), None, 0.7)
    xa, ha, sa = _t(x), torch.empty(nt, d, dtype=td, device=DEV), _t(st)
    K.gated_add_rmsnorm(xa, _t(w), eps, ha, pend())
    hsa = K.token_shift(ha, torch.empty_like(ha), _t(mu), sa, cu, slots)
    xb, hb, sb, hsb = _t(x), torch.empty(nt, d, dtype=td, device=DEV), _t(st), torch.empty(nt, d, dtype=td, device=DEV)
    K.gated_add_rmsnorm(xb, _t(w), eps, hb, pend(), shift=(_t(mu), sb, slots, hsb))
    for a, b in ((xa, xb), (ha, hb), (hsa, hsb), (sa, sb)):
        assert torch.equal(a, b)
    v = x + 0.7 * P.sigmoid(gate) * delta
    h = P.unit_rms(v, eps) * w
    np.testing.assert_allclose(hsb.float().cpu().numpy(), h + (st[[6, 0, 3, 2, 5]] - h) * mu, atol=_atol(dtype))


def _paged(model_dtype, pages, nkv, dk, dv):
    from transformer_amd.kernels import PAGE
    kc = torch.zeros(pages, nkv, PAGE, dk, dtype=model_dtype, device=DEV)
    vc = torch.zeros(pages, nkv, dv, PAGE, dtype=model_dtype, device=DEV)
    return kc, vc


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("geom", [(6, 3, 40, 24, 16), (2, 2, 16, 72, 16), (5, 1, 23, 9, 0), (4, 2, 128, 64, 64)])
def test_attention_pieces(dtype, geom):
    """qk_prepare + attention over shuffled pages, a prompt cut in two and then single
    tokens, against the plain functions; values mixed with an earlier layer's."""
    from transformer_amd import kernels as K
    H, G, dk, dv, rot = geom
    td = torch.float32 if dtype == "float32" else torch.bfloat16
    rng = np.random.default_rng(3)
    T, eps, scale, lam, base = 150, 1e-5, 0.21, 0.3, 500.0
    q, k, v, vf = (_bf(rng.standard_normal((T, n))) for n in (H * dk, G * dk, G * dv, G * dv))
    wq, wk = 1 + 0.2 * rng.standard_normal(H * dk), 1 + 0.2 * rng.standard_normal(G * dk)
    pos = np.arange(T)
    qn = (P.unit_rms(q, eps) * wq).reshape(T, H, dk)
    kn = (P.unit_rms(k, eps) * wk).reshape(T, G, dk)
    if rot:
        qn, kn = P.rotate_partial(qn, pos, base, rot), P.rotate_partial(kn, pos, base, rot)
    vm = (1 - lam) * v + lam * vf
    want = P.softmax_attention(qn, kn, vm.reshape(T, G, dv), scale).reshape(T, H * dv)
    kc, vc = _paged(td, 9, G, dk, dv)
    table = _t([[7, 2, 5]], torch.int32)
    inv = base ** (-2.0 * np.arange(rot // 2) / rot) if rot else None
    got, at = [], 0
    for n in (70, 58, 1, 1, 20):
        rows = slice(at, at + n)
        qkv = _t(np.concatenate([q[rows], k[rows], v[rows]], 1), td)
        positions = _t(pos[rows], torch.int32)
        angles = None
        if rot:
            angles = K.rope_table(positions, _t(inv), torch.empty(n, rot // 2, 2, device=DEV))
        p = pos[rows]
        dest = _t(np.array([7, 2, 5])[p // 64] * 64 + p % 64, torch.int32)
        keep = torch.empty(n, G * dv, dtype=td, device=DEV)
        K.qk_prepare(qkv, H, G, dk, dv, eps, _t(wq), _t(wk), angles, rot, _t([lam]), _t(vf[rows], td), keep,
                     dest, kc, vc)
        np.testing.assert_allclose(keep.float().cpu().numpy(), v[rows], atol=1e-6)
        o = torch.empty(n, H * dv, dtype=td, device=DEV)
        K.attention_generic_dv(qkv, o, kc, vc, table, _t([0, n], torch.int32), _t([at], torch.int32), n,
                               H, G, dk, dv, scale)
        got.append(o.float().cpu().numpy())
        at += n
    np.testing.assert_allclose(np.concatenate(got), want, atol=1e-5 if dtype == "float32" else 3e-2)


@pytest.mark.parametrize("where", ["prompt", "decode"])
def test_attention_far_key_and_window_edges(where):
    """One key far back gets a score that stands out, so the output is that key's value; with
    a window the same key is seen just inside it and not just outside."""
    from transformer_amd import kernels as K
    H, G, dk, dv, T = 2, 1, 24, 40, 300
    rng = np.random.default_rng(4)
    k = rng.standard_normal((T, G * dk)) * 0.1
    v = rng.standard_normal((T, G * dv))
    q = rng.standard_normal((T, H * dk)) * 0.1
    far = 3
    k[far] = 0.0
    k[far, :4] = 6.0
    q[T - 1] = 0.0
    q[T - 1, :4] = 6.0
    q[T - 1, dk:dk + 4] = 6.0
    kc, vc = _paged(torch.float32, 6, G, dk, dv)
    pages = np.array([4, 1, 3, 0, 5])
    pos = np.arange(T)
    dest = _t(pages[pos // 64] * 64 + pos % 64, torch.int32)
    qkv = _t(np.concatenate([q, k, v], 1))
    K.qk_prepare(qkv, H, G, dk, dv, 0.0, None, None, None, 0, dest=dest, kcache=kc, vcache=vc)
    table = _t([pages], torch.int32)

    def last_row(window):
        if where == "prompt":
            o = torch.empty(T, H * dv, device=DEV)
            K.attention_generic_dv(qkv, o, kc, vc, table, _t([0, T], torch.int32), _t([0], torch.int32), T,
                                   H, G, dk, dv, 1.0, window)
            return o[-1].cpu().numpy()
        o = torch.empty(1, H * dv, device=DEV)
        K.attention_generic_dv(qkv[T - 1:], o, kc, vc, table, _t([0, 1], torch.int32),
                               _t([T - 1], torch.int32), 1, H, G, dk, dv, 1.0, window)
        return o[0].cpu().numpy()

    want = np.tile(v[far], H)
    np.testing.assert_allclose(last_row(None), want, atol=1e-3)
    np.testing.assert_allclose(last_row(T - far), want, atol=1e-3)          # the window's last key
    assert np.abs(last_row(T - far - 1) - want).max() > 0.1                 # one short: not seen


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("geom", [(144, 3, 4), (48, 1, 1), (80, 5, 2), (640, 2, 3), (1600, 2, 2)])
def test_diagonal_recurrence_pieces(dtype, geom):
    from transformer_amd import kernels as K
    C, nb, taps = geom
    td = torch.float32 if dtype == "float32" else torch.bfloat16
    rng = np.random.default_rng(5)
    bs, lens = C // nb, [200, 1, 70]     # more than one segment of the side-by-side scan
    w = {"y": np.zeros((C, 1)), "x": np.zeros((C, 1)), "y.b": 0.3 * rng.standard_normal(C),
         "x.b": 0.3 * rng.standard_normal(C), "conv": rng.standard_normal((C, taps)) / taps ** 0.5,
         "conv.b": 0.1 * rng.standard_normal(C), "ra": _bf(rng.standard_normal((nb, bs, bs)) / bs ** 0.5),
         "ri": _bf(rng.standard_normal((nb, bs, bs)) / bs ** 0.5), "ra.b": 0.2 * rng.standard_normal((nb, bs)),
         "ri.b": 0.2 * rng.standard_normal((nb, bs)), "lam": rng.uniform(-4, 1, C), "o": np.eye(C)}
    seqs = [(_bf(rng.standard_normal((n, C))), _bf(rng.standard_normal((n, C)))) for n in lens]

    def plain_one(ys, xs):          # the plain mixer with the projections already applied
        y = P.gelu_tanh(ys + w["y.b"])
        u = P.causal_conv(xs + w["x.b"], w["conv"], w["conv.b"])
        ub = u.reshape(len(u), nb, bs)
        r = P.sigmoid(np.einsum("tbi,boi->tbo", ub, w["ra"]) + w["ra.b"]).reshape(len(u), C)
        i = P.sigmoid(np.einsum("tbi,boi->tbo", ub, w["ri"]) + w["ri.b"]).reshape(len(u), C)
        a = np.exp(-8.0 * r * P.softplus(w["lam"]))
        S, out = np.zeros(C), []
        for t in range(len(u)):
            S = a[t] * S + np.sqrt(1 - a[t] ** 2) * i[t] * u[t]
            out.append(S * y[t])
        return np.array(out)

    want = [plain_one(*s) for s in seqs]
    state = torch.zeros(5, C, device=DEV)
    conv_state = torch.zeros(5, taps - 1, C, device=DEV)
    slots = _t([3, 0, 4], torch.int32)
    gw = _t(np.concatenate([w["ra"], w["ri"]]), td)
    gb = _t(np.concatenate([w["ra.b"], w["ri.b"]]))
    for lo, hi in ((0, 1), (1, 3), (3, 40), (40, 300)):     # one token, two tokens, portions
        part = [(y[lo:hi], x[lo:hi]) for y, x in seqs]
        keep = [i for i, p in enumerate(part) if len(p[0])]
        yx = _t(np.concatenate([np.concatenate(part[i], 1) for i in keep]), td)
        nt = yx.shape[0]
        cu, sl = _tables([len(part[i][0]) for i in keep]), slots[keep].contiguous()
        a, b = torch.empty(nt, C, device=DEV), torch.empty(nt, C, device=DEV)
        K.rglru_gates(yx, C, _t(w["x.b"]), _t(w["conv"]), _t(w["conv.b"]), conv_state, gw, gb, _t(w["lam"]),
                      8.0, cu, sl, a, b)
        out = K.rglru_scan(yx, C, _t(w["y.b"]), _t(w["x.b"]), a, b, state, conv_state, cu, sl,
                           torch.empty(nt, C, dtype=td, device=DEV), max(len(part[i][0]) for i in keep),
                           torch.empty(len(keep), C, device=DEV))
        got, at = out.float().cpu().numpy(), 0
        for i in keep:
            n = len(part[i][0])
            np.testing.assert_allclose(got[at:at + n], want[i][lo:lo + n], atol=_atol(dtype), rtol=_rtol(dtype))
            at += n


@pytest.mark.parametrize("geom", [(144, 3, 4), (512, 2, 2)])
def test_recurrence_gates_of_long_steps_match_the_plain_kernel(geom):
    """From 256 tokens on a bfloat16 step forms its gates through the library (u split into
    two bfloat16 halves, float32 sums): the same decays and input terms as the 32-bit kernel."""
    from transformer_amd import kernels as K
    from transformer_amd.parts.linear import Workspace
    C, nb, taps = geom
    rng = np.random.default_rng(8)
    bs, lens = C // nb, [290, 31]
    nt = sum(lens)
    yx = _t(rng.standard_normal((nt, 2 * C)) * 2, torch.bfloat16)
    gw = _t(rng.standard_normal((2 * nb, bs, bs)) / bs ** 0.5, torch.bfloat16)
    gb, xb, cb, lam = (_t(rng.standard_normal(n) * 0.3) for n in ((2 * nb, bs), C, C, C))
    tp = _t(rng.standard_normal((C, taps)) / taps ** 0.5)
    conv_state = _t(rng.standard_normal((3, taps - 1, C)))
    cu, sl = _tables(lens), _t([2, 0], torch.int32)
    out = []
    for split in (False, True):
        a, b = torch.empty(nt, C, device=DEV), torch.empty(nt, C, device=DEV)
        if split:
            K.rglru_gates_split(yx, C, xb, tp, cb, conv_state, gw, gb, lam, 8.0, cu, sl, a, b, Workspace(DEV))
        else:
            K.rglru_gates(yx, C, xb, tp, cb, conv_state, gw, gb, lam, 8.0, cu, sl, a, b)
        out.append((a.cpu().numpy(), b.cpu().numpy()))
    np.testing.assert_allclose(out[1][0], out[0][0], atol=2e-5)
    np.testing.assert_allclose(out[1][1], out[0][1], atol=2e-4, rtol=1e-4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("geom", [(3, 20, 28, 5), (1, 64, 16, 2), (2, 36, 12, 9), (2, 128, 96, 16), (1, 250, 130, 3)])
def test_gated_linear_attention_pieces(dtype, geom):
    from transformer_amd import kernels as K
    H, dk, dv, rank = geom
    td = torch.float32 if dtype == "float32" else torch.bfloat16
    rng = np.random.default_rng(6)
    tau, eps, lens = 4.0, 1e-5, [61, 1, 10]
    a2, a2b = _bf(rng.standard_normal((H * dk, rank))), rng.standard_normal(H * dk) + 2.0
    nw = 1 + 0.2 * rng.standard_normal(dv)
    width = 2 * H * dk + 2 * H * dv + rank
    seqs = [_bf(rng.standard_normal((n, width))) for n in lens]

    def plain_one(p):
        T = len(p)
        q, k, v, g, low = np.split(p, np.cumsum([H * dk, H * dk, H * dv, H * dv]), axis=1)
        alpha = P.sigmoid(low @ a2.T + a2b) ** (1.0 / tau)
        q, k, alpha, v = (t.reshape(T, H, -1) for t in (q * dk ** -0.5, k, alpha, v))
        S, o = np.zeros((H, dk, dv)), np.empty((T, H, dv))
        for t in range(T):
            S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
            o[t] = np.einsum("hkv,hk->hv", S, q[t])
        return (P.unit_rms(o, eps) * nw).reshape(T, H * dv) * P.silu(g)

    want = [plain_one(s) for s in seqs]
    state = torch.zeros(4, H, dk, dv, device=DEV)
    slots = _t([1, 3, 0], torch.int32)
    for lo, hi in ((0, 1), (1, 3), (3, 70)):
        part = [s[lo:hi] for s in seqs]
        keep = [i for i, p in enumerate(part) if len(p)]
        proj = _t(np.concatenate([part[i] for i in keep]), td)
        nt = proj.shape[0]
        cu, sl = _tables([len(part[i]) for i in keep]), slots[keep].contiguous()
        o = K.gla_recurrent(proj, H, dk, dv, rank, _t(a2, td), _t(a2b), tau, state, cu, sl,
                            torch.empty(K.gla_row_parts(dk), nt, H, dv, device=DEV),
                            torch.empty(nt, H * dk, device=DEV))
        out = K.gla_out(o, proj, H, dk, dv, _t(nw), eps, torch.empty(nt, H * dv, dtype=td, device=DEV))
        got, at = out.float().cpu().numpy(), 0
        for i in keep:
            n = len(part[i])
            np.testing.assert_allclose(got[at:at + n], want[i][lo:lo + n], atol=1e-4 if dtype == "float32" else 3e-2,
                                       rtol=_rtol(dtype))
            at += n


@pytest.mark.parametrize("dtype", DTYPES)
def test_gelu_gate(dtype):
    from transformer_amd import kernels as K
    td = torch.float32 if dtype == "float32" else torch.bfloat16
    gu = _bf(np.random.default_rng(7).standard_normal((5, 2 * 37)) * 2)
    out = K.glu(_t(gu, td), torch.empty(5, 37, dtype=td, device=DEV), "gelu_tanh")
    np.testing.assert_allclose(out.float().cpu().numpy(), P.gelu_tanh(gu[:, :37]) * gu[:, 37:], atol=_atol(dtype) * 3)


# ----------------------------------------------------------------------------- the engine
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B"])
def test_layers_and_whole_prompt(name, dtype):
    model, toks = U.engine(name, dtype), U.tokens(name, 90, 1)
    layers = []
    want = U.plain(name, dtype).forward(toks, layers)
    dumps = {}
    model.dump = lambda n, t: dumps.__setitem__(n, t.detach().float().cpu().numpy().copy())
    try:
        cache = model.new_cache(256)
        from transformer_amd import Entry
        got = model.step(cache, [Entry(cache.alloc_slot(), toks, list(range(len(toks))))]).cpu().numpy()
    finally:
        model.dump = None
    tol = 1e-4 if dtype == "float32" else 0.15
    for i, l in enumerate(layers):
        assert np.abs(dumps[f"run.{i}"] - l).max() < tol * max(1.0, np.abs(l).max()), f"layer {i}"
    assert U.row_error(got, want).max() < U.TOL[dtype]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,edit", [("A", None), ("B", None), ("D", None), ("A", "slow"), ("A", "sharp"),
                                       ("D", "sharp")])
def test_cuts_agree_with_plain(name, edit, dtype):
    """Whole, portions down to two tokens, and every token alone: all against the plain model."""
    model, toks = U.engine(name, dtype, edit), U.tokens(name, 150, 2)
    want = U.plain_logits(name, dtype, edit, tuple(toks))
    cache = model.new_cache(512, max_slots=3)
    for cuts in ([150], [2, 2, 61, 3, 64, 17], [130], []):
        slot = cache.alloc_slot()
        got = U.run_cuts(model, cache, slot, toks, cuts)
        cache.free_slot(slot)                      # the next cut takes the same slot and pages
        assert U.row_error(got, want).max() < U.TOL[dtype], f"cuts {cuts}"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "D"])
def test_long_prompt_in_portions_at_the_kernels_edges(name, dtype):
    """Portions that end at, just before and just behind the places where the recurrent kernels
    change their ways: chunks of 8 and 32 tokens, tiles of 16, segments of 64, and the 256 tokens
    from which a bfloat16 step forms the recurrence's gates through the library."""
    model, toks = U.engine(name, dtype, "slow"), U.tokens(name, 400, 7)
    want = U.plain_logits(name, dtype, "slow", tuple(toks))
    cache = model.new_cache(512, max_slots=1)
    for cuts in ([400], [257, 63, 65, 15], [64, 256, 33, 31, 16], [255, 129, 8, 7, 1]):
        slot = cache.alloc_slot()
        got = U.run_cuts(model, cache, slot, toks, cuts)
        cache.free_slot(slot)
        assert U.row_error(got, want).max() < U.TOL[dtype], f"cuts {cuts}"


@pytest.mark.parametrize("dtype", DTYPES)
def test_unequal_batch_then_decoding_in_used_slots(dtype):
    from transformer_amd import Entry
    name = "A"
    model = U.engine(name, dtype)
    cache = model.new_cache(1024, max_slots=4)
    # a first batch dirties every slot and page, then leaves
    old = [cache.alloc_slot() for _ in range(4)]
    model.step(cache, [Entry(s, U.tokens(name, 100 + 7 * s, 50 + s), [0]) for s in old])
    for s in old:
        cache.free_slot(s)
    lens = [1, 70, 131, 2]
    seqs = [U.tokens(name, n + 40, 10 + i) for i, n in enumerate(lens)]
    want = [U.plain_logits(name, dtype, None, tuple(s)) for s in seqs]
    slots = [cache.alloc_slot() for _ in seqs]
    got = [[] for _ in seqs]
    lg = model.step(cache, [Entry(sl, s[:n], list(range(n))) for sl, s, n in zip(slots, seqs, lens)]).cpu().numpy()
    at = 0
    for i, n in enumerate(lens):
        got[i].append(lg[at:at + n].copy())
        at += n
    live = list(range(len(seqs)))
    for step in range(40):
        if step == 25:                             # one sequence leaves early, its slot is taken again
            cache.free_slot(slots[1])
            live.remove(1)
            slots[1] = cache.alloc_slot()
        lg = model.step(cache, [Entry(slots[i], [seqs[i][lens[i] + step]], [0]) for i in live]).cpu().numpy()
        for j, i in enumerate(live):
            got[i].append(lg[j:j + 1].copy())
    for i in range(len(seqs)):
        g = np.concatenate(got[i])
        assert U.row_error(g, want[i][:len(g)]).max() < U.TOL[dtype], f"sequence {i}"
    cache.pool.check()


@pytest.mark.parametrize("dtype", DTYPES)
def test_recorded_steps_match_eager_steps(dtype):
    """Single-token steps are replayed from recorded graphs; state must move exactly once per
    step, also in the step that is recorded and tried."""
    from transformer_amd import Entry
    name = "B"
    model = U.engine(name, dtype)
    seqs = [U.tokens(name, 60, 20 + i) for i in range(3)]
    outs = []
    for graphs in (True, False):
        model.use_graphs = graphs
        try:
            cache = model.new_cache(512, max_slots=4)
            slots = [cache.alloc_slot() for _ in seqs]
            rows = []
            for t in range(60):
                lg = model.step(cache, [Entry(sl, [s[t]], [0]) for sl, s in zip(slots, seqs)])
                rows.append(lg.cpu().numpy().copy())
            outs.append(np.stack(rows))
        finally:
            model.use_graphs = True
    assert np.abs(outs[0] - outs[1]).max() < (1e-5 if dtype == "float32" else 3e-2)
    want = np.stack([U.plain_logits(name, dtype, None, tuple(s)) for s in seqs], 1)
    assert U.row_error(outs[0], want).max() < U.TOL[dtype]


@pytest.mark.parametrize("dtype", DTYPES)
def test_wide_model_in_three_cuts(dtype):
    """Width 1024 and heads of 128: the products of 17 to 64 rows leave planes that the gated
    add sums, prompts go to the library, single tokens to the few-rows products."""
    name = "C"
    model, toks = U.engine(name, dtype), U.tokens(name, 200, 3)
    want = U.plain_logits(name, dtype, None, tuple(toks))
    cache = model.new_cache(512, max_slots=2)
    for cuts in ([200], [100, 40, 20, 9], [190]):
        slot = cache.alloc_slot()
        got = U.run_cuts(model, cache, slot, toks, cuts)
        cache.free_slot(slot)
        assert U.row_error(got, want).max() < U.TOL[dtype], f"cuts {cuts}"


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_over_page_borders(dtype):
    name = "A"
    model, toks = U.engine(name, dtype, "sharp"), U.tokens(name, 330, 4)
    want = U.plain_logits(name, dtype, "sharp", tuple(toks))
    cache = model.new_cache(512, max_slots=1)
    got = U.run_cuts(model, cache, cache.alloc_slot(), toks, [60])      # 270 single tokens over 4 borders
    assert U.row_error(got, want).max() < U.TOL[dtype]


def test_greedy_generation_through_the_entry_point():
    import transformer_amd as ta
    from transformer_amd.engine.generate import generate
    name, dtype = "A", "float32"
    model, plain = U.engine(name, dtype), U.plain(name, dtype)
    prompts = [U.tokens(name, n, 30 + n) for n in (5, 1, 23)]
    res = generate(model, prompts, max_new_tokens=12, sample_args=ta.SampleArgs(), stop_ids=())
    for p, out in zip(prompts, res.tokens):
        assert len(out) == 12
        seq = list(p)
        for t in out:                         # the engine's choice is the plain model's best, or ties with it
            lg = plain.forward(seq)[-1]
            assert lg.max() - lg[t] < 1e-3
            seq.append(t)
    # the next call reuses nothing of the first: same result
    again = generate(model, prompts, max_new_tokens=12, sample_args=ta.SampleArgs(), stop_ids=())
    assert again.tokens == res.tokens


def test_replayer_and_command_line():
    name, dtype = "B", "float32"
    folder = U.folder(name, dtype)
    toks = U.tokens(name, 40, 5)
    want = U.plain_logits(name, dtype, None, tuple(toks))
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    import tempfile
    with tempfile.TemporaryDirectory() as out:
        lines = [{"step": 0, "entries": [{"id": "a", "tokens": toks[:30], "want": [0, 29]},
                                         {"id": "b", "tokens": toks[:1], "want": [0]}], "end": ["b"]}]
        lines += [{"step": 1 + i, "entries": [{"id": "a", "tokens": [toks[30 + i]], "want": [0]}],
                   "end": ["a"] if i == 9 else []} for i in range(10)]
        r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype",
                            dtype, "--out", out, "--max-tokens", "128"],
                           input="\n".join(json.dumps(l) for l in lines) + "\n", capture_output=True, text=True,
                           timeout=600)
        assert r.returncode == 0, r.stderr[-2000:]
        assert [l for l in r.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(11)]
        first = np.fromfile(os.path.join(out, "0.f32"), dtype="<f4").reshape(3, -1)
        assert U.row_error(first, want[[0, 29, 0]]).max() < U.TOL[dtype]
        last = np.fromfile(os.path.join(out, "10.f32"), dtype="<f4").reshape(1, -1)
        assert U.row_error(last, want[39:40]).max() < U.TOL[dtype]
    r = subprocess.run([sys.executable, "-m", "transformer_amd", "generate", "--model", folder, "--dtype", dtype,
                        "--prompt", ",".join(map(str, toks[:6])), "--max-steps", "5"],
                       capture_output=True, text=True, timeout=600, cwd=root)
    assert r.returncode == 0, r.stderr[-2000:]


def test_random_weights_and_save_round_trip():
    import tempfile
    import transformer_amd as ta
    from transformer_amd import Entry
    model = ta.random_model(U.CFG_B, seed=3, dtype="float32", architecture="Vametar")
    toks = U.tokens("B", 20, 6)
    cache = model.new_cache(128)
    a = model.step(cache, [Entry(cache.alloc_slot(), toks, [19])]).cpu().numpy().copy()
    with tempfile.TemporaryDirectory() as d:
        ta.save_model(model, d)
        want = P.PlainVametar(d).forward(toks)[-1:]
        again = ta.load_model(d, "float32")
        cache = again.new_cache(128)
        b = again.step(cache, [Entry(cache.alloc_slot(), toks, [19])]).cpu().numpy()
    assert np.abs(a - b).max() < 1e-6
    assert U.row_error(a, want).max() < U.TOL["float32"]
