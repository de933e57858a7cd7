"""The Kunitar decoder on the GPU against the plain implementation in ``plain_kunitar``.

Each mechanism alone (its kernels against the plain function, with the state carried over a
cut), then the engine: layers, whole prompts, portions, token-by-token decoding, unequal batches,
slots and pages used again, recorded steps, far and edge keys, greedy generation, the replayer."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import kunitar_util as U
import plain_kunitar as P

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = ["float32", "bfloat16"]
TD = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def _t(a, dtype=torch.float32):
    return torch.tensor(np.asarray(a), dtype=dtype, device=DEV)


def _bf(a, dtype="bfloat16"):
    from plain_llama import round_bf16
    a = np.asarray(a, dtype=np.float64)
    return round_bf16(a) if dtype == "bfloat16" else a.astype(np.float32).astype(np.float64)


def _np(t):
    return t.detach().float().cpu().numpy().astype(np.float64)


def _close(got, want, dtype, what=""):
    tol = 3e-5 if dtype == "float32" else 2.5e-2
    assert np.abs(got - want).max() <= tol * max(1.0, np.abs(want).max()), what


# ----------------------------------------------------------------------------- mechanisms alone
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("d", [72, 90, 1024, 4100])
def test_normed_add_with_the_next_norm(dtype, d):
    from transformer_amd import kernels
    rng = np.random.default_rng(d)
    nt = 7
    x, delta = rng.standard_normal((nt, d)), 3.0 * rng.standard_normal((2, nt, d))
    w, w2 = 1 + 0.2 * rng.standard_normal(d), 1 + 0.2 * rng.standard_normal(d)
    xt, out, xc = _t(x), torch.empty(nt, d, dtype=TD[dtype], device=DEV), torch.empty(nt, d, dtype=TD[dtype], device=DEV)
    kernels.postnorm_add(xt, _t(delta), _t(w), 1e-5, xcast=xc, next_weight=_t(w2), next_eps=1e-6, out=out)
    want = x + P.rms_norm(delta.astype(np.float32).astype(np.float64).sum(0), w, 1e-5)
    assert np.abs(_np(xt) - want).max() < 2e-5
    _close(_np(xc), want, dtype)
    _close(_np(out), P.rms_norm(want, w2, 1e-6), dtype)
    xt2 = _t(x)
    kernels.postnorm_add(xt2, _t(delta[0]), _t(w), 1e-5)                   # one plane, nothing else
    assert np.abs(_np(xt2) - (x + P.rms_norm(delta[0], w, 1e-5))).max() < 2e-5


@pytest.mark.parametrize("dtype", DTYPES)
def test_shift_with_several_weights_carries_the_last_row(dtype):
    from transformer_amd import kernels
    rng = np.random.default_rng(1)
    d, lens, n = 52, [5, 1, 9], 5
    mu = rng.uniform(0, 1, (n, d))
    seqs = [_bf(rng.standard_normal((L + 4, d)), dtype) for L in lens]
    state = torch.zeros(6, d, device=DEV)
    state[4] = 7.0                                                          # a slot nobody uses stays as it is
    slots = _t([3, 0, 5], torch.int32)
    got = [[] for _ in lens]
    for part in (lambda L: (0, L), lambda L: (L, L + 1), lambda L: (L + 1, L + 4)):
        rows = [s[slice(*part(L))] for s, L in zip(seqs, lens)]
        h = _t(np.concatenate(rows), TD[dtype])
        cu = _t(np.concatenate([[0], np.cumsum([len(r) for r in rows])]), torch.int32)
        out = torch.empty(n, h.shape[0], d, dtype=TD[dtype], device=DEV)
        kernels.token_shift_multi(h, out, _t(mu), state, cu, slots)
        at = 0
        for i, r in enumerate(rows):
            got[i].append(_np(out[:, at:at + len(r)]))
            at += len(r)
    for i, s in enumerate(seqs):
        prev = np.vstack([np.zeros((1, d)), s[:-1]])
        want = np.stack([s + (prev - s) * mu[j] for j in range(n)])
        _close(np.concatenate(got[i], 1), want, dtype, f"sequence {i}")
    assert float(state[4].min()) == 7.0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", ["gelu", "gelu_tanh", "relu2", "silu"])
def test_activations(dtype, kind):
    from transformer_amd import kernels
    rng = np.random.default_rng(3)
    x = _bf(3 * rng.standard_normal((9, 37)), dtype)
    side = rng.standard_normal((9, 50)).astype(np.float32)
    f = {"gelu": P.gelu_erf, "gelu_tanh": P.gelu_tanh, "relu2": P.relu_squared, "silu": P.silu}[kind]
    out = torch.empty(9, 37, dtype=TD[dtype], device=DEV)
    kernels.activation(_t(x, TD[dtype]), out, kind)
    _close(_np(out), f(x), dtype)
    kernels.activation(_t(x, TD[dtype]), out, kind, side=_t(side)[:, 5:42])
    _close(_np(out), f(x) * side[:, 5:42], dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("geom", [(3, 24, 6), (1, 64, 2), (4, 8, 5), (2, 100, 1), (16, 64, 16)])
def test_bonus_recurrence_pieces(dtype, geom):
    """Decay, recurrence with the state carried over cuts of many, one and two tokens, head norm
    and gate; three sequences of unequal lengths in used slots."""
    from transformer_amd import kernels
    H, n, rank = geom
    rng = np.random.default_rng(H * 100 + n)
    lens, N = [37, 1, 12], H * n
    w2 = _bf(rng.standard_normal((N, rank)) / np.sqrt(rank), dtype)
    w0, u = rng.uniform(-6, 0, N), 0.5 * rng.standard_normal((H, n))
    nw = 1 + 0.2 * rng.standard_normal(N)
    seqs = [dict(rkvg=_bf(rng.standard_normal((4, L + 3, N)), dtype), low=_bf(rng.standard_normal((L + 3, rank)), dtype))
            for L in lens]
    state = torch.full((5, H, n, n), 3.0, device=DEV)
    slots_host = [4, 0, 2]
    for s in slots_host:
        state[s].zero_()
    slots = _t(slots_host, torch.int32)
    got = [[] for _ in lens]
    for part in (lambda L: (0, L), lambda L: (L, L + 1), lambda L: (L + 1, L + 3)):
        sl = [slice(*part(L)) for L in lens]
        rkvg = _t(np.concatenate([s["rkvg"][:, c] for s, c in zip(seqs, sl)], 1), TD[dtype])
        low = _t(np.concatenate([s["low"][c] for s, c in zip(seqs, sl)]), TD[dtype])
        nt = rkvg.shape[1]
        cu = _t(np.concatenate([[0], np.cumsum([c.stop - c.start for c in sl])]), torch.int32)
        o = torch.empty(kernels.gla_row_parts(n), nt, H, n, device=DEV)
        kernels.wkv_recurrent(rkvg, low, H, n, n, _t(w2, TD[dtype]), _t(w0), _t(u), state, cu, slots, o,
                              torch.empty(nt, N, device=DEV))
        out = kernels.head_norm_gate(o, rkvg[3], H, n, _t(nw), 1e-5, torch.empty(nt, N, dtype=TD[dtype], device=DEV))
        at = 0
        for i, c in enumerate(sl):
            got[i].append(_np(out[at:at + c.stop - c.start]))
            at += c.stop - c.start
    for i, (s, L) in enumerate(zip(seqs, lens)):
        T = L + 3
        decay = np.exp(-np.exp(np.tanh(s["low"]) @ w2.T + w0)).reshape(T, H, n)
        r, k, v = (s["rkvg"][j].reshape(T, H, n) for j in range(3))
        o, S = P.wkv_recurrence(r, k, v, decay, u)
        want = P.unit_rms(o, 1e-5).reshape(T, N) * nw * P.silu(s["rkvg"][3])
        _close(np.concatenate(got[i]), want, dtype, f"sequence {i}")
        assert np.abs(_np(state[slots_host[i]]) - S).max() < 1e-3 * max(1.0, np.abs(S).max())
    assert float(state[1].min()) == 3.0 and float(state[3].max()) == 3.0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("geom", [(5, 2, 24, 72, True, 40), (3, 3, 16, 72, False, None), (1, 1, 32, 64, True, 8),
                                  (9, 4, 10, 90, True, 3), (8, 2, 256, 1024, True, 512), (64, 6, 40, 128, False, None)])
def test_routed_feed_forward_pieces(dtype, geom):
    """Router, ordering by expert, the experts' products and the way back, against the plain
    function; chosen experts are checked token by token."""
    import transformer_amd as ta
    from transformer_amd.config.spec import RoutedMLPSpec
    from transformer_amd.parts.base import build_part
    from transformer_amd.parts.linear import Workspace
    E, top, ff, d, shared, sff = geom
    rng = np.random.default_rng(E * 10 + top)
    w = {"router": _bf(2 * rng.standard_normal((E, d)) / np.sqrt(d))}
    for e in range(E):
        w[f"e{e}.up"], w[f"e{e}.down"] = _bf(rng.standard_normal((ff, d)) / np.sqrt(d)), _bf(rng.standard_normal((d, ff)) / np.sqrt(ff))
    if shared:
        w["shared.up"], w["shared.down"] = _bf(rng.standard_normal((sff, d)) / np.sqrt(d)), _bf(rng.standard_normal((d, sff)) / np.sqrt(sff))
        w["shared.sg"] = _bf(rng.standard_normal((1, d)) / np.sqrt(d))
    part = build_part(RoutedMLPSpec(hidden=d, experts=E, top=top, intermediate=ff, shared_intermediate=sff if shared else None),
                      TD[dtype], DEV)
    bound = {"router.weight": np.concatenate([w["router"]] + ([w["shared.sg"]] if shared else [])),
             "experts.up.weight": np.concatenate([w[f"e{e}.up"] for e in range(E)]),
             "experts.down.weight": np.concatenate([w[f"e{e}.down"] for e in range(E)])}
    if shared:
        bound["shared.up.weight"], bound["shared.down.weight"] = w["shared.up"], w["shared.down"]
    part.bind({k: _t(v, TD[dtype]) for k, v in bound.items()})

    class Ctx:
        ws = Workspace(DEV)
    m = {"router": {"top": top}, "shared": {"ff": sff} if shared else None}
    for nt in (1, 5, 77):
        h = _bf(rng.standard_normal((nt, d)), dtype)
        delta, bias = part.run(_t(h, TD[dtype]), Ctx)
        want = P.moe(h, w, "", m)
        chosen = _np(Ctx.ws.take("moe.chosen", (nt, top), torch.int32)).astype(int)
        assert (chosen == P.route(h, w["router"], top)[0]).all()
        _close(_np(delta), want, dtype, f"{nt} tokens")


@pytest.mark.parametrize("form", ["split_k", "direct", "lds"])
@pytest.mark.parametrize("geom", [(5, 3, 40, 72, 700), (3, 1, 264, 200, 300), (16, 2, 130, 136, 90), (2, 2, 64, 64, 5)])
def test_experts_products_in_every_form(form, geom):
    """The three bfloat16 kernels of the experts' products on the same ordered rows: runs of one to
    many tiles per expert, an expert that nobody chose, widths that end inside tiles and steps."""
    from transformer_amd import kernels
    E, top, N, K, nt = geom
    rng = np.random.default_rng(E + nt)
    chosen = np.stack([rng.choice(E - 1 if E > 2 else E, top, replace=False) for _ in range(nt)]).astype(np.int32)
    rows = kernels.moe_max_rows(nt * top, E)
    row_pair = torch.empty(rows, dtype=torch.int32, device=DEV)
    tile_expert = torch.empty(rows // 16, dtype=torch.int32, device=DEV)
    pair_row = torch.empty(nt * top, dtype=torch.int32, device=DEV)
    kernels.moe_plan(_t(chosen, torch.int32), E, row_pair, tile_expert, pair_row)
    h = _bf(rng.standard_normal((nt, K)))
    w = _bf(rng.standard_normal((E, N, K)) / np.sqrt(K))
    a = kernels.moe_gather(_t(h, torch.bfloat16), top, row_pair, None, torch.empty(rows, K, dtype=torch.bfloat16, device=DEV))
    for out_dtype, act in ((torch.float32, None), (torch.bfloat16, "relu2")):
        out = torch.full((rows, N), float("nan"), dtype=out_dtype, device=DEV)
        kernels.moe_gemm(a, _t(w, torch.bfloat16), tile_expert, out, act, form=form)
        got = _np(out)[_np(pair_row).astype(int)].reshape(nt, top, N)
        want = np.einsum("tk,tjnk->tjn", h, w[chosen])
        if act:
            want = P.relu_squared(want)
        _close(got, want, "bfloat16" if out_dtype == torch.bfloat16 else "float32", f"{out_dtype}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("geom", [(3, 20, 8, 8, 48, 33), (1, 16, 16, 16, 16, 1), (5, 7, 6, 4, 19, 9), (2, 12, 8, 8, 48, None),
                                  (8, 64, 32, 32, 128, 150), (4, 16, 0, 0, 300, 70)])
def test_latent_attention_pieces(dtype, geom):
    """The whole mixer (first product, norms, rotation, cache rows, per-head maps, attention,
    gate) of one layer against the plain function: a prompt over several pages, a portion of two
    tokens, then single tokens, in pages that were used before."""
    from transformer_amd.cache.storage import SequenceCache
    from transformer_amd.config.spec import LatentAttentionSpec
    from transformer_amd.engine.batch import Entry, Uploader, plan_step
    from transformer_amd.parts.base import build_part
    from transformer_amd.parts.linear import Workspace
    H, dn, dr, dims, r, window = geom
    d, dv, qr = 56, dn + 3, r // 2 + 5
    rng = np.random.default_rng(H + r)
    spec = LatentAttentionSpec(hidden=d, num_heads=H, nope_dim=dn, rope_dim=dr, value_dim=dv, q_rank=qr, kv_rank=r,
                               scale=0.3, eps=1e-5, rot_dims=dims, rot_base=500.0, window=window, cache_window=window)
    part = build_part(spec, TD[dtype], DEV)
    w = {"dq": rng.standard_normal((qr, d)) / np.sqrt(d), "dkv": rng.standard_normal((r + dr, d)) / np.sqrt(d),
         "g": rng.standard_normal((H, d)) / np.sqrt(d), "dq.norm": 1 + 0.2 * rng.standard_normal(qr),
         "dkv.norm": 1 + 0.2 * rng.standard_normal(r), "uq": 4 * rng.standard_normal((H * (dn + dr), qr)) / np.sqrt(qr),
         "uk": rng.standard_normal((H * dn, r)) / np.sqrt(r), "uv": rng.standard_normal((H * dv, r)) / np.sqrt(r),
         "o": rng.standard_normal((d, H * dv)) / np.sqrt(H * dv)}
    w = {k: _bf(v) for k, v in w.items()}
    mat = TD[dtype]
    part.bind({"in.weight": _t(np.concatenate([w["dq"], w["dkv"], w["g"]]), mat), "q_norm.weight": _t(w["dq.norm"]),
               "kv_norm.weight": _t(w["dkv.norm"]), "uq.weight": _t(w["uq"], mat), "uk.weight": _t(w["uk"], mat),
               "uv.weight": _t(w["uv"], mat), "out.weight": _t(w["o"], mat)})
    cache = SequenceCache([part.cache_need()], 1024, 3, TD[dtype], DEV)
    cache.keys[0].fill_(float("nan"))                                     # whatever is read unwritten shows
    junk = cache.alloc_slot()
    ws, up = Workspace(DEV), Uploader(DEV)
    T = 200
    h = _bf(rng.standard_normal((T, d)), dtype)
    m = {"heads": H, "dim": dn, "rot_dim": dr, "vdim": dv, "kv_rank": r, "scale": 0.3, "rot": {"base": 500.0, "dims": dims},
         "mask": None if window is None else {"size": window}}
    kv = P.latent_kv(h, w, "", m, 1e-5, np.arange(T))
    want = P.latent_attention(h, w, "", m, 1e-5, np.arange(T), kv)
    slot = cache.alloc_slot()
    got, at = [], 0
    for n in [150, 2] + [1] * 48:
        entries = [Entry(slot, [0] * n, [])]
        ctx = plan_step(entries, cache, 10, up, ws)
        delta, _ = part.run(_t(h[at:at + n], TD[dtype]), ctx, cache, 0, True)
        got.append(_np(delta if delta.dim() == 2 else delta.sum(0)))
        cache.pool.advance(slot, n)
        cache.release_outside_windows(slot)
        at += n
    _close(np.concatenate(got), want, dtype)
    cache.pool.check()


@pytest.mark.parametrize("geom", [(3, 48, 8, 33), (2, 16, 0, 1), (5, 19, 6, None), (16, 128, 32, 150), (4, 300, 4, 70),
                                  (2, 512, 64, 100), (7, 200, 64, 40)])
def test_latent_attention_kernels_agree(geom):
    """The matrix-core kernels (a workgroup's waves sharing their chunks, for steps of many rows; a wave
    alone, with a row's keys dealt to one, three and seven waves) against the float32 kernel on the
    same bfloat16 values: sequences of unequal lengths that go on from unequal starts, in pages
    handed out in a scrambled order, with a gate."""
    from transformer_amd import kernels
    from transformer_amd.cache.storage import PAGE
    H, r, dr, window = geom
    rng = np.random.default_rng(H * 1000 + r)
    W = kernels.latent_row_width(r, dr, torch.bfloat16)
    starts, lens = [0, 130, 65, 7], [90, 75, 1, 140]
    total = sum(lens)
    npages = sum(-(-(a + n) // PAGE) for a, n in zip(starts, lens))
    order = rng.permutation(npages)
    table = np.zeros((len(lens), max(-(-(a + n) // PAGE) for a, n in zip(starts, lens))), dtype=np.int32)
    at = 0
    for i, (a, n) in enumerate(zip(starts, lens)):
        k = -(-(a + n) // PAGE)
        table[i, :k] = order[at:at + k]
        at += k
    rows = _bf(rng.standard_normal((npages + 1, 1, PAGE, W)))
    rows[..., r + dr:] = 0.0
    qa = _bf(2.0 * rng.standard_normal((total, H, W)))
    qa[..., r + dr:] = 0.0
    gate = _bf(rng.standard_normal((total, H + 3)))
    cu = _t(np.concatenate([[0], np.cumsum(lens)]), torch.int32)
    args = (_t(table, torch.int32), cu, _t(starts, torch.int32), max(lens), r, dr, 0.2, window)
    want = torch.empty(total, H, r, device=DEV)
    kernels.latent_attention(_t(qa[..., :r + dr]), want, _t(rows[..., :r + dr]), *args, gate=_t(gate)[:, 2:])
    for shares in (1, 3, 7):
        out = torch.full((total, H, r), float("nan"), dtype=torch.bfloat16, device=DEV)
        kernels.latent_attention(_t(qa, torch.bfloat16), out, _t(rows, torch.bfloat16), *args,
                                 gate=_t(gate, torch.bfloat16)[:, 2:], shares=shares)
        _close(_np(out), _np(want), "bfloat16", f"{shares} shares")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("where", ["prompt", "decode"])
def test_far_key_and_window_edges_stand_out(where, dtype):
    """One key is made to dominate the softmax: the last key inside the window, then the first
    one outside it (which must not count), then a key hundreds of tokens back without a window.
    The cached rows and the queries are written by hand so that nothing else hides a miss."""
    from transformer_amd import kernels
    from transformer_amd.cache.storage import PAGE
    r, dr, H, T = 24, 4, 2, 300
    D = r + dr
    rng = np.random.default_rng(5)
    rows = _bf(rng.standard_normal((T, D)), dtype)
    pages = np.arange(8)[::-1].copy()                                     # the sequence's pages in reverse order
    W = D if dtype == "float32" else 32                                   # bfloat16 rows are padded to 16-byte pieces
    kc = torch.zeros(9, 1, PAGE, W, dtype=TD[dtype], device=DEV)
    for t in range(T):
        kc[pages[t // PAGE], 0, t % PAGE, :D] = _t(rows[t], TD[dtype])
    table = _t(pages[None, :], torch.int32)
    for window, mark, counts in ((40, T - 40, True), (40, T - 41, False), (None, 7, True)):
        qa = np.zeros((1, H, W))
        qa[0, :, :D] = _bf(6.0 * rows[mark] / np.linalg.norm(rows[mark]), dtype)   # points at the marked key
        lo = 0 if window is None else T - window
        s = rows[lo:T] @ qa[0, :, :D].T * 1.0
        p = np.exp(s - s.max(0))
        want = (p / p.sum(0)).T @ rows[lo:T, :r]
        if where == "decode":
            cu, pos0, q, nq = _t([0, 1], torch.int32), _t([T - 1], torch.int32), _t(qa, TD[dtype]), 1
        else:                                                             # the last of a portion of 70 tokens
            nq = 70
            q = torch.zeros(nq, H, W, dtype=TD[dtype], device=DEV)
            q[-1] = _t(qa[0], TD[dtype])
            cu, pos0 = _t([0, nq], torch.int32), _t([T - nq], torch.int32)
        out = torch.empty(nq, H, r, dtype=TD[dtype], device=DEV)
        shares = 3 if where == "decode" else 1                            # the keys dealt to three waves
        kernels.latent_attention(q, out, kc, table, cu, pos0, nq, r, dr, 1.0, window, shares=shares)
        got = _np(out[-1])
        assert np.abs(got - want).max() < (1e-4 if dtype == "float32" else 2e-2)
        weight_of_mark = np.abs(got - rows[mark, :r]).max() < 0.35 * np.abs(rows[mark, :r]).max()
        assert weight_of_mark == counts, (window, mark)


# ----------------------------------------------------------------------------- the engine
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "D"])
def test_layers_and_whole_prompt(name, dtype):
    from transformer_amd import Entry
    model, toks = U.engine(name, dtype), U.tokens(name, 90, 1)
    dumps = {}
    model.dump = lambda n, t: dumps.__setitem__(n, t.detach().float().cpu().numpy().copy())
    try:
        cache = model.new_cache(256)
        got = model.step(cache, [Entry(cache.alloc_slot(), toks, list(range(len(toks))))]).cpu().numpy()
    finally:
        model.dump = None
    layers = []
    routes = None if dtype == "float32" else \
        {int(n.split(".")[1]): t.astype(np.int64) for n, t in dumps.items() if n.endswith(".experts")}
    want = U.plain(name, dtype).forward(toks, layers, routes=routes)
    tol = 1e-4 if dtype == "float32" else 0.15
    for i, l in enumerate(layers):
        assert np.abs(dumps[f"run.{i}"] - l).max() < tol * max(1.0, np.abs(l).max()), f"layer {i}"
    assert U.row_error(got, want).max() < U.TOL[dtype]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,edit", [("A", None), ("B", None), ("D", None), ("A", "slow"), ("A", "sharp"), ("D", "sharp")])
def test_cuts_agree_with_plain(name, edit, dtype):
    """Whole, portions down to two tokens, and every token alone: all against the plain model."""
    if (name, edit, dtype) == ("D", "sharp", "bfloat16"):
        pytest.skip("widths of a few coordinates and a softmax this peaked: bfloat16 rounding of q and k "
                    "decides which key wins; the float32 run holds the case")
    model, toks, EDIT = U.engine(name, dtype, edit), U.tokens(name, 150, 2), edit
    cache = model.new_cache(512, max_slots=3)
    for cuts in ([150], [2, 2, 61, 3, 64, 17], [130], []):
        slot = cache.alloc_slot()
        got, routes = U.run_cuts(model, cache, slot, toks, cuts, routes=True)
        cache.free_slot(slot)                      # the next cut takes the same slot and pages
        U.check_against_plain(name, dtype, EDIT, toks, got, routes, f"cuts {cuts}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_prompt_in_portions_over_windows_and_pages(dtype):
    """400 tokens: windows of 33, 70 and 20 pass over page borders, pages that left every window
    go back to the pool, portions end at and around the recurrence's chunks of 8 and 32."""
    name = "A"
    model, toks, EDIT = U.engine(name, dtype, "sharp"), U.tokens(name, 400, 7), "sharp"
    cache = model.new_cache(512, max_slots=1)
    for cuts in ([400], [257, 63, 65, 15], [64, 256, 33, 31, 16], [255, 129, 8, 7, 1]):
        slot = cache.alloc_slot()
        got, routes = U.run_cuts(model, cache, slot, toks, cuts, routes=True)
        cache.free_slot(slot)                      # the next cut takes the same slot and pages
        U.check_against_plain(name, dtype, EDIT, toks, got, routes, f"cuts {cuts}")
    cache.pool.check()


@pytest.mark.parametrize("dtype", DTYPES)
def test_unequal_batch_then_decoding_in_used_slots(dtype):
    from transformer_amd import Entry
    name = "A"
    model = U.engine(name, dtype)
    cache = model.new_cache(1024, max_slots=4)
    old = [cache.alloc_slot() for _ in range(4)]          # a first batch dirties every slot and page, then leaves
    model.step(cache, [Entry(s, U.tokens(name, 100 + 7 * s, 50 + s), [0]) for s in old])
    for s in old:
        cache.free_slot(s)
    lens = [1, 70, 131, 2]
    seqs = [U.tokens(name, n + 40, 10 + i) for i, n in enumerate(lens)]
    slots = [cache.alloc_slot() for _ in seqs]
    got, rows = [[] for _ in seqs], [[] for _ in seqs]
    graphs = dtype == "float32"                    # float32: recorded steps, the plain model's own routing
    rec = U.Routes(model)
    if not graphs:
        rec.__enter__()
    try:
        lg = model.step(cache, [Entry(sl, s[:n], list(range(n))) for sl, s, n in zip(slots, seqs, lens)]).cpu().numpy()
        at = 0
        for i, n in enumerate(lens):
            got[i].append(lg[at:at + n].copy())
            rows[i].append(slice(at, at + n))
            at += n
        live = list(range(len(seqs)))
        for step in range(40):
            if step == 25:                             # one sequence leaves early, its slot is taken again
                cache.free_slot(slots[1])
                live.remove(1)
                slots[1] = cache.alloc_slot()
            rec.next_step()
            lg = model.step(cache, [Entry(slots[i], [seqs[i][lens[i] + step]], [0]) for i in live]).cpu().numpy()
            for i in range(len(seqs)):
                rows[i].append(slice(live.index(i), live.index(i) + 1) if i in live else None)
            for j, i in enumerate(live):
                got[i].append(lg[j:j + 1].copy())
    finally:
        if not graphs:
            rec.__exit__()
    for i in range(len(seqs)):
        U.check_against_plain(name, dtype, None, seqs[i], np.concatenate(got[i]),
                              None if graphs else rec.of_rows(rows[i]), f"sequence {i}")
    cache.pool.check()


@pytest.mark.parametrize("dtype", DTYPES)
def test_recorded_steps_match_eager_steps(dtype):
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
    assert np.abs(outs[0] - outs[1]).max() < (1e-5 if dtype == "float32" else 3e-2) * np.abs(outs[1]).max()
    if dtype == "float32":          # bfloat16 against the plain model: the tests that follow the engine's routing
        want = np.stack([U.plain_logits(name, dtype, None, tuple(s)) for s in seqs], 1)
        assert U.row_error(outs[0], want).max() < U.TOL[dtype]


@pytest.mark.parametrize("dtype", DTYPES)
def test_wide_model_in_three_cuts(dtype):
    """Width 1024: the experts' products run on the matrix cores, products of 17 to 64 rows leave
    planes, prompts go to the library, single tokens to the few-rows products; windows of 150
    and 100 over the borders of pages."""
    name = "C"
    model, toks, EDIT = U.engine(name, dtype), U.tokens(name, 260, 3), None
    cache = model.new_cache(512, max_slots=2)
    for cuts in ([260], [100, 40, 70, 20, 9], [250]):
        slot = cache.alloc_slot()
        got, routes = U.run_cuts(model, cache, slot, toks, cuts, routes=True)
        cache.free_slot(slot)                      # the next cut takes the same slot and pages
        U.check_against_plain(name, dtype, EDIT, toks, got, routes, f"cuts {cuts}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_over_page_borders(dtype):
    name = "A"
    model, toks = U.engine(name, dtype, "slow"), U.tokens(name, 330, 4)
    cache = model.new_cache(512, max_slots=1)
    slot = cache.alloc_slot()
    got, routes = U.run_cuts(model, cache, slot, toks, [60], routes=True)   # 270 single tokens over 4 borders
    U.check_against_plain(name, dtype, "slow", toks, got, routes)
    if dtype == "float32":                            # once more as generation runs it: recorded steps
        cache.free_slot(slot)
        got = U.run_cuts(model, cache, cache.alloc_slot(), toks, [60])
        U.check_against_plain(name, dtype, "slow", toks, got)


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
    model = ta.random_model(U.CFG_B, seed=3, dtype="float32", architecture="Kunitar")
    toks = U.tokens("B", 20, 6)
    cache = model.new_cache(128)
    a = model.step(cache, [Entry(cache.alloc_slot(), toks, [19])]).cpu().numpy().copy()
    with tempfile.TemporaryDirectory() as d:
        ta.save_model(model, d)
        want = P.PlainKunitar(d).forward(toks)[-1:]
        again = ta.load_model(d, "float32")
        cache = again.new_cache(128)
        b = again.step(cache, [Entry(cache.alloc_slot(), toks, [19])]).cpu().numpy()
    assert np.abs(a - b).max() < 1e-6 * max(1.0, np.abs(a).max())
    assert U.row_error(a, want).max() < U.TOL["float32"]


def _draw_config(case):
    """A random Kunitar configuration: any order of the two mixers, readers of earlier layers' rows
    with windows of their own, every kind of feed-forward or none, sizes that are odd or no power
    of two."""
    r = np.random.default_rng(case)
    width = int(r.choice([40, 66, 100, 136, 33, 257]))
    layers, sources = [], []
    for i in range(int(r.integers(1, 6))):
        mlp = [None, U._dense(int(r.choice([24, 57, 130]))),
               U._moe(int(r.choice([1, 2, 5, 9, 16])), 1, int(r.choice([8, 20, 33])),
                      shared=None if r.integers(0, 2) else int(r.choice([6, 24])))][int(r.integers(0, 3))]
        if mlp is not None and mlp["kind"] == "moe":
            mlp["router"]["top"] = int(r.integers(1, mlp["router"]["experts"] + 1))
        if r.integers(0, 2):
            layers.append(U._wkv(int(r.choice([1, 2, 3, 5])), int(r.choice([8, 12, 20, 32, 40])), int(r.choice([1, 3, 8])), mlp))
            continue
        window = None if r.integers(0, 4) == 0 else int(r.choice([1, 2, 7, 31, 64, 65, 100]))
        if sources and r.integers(0, 2):
            j = int(r.choice(sources))
            m = layers[j]["mixer"]
            layers.append(U._lat(int(r.choice([1, 2, 4, 7])), int(r.choice([4, 10, 16, 24])), m["rot_dim"], int(r.choice([6, 16, 30])),
                                 int(r.choice([8, 20, 48])), m["kv_rank"], float(r.choice([0.1, 0.25])), m["rot"]["base"],
                                 window=window, kv_from=j, mlp=mlp, dims=m["rot"]["dims"]))
            continue
        rot_dim = int(r.choice([2, 4, 8, 10, 16]))
        sources.append(i)
        layers.append(U._lat(int(r.choice([1, 2, 3, 6])), int(r.choice([4, 10, 16, 24])), rot_dim, int(r.choice([6, 16, 30])),
                             int(r.choice([8, 20, 48])), int(r.choice([8, 24, 40, 72])), float(r.choice([0.1, 0.25])),
                             float(r.choice([100.0, 1e4, 5e5])), window=window, mlp=mlp,
                             dims=rot_dim if r.integers(0, 2) else 2 * int(r.integers(1, rot_dim // 2 + 1))))
    cfg = {"architecture": "Kunitar", "vocab": int(r.choice([5, 97, 300, 1001])), "width": width,
           "norm": {"eps": float(r.choice([1e-6, 1e-5, 1e-3]))}, "embedding": {"scale": float(r.choice([1.0, 0.5, 3.0]))},
           "layers": layers}
    if r.integers(0, 3):
        cfg["token_side"] = {"dim": int(r.choice([1, 4, 7, 16]))}
    lens = [int(x) for x in r.integers(1, 150, size=int(r.integers(1, 5)))]
    return cfg, lens, r


@pytest.mark.parametrize("first", [2000, 2006, 2012])
def test_random_configurations_against_the_plain_model(first):
    """float32, the plain model's own routing, every row: a batch of unequal prompts in one step into
    poisoned pages, then eight single tokens each (recorded steps)."""
    import tempfile
    import transformer_amd as ta
    from gpu_util import poison
    for case in range(first, first + 6):
        cfg, lens, r = _draw_config(case)
        with tempfile.TemporaryDirectory(prefix="ku_rand_") as d:
            P.make_model_folder(d, cfg, case, storage="F32")
            ref = P.PlainKunitar(d)
            model = ta.load_model(d, "float32", "cuda:0")
        toks = [[int(t) for t in r.integers(0, cfg["vocab"], size=n + 8)] for n in lens]
        cache = model.new_cache(64 * sum(-(-(n + 8) // 64) for n in lens), max_slots=len(lens))
        poison(cache)
        slots = [cache.alloc_slot() for _ in lens]
        want = [ref.forward(t) for t in toks]
        what = f"case {case} {json.dumps(cfg)} prompts {lens}"
        got = model.step(cache, [ta.Entry(s, t[:n], [n - 1]) for s, t, n in zip(slots, toks, lens)]).cpu().numpy()
        for i, n in enumerate(lens):
            assert U.row_error(got[i], want[i][n - 1]) < U.TOL["float32"], what
        for j in range(8):
            got = model.step(cache, [ta.Entry(s, [t[n + j]], [0]) for s, t, n in zip(slots, toks, lens)]).cpu().numpy()
            for i, n in enumerate(lens):
                assert U.row_error(got[i], want[i][n + j]) < U.TOL["float32"], (what, j)
        for s in slots:
            cache.free_slot(s)
        cache.pool.check()
        # the same in bfloat16 (matrix cores, odd widths): rows are finite, and all but the few that a
        # close call between two experts moves lie within rounding of the plain model
        with tempfile.TemporaryDirectory(prefix="ku_rand_") as d:
            P.make_model_folder(d, cfg, case, storage="BF16")
            model = ta.load_model(d, "bfloat16", "cuda:0")
        cache = model.new_cache(64 * sum(-(-(n + 8) // 64) for n in lens), max_slots=len(lens))
        poison(cache)
        slots = [cache.alloc_slot() for _ in lens]
        errs = []
        got = model.step(cache, [ta.Entry(s, t[:n], list(range(n))) for s, t, n in zip(slots, toks, lens)]).cpu().numpy()
        at = 0
        for i, n in enumerate(lens):
            errs += list(U.row_error(got[at:at + n], want[i][:n]))
            at += n
        for j in range(8):
            got = model.step(cache, [ta.Entry(s, [t[n + j]], [0]) for s, t, n in zip(slots, toks, lens)]).cpu().numpy()
            errs += [U.row_error(got[i], want[i][n + j]) for i, n in enumerate(lens)]
        errs = np.asarray(errs)
        assert np.isfinite(errs).all() and np.median(errs) < U.TOL["bfloat16"], (what, np.median(errs))
