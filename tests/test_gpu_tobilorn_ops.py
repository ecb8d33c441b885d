"""The mechanisms of the Tobilorn design, each alone, against the float64 restatement in oracle/tobilorn.py: the offset norm and the
fused residual step, table rows with a scale, differential grouped-query attention (two maps, half-split rotation, biases, window
with kept first keys, pages, several runs with a cache each), the routed feed-forward (score routing with a correction, identity
experts, a shared expert) and the per-layer token input."""
import math

import numpy as np
import pytest
import torch

from oracle import tobilorn as ot
from tests.conftest import load_pkg
from tests.seq_helpers import MixerRig, dev_weights, rel_err

pytestmark = pytest.mark.gpu
bf = ot.bf16_values


@pytest.fixture(scope="module")
def so():
    load_pkg()
    from dash_infer_amd import seq_ops
    return seq_ops


def dev(a, dt=torch.float32):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(dt).cuda()


def i32(a):
    return torch.tensor(a, dtype=torch.int32, device="cuda")


# ---------------------------------------------------------------------------------------------------------------- norms, tables
def test_offset_norm_with_rows_and_scale(so):
    rng = np.random.default_rng(0)
    T, K = 29, 100
    x = rng.normal(0, 2.0, (T, K)).astype(np.float32)
    w = bf(0.3 * rng.normal(size=K))
    rows = [3, 0, 28, 3]
    got = so.rmsnorm(dev(x), dev(w, torch.bfloat16), 1e-4, row_idx=i32(rows), gamma_add=1.0, out_scale=0.625)
    assert rel_err(got.cpu().numpy(), ot.offset_norm(x, w, 1e-4)[rows] * 0.625) < 2e-6
    plain = so.rmsnorm(dev(x), dev(w), 1e-4)                                # the plain weight is what it was
    assert rel_err(plain.cpu().numpy(), ot.unit_rms(x, 1e-4) * w) < 2e-6


@pytest.mark.parametrize("K", [72, 1024 + 41, 5000])     # a row in registers, the generic kernel (no multiple of 4), the widest register form
def test_residual_step_fused_with_the_next_norm(so, K):
    rng = np.random.default_rng(1)
    T, eps = 19, 1e-5
    x, m = rng.normal(0, 1.5, (T, K)).astype(np.float32), rng.normal(0, 0.2, (T, K)).astype(np.float32)
    gm, gh = bf(0.2 * rng.normal(size=K)), bf(0.2 * rng.normal(size=K))
    xo = x.astype(np.float64) + ot.offset_norm(m, gm, eps)
    want_h = ot.offset_norm(xo, gh, eps)
    wide = dev(np.concatenate([m, m], 1))                                   # the sublayer's output as a column slice
    xd, h = dev(x), torch.empty(T, K, device="cuda")
    pair = torch.zeros(T, 2 * K, device="cuda")
    out = so.residual_norm_step(xd, eps, m=wide[:, K:], gamma_m=dev(gm, torch.bfloat16), add_m=1.0, gamma_h=dev(gh, torch.bfloat16), add_h=1.0,
                                h=h, copy=pair[:, :K])
    assert out.data_ptr() == xd.data_ptr()                                  # in place
    assert rel_err(xd.cpu().numpy(), xo) < 1e-6 and rel_err(h.cpu().numpy(), want_h) < 3e-6
    assert torch.equal(pair[:, :K], xd) and float(pair[:, K:].abs().max()) == 0.0
    # bf16 outputs are the roundings of the f32 ones; a plain weight on the sublayer's output; no next norm
    xd2, h16, c16 = dev(x), torch.empty(T, K, dtype=torch.bfloat16, device="cuda"), torch.empty(T, K, dtype=torch.bfloat16, device="cuda")
    so.residual_norm_step(xd2, eps, m=dev(m), gamma_m=dev(gm), add_m=1.0, gamma_h=dev(gh), add_h=1.0, h=h16, copy=c16)
    assert torch.equal(h16, h.to(torch.bfloat16)) and torch.equal(c16, xd2.to(torch.bfloat16))
    xd3 = dev(x)
    so.residual_norm_step(xd3, eps, m=dev(m), gamma_m=dev(gm), add_m=0.0)
    assert rel_err(xd3.cpu().numpy(), x.astype(np.float64) + ot.unit_rms(m, eps) * gm) < 1e-6
    # no sublayer output: the norm alone, the stream untouched
    xd4, h4 = dev(x), torch.empty(T, K, device="cuda")
    assert so.residual_norm_step(xd4, eps, gamma_h=dev(gh), add_h=1.0, h=h4).data_ptr() == xd4.data_ptr()
    assert torch.equal(xd4, dev(x)) and rel_err(h4.cpu().numpy(), ot.offset_norm(x, gh, eps)) < 3e-6


def test_table_rows_with_scale_and_columns(so):
    rng = np.random.default_rng(2)
    table = bf(rng.normal(size=(11, 30)))
    ids = [4, 0, 10, 4, 7]
    got = so.embed_rows(i32(ids), dev(table, torch.bfloat16), scale=3.5)
    assert np.allclose(got.cpu().numpy(), table[ids] * np.float32(3.5), rtol=1e-7, atol=0)
    wide = torch.zeros(5, 16, device="cuda")
    so.embed_rows(i32(ids), dev(table, torch.bfloat16), col0=12, cols=6, out=wide[:, 10:])
    assert np.array_equal(wide[:, 10:].cpu().numpy(), table[ids][:, 12:18]) and float(wide[:, :10].abs().max()) == 0.0
    b16 = torch.empty(5, 30, dtype=torch.bfloat16, device="cuda")
    so.embed_rows(i32(ids), dev(table), scale=0.5, out=b16)
    assert torch.equal(b16.cpu(), torch.from_numpy(table[ids] * np.float32(0.5)).to(torch.bfloat16))


def test_two_maps_to_one(so):
    rng = np.random.default_rng(3)
    T, H, V = 13, 3, 70
    x = rng.normal(size=(T, H, 2, V)).astype(np.float32)
    lam, sc, eps = 0.8125, 0.75, 1e-5
    want = ot.unit_rms(x[:, :, 0].astype(np.float64) - lam * x[:, :, 1], eps) * sc
    got = so.maps_diff_norm(dev(x.reshape(T, -1)), lam, sc, eps, H, V)
    assert rel_err(got.cpu().numpy(), want.reshape(T, -1)) < 2e-6
    o16 = torch.empty(T, H * V, dtype=torch.bfloat16, device="cuda")
    so.maps_diff_norm(dev(x.reshape(T, -1)), lam, sc, eps, H, V, out=o16)
    assert torch.equal(o16, got.to(torch.bfloat16))


# ---------------------------------------------------------------------------------------------------------------- attention
def attention_weights(rng, width, H, G, D, V, aligned=False):
    r = lambda *s, sd=None: bf(rng.normal(0, sd if sd is not None else 1.0 / math.sqrt(s[-1]), s))
    w = {"q": r(H * 2 * D, width), "k": r(G * 2 * D, width), "v": r(G * V, width), "o": r(width, H * V), "o.b": bf(0.1 * rng.normal(size=width)),
         "q.b": bf(0.2 * rng.normal(size=H * 2 * D)), "k.b": bf(0.2 * rng.normal(size=G * 2 * D)), "v.b": bf(0.2 * rng.normal(size=G * V))}
    for nm in ("lq1", "lk1", "lq2", "lk2"):
        w[nm] = bf(rng.normal(0, 0.6 / math.sqrt(D), D))
    if aligned:     # every query map projects as the key map it reads: rows of the same direction score high on each other
        q = w["k"].reshape(G, 2, D, width)[np.arange(H) // (H // G)]
        w["q"] = np.ascontiguousarray(q).reshape(H * 2 * D, width)
        w["q.b"], w["k.b"] = 0 * w["q.b"], 0 * w["k.b"]
    return w


def mixer_config(H, G, D, V, rot_dims, window, keep, diff=0.25, scale=None, base=10000.0):
    return {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "diff": diff, "scale": scale if scale is not None else D ** -0.5,
            "mask": {"size": window, "keep_first": keep}, "rot": {"dims": rot_dims, "base": base}}


def attention_rig(w, m, dtype, runs=1, **kw):
    load_pkg()
    from dash_infer_amd import mixers
    lam = ot.differential_lambda(w, m["diff"])
    build = lambda state, dt: mixers.GroupedQueryAttention(
        "t", m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["scale"], dev_weights(w), state, dt, rot_dims=m["rot"]["dims"],
        rot_base=m["rot"]["base"], rot_layout="halves", window=m["mask"]["size"], keep_first=m["mask"]["keep_first"],
        differential=(lam, 1.0 - m["diff"]), runs=runs)
    return MixerRig(build, dtype, **kw)


SHAPES = [  # width, heads, kv heads, dim, vdim, rotated dims, window, kept first
    (72, 6, 2, 24, 16, 24, 40, 5),       # head sizes that are no multiple of 32 / 16
    (64, 4, 4, 32, 32, 16, 64, 64),      # as many key/value heads as query heads, half of the map rotated, the window one page
    (80, 5, 1, 40, 8, 40, 1, 3),         # one key/value head, an odd number of query heads, a window of the row itself
    (60, 3, 1, 20, 12, 8, 33, 0),        # head sizes the matrix-core form does not serve, no kept keys
    (64, 2, 1, 64, 128, 64, 1000, 2),    # the widest value tiles, a window that never binds
]


@pytest.mark.parametrize("shape", SHAPES)
def test_differential_attention_against_the_oracle(shape):
    width, H, G, D, V, rd, window, keep = shape
    rng = np.random.default_rng(H * 100 + D)
    w = attention_weights(rng, width, H, G, D, V)
    m = mixer_config(H, G, D, V, rd, window, keep)
    n = 150
    h = bf(rng.normal(size=(n, width)))
    want = ot.differential_attention(h, w, m, 1e-5)
    rig = attention_rig(w, m, torch.float32)
    assert rel_err(rig.step([("a", h)])[0], want) < 3e-5
    cut = np.concatenate([rig.step([("b", h[:70])])[0], rig.step([("b", h[70:72])])[0], rig.step([("b", h[72:])])[0]])
    assert rel_err(cut, want) < 3e-5
    one = np.concatenate([rig.step([("c", h[:130])])[0]] + [rig.step([("c", h[i:i + 1])])[0] for i in range(130, n)])
    assert rel_err(one, want) < 3e-5
    rig16 = attention_rig(w, m, torch.bfloat16)
    got16 = rig16.step([("a", h)])[0]
    assert rel_err(got16, want) < 0.04, rel_err(got16, want)
    one16 = np.concatenate([rig16.step([("c", h[:130])])[0]] + [rig16.step([("c", h[i:i + 1])])[0] for i in range(130, n)])
    assert rel_err(one16, want) < 0.04                                      # one row at a time: the key walk is split


def test_two_maps_are_two_softmaxes_over_the_same_values():
    """lambda = 0 leaves the first map alone: with diff = 0 and the four lambda vectors zero, lambda = exp(0) - exp(0) + 0"""
    rng = np.random.default_rng(5)
    width, H, G, D, V = 48, 4, 2, 16, 24
    w = attention_weights(rng, width, H, G, D, V)
    for nm in ("lq1", "lk1", "lq2", "lk2"):
        w[nm] = 0 * w[nm]
    m = mixer_config(H, G, D, V, 16, 30, 4, diff=0.0)
    h = bf(rng.normal(size=(90, width)))
    maps = []
    want = ot.differential_attention(h, w, m, 1e-5, maps_out=maps)
    first = np.stack([ot.unit_rms(a1, 1e-5) for a1, _ in maps], 1).reshape(90, H * V) @ np.asarray(w["o"], np.float64).T + w["o.b"]
    assert np.allclose(want, first)
    assert rel_err(attention_rig(w, m, torch.float32).step([("a", h)])[0], want) < 3e-5


def marked_rows(rng, n, width, reader, marker=None):
    """small random rows; the reading row points along u, the marked row more strongly along u and along a second direction that
    gives it values of its own (the output is normed per head: a key with the reader's own values would not show)"""
    u, u2 = rng.normal(size=width), rng.normal(size=width)
    u, u2 = u / np.linalg.norm(u), u2 / np.linalg.norm(u2)
    h = 0.3 * rng.normal(size=(n, width))
    h[reader] = 4.0 * u
    if marker is not None:
        h[marker] = 8.0 * u + 8.0 * u2
    return bf(h)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("edge", ["window", "first", "page"])
def test_a_key_just_inside_and_just_outside(dtype, edge):
    """Queries and keys project alike (and mostly unrotated), so a marked row far back takes a large share of the softmax of a later
    marked row -- if the mask lets it.  The marked key stands just inside and just outside the window / the kept first keys, and on
    both sides of a page border; the reading row comes in a prompt's portion and decoded alone."""
    rng = np.random.default_rng(11)
    width, H, G, D, V, window, keep = 64, 4, 2, 32, 16, 70, 6
    w = attention_weights(rng, width, H, G, D, V, aligned=True)
    m = mixer_config(H, G, D, V, 8, window, keep, scale=1.0)
    i = 200                                                                  # the reading row, in the fourth page
    cases = {"window": [i - window + 1, i - window], "first": [keep - 1, keep], "page": [191, 192, 127, 128, 64, 63]}[edge]
    inside = {"window": [True, False], "first": [True, False], "page": [True, True, False, False, False, False]}[edge]
    plain = ot.differential_attention(marked_rows(np.random.default_rng(3), i + 1, width, i), w, m, 1e-5)[i]
    tol = 5e-5 if dtype == torch.float32 else 0.05
    rig = attention_rig(w, m, dtype)
    for j, seen in zip(cases, inside):
        h = marked_rows(np.random.default_rng(3), i + 1, width, i, j)
        want = ot.differential_attention(h, w, m, 1e-5)
        moved = rel_err(want[i], plain)
        assert (moved > 0.1) if seen else (moved < 1e-9), (j, moved)         # the oracle itself: the key counts, or not at all
        whole = rig.step([("w", h)])[0]
        rig.release("w")
        assert rel_err(whole[i], want[i]) < tol and rel_err(whole, want) < tol, (j, rel_err(whole, want))
        rig.step([("d", h[:i - 1])])
        rig.step([("d", h[i - 1:i])])
        alone = rig.step([("d", h[i:])])[0]                                  # the reading row decoded alone
        rig.release("d")
        assert rel_err(alone[0], want[i]) < tol, (j, rel_err(alone[0], want[i]))


def test_runs_of_a_looped_layer_keep_caches_apart():
    rng = np.random.default_rng(6)
    width, H, G, D, V = 48, 2, 2, 16, 16
    w = attention_weights(rng, width, H, G, D, V)
    m = mixer_config(H, G, D, V, 16, 20, 2)
    ha, hb = bf(rng.normal(size=(50, width))), bf(rng.normal(size=(50, width)))
    rig = attention_rig(w, m, torch.float32, runs=2)
    load_pkg()
    mixer, step = rig.mixer, rig.step

    class Both:         # the rig calls one mixer per step: run 0 on the rows, run 1 on other rows of the same positions
        def __call__(self, ctx, h, h16=None):
            self.second = mixer(ctx, torch.from_numpy(hb[self.lo:self.lo + h.shape[0]].astype(np.float32)).cuda(), run=1).cpu().numpy()
            return mixer(ctx, h, run=0)
    both = Both()
    rig.mixer = both
    got_a, got_b = [], []
    for lo, hi in ((0, 30), (30, 31), (31, 50)):
        both.lo = lo
        got_a.append(step([("s", ha[lo:hi])])[0])
        got_b.append(both.second)
    assert rel_err(np.concatenate(got_a), ot.differential_attention(ha, w, m, 1e-5)) < 3e-5
    assert rel_err(np.concatenate(got_b), ot.differential_attention(hb, w, m, 1e-5)) < 3e-5


def test_batch_of_unequal_portions_and_reused_pages():
    rng = np.random.default_rng(7)
    width, H, G, D, V = 72, 6, 2, 24, 16
    w = attention_weights(rng, width, H, G, D, V)
    m = mixer_config(H, G, D, V, 24, 50, 3)
    hs = [bf(rng.normal(size=(n, width))) for n in (140, 9, 66, 100)]
    wants = [ot.differential_attention(h, w, m, 1e-5) for h in hs]
    for dtype, tol in ((torch.float32, 3e-5), (torch.bfloat16, 0.04)):
        rig = attention_rig(w, m, dtype, max_tokens=384, slots=3)            # 6 pages, all in use
        a0 = rig.step([("a", hs[0][:100]), ("b", hs[1][:1])])
        a1 = rig.step([("a", hs[0][100:101]), ("b", hs[1][1:]), ("c", hs[2][:64])])
        a2 = rig.step([("a", hs[0][101:]), ("c", hs[2][64:])])
        assert rel_err(np.concatenate([a0[0], a1[0], a2[0]]), wants[0]) < tol
        assert rel_err(np.concatenate([a0[1], a1[1]]), wants[1]) < tol and rel_err(np.concatenate([a1[2], a2[1]]), wants[2]) < tol
        for name in "abc":
            rig.release(name)
        d = rig.step([("d", hs[3])])[0]                                      # pages and a slot that others wrote
        assert rel_err(d, wants[3]) < tol


# ---------------------------------------------------------------------------------------------------------------- feed-forward
def ff_weights(rng, width, E, I, ff, shared_ff):
    r = lambda *s, sd=None: bf(rng.normal(0, sd if sd is not None else 1.0 / math.sqrt(s[-1]), s))
    w = {"router": r(E + I, width, sd=2.0 / math.sqrt(width)), "correction": bf(0.1 * rng.normal(size=E + I))}
    for e in range(E):
        w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"] = r(ff, width), r(ff, width), r(width, ff)
    if shared_ff:
        w["shared.gate"], w["shared.up"], w["shared.down"] = r(shared_ff, width), r(shared_ff, width), r(width, shared_ff)
    return w


def ff_rig(w, fc, dtype):
    load_pkg()
    from dash_infer_amd import mixers
    E, I = fc["router"]["experts"], fc["router"]["identity"]

    def build(state, dt):
        d = dev_weights(w)
        shared = mixers.GatedMlp(d["shared.gate"], d["shared.up"], d["shared.down"], "silu") if fc.get("shared") else None
        return mixers.ExpertMlp(d["router"], None, [d[f"e{e}.gate"] for e in range(E)], [d[f"e{e}.up"] for e in range(E)],
                                [d[f"e{e}.down"] for e in range(E)], fc["router"]["top"], unit="silu", scoring="scores",
                                correction=d.get("correction"), identity=I, shared=shared)
    return MixerRig(build, dtype)


@pytest.mark.parametrize("sizes", [(72, 5, 2, 2, 24, 40), (64, 4, 0, 1, 32, 0), (40, 2, 3, 5, 12, 16), (96, 8, 1, 3, 40, 64)])
def test_routed_feed_forward_against_the_oracle(sizes):
    width, E, I, top, ff, shared_ff = sizes
    rng = np.random.default_rng(E * 10 + I)
    w = ff_weights(rng, width, E, I, ff, shared_ff)
    fc = {"router": {"experts": E, "identity": I, "top": top}, "expert": {"ff": ff}, "shared": {"ff": shared_ff} if shared_ff else None}
    h = bf(rng.normal(size=(150, width)))
    chosen = []
    want = ot.moe_ff(h, w, fc, chosen)
    if I:
        assert any(max(c) >= E for c in chosen)                              # identity experts are chosen somewhere
    got = ff_rig(w, fc, torch.float32).step([("a", h)])[0]
    assert rel_err(got, want) < 3e-5
    few = ff_rig(w, fc, torch.float32).step([("a", h[:3])])[0]                # few rows: the weight-streaming products
    assert rel_err(few, want[:3]) < 3e-5
    got16 = ff_rig(w, fc, torch.bfloat16).step([("a", h)])[0]
    err = np.abs(got16 - want).max(1) / np.abs(want).max()
    assert np.mean(err < 0.03) > 0.9                                         # a rounding may tip a narrow choice


def test_correction_moves_the_choice_but_not_the_weights():
    rng = np.random.default_rng(8)
    width, E, I, top = 32, 3, 1, 2
    w = ff_weights(rng, width, E, I, 8, 0)
    w["correction"] = bf(np.array([0.0, 0.0, 5.0, 5.0]))                       # the last real expert and the identity expert always win
    fc = {"router": {"experts": E, "identity": I, "top": top}, "expert": {"ff": 8}, "shared": None}
    h = bf(rng.normal(size=(40, width)))
    chosen = []
    want = ot.moe_ff(h, w, fc, chosen)
    assert all(sorted(c) == [2, 3] for c in chosen)
    idx, ws = ot.route(h, w, top)
    assert np.allclose(ws.sum(1), 1.0) and ws.min() > 0 and ws.max() < 1      # the weights are scores, not corrected ones
    assert rel_err(ff_rig(w, fc, torch.float32).step([("a", h)])[0], want) < 3e-5


# ---------------------------------------------------------------------------------------------------------------- token side input
def test_token_side_input(so):
    rng = np.random.default_rng(9)
    T, width, sd, layers, layer = 21, 56, 10, 3, 1
    x = rng.normal(0, 2.0, (T, width)).astype(np.float32)
    table = bf(rng.normal(size=(17, layers * sd)))
    ids = rng.integers(0, 17, T).tolist()
    w = {"gate": bf(rng.normal(0, 0.2, (sd, width))), "proj": bf(rng.normal(0, 0.3, (width, sd))), "norm": bf(0.5 + 0.1 * rng.normal(size=width))}
    want = x.astype(np.float64) + ot.token_side(x, table[ids][:, layer * sd:(layer + 1) * sd], w, 1e-5)
    e = so.embed_rows(i32(ids), dev(table, torch.bfloat16), col0=layer * sd, cols=sd)
    g = so.linear(dev(x), dev(w["gate"], torch.bfloat16), act="gelu_tanh", mul=e, math=so.MATH_F32)
    y = so.linear(g, dev(w["proj"], torch.bfloat16), math=so.MATH_F32)
    xd = dev(x)
    so.residual_norm_step(xd, 1e-5, m=y, gamma_m=dev(w["norm"], torch.bfloat16), add_m=0.0)
    assert rel_err(xd.cpu().numpy(), want) < 3e-6
