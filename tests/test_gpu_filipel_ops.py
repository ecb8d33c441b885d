"""The mechanisms of the Filipel design, each alone, against the float64 restatement in oracle/filipel.py: the layer norm fused with
the residual step of two sublayers, the cubic of row-normalised powers, the join of two normed branches, attention through a latent
with a shared rotated key part (own and borrowed cache), windowed attention with softmax maps mixed between the heads, the
state-space mixer, group-limited routing."""
import numpy as np
import pytest
import torch

from oracle import filipel as of
from tests.conftest import load_pkg
from tests.seq_helpers import MixerRig, dev_weights, rel_err

pytestmark = pytest.mark.gpu
bf = of.bf16_values
EPS = 1e-5


@pytest.fixture(scope="module")
def so():
    load_pkg()
    from dash_infer_amd import seq_ops
    return seq_ops


def mixers():
    load_pkg()
    from dash_infer_amd import mixers as m
    return m


def dev(a, dt=torch.float32):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(dt).cuda()


def i32(a):
    return torch.tensor(a, dtype=torch.int32, device="cuda")


def rows(rng, n, width, scale=1.0):
    """hidden rows whose values are 16-bit ones, so that both engines read the same numbers"""
    return bf(rng.normal(0, scale, (n, width)))


# ---------------------------------------------------------------------------------------------------------------- row operators
# widths of every form of the row kernels: 256, 512 and 1024 threads with 4, 8 and 16 elements each, and the looping form beyond
@pytest.mark.parametrize("K", [50, 72, 1024 + 41, 3000, 4096 + 8, 9001, 16384 + 40])
def test_layer_norm_fused_with_the_residual_step(so, K):
    rng = np.random.default_rng(0)
    T = 23
    x = (rng.normal(0, 1.5, (T, K)) + 0.7).astype(np.float32)                   # a mean that matters
    a, b = rng.normal(0, 0.5, (T, K)).astype(np.float32), rng.normal(0, 0.5, (T, K)).astype(np.float32)
    w = bf(1.0 + 0.3 * rng.normal(size=K))
    xo = x.astype(np.float64) + 0.25 * (a.astype(np.float64) + b)
    wide = dev(np.concatenate([b, b], 1))                                       # a sublayer's output as a column slice
    xd = dev(x)
    h = so.residual_layernorm(xd, dev(w, torch.bfloat16), a=dev(a), b=wide[:, K:], mult=0.25, eps=1e-4, x_out=xd)
    assert rel_err(xd.cpu().numpy(), xo) < 1e-6 and rel_err(h.cpu().numpy(), of.layer_norm(xo, w, 1e-4)) < 3e-6
    xd2 = dev(x)
    h16 = so.residual_layernorm(xd2, dev(w), a=dev(a), b=dev(b), mult=0.25, eps=1e-4, x_out=xd2, out_dtype=torch.bfloat16)
    assert torch.equal(h16, h.to(torch.bfloat16))
    xd3 = dev(x)
    assert so.residual_layernorm(xd3, None, a=dev(a), mult=2.0, x_out=xd3) is None    # one sublayer, no next norm
    assert rel_err(xd3.cpu().numpy(), x.astype(np.float64) + 2.0 * a) < 1e-6
    pick = [5, 0, 22, 5]
    hr = so.residual_layernorm(dev(x), dev(w, torch.bfloat16), eps=1e-4, row_idx=i32(pick))   # the norm of chosen rows, the stream untouched
    assert rel_err(hr.cpu().numpy(), of.layer_norm(x, w, 1e-4)[pick]) < 3e-6
    # not an RMS norm: the mean is taken off
    assert rel_err(hr.cpu().numpy(), of.unit_rms(x, 1e-4)[pick] * w) > 1e-2


def test_cubic_of_normalised_powers_and_the_dense_feed_forward(so):
    rng = np.random.default_rng(1)
    coef = bf(np.array([0.7, -0.4, 0.25, 0.1]))
    for F in (333, 2500, 8192, 14336 + 3, 17001):
        z = rng.normal(0, 1.3, (17, F)).astype(np.float32)
        out = torch.empty(17, F, device="cuda")
        so.polynorm(dev(z), dev(coef, torch.bfloat16), 1e-4, out)
        assert rel_err(out.cpu().numpy(), of.poly_norm(z, coef, 1e-4)) < 3e-6, F
    width, ff = 72, 50
    w = of.ff_weights(rng, width, {"kind": "dense", "ff": ff})
    h = rows(rng, 40, width)
    for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 0.03)):
        rig = MixerRig(lambda st, dt: mixers().DenseMlp(*[dev_weights(w)[k] for k in ("up", "down")], ("polynorm", dev_weights(w)["act"])), dtype)
        assert rel_err(rig.step([("a", h)])[0], of.dense_ff(h, w, EPS)) < tol


@pytest.mark.parametrize("K", [70, 1500, 4100, 8192, 20000])
def test_two_normed_branches_joined(so, K):
    rng = np.random.default_rng(2)
    a, b = rng.normal(0, 3.0, (9, K)).astype(np.float32), rng.normal(0, 0.1, (9, K)).astype(np.float32)
    wa, wb = bf(1 + 0.2 * rng.normal(size=K)), bf(1 + 0.2 * rng.normal(size=K))
    wide = dev(np.concatenate([a, a], 1))
    got = so.rmsnorm_pair(wide[:, K:], dev(wa, torch.bfloat16), dev(b), dev(wb, torch.bfloat16), 0.5, 1e-5)
    assert rel_err(got.cpu().numpy(), 0.5 * (of.unit_rms(a, 1e-5) * wa + of.unit_rms(b, 1e-5) * wb)) < 3e-6


@pytest.mark.parametrize("heads,P,groups", [(3, 20, 2), (64, 64, 1), (64, 64, 4), (40, 250, 1), (70, 256, 1), (70, 256, 7)])
def test_skip_gate_and_grouped_norm(so, heads, P, groups):
    """v = (o + D[head] x) silu(z), every one of `groups` equal parts of the row divided by its own root mean square, times the weight"""
    rng = np.random.default_rng(3)
    T, n = 7, heads * P
    o, x, z = (rng.normal(0, 1.2, (T, n)).astype(np.float32) for _ in range(3))
    skip, w = bf(rng.normal(size=heads)), bf(1 + 0.2 * rng.normal(size=n))
    v = (o.astype(np.float64) + np.repeat(skip.astype(np.float64), P)[None] * x) * of.silu(z.astype(np.float64))
    parts = v.reshape(T, groups, n // groups)
    want = (parts / np.sqrt((parts ** 2).mean(-1, keepdims=True) + 1e-5)).reshape(T, n) * w
    got = so.gate_group_rmsnorm(dev(o), dev(z), dev(w, torch.bfloat16), 1e-5, heads, P, groups, x=dev(x), skip=dev(skip, torch.bfloat16))
    assert rel_err(got.cpu().numpy(), want) < 3e-6
    plain = so.gate_group_rmsnorm(dev(o), dev(z), dev(w), 1e-5, heads, P, groups)         # no skip term
    v0 = (o.astype(np.float64) * of.silu(z.astype(np.float64))).reshape(T, groups, n // groups)
    assert rel_err(plain.cpu().numpy(), (v0 / np.sqrt((v0 ** 2).mean(-1, keepdims=True) + 1e-5)).reshape(T, n) * w) < 3e-6


# ---------------------------------------------------------------------------------------------------------------- latent attention
def latent_rig(w, o, dtype, kv_from=None, width=72):
    m = mixers()
    def build(st, dt):
        first = None
        if kv_from is not None:        # the layer whose cache is read: built first, on the same state manager
            first = m.LatentWindowAttention("src", kv_from[1]["heads"], kv_from[1]["dim"], kv_from[1]["vdim"], kv_from[1]["kv_rank"], kv_from[1]["q_rank"], 0,
                                            of.latent_config(kv_from[1])["scale"], dev_weights(kv_from[0]), st, dt, rot_dim=kv_from[1]["rot_dim"],
                                            rot_base=kv_from[1]["base"])
        mine = m.LatentWindowAttention("mine", o["heads"], o["dim"], o["vdim"], o["kv_rank"], o["q_rank"], 0, of.latent_config(o)["scale"],
                                       dev_weights(w), st, dt, kv_from_key="src" if first is not None else None, rot_dim=o["rot_dim"], rot_base=o["base"])
        if first is None:
            return mine
        return lambda ctx, h, h16=None: (first(ctx, h, h16), mine(ctx, h, h16))[1]
    return MixerRig(build, dtype)


LATENT_SHAPES = {
    "plain": {},
    "one_head_odd": dict(heads=1, dim=12, rot_dim=2, vdim=9, kv_rank=11, q_rank=5),
    "one_row_of_64": dict(heads=4, dim=32, rot_dim=16, vdim=32, kv_rank=48, q_rank=40, base=100.0),
    "padded_row": dict(heads=5, dim=8, rot_dim=24, vdim=16, kv_rank=80, q_rank=16, scale=0.7),
}


@pytest.mark.parametrize("shape", list(LATENT_SHAPES))
def test_latent_attention_whole_portions_and_decoding(shape):
    rng = np.random.default_rng(3)
    o = dict(of.LATENT, **LATENT_SHAPES[shape])
    w = of.latent_weights(rng, 72, o)
    n = 150
    h = rows(rng, n, 72)
    want = of.latent_attention(h, w, of.latent_config(o), EPS)
    for dtype, tol in ((torch.float32, 2e-5), (torch.bfloat16, 0.05)):
        rig = latent_rig(w, o, dtype)
        assert rel_err(rig.step([("a", h)])[0], want) < tol
        cuts = [0, 3, 5, 64, 65, 70, 128, 130, n]                              # portions that end inside a page, at its border, one row after
        got = np.concatenate([rig.step([("b", h[a:b])])[0] for a, b in zip(cuts, cuts[1:])])
        assert rel_err(got, want) < tol
        dec = np.concatenate([rig.step([("c", h[i:i + 1])])[0] for i in range(80)])
        assert rel_err(dec, want[:80]) < tol


def test_latent_attention_on_another_layers_cache():
    rng = np.random.default_rng(4)
    src = dict(of.LATENT)
    mine = dict(of.LATENT, heads=2, dim=8, vdim=12, q_rank=10, kv_from=0)
    ws, wm = of.latent_weights(rng, 72, src), of.latent_weights(rng, 72, mine)
    assert "dkv" not in wm
    h = rows(rng, 140, 72)
    cached = of.latent_keys(h, ws, of.latent_config(src), EPS)
    want = of.latent_attention(h, wm, of.latent_config(mine), EPS, cached=cached)
    for dtype, tol in ((torch.float32, 2e-5), (torch.bfloat16, 0.05)):
        rig = latent_rig(wm, mine, dtype, kv_from=(ws, src))
        got = np.concatenate([rig.step([("a", h[:100])])[0]] + [rig.step([("a", h[i:i + 1])])[0] for i in range(100, 140)])
        assert rel_err(got, want) < tol


def test_latent_attention_reads_one_far_key_across_pages():
    """sharp scores: the last rows put most of their weight on single keys, hundreds of positions and several pages back; the rotated
    part decides too (shown by an oracle without it)"""
    rng = np.random.default_rng(5)
    o = dict(of.LATENT, scale=3.0, rot_dim=16, base=50.0)
    w = of.latent_weights(rng, 72, o)
    n = 400
    h = rows(rng, n, 72)
    m = of.latent_config(o)
    want = of.latent_attention(h, w, m, EPS)
    moved = h.copy()
    moved[:100] = rows(rng, 100, 72)                                            # other far keys: the last rows change
    assert rel_err(of.latent_attention(moved, w, m, EPS)[-40:], want[-40:]) > 0.05
    w0 = dict(w, uq=w["uq"].copy())
    w0["uq"].reshape(o["heads"], o["dim"] + o["rot_dim"], -1)[:, o["dim"]:] = 0.0  # no rotated query part
    assert rel_err(of.latent_attention(h, w0, m, EPS)[-40:], want[-40:]) > 0.05
    for dtype, tol in ((torch.float32, 5e-5), (torch.bfloat16, 0.08)):
        rig = latent_rig(w, o, dtype)
        got = np.concatenate([rig.step([("a", h[:360])])[0]] + [rig.step([("a", h[i:i + 1])])[0] for i in range(360, n)])
        assert rel_err(got[:360], want[:360]) < tol and rel_err(got[360:], want[360:]) < tol


# ---------------------------------------------------------------------------------------------------------------- mixed softmax maps
def talk_rig(w, o, dtype, width=72, max_tokens=2048):
    m = mixers()
    def build(st, dt):
        d = dev_weights(w)
        return m.GroupedQueryAttention("att", o["heads"], o["kv_heads"], o["dim"], o["vdim"], of.left_config(o)["scale"], d, st, dt,
                                       rot_dims=o["rot_dims"], rot_base=o["base"], rot_layout="halves", window=o["window"], head_temp=d["temp"],
                                       talk=d["talk"], elem_gate=True)
    return MixerRig(build, dtype, max_tokens=max_tokens)


TALK_SHAPES = {
    "plain": {},
    "odd_one_kv_head": dict(heads=3, kv_heads=1, dim=20, vdim=12, rot_dims=20, window=17, scale=0.4),
    "as_many_kv_heads": dict(heads=4, kv_heads=4, dim=32, vdim=64, rot_dims=16, window=64),
    "one_key": dict(heads=2, kv_heads=2, dim=8, vdim=200, rot_dims=0, window=1),
    "never_binds": dict(heads=16, kv_heads=4, dim=8, vdim=8, rot_dims=4, window=1000, base=77.0),
    # sizes of the matrix-core form: two and four heads per wave, output heads shared between two workgroups, heads past a multiple of 8
    "tiles_16_heads": dict(heads=16, kv_heads=2, dim=64, vdim=32, rot_dims=32, window=50),
    "tiles_32_heads": dict(heads=32, kv_heads=8, dim=32, vdim=16, rot_dims=32, window=33),
    "tiles_12_heads": dict(heads=12, kv_heads=3, dim=96, vdim=80, rot_dims=48, window=129),
}


@pytest.mark.parametrize("shape", list(TALK_SHAPES))
def test_mixed_maps_attention_whole_portions_and_decoding(shape):
    rng = np.random.default_rng(6)
    o = dict(of.LEFT, **TALK_SHAPES[shape])
    w = of.left_weights(rng, 72, o)
    n = 150
    h = rows(rng, n, 72)
    want = of.talking_attention(h, w, of.left_config(o))
    plain = of.talking_attention(h, dict(w, talk=np.eye(o["heads"])), of.left_config(o))
    assert rel_err(plain, want) > 0.05                                          # the mix matters
    for dtype, tol in ((torch.float32, 2e-5), (torch.bfloat16, 0.05)):
        rig = talk_rig(w, o, dtype)
        assert rel_err(rig.step([("a", h)])[0], want) < tol
        cuts = [0, 3, 5, 64, 65, 70, 128, 130, n]
        got = np.concatenate([rig.step([("b", h[a:b])])[0] for a, b in zip(cuts, cuts[1:])])
        assert rel_err(got, want) < tol
        dec = np.concatenate([rig.step([("c", h[i:i + 1])])[0] for i in range(90)])
        assert rel_err(dec, want[:90]) < tol


@pytest.mark.parametrize("window,n", [(40, 150), (64, 193), (129, 321), (300, 700)])
def test_keys_just_inside_and_just_outside_the_window(window, n):
    """the row that is scaled up has a large key and value: the last row's result changes when that row is the oldest key of its
    window (also where that key is the first or last row of a page, or lies in another part of a split walk), and does not change at
    all when it lies one position further back"""
    rng = np.random.default_rng(7)
    o = dict(of.LEFT, window=window)
    w = of.left_weights(rng, 72, o)
    m = of.left_config(o)
    h = rows(rng, n, 72)
    inside, outside = h.copy(), h.copy()
    inside[n - window] *= 8.0
    outside[n - window - 1] *= 8.0
    base = of.talking_attention(h, w, m)[-1:]
    w_in, w_out = of.talking_attention(inside, w, m)[-1:], of.talking_attention(outside, w, m)[-1:]
    assert rel_err(w_in, base) > 0.1 and rel_err(w_out, base) == 0.0
    one_more = of.talking_attention(outside, w, dict(m, mask={"size": window + 1}))[-1:]
    assert rel_err(one_more, w_out) > 0.1                                       # a window one key too long would show
    for dtype, tol in ((torch.float32, 2e-5), (torch.bfloat16, 0.05)):
        rig = talk_rig(w, o, dtype)
        for name, x, want in (("i", inside, w_in), ("o", outside, w_out)):
            whole = rig.step([(name, x)])[0][-1:]                               # as the last row of a prompt
            rig.step([(name + "d", x[:-1])])
            alone = rig.step([(name + "d", x[-1:])])[0]                         # decoded alone
            assert rel_err(whole, want) < tol and rel_err(alone, want) < tol
            rig.release(name)
            rig.release(name + "d")


def test_unequal_portions_in_one_batch_and_pages_used_again():
    rng = np.random.default_rng(8)
    o = dict(of.LEFT, window=70)
    w = of.left_weights(rng, 72, o)
    m = of.left_config(o)
    hs = [rows(rng, n, 72) for n in (130, 1, 77)]
    want = [of.talking_attention(x, w, m) for x in hs]
    rig = talk_rig(w, o, torch.float32, max_tokens=384)                          # 6 pages
    for rnd in range(3):                                                         # pages and slots come back dirty
        first = rig.step([("a", hs[0][:60]), ("b", hs[1]), ("c", hs[2][:2])])
        second = rig.step([("a", hs[0][60:]), ("c", hs[2][2:])])
        assert rel_err(np.concatenate([first[0], second[0]]), want[0]) < 2e-5
        assert rel_err(first[1], want[1]) < 2e-5 and rel_err(np.concatenate([first[2], second[1]]), want[2]) < 2e-5
        for name in "abc":
            rig.release(name)


# ---------------------------------------------------------------------------------------------------------------- state-space mixer
def ssm_rig(w, o, dtype, slots=4):
    m = mixers()
    return MixerRig(lambda st, dt: m.StateSpaceMixer("ssm", o["heads"], o["vdim"], o["state"], o["groups"], o["conv"], o["norm_groups"],
                                                     dev_weights(w), st), dtype, slots=slots)


SSM_SHAPES = {
    "plain": {},
    "groups": dict(heads=6, vdim=8, state=16, groups=3, conv=4, norm_groups=3),
    "one_of_each": dict(heads=1, vdim=9, state=3, groups=1, conv=1, norm_groups=1),
    "wide": dict(heads=2, vdim=200, state=64, groups=2, conv=2, norm_groups=8),
}


@pytest.mark.parametrize("shape", list(SSM_SHAPES))
def test_state_space_mixer_whole_rows_and_portions(shape):
    rng = np.random.default_rng(9)
    o = dict(of.RIGHT, **SSM_SHAPES[shape])
    w = of.right_weights(rng, 72, o)
    n = 330
    h = rows(rng, n, 72)
    want = of.state_space(h, w, of.right_config(o), EPS)
    for dtype, tol in ((torch.float32, 3e-5), (torch.bfloat16, 0.05)):
        rig = ssm_rig(w, o, dtype)
        assert rel_err(rig.step([("a", h)])[0], want) < tol                     # chunks side by side
        dec = np.concatenate([rig.step([("b", h[i:i + 1])])[0] for i in range(n)])
        assert rel_err(dec, want) < tol
        cuts = [0, 2, 3, 64, 65, 66, 200, 202, 329, n]
        got = np.concatenate([rig.step([("c", h[a:b])])[0] for a, b in zip(cuts, cuts[1:])])
        assert rel_err(got, want) < tol


def test_state_space_sequences_side_by_side_and_a_slot_used_again():
    rng = np.random.default_rng(10)
    o = dict(of.RIGHT)
    w = of.right_weights(rng, 72, o)
    m = of.right_config(o)
    hs = [rows(rng, n, 72) for n in (90, 140, 7)]
    want = [of.state_space(x, w, m, EPS) for x in hs]
    rig = ssm_rig(w, o, torch.float32, slots=3)
    for rnd in range(2):                                                         # the second round takes slots that hold old state
        first = rig.step([("a", hs[0][:50]), ("b", hs[1][:1]), ("c", hs[2])])
        second = rig.step([("b", hs[1][1:131]), ("a", hs[0][50:])])
        third = rig.step([("b", hs[1][131:])])
        assert rel_err(np.concatenate([first[0], second[1]]), want[0]) < 3e-5
        assert rel_err(np.concatenate([first[1], second[0], third[0]]), want[1]) < 3e-5 and rel_err(first[2], want[2]) < 3e-5
        for name in "abc":
            rig.release(name)
    # the oracle carries its state the same way
    parts = []
    state = {"S": np.zeros((o["heads"], o["state"], o["vdim"])), "tail": np.zeros((o["conv"] - 1, o["heads"] * o["vdim"] + 2 * o["groups"] * o["state"]))}
    for a, b in ((0, 1), (1, 60), (60, 90)):
        parts.append(of.state_space(hs[0][a:b], w, m, EPS, state))
    assert rel_err(np.concatenate(parts), want[0]) < 1e-12


# ---------------------------------------------------------------------------------------------------------------- routed experts
@pytest.mark.parametrize("experts,count,keep,top", [(6, 3, 2, 2), (8, 4, 1, 2), (4, 1, 1, 4), (9, 3, 1, 3), (8, 4, 2, 3), (5, 5, 2, 1)])
def test_group_limited_routing(so, experts, count, keep, top):
    rng = np.random.default_rng(11)
    width, ff, n = 72, 20, 300
    fc = of.ff_config(("moe", dict(experts=experts, count=count, keep=keep, top=top, ff=ff)))
    w = of.ff_weights(rng, width, fc)
    h = rows(rng, n, width)
    idx, ws = of.route(h, w, fc)
    z = (h.astype(np.float64) @ w["router"].astype(np.float64).T).astype(np.float32)
    ids, wts, seg, src_row, dst = so.moe_route(dev(z), top, so.ROUTE_SCORES, None, (count, keep))
    assert np.array_equal(ids.cpu().numpy(), idx) and rel_err(wts.cpu().numpy(), ws) < 1e-5
    if count > keep and top > keep:                                              # the limit matters: plain top-k would choose otherwise somewhere
        plain = np.argsort(-z, axis=1, kind="stable")[:, :top]
        assert any(set(a) != set(b) for a, b in zip(plain.tolist(), idx.tolist()))
    m = mixers()
    d = dev_weights(w)
    for dtype, tol, few in ((torch.float32, 2e-5, 1.0), (torch.bfloat16, 0.05, 0.9)):
        rig = MixerRig(lambda st, dt: m.ExpertMlp(d["router"], None, [d[f"e{e}.gate"] for e in range(experts)], [d[f"e{e}.up"] for e in range(experts)],
                                                  [d[f"e{e}.down"] for e in range(experts)], top, unit="silu", scoring="scores", groups=(count, keep)), dtype)
        want = of.moe_ff(h, w, fc)
        got = rig.step([("a", h)])[0]
        err = np.abs(got - want).max(1) / np.abs(want).max()
        assert np.mean(err < tol) >= few
        alone = rig.step([("b", h[7:8])])[0]                                    # a token alone (the one-launch routing) against the batch
        assert rel_err(alone, got[7:8]) < (1e-6 if dtype == torch.float32 else 0.05)


# ---------------------------------------------------------------------------------------------------------------- the pair of mixers
def test_two_mixers_side_by_side():
    rng = np.random.default_rng(12)
    lo, ro = dict(of.LEFT), dict(of.RIGHT)
    wl, wr = of.left_weights(rng, 72, lo), of.right_weights(rng, 72, ro)
    mcfg = {"left": of.left_config(lo), "right": of.right_config(ro)}
    h = rows(rng, 100, 72)
    want = of.side_by_side(h, wl, wr, mcfg, EPS)
    m = mixers()
    def build(st, dt):
        dl, dr = dev_weights(wl), dev_weights(wr)
        left = m.GroupedQueryAttention("att", lo["heads"], lo["kv_heads"], lo["dim"], lo["vdim"], mcfg["left"]["scale"], dl, st, dt, rot_dims=lo["rot_dims"],
                                       rot_base=lo["base"], rot_layout="halves", window=lo["window"], head_temp=dl["temp"], talk=dl["talk"], elem_gate=True)
        right = m.StateSpaceMixer("ssm", ro["heads"], ro["vdim"], ro["state"], ro["groups"], ro["conv"], ro["norm_groups"], dr, st)
        return m.SideBySide(left, right, dl["out"], dr["out"], 0.5)
    rig = MixerRig(build, torch.float32)
    got = np.concatenate([rig.step([("a", h[:37])])[0], rig.step([("a", h[37:])])[0]])
    assert rel_err(got, want) < 2e-5
