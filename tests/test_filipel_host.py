"""Host-side checks of the Filipel design (no GPU): the registry, and the float64 restatement against closed forms and against
itself -- rotation, the mixed softmax maps, the state-space recurrence, group-limited routing, the cubic of normalised powers."""
import numpy as np

from oracle import filipel as of
from tests.conftest import load_pkg


def test_the_registry_resolves_the_architecture():
    load_pkg()
    from dash_infer_amd import models
    assert "Filipel" in models.known()
    cls = models.resolve({"architecture": "Filipel"})
    assert cls.engine == "sequence" and cls.__name__ == "Filipel"


def test_rotation_is_relative_and_leaves_the_rest():
    rng = np.random.default_rng(0)
    q, k = rng.normal(size=12), rng.normal(size=12)
    dots = [of.rotate_halves(q, p + 5, 8, 100.0) @ of.rotate_halves(k, p, 8, 100.0) for p in (0, 3, 40)]
    assert np.allclose(dots, dots[0], rtol=1e-5)
    assert np.array_equal(of.rotate_halves(q, 9, 8, 100.0)[8:], q[8:]) and np.allclose(of.rotate_halves(q, 0, 8, 100.0), q)
    r = of.rotate_halves(np.array([1.0, 0.0, 0.0, 0.0]), 1, 4, 100.0)           # dimension 0 pairs with dimension 2
    assert np.allclose(r, [np.cos(1.0), 0.0, np.sin(1.0), 0.0], atol=1e-6)


def test_mixed_maps_with_the_identity_are_plain_windowed_attention():
    rng = np.random.default_rng(1)
    o = dict(of.LEFT, heads=4, kv_heads=2, window=5, rot_dims=0)
    w = of.left_weights(rng, 24, o)
    w["talk"], w["temp"] = np.eye(4), np.ones(4)
    w["g"] = np.zeros_like(w["g"])                                              # a gate of one half everywhere
    w["o"] = np.zeros_like(w["o"])
    w["o"][:, 72:] = np.eye(24)                                                 # the output is head 3's
    h = rng.normal(size=(12, 24))
    seen = []
    got = of.talking_attention(h, w, of.left_config(o), weights_out=seen)
    lo, maps, mixed = seen[-1]
    assert lo == 12 - 5 and maps.shape == (4, 5) and np.allclose(maps.sum(1), 1.0) and np.array_equal(maps, mixed)
    q, k, v = h @ w["q"].T.astype(np.float64), h @ w["k"].T.astype(np.float64), h @ w["v"].T.astype(np.float64)
    s = (k[7:, 16:32] @ q[11, 48:64]) * o["dim"] ** -0.5                        # head 3 reads key/value head 1
    p = np.exp(s - s.max())
    assert np.allclose(got[11], 0.5 * ((p / p.sum()) @ v[7:, 24:48]))


def test_state_space_recurrence_against_its_closed_form():
    rng = np.random.default_rng(2)
    o = dict(of.RIGHT, heads=2, vdim=3, state=4, groups=1, conv=1, norm_groups=1)
    w = of.right_weights(rng, 10, o)
    w["conv"], w["conv.b"] = np.ones_like(w["conv"]), np.zeros_like(w["conv.b"])
    w["norm"], w["o"] = np.ones(6), np.eye(6)
    h = rng.normal(size=(7, 10))
    got = of.state_space(h, w, of.right_config(o), 0.0)
    a = h @ w["in"].T.astype(np.float64)
    z, u, dt = a[:, :6], of.silu(a[:, 6:20]), of.softplus(a[:, 20:] + w["dt_bias"])
    x, B, C = u[:, :6].reshape(7, 2, 3), u[:, 6:10], u[:, 10:14]
    la = -np.exp(w["A_log"].astype(np.float64)) * dt
    y = np.zeros((7, 2, 3))
    for t in range(7):
        for hd in range(2):
            for s in range(t + 1):                                              # y_t = sum_s exp(sum of the log decays after s) dt_s (C_t . B_s) x_s
                y[t, hd] += np.exp(la[s + 1: t + 1, hd].sum()) * dt[s, hd] * (C[t] @ B[s]) * x[s, hd]
            y[t, hd] += w["D"][hd] * x[t, hd]
    want = of.unit_rms(y.reshape(7, 6) * of.silu(z), 0.0)
    assert np.allclose(got, want, rtol=1e-9, atol=1e-12)


def test_routing_keeps_to_the_best_groups():
    rng = np.random.default_rng(3)
    fc = of.ff_config(("moe", dict(experts=8, count=4, keep=2, top=3, ff=4)))
    w = of.ff_weights(rng, 16, fc)
    h = rng.normal(size=(200, 16))
    idx, ws = of.route(h, w, fc)
    z = h @ w["router"].T.astype(np.float64)
    for t in range(200):
        best = np.argsort(-z[t].reshape(4, 2).max(1), kind="stable")[:2]
        assert {i // 2 for i in idx[t]} <= set(best.tolist()) and len(set(idx[t])) == 3
        allowed = sorted((e for e in range(8) if e // 2 in best), key=lambda e: -z[t, e])[:3]
        assert list(idx[t]) == allowed
    assert np.allclose(ws.sum(1), 1.0) and (ws > 0).all()
    dense = of.moe_ff(h[:5], w, fc)
    assert dense.shape == (5, 16)


def test_cubic_of_normalised_powers():
    z = np.array([[1.0, -2.0, 3.0, 0.5]])
    got = of.poly_norm(z, np.array([2.0, 0.0, 0.0, 1.0]), 0.0)
    assert np.allclose(got, 2.0 * z / np.sqrt((z * z).mean()) + 1.0)
    got = of.poly_norm(z, np.array([0.0, 1.0, 1.0, 0.0]), 0.0)
    assert np.allclose(got, z ** 2 / np.sqrt((z ** 4).mean()) + z ** 3 / np.sqrt((z ** 6).mean()))


def test_a_random_model_runs_and_its_layers_are_as_asked():
    rng = np.random.default_rng(4)
    cfg, t = of.random_filipel(rng, [("latent_attention", None, ("moe",)), ("parallel", None, ("dense", 30)), ("latent_attention", {"kv_from": 0}, None)])
    assert [l["type"] for l in cfg["layers"]] == ["latent_attention", "parallel", "latent_attention"]
    assert "l2.mix.dkv" not in t and "l0.mix.dkv" in t and t["l1.mix.left.talk"].shape == (6, 6)
    streams = []
    lg = of.forward(cfg, t, [3, 1, 4, 1, 5], streams)
    assert lg.shape == (5, cfg["vocab"]) and len(streams) == 3 and np.isfinite(lg).all()
    assert np.allclose(of.forward(cfg, t, [3, 1, 4])[:3], lg[:3])               # causal
