"""Host-side parts of the Tobilorn design (no GPU): the registry, the order of layer runs, and the oracle against itself (its mask,
its routing with identity experts against dense evaluation, the half-split rotation)."""
import math

import numpy as np
import pytest

from oracle import tobilorn as ot
from tests.conftest import load_pkg


def test_registry_knows_the_design():
    load_pkg()
    from dash_infer_amd import models
    cls = models.resolve({"architecture": "Tobilorn"})
    assert cls.engine == "sequence" and "Tobilorn" in models.known()


def test_order_of_layer_runs_matches_the_oracle():
    load_pkg()
    from dash_infer_amd.models.tobilorn import layer_runs
    for n, loop in ((5, (1, 3, 3)), (3, (0, 3, 2)), (4, None), (3, (2, 3, 1)), (6, (0, 1, 4))):
        cfg = {"layers": [None] * n}
        if loop:
            cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
        want = ot.layer_runs(cfg)
        got = layer_runs(n, cfg.get("loop"))
        assert [g[0] for g in got] == [w[0] for w in want]
        assert [g[2] for g in got] == [w[1] if w[2] else None for w in want]          # the pass that starts at this run
        seen = {}
        for layer, run, _ in got:                                                      # a layer's runs count from 0
            assert run == seen.get(layer, 0)
            seen[layer] = run + 1
        assert len(got) == n + ((loop[1] - loop[0]) * (loop[2] - 1) if loop else 0)
    with pytest.raises(ValueError):
        layer_runs(3, {"start": 2, "stop": 5, "times": 2})


def test_oracle_mask():
    vis = lambda i, w, k: [j for j in range(i + 1) if ot.visible(i, j, w, k)]
    assert vis(10, 3, 2) == [0, 1, 8, 9, 10]
    assert vis(10, 3, 0) == [8, 9, 10] and vis(10, 1, 0) == [10]
    assert vis(3, 3, 2) == [0, 1, 2, 3] and vis(1, 5, 4) == [0, 1]                      # kept keys never lie ahead of the row
    assert vis(10, 100, 0) == list(range(11))


def test_oracle_rotation_is_relative_and_leaves_the_rest():
    rng = np.random.default_rng(0)
    q, k = rng.normal(size=12), rng.normal(size=12)
    dots = [ot.rotate_halves(q, p + 5, 8, 100.0) @ ot.rotate_halves(k, p, 8, 100.0) for p in (0, 3, 40)]
    assert np.allclose(dots, dots[0], atol=1e-5)
    r = ot.rotate_halves(q, 7, 8, 100.0)
    assert np.array_equal(r[8:], q[8:]) and not np.allclose(r[:8], q[:8])
    assert math.isclose(r[0], q[0] * math.cos(7.0) - q[4] * math.sin(7.0), rel_tol=1e-6)   # pair (0, 4) turns by 7 * 100^0


def test_oracle_routing_with_identity_experts():
    rng = np.random.default_rng(1)
    width, E, I, ff = 16, 3, 2, 6
    w = {"router": rng.normal(size=(E + I, width)), "correction": np.zeros(E + I)}
    for e in range(E):
        w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"] = rng.normal(size=(ff, width)), rng.normal(size=(ff, width)), rng.normal(size=(width, ff))
    h = rng.normal(size=(5, width))
    fc = {"router": {"experts": E, "identity": I, "top": E + I}, "expert": {"ff": ff}, "shared": None}
    out = ot.moe_ff(h, w, fc)                                                 # every expert: the softmax itself weighs them
    z = h @ w["router"].T
    p = np.exp(z - z.max(1, keepdims=True))
    p /= p.sum(1, keepdims=True)
    dense = sum(p[:, e:e + 1] * ot.gated_unit(h, w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"]) for e in range(E)) + p[:, E:].sum(1, keepdims=True) * h
    assert np.allclose(out, dense)
    fc["router"]["top"] = 2
    idx, ws = ot.route(h, w, 2)
    assert np.allclose(ws.sum(1), 1.0) and np.all(np.take_along_axis(p, idx, 1)[:, 0] >= np.take_along_axis(p, idx, 1)[:, 1])


def test_oracle_lambda():
    w = {"lq1": [1.0, 2.0], "lk1": [0.5, 0.25], "lq2": [0.0, 0.0], "lk2": [3.0, 3.0]}
    assert math.isclose(ot.differential_lambda(w, 0.3), math.exp(1.0) - 1.0 + 0.3)
