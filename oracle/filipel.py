"""Plain, slow float64 restatement of the Filipel design, one function per mechanism, row by row.  Test infrastructure only:
numpy, no kernels, no code shared with the product path.

Notation: h [n, width] the rows of ONE sequence in order (row p is position p); weights as the checkpoint stores them
([out, in]); w maps the names below '<layer>.mix.' / '<layer>.mix.left.' / '<layer>.mix.right.' / '<layer>.mlp.' to arrays."""
import math

import numpy as np


def f64(a):
    return np.asarray(a, np.float64)


def silu(z):
    return z / (1.0 + np.exp(-z))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def softplus(z):
    return np.logaddexp(0.0, z)


def unit_rms(x, eps):
    x = f64(x)
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def layer_norm(x, w, eps):
    """mean and variance over the row, a weight and no bias"""
    x = f64(x)
    d = x - x.mean(axis=-1, keepdims=True)
    return d / np.sqrt(np.mean(d * d, axis=-1, keepdims=True) + eps) * f64(w)


# -- rotary positions -----------------------------------------------------------------------------------------------------
def rotate_halves(x, pos, dims, base):
    """x [.., dim] of the token at position pos: dimension i turns with dimension i + dims / 2 by pos * base^(-2 i / dims); the
    dimensions from dims on stay.  The angle is the 32-bit product of position and frequency."""
    half = dims // 2
    f = np.array([float(base) ** (-2.0 * i / dims) for i in range(half)])
    ang = (np.float32(pos) * f.astype(np.float32)).astype(np.float64)
    c, s = np.cos(ang), np.sin(ang)
    out = f64(x).copy()
    u, v = f64(x)[..., :half], f64(x)[..., half:dims]
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


def softmax_weights(scores):
    e = np.exp(scores - scores.max())
    return e / e.sum()


# -- attention through a latent with a shared rotated key part ------------------------------------------------------------
def latent_keys(h, w, m, eps):
    """what the layer caches: (latent c [n, kv_rank], rotated key part [n, rot_dim])"""
    R, Rd = int(m["kv_rank"]), int(m["rot_dim"])
    kv = f64(h) @ f64(w["dkv"]).T
    c = unit_rms(kv[:, :R], eps) * f64(w["dkv.norm"])
    kr = np.stack([rotate_halves(kv[p, R:], p, Rd, float(m["rot"]["base"])) for p in range(h.shape[0])])
    return c, kr


def latent_attention(h, w, m, eps, cached=None):
    """cached: (c, kr) of the layer whose cache this one reads (kv_from), else its own"""
    n = h.shape[0]
    H, D, Rd, V = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"])
    h = f64(h)
    cq = unit_rms(h @ f64(w["dq"]).T, eps) * f64(w["dq.norm"])
    q = (cq @ f64(w["uq"]).T).reshape(n, H, D + Rd)
    c, kr = cached if cached is not None else latent_keys(h, w, m, eps)
    k = (c @ f64(w["uk"]).T).reshape(n, H, D)
    v = (c @ f64(w["uv"]).T).reshape(n, H, V)
    out = np.zeros((n, H, V))
    for i in range(n):
        qr = rotate_halves(q[i, :, D:], i, Rd, float(m["rot"]["base"]))
        for hd in range(H):
            s = (k[: i + 1, hd] @ q[i, hd, :D] + kr[: i + 1] @ qr[hd]) * float(m["scale"])
            out[i, hd] = softmax_weights(s) @ v[: i + 1, hd]
    return (out.reshape(n, H * V) * sigmoid(h @ f64(w["g"]).T)) @ f64(w["o"]).T


# -- windowed grouped-query attention whose softmax maps are mixed between the heads ----------------------------------------
def talking_attention(h, w, m, weights_out=None):
    n = h.shape[0]
    H, G, D, V = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    window, rd, base = int(m["mask"]["size"]), int(m["rot"]["dims"]), float(m["rot"]["base"])
    h = f64(h)
    q = (h @ f64(w["q"]).T).reshape(n, H, D)
    k = (h @ f64(w["k"]).T).reshape(n, G, D)
    v = (h @ f64(w["v"]).T).reshape(n, G, V)
    q = np.stack([rotate_halves(q[p], p, rd, base) for p in range(n)])
    k = np.stack([rotate_halves(k[p], p, rd, base) for p in range(n)])
    talk, temp = f64(w["talk"]), f64(w["temp"])
    out = np.zeros((n, H, V))
    for i in range(n):
        lo = max(0, i - window + 1)
        maps = np.stack([softmax_weights((k[lo: i + 1, hd // (H // G)] @ q[i, hd]) * float(m["scale"]) * temp[hd]) for hd in range(H)])
        mixed = talk @ maps                                   # [H, keys]
        if weights_out is not None:
            weights_out.append((lo, maps, mixed))
        for hd in range(H):
            out[i, hd] = mixed[hd] @ v[lo: i + 1, hd // (H // G)]
    return (out.reshape(n, H * V) * sigmoid(h @ f64(w["g"]).T)) @ f64(w["o"]).T


# -- state-space mixer (scalar decay per head, matrix state) ----------------------------------------------------------------
def state_space(h, w, m, eps, state=None):
    """state: None (a fresh sequence) or {'S': [heads, N, vdim], 'tail': [taps - 1, channels]} carried between calls (updated in place)"""
    n = h.shape[0]
    Hn, P, N, G, taps, ng = int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m["groups"]), int(m["conv"]), int(m["norm_groups"])
    inner, ch = Hn * P, Hn * P + 2 * G * N
    a = f64(h) @ f64(w["in"]).T
    z, xbc, dt = a[:, :inner], a[:, inner: inner + ch], a[:, inner + ch:]
    if state is None:
        state = {"S": np.zeros((Hn, N, P)), "tail": np.zeros((taps - 1, ch))}
    padded = np.concatenate([state["tail"], xbc], 0)
    cw, cb = f64(w["conv"]), f64(w["conv.b"])
    u = np.stack([silu((padded[t: t + taps] * cw.T).sum(0) + cb) for t in range(n)])
    if taps > 1:
        state["tail"][:] = padded[n:]
    x, B, C = u[:, :inner].reshape(n, Hn, P), u[:, inner: inner + G * N].reshape(n, G, N), u[:, inner + G * N:].reshape(n, G, N)
    dt = softplus(dt + f64(w["dt_bias"]))
    decay = np.exp(-np.exp(f64(w["A_log"])) * dt)             # [n, heads]
    y = np.zeros((n, Hn, P))
    S = state["S"]
    for t in range(n):
        for hd in range(Hn):
            g = hd // (Hn // G)
            S[hd] = decay[t, hd] * S[hd] + dt[t, hd] * np.outer(B[t, g], x[t, hd])
            y[t, hd] = S[hd].T @ C[t, g] + f64(w["D"])[hd] * x[t, hd]
    y = y.reshape(n, inner) * silu(z)
    y = unit_rms(y.reshape(n, ng, inner // ng), eps).reshape(n, inner) * f64(w["norm"])
    return y @ f64(w["o"]).T


def side_by_side(h, w_left, w_right, m, eps, state=None):
    """the mean of the two mixers' results, each brought to unit root mean square over the width and weighted"""
    a = unit_rms(talking_attention(h, w_left, m["left"]), eps) * f64(w_left["out"])
    b = unit_rms(state_space(h, w_right, m["right"], eps, state), eps) * f64(w_right["out"])
    return 0.5 * (a + b)


# -- feed-forward -----------------------------------------------------------------------------------------------------------
def poly_norm(z, coef, eps):
    """a N(z) + b N(z^2) + c N(z^3) + e with the powers taken per element and N = division by the row's root mean square"""
    a, b, c, e = [float(t) for t in f64(coef)]
    return a * unit_rms(z, eps) + b * unit_rms(z * z, eps) + c * unit_rms(z * z * z, eps) + e


def dense_ff(h, w, eps):
    return poly_norm(f64(h) @ f64(w["up"]).T, w["act"], eps) @ f64(w["down"]).T


def route(h, w, fc):
    """-> (chosen experts [n, top], weights [n, top]): scores = softmax over all experts; only the experts of the `keep` groups
    with the largest best score can be chosen; weights = the chosen scores over their sum"""
    r = fc["router"]
    E, top, count, keep = int(r["experts"]), int(r["top"]), int(r["groups"]["count"]), int(r["groups"]["keep"])
    z = f64(h) @ f64(w["router"]).T
    s = np.exp(z - z.max(1, keepdims=True))
    s /= s.sum(1, keepdims=True)
    n = h.shape[0]
    idx, ws = np.zeros((n, top), np.int64), np.zeros((n, top))
    for t in range(n):
        best = s[t].reshape(count, E // count).max(1)
        kept = np.argsort(-best, kind="stable")[:keep]
        allowed = np.full(E, -1.0)
        for g in kept:
            allowed[g * (E // count): (g + 1) * (E // count)] = s[t, g * (E // count): (g + 1) * (E // count)]
        idx[t] = np.argsort(-allowed, kind="stable")[:top]
        ws[t] = s[t, idx[t]] / (s[t, idx[t]].sum() + 1e-20)
    return idx, ws


def moe_ff(h, w, fc, chosen=None):
    h = f64(h)
    idx, ws = route(h, w, fc)
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        if chosen is not None:
            chosen.append(idx[t].tolist())
        for e, wt in zip(idx[t], ws[t]):
            unit = silu(h[t] @ f64(w[f"e{e}.gate"]).T) * (h[t] @ f64(w[f"e{e}.up"]).T)
            out[t] += wt * (unit @ f64(w[f"e{e}.down"]).T)
    return out


# -- the model --------------------------------------------------------------------------------------------------------------
def sub(tensors, prefix):
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def forward(cfg, tensors, tokens, streams=None):
    """tokens of ONE sequence from position 0 -> logits [n, vocab]; streams: a list that receives the residual stream after every layer"""
    eps, mult = float(cfg["norm"]["eps"]), float(cfg["residual_mult"])
    x = f64(tensors["embed"])[np.asarray(tokens)]
    caches = {}
    for i, lc in enumerate(cfg["layers"]):
        w, m = sub(tensors, f"l{i}."), lc["mixer"]
        h = layer_norm(x, w["norm1"], eps)
        if lc["type"] == "latent_attention":
            mw = sub(w, "mix.")
            if m.get("kv_from") is None:
                caches[i] = latent_keys(h, mw, m, eps)
            mo = latent_attention(h, mw, m, eps, cached=caches[i if m.get("kv_from") is None else int(m["kv_from"])])
        elif lc["type"] == "parallel":
            mo = side_by_side(h, sub(w, "mix.left."), sub(w, "mix.right."), m, eps)
        else:
            raise ValueError(lc["type"])
        fc = lc.get("mlp")
        fo = 0.0
        if fc is not None:
            fo = dense_ff(h, sub(w, "mlp."), eps) if fc["kind"] == "dense" else moe_ff(h, sub(w, "mlp."), fc)
        x = x + mult * (mo + fo)
        if streams is not None:
            streams.append(x.copy())
    return layer_norm(x, tensors["final.norm"], eps) @ f64(tensors["head"]).T


# -- small random models (tests) --------------------------------------------------------------------------------------------
def bf16_values(a):
    """float32 array whose values are exactly representable in bfloat16 (round to nearest even)"""
    u = np.asarray(a, np.float32).view(np.uint32)
    u = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    return u.astype(np.uint32).view(np.float32)


LEFT = dict(heads=6, kv_heads=2, dim=16, vdim=24, window=40, rot_dims=8, base=10000.0, scale=None)
RIGHT = dict(heads=3, vdim=20, state=12, groups=1, conv=3, norm_groups=2)
LATENT = dict(heads=3, dim=16, rot_dim=8, vdim=20, kv_rank=24, q_rank=28, base=5000.0, scale=None, kv_from=None)
MOE = dict(experts=6, count=3, keep=2, top=2, ff=20)


def left_weights(rng, width, o):
    bf = bf16_values
    r = lambda *s: bf(rng.normal(0, 1.0 / math.sqrt(s[-1]), s))
    H, G, D, V = o["heads"], o["kv_heads"], o["dim"], o["vdim"]
    return {"q": r(H * D, width), "k": r(G * D, width), "v": r(G * V, width), "g": r(H * V, width), "o": r(width, H * V),
            "talk": bf(np.eye(H) * 0.8 + 0.3 * rng.normal(size=(H, H))), "temp": bf(rng.uniform(0.6, 1.6, H)),
            "out": bf(1.0 + 0.2 * rng.normal(size=width))}


def left_config(o):
    return {"heads": o["heads"], "kv_heads": o["kv_heads"], "dim": o["dim"], "vdim": o["vdim"], "mask": {"size": o["window"]},
            "rot": {"base": o["base"], "dims": o["rot_dims"]}, "scale": o["scale"] if o["scale"] is not None else o["dim"] ** -0.5}


def right_weights(rng, width, o):
    bf = bf16_values
    r = lambda *s: bf(rng.normal(0, 1.0 / math.sqrt(s[-1]), s))
    Hn, P, N, G, taps = o["heads"], o["vdim"], o["state"], o["groups"], o["conv"]
    inner, ch = Hn * P, Hn * P + 2 * G * N
    return {"in": r(2 * inner + 2 * G * N + Hn, width), "conv": bf(rng.normal(0, 0.6, (ch, taps))), "conv.b": bf(0.1 * rng.normal(size=ch)),
            "dt_bias": bf(rng.uniform(-3.0, 0.5, Hn)), "A_log": bf(np.log(rng.uniform(0.3, 4.0, Hn))), "D": bf(rng.normal(size=Hn)),
            "norm": bf(1.0 + 0.2 * rng.normal(size=inner)), "o": r(width, inner), "out": bf(1.0 + 0.2 * rng.normal(size=width))}


def right_config(o):
    return {k: o[k] for k in ("heads", "vdim", "state", "groups", "conv", "norm_groups")}


def latent_weights(rng, width, o):
    bf = bf16_values
    r = lambda *s: bf(rng.normal(0, 1.0 / math.sqrt(s[-1]), s))
    H, D, Rd, V, R, Q = o["heads"], o["dim"], o["rot_dim"], o["vdim"], o["kv_rank"], o["q_rank"]
    w = {"dq": r(Q, width), "dq.norm": bf(1.0 + 0.2 * rng.normal(size=Q)), "uq": r(H * (D + Rd), Q), "uk": r(H * D, R), "uv": r(H * V, R),
         "g": r(H * V, width), "o": r(width, H * V)}
    if o.get("kv_from") is None:
        w["dkv"], w["dkv.norm"] = r(R + Rd, width), bf(1.0 + 0.2 * rng.normal(size=R))
    return w


def latent_config(o):
    m = {"heads": o["heads"], "dim": o["dim"], "rot_dim": o["rot_dim"], "vdim": o["vdim"], "kv_rank": o["kv_rank"], "q_rank": o["q_rank"],
         "rot": {"base": o["base"], "dims": o["rot_dim"]}, "scale": o["scale"] if o["scale"] is not None else (o["dim"] + o["rot_dim"]) ** -0.5}
    if o.get("kv_from") is not None:
        m["kv_from"] = o["kv_from"]
    return m


def ff_weights(rng, width, fc):
    bf = bf16_values
    r = lambda *s: bf(rng.normal(0, 1.0 / math.sqrt(s[-1]), s))
    if fc["kind"] == "dense":
        return {"up": r(fc["ff"], width), "down": r(width, fc["ff"]), "act": bf(np.array([0.7, 0.35, -0.2, 0.05]) + 0.05 * rng.normal(size=4))}
    w = {"router": bf(rng.normal(0, 2.0 / math.sqrt(width), (fc["router"]["experts"], width)))}
    for e in range(fc["router"]["experts"]):
        w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"] = r(fc["expert"]["ff"], width), r(fc["expert"]["ff"], width), r(width, fc["expert"]["ff"])
    return w


def ff_config(spec):
    """spec: None, ("dense", ff) or ("moe", overrides of MOE)"""
    if spec is None:
        return None
    if spec[0] == "dense":
        return {"kind": "dense", "ff": int(spec[1])}
    o = dict(MOE, **(spec[1] if len(spec) > 1 else {}))
    return {"kind": "moe", "expert": {"ff": o["ff"]}, "router": {"experts": o["experts"], "top": o["top"], "groups": {"count": o["count"], "keep": o["keep"]}}}


def random_filipel(rng, layers, width=72, vocab=97, eps=1e-5, residual_mult=0.5):
    """A small random model -> (config, tensors as float32 arrays of bf16 values).  layers: a list of (type, mixer overrides, ff spec):
    type "parallel" with overrides {"left": {..}, "right": {..}} of LEFT / RIGHT, or "latent_attention" with overrides of LATENT;
    ff spec as ff_config takes it."""
    bf = bf16_values
    cfg = {"architecture": "Filipel", "width": width, "vocab": vocab, "norm": {"eps": eps}, "residual_mult": residual_mult, "layers": []}
    t = {"embed": bf(rng.normal(size=(vocab, width))), "head": bf(rng.normal(0, 1.0 / math.sqrt(width), (vocab, width))),
         "final.norm": bf(1.0 + 0.2 * rng.normal(size=width))}
    for i, (kind, over, ff) in enumerate(layers):
        p = f"l{i}."
        t[p + "norm1"] = bf(1.0 + 0.2 * rng.normal(size=width))
        if kind == "parallel":
            lo, ro = dict(LEFT, **(over or {}).get("left", {})), dict(RIGHT, **(over or {}).get("right", {}))
            m = {"left": left_config(lo), "right": right_config(ro)}
            for k, v in left_weights(rng, width, lo).items():
                t[p + "mix.left." + k] = v
            for k, v in right_weights(rng, width, ro).items():
                t[p + "mix.right." + k] = v
        else:
            o = dict(LATENT, **(over or {}))
            m = latent_config(o)
            for k, v in latent_weights(rng, width, o).items():
                t[p + "mix." + k] = v
        fc = ff_config(ff)
        if fc is not None:
            for k, v in ff_weights(rng, width, fc).items():
                t[p + "mlp." + k] = v
        cfg["layers"].append({"type": kind, "mixer": m, "mlp": fc})
    return cfg, t
