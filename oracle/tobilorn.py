"""Plain, slow float64 restatement of the Tobilorn design, one function per mechanism, row by row.  Test infrastructure only:
numpy, no kernels, no code shared with the product path.

Notation: h [n, width] the rows of ONE sequence in order (row p is position p); weights as the checkpoint stores them
([out, in]); w maps the names below '<layer>.mix.' / '<layer>.mlp.' / '<layer>.side.' to arrays."""
import math

import numpy as np


def f64(a):
    return np.asarray(a, np.float64)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z / (1.0 + np.exp(-z))


def unit_rms(x, eps):
    x = f64(x)
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def offset_norm(x, w, eps):
    """RMS norm whose stored weight is the deviation from one"""
    return unit_rms(x, eps) * (1.0 + f64(w))


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


# -- attention ------------------------------------------------------------------------------------------------------------
def visible(i, j, window, keep_first):
    """may the row at position i read the key at position j"""
    return j <= i and (i - j < window or j < keep_first)


def masked_softmax_rows(q, k, v, scale, window, keep_first):
    """q [n, D], k [n, D], v [n, V] of one map of one head -> [n, V]"""
    n = q.shape[0]
    out = np.zeros((n, v.shape[1]))
    for i in range(n):
        js = [j for j in range(i + 1) if visible(i, j, window, keep_first)]
        s = (k[js] @ q[i]) * scale
        e = np.exp(s - s.max())
        out[i] = (e / e.sum()) @ v[js]
    return out


def differential_lambda(w, diff):
    return math.exp(float(f64(w["lq1"]) @ f64(w["lk1"]))) - math.exp(float(f64(w["lq2"]) @ f64(w["lk2"]))) + float(diff)


def differential_attention(h, w, m, eps, maps_out=None):
    """Two softmax maps per head over the same values, the second subtracted lambda times; the difference is divided by its root
    mean square per head and scaled by 1 - diff.  m: the layer's mixer config."""
    n = h.shape[0]
    H, G, D, V = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    window, keep = int(m["mask"]["size"]), int(m["mask"]["keep_first"])
    rd, base, diff = int(m["rot"]["dims"]), float(m["rot"]["base"]), float(m["diff"])
    h = f64(h)
    q = (h @ f64(w["q"]).T + f64(w["q.b"])).reshape(n, H, 2, D)
    k = (h @ f64(w["k"]).T + f64(w["k.b"])).reshape(n, G, 2, D)
    v = (h @ f64(w["v"]).T + f64(w["v.b"])).reshape(n, G, V)
    q = np.stack([rotate_halves(q[p], p, rd, base) for p in range(n)])
    k = np.stack([rotate_halves(k[p], p, rd, base) for p in range(n)])
    lam = differential_lambda(w, diff)
    out = np.zeros((n, H, V))
    for hd in range(H):
        g = hd // (H // G)
        a1 = masked_softmax_rows(q[:, hd, 0], k[:, g, 0], v[:, g], float(m["scale"]), window, keep)
        a2 = masked_softmax_rows(q[:, hd, 1], k[:, g, 1], v[:, g], float(m["scale"]), window, keep)
        if maps_out is not None:
            maps_out.append((a1, a2))
        out[:, hd] = unit_rms(a1 - lam * a2, eps) * (1.0 - diff)
    return out.reshape(n, H * V) @ f64(w["o"]).T + f64(w["o.b"])


# -- feed-forward -----------------------------------------------------------------------------------------------------------
def gated_unit(h, gate, up, down):
    return (silu(h @ f64(gate).T) * (h @ f64(up).T)) @ f64(down).T


def route(h, w, top):
    """-> (chosen expert indices [n, top], their weights [n, top]): softmax over every router output; the choice adds a
    correction per expert to the scores, the weights do not"""
    z = f64(h) @ f64(w["router"]).T
    s = np.exp(z - z.max(1, keepdims=True))
    s /= s.sum(1, keepdims=True)
    pick = s + f64(w["correction"])
    idx = np.argsort(-pick, axis=1, kind="stable")[:, :top]
    ws = np.take_along_axis(s, idx, 1)
    return idx, ws / (ws.sum(1, keepdims=True) + 1e-20)


def moe_ff(h, w, fc, chosen=None):
    """fc: the layer's mlp config.  The last router.identity router outputs stand for experts that return their input."""
    h = f64(h)
    n_real, top = int(fc["router"]["experts"]), int(fc["router"]["top"])
    idx, ws = route(h, w, top)
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        if chosen is not None:
            chosen.append(idx[t].tolist())
        for e, p in zip(idx[t], ws[t]):
            out[t] += p * (h[t] if e >= n_real else gated_unit(h[t:t + 1], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"])[0])
    if fc.get("shared") is not None:
        out += gated_unit(h, w["shared.gate"], w["shared.up"], w["shared.down"])
    return out


# -- per-layer token input ----------------------------------------------------------------------------------------------------
def token_side(x, e, w, eps):
    """x [n, width] the stream, e [n, dim] the tokens' rows of this layer's part of the side table"""
    y = (gelu_tanh(f64(x) @ f64(w["gate"]).T) * f64(e)) @ f64(w["proj"]).T
    return unit_rms(y, eps) * f64(w["norm"])


# -- the model --------------------------------------------------------------------------------------------------------------
def _sub(tensors, prefix):
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def layer_runs(config):
    """[(layer index, pass number or None, first of its pass)] in the order the layers run"""
    n, loop = len(config["layers"]), config.get("loop")
    if not loop:
        return [(i, None, False) for i in range(n)]
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    runs = [(i, None, False) for i in range(a)]
    for t in range(times):
        runs += [(i, t, i == a) for i in range(a, b)]
    return runs + [(i, None, False) for i in range(b, n)]


def tobilorn_forward(config, tensors, tokens, layer_streams=None):
    """tensors: name -> numpy array.  -> logits [n, vocab] (float64); layer_streams collects the stream after every layer run"""
    eps = float(config["norm"]["eps"])
    tokens = list(tokens)
    x0 = f64(tensors["embed"])[tokens] * float(config["embedding"]["scale"])
    x = x0
    sd = int(config["token_side"]["dim"]) if config.get("token_side") else 0
    for i, t, first in layer_runs(config):
        if first:
            x = np.concatenate([x, x0], 1) @ f64(tensors["loop.in"]).T + f64(tensors["loop.step"])[t]
        lc, p = config["layers"][i], f"l{i}."
        if lc["type"] != "attention":
            raise ValueError(lc["type"])
        mo = differential_attention(offset_norm(x, tensors[p + "norm1"], eps), _sub(tensors, p + "mix."), lc["mixer"], eps)
        x = x + offset_norm(mo, tensors[p + "norm1b"], eps)
        if lc.get("mlp") is not None:
            fo = moe_ff(offset_norm(x, tensors[p + "norm2"], eps), _sub(tensors, p + "mlp."), lc["mlp"])
            x = x + offset_norm(fo, tensors[p + "norm2b"], eps)
        if sd:
            x = x + token_side(x, f64(tensors["side.embed"])[tokens][:, i * sd:(i + 1) * sd], _sub(tensors, p + "side."), eps)
        if layer_streams is not None:
            layer_streams.append(x)
    return offset_norm(x, tensors["final.norm"], eps) @ f64(tensors["head"]).T * float(config["logit_scale"])


def bf16_values(a):
    """float32 array whose values are exactly representable in bfloat16 (round to nearest even)"""
    u = np.asarray(a, np.float32).view(np.uint32)
    u = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    return u.astype(np.uint32).view(np.float32)


def random_tobilorn(rng, width=72, vocab=97, layers=5, loop=(1, 3, 3), heads=6, kv_heads=2, dim=16, vdim=24, rot_dims=None, base=10000.0,
                    scale=None, diff=0.25, window=40, keep_first=5, experts=5, identity=1, top=3, expert_ff=20, shared_ff=36, side_dim=12,
                    embed_scale=3.0, logit_scale=0.7, eps=1e-5, no_mlp=(), per_layer=None):
    """A small random model -> (config, tensors as float32 arrays of bf16 values).  loop: (start, stop, times) or None; no_mlp:
    layers without a feed-forward; per_layer: {layer index: overrides of the sizes above for that layer}."""
    bf = bf16_values
    r = lambda *s, sd=None: bf(rng.normal(0, sd if sd is not None else 1.0 / math.sqrt(s[-1]), s))
    cfg = {"architecture": "Tobilorn", "width": width, "vocab": vocab, "norm": {"eps": eps}, "embedding": {"scale": embed_scale},
           "logit_scale": logit_scale, "layers": []}
    t = {"embed": r(vocab, width, sd=1.0), "head": r(vocab, width), "final.norm": bf(0.2 * rng.normal(size=width))}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
        t["loop.in"], t["loop.step"] = r(width, 2 * width, sd=1.0 / math.sqrt(width)), bf(0.5 * rng.normal(size=(loop[2], width)))
    if side_dim:
        cfg["token_side"] = {"dim": side_dim}
        t["side.embed"] = r(vocab, layers * side_dim, sd=1.0)
    for i in range(layers):
        o = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, rot_dims=rot_dims, base=base, scale=scale, diff=diff, window=window,
                 keep_first=keep_first, experts=experts, identity=identity, top=top, expert_ff=expert_ff, shared_ff=shared_ff)
        o.update((per_layer or {}).get(i, {}))
        H, G, D, V = o["heads"], o["kv_heads"], o["dim"], o["vdim"]
        p = f"l{i}."
        m = {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "diff": o["diff"], "scale": o["scale"] if o["scale"] is not None else D ** -0.5,
             "mask": {"size": o["window"], "keep_first": o["keep_first"]},
             "rot": {"base": o["base"], "dims": o["rot_dims"] if o["rot_dims"] is not None else D}}
        for nm in ("norm1", "norm1b"):
            t[p + nm] = bf(0.2 * rng.normal(size=width))
        t[p + "mix.q"], t[p + "mix.k"], t[p + "mix.v"] = r(H * 2 * D, width), r(G * 2 * D, width), r(G * V, width)
        t[p + "mix.o"], t[p + "mix.o.b"] = r(width, H * V), bf(0.1 * rng.normal(size=width))
        for nm, rows in (("q", H * 2 * D), ("k", G * 2 * D), ("v", G * V)):
            t[p + f"mix.{nm}.b"] = bf(0.2 * rng.normal(size=rows))
        for nm in ("lq1", "lk1", "lq2", "lk2"):
            t[p + "mix." + nm] = bf(rng.normal(0, 0.6 / math.sqrt(D), D))
        layer = {"type": "attention", "mixer": m, "mlp": None}
        if i not in no_mlp:
            E, I = o["experts"], o["identity"]
            layer["mlp"] = {"kind": "moe", "expert": {"ff": o["expert_ff"]}, "router": {"experts": E, "identity": I, "top": o["top"]},
                            "shared": {"ff": o["shared_ff"]} if o["shared_ff"] else None}
            for nm in ("norm2", "norm2b"):
                t[p + nm] = bf(0.2 * rng.normal(size=width))
            for e in range(E):
                t[p + f"mlp.e{e}.gate"], t[p + f"mlp.e{e}.up"] = r(o["expert_ff"], width), r(o["expert_ff"], width)
                t[p + f"mlp.e{e}.down"] = r(width, o["expert_ff"])
            t[p + "mlp.router"] = r(E + I, width, sd=2.0 / math.sqrt(width))
            t[p + "mlp.correction"] = bf(0.05 * rng.normal(size=E + I))
            if o["shared_ff"]:
                t[p + "mlp.shared.gate"], t[p + "mlp.shared.up"] = r(o["shared_ff"], width), r(o["shared_ff"], width)
                t[p + "mlp.shared.down"] = r(width, o["shared_ff"])
        if side_dim:
            t[p + "side.gate"], t[p + "side.proj"] = r(side_dim, width), r(width, side_dim)
            t[p + "side.norm"] = bf(0.5 + 0.1 * rng.normal(size=width))
        cfg["layers"].append(layer)
    return cfg, t
