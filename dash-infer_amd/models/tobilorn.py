"""Tobilorn: a decoder-only model of differential-attention layers with routed feed-forwards, a looped block of layers and a
per-layer token input.

  embedding   x0 = embed[token] * embedding.scale
  layer i     x <- x + norm1b(mixer(norm1(x)));  x <- x + norm2b(ff(norm2(x))) where the layer has a feed-forward;
              norm(v) = v / rms(v) * (1 + w): the stored weight is the deviation from one
              then the token's side input:  x <- x + unit_rms(side.proj(gelu(side.gate x) * side.embed[token, part i])) * side.norm
              mixer 'attention': grouped-query differential attention -- two softmax maps per head (queries and keys of the two maps
                    side by side) over the same values, biases, rotary positions on the two halves of the rotated part of every
                    map, a sliding window that keeps the first keys; out = unit_rms(map1 - lambda map2) (1 - diff) per head with
                    lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff
              ff:   routed experts (silu units): scores = softmax over all router outputs, the choice by score + correction, weights
                    = the chosen scores over their sum; the last router outputs are identity experts; a shared expert is added
  loop        layers start .. stop - 1 run `times` times in a row with the same weights and a cache per pass; every pass starts
              with x <- loop.in [x; x0] + loop.step[pass]
  head        logits = head . norm(x; final.norm) * logit_scale
Sizes, layer order and constants come from config.json; tensor names are those of the checkpoint ('l<i>.mix.*', 'l<i>.mlp.*',
'l<i>.side.*').
"""
import math

import torch

from .. import mixers
from .. import seq_ops as so
from . import register


def _sub(tensors, prefix):
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def layer_runs(n_layers, loop):
    """[(layer, which run of that layer, pass that starts here or None)] in the order the layers run"""
    if not loop:
        return [(i, 0, None) for i in range(n_layers)]
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    if not 0 <= a < b <= n_layers or times < 1:
        raise ValueError(f"loop {loop!r} does not fit {n_layers} layers")
    runs = [(i, 0, None) for i in range(a)]
    for t in range(times):
        runs += [(i, t, t if i == a else None) for i in range(a, b)]
    return runs + [(i, 0, None) for i in range(b, n_layers)]


class _Layer:
    __slots__ = ("norm1", "norm1b", "mixer", "norm2", "norm2b", "ff", "side")


class _Side:
    """the per-layer token input: columns [col0, col0 + dim) of the shared side table"""
    __slots__ = ("col0", "dim", "gate", "proj", "norm")


@register("Tobilorn")
class Tobilorn:
    engine = "sequence"

    def __init__(self, config, tensors, state, dtype):
        self.config = config
        self.width, self.vocab = int(config["width"]), int(config["vocab"])
        self.eps = float(config["norm"]["eps"])
        self.dtype = dtype
        self.math = so.MATH_BF16 if dtype == torch.bfloat16 else so.MATH_F32
        self.embed = tensors["embed"].contiguous()
        assert self.embed.shape == (self.vocab, self.width)
        self.embed_scale = float((config.get("embedding") or {}).get("scale", 1.0))
        self.logit_scale = float(config.get("logit_scale", 1.0))
        self.final_norm, self.head = tensors["final.norm"].contiguous(), tensors["head"].contiguous()
        n = len(config["layers"])
        self.loop = config.get("loop") or None
        self.runs = layer_runs(n, self.loop)
        if self.loop:
            self.loop_in, self.loop_step = tensors["loop.in"].contiguous(), tensors["loop.step"].contiguous()
            assert self.loop_in.shape == (self.width, 2 * self.width) and self.loop_step.shape == (int(self.loop["times"]), self.width)
        side = config.get("token_side") or None
        self.side_dim = int(side["dim"]) if side else 0
        if self.side_dim:
            self.side_embed = tensors["side.embed"].contiguous()
            assert self.side_embed.shape == (self.vocab, n * self.side_dim)
        times = {i: sum(1 for r in self.runs if r[0] == i) for i in range(n)}
        self.layers = []
        for i, lc in enumerate(config["layers"]):
            w, m = _sub(tensors, f"l{i}."), lc["mixer"]
            L = _Layer()
            L.norm1, L.norm1b = w["norm1"].contiguous(), w["norm1b"].contiguous()
            if lc["type"] != "attention":
                raise ValueError(f"layer {i}: unknown mixer type {lc['type']!r}")
            mw = _sub(w, "mix.")
            diff = float(m["diff"])
            dot = lambda a, b: float((mw[a].double() * mw[b].double()).sum().item())        # once, at load
            lam = math.exp(dot("lq1", "lk1")) - math.exp(dot("lq2", "lk2")) + diff
            mask, rot = m.get("mask") or {}, m.get("rot") or {}
            L.mixer = mixers.GroupedQueryAttention(
                f"l{i}.attn", int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"]), float(m["scale"]), mw, state, dtype,
                rot_dims=int(rot.get("dims", 0)), rot_base=float(rot.get("base", 10000.0)), rot_layout="halves",
                window=int(mask.get("size", 0)), keep_first=int(mask.get("keep_first", 0)), differential=(lam, 1.0 - diff), runs=times[i])
            L.ff, fc = None, lc.get("mlp")
            L.norm2 = L.norm2b = None
            if fc is not None:
                if fc.get("kind", "moe") != "moe":
                    raise ValueError(f"layer {i}: unknown feed-forward kind {fc['kind']!r}")
                fw = _sub(w, "mlp.")
                L.norm2, L.norm2b = w["norm2"].contiguous(), w["norm2b"].contiguous()
                ne, ident = int(fc["router"]["experts"]), int(fc["router"].get("identity", 0))
                shared = None
                if fc.get("shared") is not None:
                    shared = mixers.GatedMlp(fw["shared.gate"], fw["shared.up"], fw["shared.down"], "silu")
                    assert fw["shared.gate"].shape == (int(fc["shared"]["ff"]), self.width)
                L.ff = mixers.ExpertMlp(fw["router"], None, [fw[f"e{e}.gate"] for e in range(ne)], [fw[f"e{e}.up"] for e in range(ne)],
                                        [fw[f"e{e}.down"] for e in range(ne)], int(fc["router"]["top"]), unit="silu", scoring="scores",
                                        correction=fw.get("correction"), identity=ident, shared=shared)
                assert fw["e0.gate"].shape == (int(fc["expert"]["ff"]), self.width)
            L.side = None
            if self.side_dim:
                S = _Side()
                S.col0, S.dim = i * self.side_dim, self.side_dim
                S.gate, S.proj, S.norm = w["side.gate"].contiguous(), w["side.proj"].contiguous(), w["side.norm"].contiguous()
                assert S.gate.shape == (S.dim, self.width) and S.proj.shape == (self.width, S.dim)
                L.side = S
            self.layers.append(L)

    @classmethod
    def from_config(cls, config, tensors, state, dtype):
        return cls(config, tensors, state, dtype)

    def second_rows(self, prev, tokens):
        return None      # the side table is read by the token's own id

    def forward(self, ctx):
        """-> the residual stream after the last layer, [T, width] f32.

        Every sublayer leaves (its output m, the weight of the norm on it); the residual step x <- x + norm(m) runs fused with what
        the NEXT sublayer reads: its input norm, a copy of the stream in the products' type, or the left half of the loop's input."""
        T, W, eps = ctx.T, self.width, ctx.eps
        dev = self.embed.device
        act = torch.bfloat16 if self.math == so.MATH_BF16 else torch.float32
        x = so.embed_rows(ctx.ids, self.embed, scale=self.embed_scale)
        cat = None
        if self.loop:     # [x | x0] as the pass entry reads it; x0 is written once
            cat = torch.empty(T, 2 * W, dtype=act, device=dev)
            so.embed_rows(ctx.ids, self.embed, scale=self.embed_scale, out=cat[:, W:])
        side = so.embed_rows(ctx.ids, self.side_embed) if self.side_dim else None      # every layer's part of the tokens' side rows, once
        pending = None    # (m, gamma, gamma_add) of the sublayer that ran last

        def advance(norm=None, raw=False, left=False):
            """apply the pending residual step -> what the next sublayer reads (norm: its input norm's weight; raw: the stream as
            the products read it; left: nothing, the stream goes into the left half of `cat`)"""
            nonlocal x, pending
            m, gm, am = pending if pending is not None else (None, None, 0.0)
            pending = None
            h = torch.empty(T, W, dtype=act, device=dev) if norm is not None else None
            copy = cat[:, :W] if left else (torch.empty(T, W, dtype=act, device=dev) if raw and act != torch.float32 else None)
            if m is not None or h is not None or copy is not None:
                x = so.residual_norm_step(x, eps, m=m, gamma_m=gm, add_m=am, gamma_h=norm, add_h=1.0, h=h, copy=copy)
            return h if norm is not None else (copy if copy is not None else x)

        for r, (li, run, enter) in enumerate(self.runs):
            L = self.layers[li]
            if enter is not None:
                advance(left=True)
                x = so.linear(cat, self.loop_in, self.loop_step[enter], math=ctx.math)
            pending = (L.mixer(ctx, advance(norm=L.norm1), run=run), L.norm1b, 1.0)
            if L.ff is not None:
                pending = (L.ff(ctx, advance(norm=L.norm2)), L.norm2b, 1.0)
            if L.side is not None:
                S = L.side
                g = so.linear(advance(raw=True), S.gate, act="gelu_tanh", mul=side[:, S.col0: S.col0 + S.dim], math=ctx.math,
                              out=ctx.act_buffer(S.dim))
                pending = (so.linear(g, S.proj, math=ctx.math), S.norm, 0.0)
            if ctx.taps is not None:
                advance()
                ctx.taps[r] = x.clone()
        advance()
        return x

    def logits(self, ctx, x, rows):
        """rows: int32 device tensor of the row indices whose logits are wanted -> f32 [len(rows), vocab]"""
        hn = torch.empty(rows.shape[0], self.width, dtype=torch.bfloat16 if self.math == so.MATH_BF16 else torch.float32, device=x.device)
        so.rmsnorm(x, self.final_norm, ctx.eps, row_idx=rows, out=hn, gamma_add=1.0, out_scale=self.logit_scale)
        return so.linear(hn, self.head, math=ctx.math)
