"""Filipel: a decoder-only model whose layers run their token mixer and their feed-forward side by side on ONE layer-normed copy of
the stream.

  embedding   x = embed[token]
  layer i     h = layer_norm(x) * norm1 (mean and variance, no bias);  x <- x + residual_mult * (mixer(h) + ff(h))
              mixer 'latent_attention': causal attention through a low-rank latent; queries through a normed latent of their own; every
                    head's query is [dim plain | rot_dim rotated], the key is [W_uk c | one rotated part shared by the heads]; only the
                    normed latent c and the rotated key part are cached; sigmoid gate per output element; a layer with kv_from reads
                    the cache of an earlier layer (with its own W_uk, W_uv and queries)
              mixer 'parallel': two mixers on the same h, each result RMS-normed over the width and weighted, then averaged --
                    left:  grouped-query attention, rotary positions on the two halves of the rotated part, a multiplier per head on
                           the scores, a sliding window, softmax maps mixed between the heads by a matrix, sigmoid gate per element
                    right: a state-space mixer: short causal convolution + silu on [x | B | C], softplus step sizes, a scalar decay
                           per head, a matrix state, skip term, silu gate before a grouped RMS norm
              ff:   dense: down(polynorm(up h)) with a cubic of row-normalised powers; or routed experts (silu units): scores =
                    softmax over all experts, only the experts of the best groups can be chosen, weights = the chosen scores over
                    their sum; or none
  head        logits = head . layer_norm(x; final.norm)
Sizes, the order of the layers and every constant come from config.json; tensor names are those of the checkpoint
('l<i>.norm1', 'l<i>.mix.*', 'l<i>.mix.left.*', 'l<i>.mix.right.*', 'l<i>.mlp.*').
"""
import torch

from .. import mixers
from .. import seq_ops as so
from . import register


def _sub(tensors, prefix):
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


@register("Filipel")
class Filipel:
    engine = "sequence"

    def __init__(self, config, tensors, state, dtype):
        self.config = config
        self.width, self.vocab = int(config["width"]), int(config["vocab"])
        self.eps = float(config["norm"]["eps"])
        self.mult = float(config.get("residual_mult", 1.0))
        self.dtype = dtype
        self.math = so.MATH_BF16 if dtype == torch.bfloat16 else so.MATH_F32
        self.embed = tensors["embed"]
        assert self.embed.shape == (self.vocab, self.width)
        self.final_norm, self.head = tensors["final.norm"].contiguous(), tensors["head"].contiguous()
        self.layers = []
        for i, lc in enumerate(config["layers"]):
            w, m, kind = _sub(tensors, f"l{i}."), lc["mixer"], lc["type"]
            if kind == "latent_attention":
                mixer = self._latent(i, m, _sub(w, "mix."), state, dtype)
            elif kind == "parallel":
                lw, rw = _sub(w, "mix.left."), _sub(w, "mix.right.")
                mixer = mixers.SideBySide(self._windowed(i, m["left"], lw, state, dtype), self._state_space(i, m["right"], rw, state),
                                          lw["out"], rw["out"], coef=0.5)
            else:
                raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
            self.layers.append((w["norm1"].contiguous(), mixer, self._feed_forward(i, lc.get("mlp"), _sub(w, "mlp."))))

    # -- the parts of a layer, each from its piece of the configuration ---------------------------------------------------------
    def _latent(self, i, m, mw, state, dtype):
        src, key_from = m.get("kv_from"), None
        if src is not None:
            src = int(src)
            sm = self.config["layers"][src]["mixer"] if 0 <= src < i else None
            if sm is None or self.config["layers"][src]["type"] != "latent_attention" or sm.get("kv_from") is not None:
                raise ValueError(f"layer {i}: kv_from {src} is no earlier latent-attention layer with a cache of its own")
            if (int(sm["kv_rank"]), int(sm["rot_dim"]), float(sm["rot"]["base"])) != (int(m["kv_rank"]), int(m["rot_dim"]), float(m["rot"]["base"])):
                raise ValueError(f"layer {i}: the cache of layer {src} has another latent size or rotation")
            key_from = f"l{src}.latent"
        rot = m.get("rot") or {}
        if int(rot.get("dims", m.get("rot_dim", 0))) != int(m.get("rot_dim", 0)):
            raise ValueError(f"layer {i}: the rotated part is rot_dim wide")
        return mixers.LatentWindowAttention(f"l{i}.latent", int(m["heads"]), int(m["dim"]), int(m["vdim"]), int(m["kv_rank"]), int(m["q_rank"]), 0,
                                            float(m["scale"]), mw, state, dtype, kv_from_key=key_from, rot_dim=int(m.get("rot_dim", 0)),
                                            rot_base=float(rot.get("base", 10000.0)))

    def _windowed(self, i, m, lw, state, dtype):
        rot, mask = m.get("rot") or {}, m.get("mask") or {}
        return mixers.GroupedQueryAttention(f"l{i}.attn", int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"]), float(m["scale"]), lw,
                                            state, dtype, rot_dims=int(rot.get("dims", 0)), rot_base=float(rot.get("base", 10000.0)),
                                            rot_layout="halves", window=int(mask.get("size", 0)), head_temp=lw["temp"], talk=lw["talk"],
                                            elem_gate=True)

    def _state_space(self, i, m, rw, state):
        return mixers.StateSpaceMixer(f"l{i}.ssm", int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m["groups"]), int(m["conv"]),
                                      int(m["norm_groups"]), rw, state)

    def _feed_forward(self, i, fc, fw):
        if fc is None:
            return None
        if fc["kind"] == "dense":
            assert fw["up"].shape == (int(fc["ff"]), self.width)
            return mixers.DenseMlp(fw["up"], fw["down"], ("polynorm", fw["act"]))
        if fc["kind"] == "moe":
            r = fc["router"]
            n, g = int(r["experts"]), r.get("groups") or {}
            assert fw["e0.gate"].shape == (int(fc["expert"]["ff"]), self.width)
            return mixers.ExpertMlp(fw["router"], None, [fw[f"e{e}.gate"] for e in range(n)], [fw[f"e{e}.up"] for e in range(n)],
                                    [fw[f"e{e}.down"] for e in range(n)], int(r["top"]), unit="silu", scoring="scores",
                                    groups=(int(g.get("count", 1)), int(g.get("keep", g.get("count", 1)))))
        raise ValueError(f"layer {i}: unknown feed-forward kind {fc['kind']!r}")

    @classmethod
    def from_config(cls, config, tensors, state, dtype):
        return cls(config, tensors, state, dtype)

    def second_rows(self, prev, tokens):
        return None      # one embedding table

    def forward(self, ctx):
        """-> the residual stream after the last layer, [T, width] f32.  The residual step of a layer and the input norm of the next
        one are one launch; bf16 products read a bf16 copy of the norm's output (the same bits at half the traffic)."""
        act = torch.bfloat16 if self.math == so.MATH_BF16 else torch.float32
        x = so.embed_sum(ctx.ids, self.embed)
        h = so.residual_layernorm(x, self.layers[0][0], eps=self.eps, out_dtype=act) if self.layers else None
        for i, (_, mixer, ff) in enumerate(self.layers):
            h32, h16 = (None, h) if act == torch.bfloat16 else (h, None)
            mo = mixer(ctx, h32, h16)
            fo = ff(ctx, h32, h16) if ff is not None else None
            nxt = self.layers[i + 1][0] if i + 1 < len(self.layers) else None
            h = so.residual_layernorm(x, nxt, a=mo, b=fo, mult=self.mult, eps=self.eps, x_out=x, out_dtype=act)
            if ctx.taps is not None:
                ctx.taps[i] = x.clone()
        return x

    def logits(self, ctx, x, rows):
        """rows: int32 device tensor of the row indices whose logits are wanted -> f32 [len(rows), vocab]"""
        hn = so.residual_layernorm(x, self.final_norm, eps=self.eps, row_idx=rows,
                                   out_dtype=torch.bfloat16 if self.math == so.MATH_BF16 else torch.float32)
        return so.linear(hn, self.head, math=ctx.math)
