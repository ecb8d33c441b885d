"""Token mixers and feed-forward blocks of the sequence engine, each with its constants as parameters.

A mixer maps the rows h [T, width] (f32) of one step -- portions of several sequences, described by the step context --
to rows of the same shape, reading and updating what its sequences left in the state manager:
  LatentWindowAttention  attention through a low-rank latent that alone is cached (paged), sliding window, softmax sink,
                         sigmoid output gate; a layer may read the latent cache another layer writes; option: a rotated part of
                         every head's query against ONE rotated key part per token, cached behind the latent
  GatedLinearRecurrence  two-branch recurrent block: gelu branch x (short causal convolution -> block-diagonal gates ->
                         real-gated diagonal recurrence), f32 state and convolution tail per slot
  DenseMlp               down(act(up(h))); act: an elementwise activation, or ("polynorm", coef): a cubic of row-normalised powers
  GroupedQueryAttention  causal attention over paged key and value caches with fewer key/value heads than query heads; options:
                         unit-RMS norm of queries and keys, rotary positions (paired or half-split layout, part of the head,
                         frequencies rescaled for longer contexts), biases, a sink logit (per head or the constant 0), a tanh cap
                         on the scores, a sigmoid gate per head, values mixed with those of an earlier layer of the same step,
                         a sliding window that keeps the first keys of the sequence, two softmax maps per head whose difference
                         is normed per head (differential attention), several runs per step with a cache each (looped layers),
                         a multiplier per head on the scores, softmax maps mixed between the heads after the softmax (talking
                         heads), a sigmoid gate per output element
  GatedLinearAttention   linear attention with a decay per key channel and a matrix state per head (f32, per slot), unit-RMS
                         norm per head, silu output gate
  StateSpaceMixer        state-space duality form: short causal convolution + silu on [x | B | C], a scalar decay per head from a
                         softplus step size, a matrix state per head (f32, per slot), skip term, silu gate BEFORE a grouped RMS norm
  SideBySide             two mixers on the same input, their results RMS-normed over the width, weighted and averaged
  GatedMlp               down(act(gate(h)) * up(h))
  ExpertMlp              top-k routed experts; units: clamped sigmoid-gated or silu-gated; routing: softmax over the chosen logits,
                         or softmax scores over all router outputs with a correction added for the choice alone; router outputs
                         past the real experts stand for identity experts; an always-on shared expert
Matrix products run in ctx.math (seq_ops.MATH_F32 / MATH_BF16); norms, scores, gates of the recurrence, decays and
state are f32 in both.
"""
import torch

from . import seq_ops as so


class StepContext:
    """One step's flat batch on the device.  ids / rows2: token and second-table rows; tok_*: per row; ent_*: per portion."""

    def __init__(self, T, E, ids, rows2, tok_slot, tok_pos, tok_off, ent_slot, ent_row0, ent_count, want_rows, math, eps):
        self.T, self.E = T, E
        self.ids, self.rows2, self.tok_slot, self.tok_pos, self.tok_off = ids, rows2, tok_slot, tok_pos, tok_off
        self.ent_slot, self.ent_row0, self.ent_count, self.want_rows = ent_slot, ent_row0, ent_count, want_rows
        self.math, self.eps = math, eps
        self.max_count, self.max_pos = T, 0     # host numbers: the largest portion and the last position of the step
        self.taps = None    # layer index -> [T, .] intermediate (diagnostics; None: off)
        self.shared = {}    # what a layer leaves for later layers of the SAME step (values to be mixed in)

    def act_buffer(self, n, dtype=None):
        """[T, n] for an activation that only a product reads: bf16 under bf16 products (the product would round it anyway), else f32"""
        dt = dtype or (torch.bfloat16 if self.math == so.MATH_BF16 else torch.float32)
        return torch.empty(self.T, n, dtype=dt, device=self.ids.device)


class LatentWindowAttention:
    def __init__(self, key, heads, dim, vdim, kv_rank, q_rank, window, scale, w, state, cache_dtype, kv_from_key=None, rot_dim=0,
                 rot_base=10000.0):
        """w: dq [q_rank, width], dq.norm, uq [heads*(dim+rot_dim), q_rank], dkv [kv_rank+rot_dim, width] + dkv.norm (absent with
        kv_from_key), uk [heads*dim, kv_rank], uv [heads*vdim, kv_rank], sink [heads] (optional), g [heads*vdim, width],
        o [width, heads*vdim].
        rot_dim > 0: every head's query is [dim | rot_dim] and the last rot_dim rows of dkv are one key part shared by the heads;
        both rotate with the position (halves layout, base rot_base) and add q_rot . k_rot to the score.  The page row is then
        [latent | rotated key part | zeros up to a multiple of 32]: the attention kernels see a latent of that width, the
        absorbed queries carry their rotated part behind them, and the value product's weight has zero columns there."""
        self.H, self.D, self.V, self.R, self.Q, self.window, self.scale = heads, dim, vdim, kv_rank, q_rank, int(window or 0), float(scale)
        self.rot = int(rot_dim or 0)
        assert self.rot % 2 == 0
        self.owns_cache = kv_from_key is None
        parts = [w["dq"]] + ([w["dkv"]] if self.owns_cache else []) + [w["g"]]
        self.w_in = torch.cat(parts, 0).contiguous()          # one product for everything that reads h
        self.c_lo = q_rank
        self.g_lo = q_rank + (kv_rank + self.rot if self.owns_cache else 0)
        self.n_in = self.g_lo + heads * vdim
        self.dq_norm = w["dq.norm"]
        self.dkv_norm = w.get("dkv.norm")
        assert w["uq"].shape == (heads * (dim + self.rot), q_rank) and w["o"].shape[1] == heads * vdim
        assert not self.owns_cache or w["dkv"].shape[0] == kv_rank + self.rot
        dev = w["uq"].device
        if self.rot:
            # the cache row: latent, rotated key part, padding (whole 32-element steps for the matrix-core kernel on 16-bit pages)
            self.Rp = -(-(kv_rank + self.rot) // 32) * 32 if cache_dtype == torch.bfloat16 else kv_rank + self.rot
            uq = w["uq"].view(heads, dim + self.rot, q_rank)       # queries come out as [all heads' plain parts | all heads' rotated parts]
            self.uq = torch.cat([uq[:, :dim].reshape(heads * dim, q_rank), uq[:, dim:].reshape(heads * self.rot, q_rank)], 0).contiguous()
            self.freq = rotary_frequencies(self.rot, rot_base)[0].to(dev)
        else:
            self.Rp, self.uq, self.freq = kv_rank, w["uq"].contiguous(), None
        pad = self.Rp - kv_rank
        # scores against the latent itself: q' = W_uk[h]^T q_h, so that k = W_uk c never has to be formed
        uk_t = w["uk"].view(heads, dim, kv_rank).transpose(1, 2)                          # [H, R, D]
        uv = w["uv"].view(heads, vdim, kv_rank)                                            # [H, V, R]
        if pad:
            uk_t = torch.cat([uk_t, torch.zeros(heads, pad, dim, dtype=uk_t.dtype, device=dev)], 1)
            uv = torch.cat([uv, torch.zeros(heads, vdim, pad, dtype=uv.dtype, device=dev)], 2)
        self.uk_t, self.uv = uk_t.contiguous(), uv.contiguous()
        self.sink, self.o = w.get("sink"), w["o"].contiguous()
        if self.owns_cache:
            self.table = state.add_span_cache(key, self.Rp, cache_dtype)
        else:
            self.table = state.tables[kv_from_key]
            assert self.table.row_elems == self.Rp, "a shared latent cache must have this layer's rank (and rotated part)"
        self.mc = so.latent_attn_mc_supported(self.table) and (heads * self.Rp) % 4 == 0

    def __call__(self, ctx, h, h16=None):
        """h16: the bf16 copy of h where the producer made one (bf16 products read it: the same bits at half the traffic)"""
        H, D = self.H, self.D
        a = so.linear(h16 if h16 is not None else h, self.w_in, act="sigmoid", act_cols=(self.g_lo, self.n_in), math=ctx.math)
        cq = so.rmsnorm(a[:, : self.Q], self.dq_norm, ctx.eps, out=ctx.act_buffer(self.Q))
        if self.rot:      # the rotated parts stay f32 (angles and rotation are f32); the plain parts feed a product
            q = so.linear(cq, self.uq, math=ctx.math)
            ql = so.linear(q[:, : H * D], self.uk_t, groups=H, math=ctx.math)
            so.latent_rope_append(self.table, a[:, self.c_lo: self.g_lo], self.dkv_norm, ctx.eps, self.R, self.rot, self.freq, q[:, H * D:],
                                  ql, H, ctx.tok_slot, ctx.tok_pos, append=self.owns_cache)
        else:
            q = so.linear(cq, self.uq, math=ctx.math, out=ctx.act_buffer(H * D))
            if self.owns_cache:
                so.norm_span_append(self.table, a[:, self.c_lo: self.g_lo], self.dkv_norm, ctx.eps, ctx.tok_slot, ctx.tok_pos)
            ql = so.linear(q, self.uk_t, groups=H, math=ctx.math)
        if ctx.math == so.MATH_BF16 and self.mc:
            ol = so.latent_window_attn_mc(ql, self.table, self.sink, ctx.tok_pos, ctx.ent_slot, ctx.ent_row0, ctx.ent_count, ctx.max_count,
                                          ctx.max_pos, H, self.window, self.scale)
        else:
            ol = so.latent_window_attn(ql, self.table, self.sink, ctx.tok_slot, ctx.tok_pos, H, self.window, self.scale, math=ctx.math)
        og = so.linear(ol, self.uv, groups=H, mul=a[:, self.g_lo:], math=ctx.math, out=ctx.act_buffer(H * self.V))
        return so.linear(og, self.o, math=ctx.math)


class GatedLinearRecurrence:
    def __init__(self, key, width, blocks, taps, decay, w, state):
        """w: y [width, model], y.b, x [width, model], x.b, conv [width, taps], conv.b, ra / ri [blocks, bs, bs], ra.b / ri.b
        [blocks, bs], lam [width], o [model, width]"""
        assert width % blocks == 0 and w["conv"].shape == (width, taps)
        self.C, self.B, self.taps, self.decay = width, blocks, taps, float(decay)
        self.w_in = torch.cat([w["y"], w["x"]], 0).contiguous()
        self.b_in = torch.cat([w["y.b"], w["x.b"]], 0).contiguous()
        self.conv, self.conv_b = w["conv"].contiguous(), w["conv.b"].contiguous()
        self.w_gate = torch.cat([w["ra"], w["ri"]], 0).contiguous()           # [2B, bs, bs]: recurrence gates, then input gates
        self.b_gate = torch.cat([w["ra.b"], w["ri.b"]], 0).contiguous()
        self.lam, self.o = w["lam"].contiguous(), w["o"].contiguous()
        self.S = state.add_state(key + ".S", (width,))
        self.tail = state.add_state(key + ".tail", (taps - 1, width)) if taps > 1 else None

    def __call__(self, ctx, h, h16=None):
        C = self.C
        a = so.linear(h16 if h16 is not None else h, self.w_in, self.b_in, act="gelu_tanh", act_cols=(0, C), math=ctx.math)     # [y | x]
        y, x = a[:, :C], a[:, C:]
        u = so.causal_conv_state(x, self.conv, self.conv_b, self.tail, ctx.tok_slot, ctx.tok_off)
        if self.tail is not None:
            so.conv_tail_update(self.tail, x, self.taps, ctx.ent_slot, ctx.ent_row0, ctx.ent_count)
        g = so.linear(u, self.w_gate, self.b_gate, act="sigmoid", groups=2 * self.B, x_groups=self.B,
                      math=so.MATH_F32 if ctx.math == so.MATH_F32 else so.MATH_F32_STREAM)    # f32 products in both engines
        sy = so.gated_recurrence(g[:, :C], g[:, C:], u, y, self.lam, self.decay, self.S, ctx.ent_slot, ctx.ent_row0, ctx.ent_count,
                                 max_count=ctx.max_count)
        return so.linear(sy, self.o, math=ctx.math)


class DenseMlp:
    def __init__(self, up, down, act):
        """act: the name of an elementwise activation, or ("polynorm", coef [4]): c0 N(z) + c1 N(z^2) + c2 N(z^3) + c3 with powers
        per element and N = division by the row's root mean square (f32)"""
        self.up, self.down, self.act = up.contiguous(), down.contiguous(), act
        self.coef = None
        if isinstance(act, tuple):
            assert act[0] == "polynorm"
            self.act, self.coef = None, act[1].contiguous()

    def __call__(self, ctx, h, h16=None):
        x = h16 if h16 is not None else h
        if self.coef is not None:
            act = so.polynorm(so.linear(x, self.up, math=ctx.math), self.coef, ctx.eps, ctx.act_buffer(self.up.shape[0]))
        else:
            act = so.linear(x, self.up, act=self.act, math=ctx.math, out=ctx.act_buffer(self.up.shape[0]))
        return so.linear(act, self.down, math=ctx.math)


def rotary_frequencies(dims, base, scaling=None):
    """frequency per rotated pair (f32 tensor [dims / 2], computed in f64) and the magnitude of cos and sin.  scaling: None or
    {factor, original, fast, slow}: pairs that turn fewer than `slow` times over `original` positions are slowed down by
    `factor`, pairs that turn more than `fast` times are kept, a linear ramp over the pair index between; the magnitude grows
    with 0.1 ln(factor) + 1."""
    import math
    f = [float(base) ** (-2.0 * i / dims) for i in range(dims // 2)]
    mag = 1.0
    if scaling:
        factor, orig = float(scaling["factor"]), float(scaling["original"])
        where = lambda turns: dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(float(base)))
        lo = max(math.floor(where(float(scaling["fast"]))), 0)
        hi = min(math.ceil(where(float(scaling["slow"]))), dims - 1)
        for i in range(dims // 2):
            ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            f[i] = f[i] / factor * ramp + f[i] * (1.0 - ramp)
        mag = 0.1 * math.log(factor) + 1.0
    return torch.tensor(f, dtype=torch.float64).to(torch.float32), mag


class GroupedQueryAttention:
    LAYOUTS = {"pairs": 0, "halves": 1}

    def __init__(self, key, heads, kv_heads, dim, vdim, scale, w, state, cache_dtype, rot_dims=0, rot_base=10000.0, rot_layout="pairs",
                 rot_scaling=None, qk_norm=False, sink=None, softcap=None, head_gate=False, value_mix=None, window=0, keep_first=0,
                 differential=None, runs=1, head_temp=None, talk=None, elem_gate=False):
        """w: q [heads*maps*dim, width], k [kv_heads*maps*dim, width], v [kv_heads*vdim, width] (+ q.b / k.b / v.b / o.b where
        present), q.norm / k.norm [dim] (qk_norm), g [heads, width] (head_gate), o [width, heads*vdim].  sink: None, "zero" or a
        tensor [heads].  value_mix: None, ("source", name): this layer's values are kept under `name` for the step, or
        ("mix", name, lam): v <- (1 - lam) v + lam * the values kept under `name`.
        window > 0: a row reads the keys less than `window` positions back and the first keep_first keys of its sequence.
        differential: None (maps = 1), or (lam, out_scale): two softmax maps per head (their queries and keys side by side in q
        and k) over the same values, out = unit_rms(first - lam * second) * out_scale per head.
        runs: how often the layer runs in a step (a looped layer); every run has key and value caches of its own.
        talk [heads, heads]: the heads' softmax maps are mixed after the softmax, w_h <- sum_g talk[h, g] w_g, and head h applies its
        mixed map to the values of its own key/value head; head_temp [heads]: a multiplier per head on the scaled scores;
        elem_gate: g [heads*vdim, width], the concatenated heads are multiplied by sigmoid(g h) element by element."""
        assert heads % kv_heads == 0
        self.talk = talk.contiguous() if talk is not None else None
        self.head_temp = head_temp.contiguous() if head_temp is not None else None
        self.elem_gate = bool(elem_gate)
        if self.talk is not None:
            assert self.talk.shape == (heads, heads) and differential is None and sink is None and not softcap and not keep_first and not head_gate
            assert heads <= so.TALK_MAX_HEADS, "mixed softmax maps: at most %d heads" % so.TALK_MAX_HEADS
        else:
            assert head_temp is None and not elem_gate, "a per-head score multiplier and an elementwise gate go with mixed softmax maps"
        self.H, self.G, self.D, self.V, self.scale = heads, kv_heads, dim, vdim, float(scale)
        self.maps, self.differential = (2, (float(differential[0]), float(differential[1]))) if differential is not None else (1, None)
        self.window, self.keep_first = int(window or 0), int(keep_first or 0)
        heads, kv_heads = heads * self.maps, kv_heads * self.maps     # query / key vectors per token from here on
        dev = w["q"].device
        parts = [w["q"], w["k"], w["v"]] + ([w["g"]] if head_gate or elem_gate else [])
        n = sum(p.shape[0] for p in parts)
        if n % 4:    # rows of the product's output stay 16-byte aligned for the attention kernels: zero weight rows at the end
            parts.append(torch.zeros(4 - n % 4, w["q"].shape[1], dtype=w["q"].dtype, device=dev))
        self.w_in = torch.cat(parts, 0).contiguous()
        self.k_lo, self.v_lo = heads * dim, (heads + kv_heads) * dim
        self.g_lo = self.v_lo + self.G * vdim
        self.n_in = self.w_in.shape[0]
        self.head_gate = head_gate
        self.b_in = None
        if "q.b" in w or "k.b" in w or "v.b" in w:
            zero = lambda n: torch.zeros(n, dtype=self.w_in.dtype, device=dev)
            b = [w.get("q.b", zero(heads * dim)), w.get("k.b", zero(kv_heads * dim)), w.get("v.b", zero(self.G * vdim))]
            b = torch.cat(b + ([zero(self.H)] if head_gate else []) + ([zero(self.H * vdim)] if elem_gate else []), 0)
            self.b_in = torch.cat([b, zero(self.n_in - b.shape[0])], 0).contiguous()
        self.q_norm, self.k_norm = (w["q.norm"].contiguous(), w["k.norm"].contiguous()) if qk_norm else (None, None)
        self.rot_dims, self.layout = int(rot_dims), self.LAYOUTS[rot_layout]
        assert self.rot_dims % 2 == 0 and self.rot_dims <= dim
        self.freq, self.mag = None, 1.0
        if self.rot_dims:
            f, self.mag = rotary_frequencies(self.rot_dims, rot_base, rot_scaling)
            self.freq = f.to(dev)
        self.sink_mode, self.sink = so.SINK_NONE, None
        if isinstance(sink, str):
            assert sink == "zero"
            self.sink_mode = so.SINK_ZERO
        elif sink is not None:
            self.sink_mode, self.sink = so.SINK_PER_HEAD, sink.contiguous()
        self.softcap = float(softcap or 0.0)
        self.value_mix = value_mix
        self.o, self.o_b = w["o"].contiguous(), w.get("o.b")
        assert self.o.shape[1] == self.H * vdim and w["q"].shape[0] == heads * dim and w["k"].shape[0] == kv_heads * dim
        assert w["v"].shape[0] == self.G * vdim
        names = [key] if runs == 1 else [f"{key}.run{r}" for r in range(runs)]
        self.ktables = [state.add_span_cache(n + ".k", kv_heads * dim, cache_dtype) for n in names]
        self.vtables = [state.add_span_cache(n + ".v", self.G * vdim, cache_dtype) for n in names]
        self.ktable, self.vtable = self.ktables[0], self.vtables[0]
        self.mc = so.gqa_attn_mc_supported(dim, vdim, self.ktable) and self.n_in % 4 == 0 and (heads * dim) % 4 == 0
        self.talk32, self.talk_mc = None, False
        if self.talk is not None:
            self.talk32 = self.talk.float().contiguous()
            self.talk_mc = so.talk_attn_mc_supported(self.H, self.G, dim, vdim, self.ktable) and self.n_in % 4 == 0

    def __call__(self, ctx, h, h16=None, run=0):
        H, G, D, V = self.H, self.G, self.D, self.V
        ktable, vtable = self.ktables[run], self.vtables[run]
        a = so.linear(h16 if h16 is not None else h, self.w_in, self.b_in, act="sigmoid" if self.head_gate or self.elem_gate else None,
                      act_cols=(self.g_lo, self.n_in), math=ctx.math)                                        # [q | k | v | gate]
        vin = vout = None
        lam = 0.0
        if self.value_mix is not None:
            if self.value_mix[0] == "source":
                vout = ctx.shared[self.value_mix[1]] = torch.empty(ctx.T, G * V, dtype=torch.float32, device=a.device)
            else:
                vin, lam = ctx.shared[self.value_mix[1]], self.value_mix[2]
                assert vin.shape[1] == G * V, "mixed values must have this layer's shape"
        so.qkv_prep_append(a, 0, self.k_lo, self.v_lo, H, G, D, V, self.q_norm, self.k_norm, ctx.eps, self.freq, self.rot_dims, self.layout,
                           self.mag, lam, vin, vout, ktable, vtable, ctx.tok_slot, ctx.tok_pos, maps=self.maps)
        gate = a[:, self.g_lo:] if self.head_gate else None
        if self.talk is not None and ctx.math == so.MATH_BF16 and self.talk_mc and ctx.max_count >= so.TALK_MC_MIN_ROWS:
            o = so.talk_attn_mc(a, ktable, vtable, ctx.tok_pos, ctx.ent_slot, ctx.ent_row0, ctx.ent_count, ctx.max_count, H, G, D, V, self.scale,
                                self.talk32, temp=self.head_temp, gate=a[:, self.g_lo:] if self.elem_gate else None, window=self.window,
                                out=ctx.act_buffer(H * V))
            return so.linear(o, self.o, self.o_b, math=ctx.math)
        if self.talk is not None:
            o = so.talk_attn(a, ktable, vtable, ctx.tok_slot, ctx.tok_pos, ctx.max_pos, H, G, D, V, self.scale, self.talk, temp=self.head_temp,
                             gate=a[:, self.g_lo:] if self.elem_gate else None, window=self.window, out=ctx.act_buffer(H * V))
            return so.linear(o, self.o, self.o_b, math=ctx.math)
        if ctx.math == so.MATH_BF16 and self.mc:
            o = so.gqa_attn_mc(a, ktable, vtable, ctx.tok_pos, ctx.ent_slot, ctx.ent_row0, ctx.ent_count, ctx.max_count, ctx.max_pos,
                               H, G, D, V, self.scale, self.sink, self.sink_mode, self.softcap, gate, maps=self.maps, window=self.window,
                               keep_first=self.keep_first,
                               diff=(*self.differential, ctx.eps, ctx.act_buffer(H * V)) if self.differential is not None else None)
        else:
            o = so.gqa_attn(a, ktable, vtable, ctx.tok_slot, ctx.tok_pos, H, G, D, V, self.scale, self.sink, self.sink_mode,
                            self.softcap, gate, maps=self.maps, window=self.window, keep_first=self.keep_first)
            if self.differential is not None:
                o = so.maps_diff_norm(o, self.differential[0], self.differential[1], ctx.eps, H, V, out=ctx.act_buffer(H * V))
        return so.linear(o, self.o, self.o_b, math=ctx.math)


class GatedLinearAttention:
    def __init__(self, key, heads, dim, vdim, tau, w, state, q_scale=None):
        """w: q / k [heads*dim, width], v / g [heads*vdim, width], a1 [rank, width], a2 [heads*dim, rank], a2.b, norm [vdim],
        o [width, heads*vdim].  Decay per key channel: sigmoid(a2 (a1 h) + a2.b)^(1 / tau)."""
        self.H, self.D, self.V, self.tau = heads, dim, vdim, float(tau)
        self.q_scale = float(q_scale) if q_scale is not None else dim ** -0.5
        self.w_in = torch.cat([w["q"], w["k"], w["v"], w["g"], w["a1"]], 0).contiguous()
        hd, hv = heads * dim, heads * vdim
        self.k_lo, self.v_lo, self.g_lo, self.a_lo = hd, 2 * hd, 2 * hd + hv, 2 * hd + 2 * hv
        self.a2, self.a2_b = w["a2"].contiguous(), w["a2.b"].contiguous()
        self.norm, self.o = w["norm"].contiguous(), w["o"].contiguous()
        assert w["q"].shape[0] == hd and w["v"].shape[0] == hv and self.a2.shape == (hd, w["a1"].shape[0]) and self.o.shape[1] == hv
        self.S = state.add_state(key + ".S", (heads, dim, vdim))

    def __call__(self, ctx, h, h16=None):
        H, D, V = self.H, self.D, self.V
        a = so.linear(h16 if h16 is not None else h, self.w_in, act="silu", act_cols=(self.g_lo, self.a_lo), math=ctx.math)   # [q | k | v | silu g | a1 h]
        z = so.linear(a[:, self.a_lo:], self.a2, self.a2_b, math=ctx.math)
        o = so.gla(a, a[:, self.k_lo:], a[:, self.v_lo:], z, self.q_scale, self.tau, self.S, ctx.ent_slot, ctx.ent_row0, ctx.ent_count,
                   ctx.max_count, H, D, V)
        on = so.head_rmsnorm_mul(o, self.norm, ctx.eps, H, V, mul=a[:, self.g_lo: self.a_lo], out=ctx.act_buffer(H * V))
        return so.linear(on, self.o, math=ctx.math)


class StateSpaceMixer:
    def __init__(self, key, heads, vdim, n_state, groups, taps, norm_groups, w, state):
        """w: in [2*inner + 2*groups*n_state + heads, width] laid out [z | x | B | C | dt] (inner = heads*vdim), conv [inner +
        2*groups*n_state, taps] + conv.b over [x | B | C], dt_bias / A_log / D [heads], norm [inner], o [width, inner].
        Per head (head h reads group h / (heads / groups)):  step = softplus(dt + dt_bias);  S <- exp(-exp(A_log) step) S + step B x^T;
        y = S^T C + D x;  out = o . (rms-norm over norm_groups parts of (y * silu(z)) * norm)."""
        assert heads % groups == 0 and (heads * vdim) % norm_groups == 0
        self.H, self.P, self.N, self.G, self.taps, self.norm_groups = heads, vdim, n_state, groups, int(taps), int(norm_groups)
        self.inner, self.ch = heads * vdim, heads * vdim + 2 * groups * n_state
        self.w_in = w["in"].contiguous()
        assert self.w_in.shape[0] == self.inner + self.ch + heads and w["conv"].shape == (self.ch, self.taps)
        self.conv, self.conv_b = w["conv"].contiguous(), w["conv.b"].contiguous()
        self.dt_bias, self.a_log, self.skip = w["dt_bias"].contiguous(), w["A_log"].contiguous(), w["D"].contiguous()
        self.norm, self.o = w["norm"].contiguous(), w["o"].contiguous()
        assert self.norm.shape[0] == self.inner and self.o.shape[1] == self.inner
        self.S = state.add_state(key + ".S", (heads, n_state, vdim))
        self.tail = state.add_state(key + ".tail", (self.taps - 1, self.ch)) if self.taps > 1 else None

    def __call__(self, ctx, h, h16=None):
        inner, ch, GN = self.inner, self.ch, self.G * self.N
        a = so.linear(h16 if h16 is not None else h, self.w_in, math=ctx.math)                    # [z | x B C | dt], f32
        z, xbc, dtr = a[:, :inner], a[:, inner: inner + ch], a[:, inner + ch:]
        u = so.causal_conv_state(xbc, self.conv, self.conv_b, self.tail, ctx.tok_slot, ctx.tok_off, act="silu")
        if self.tail is not None:
            so.conv_tail_update(self.tail, xbc, self.taps, ctx.ent_slot, ctx.ent_row0, ctx.ent_count)
        y = so.ssd(u, u[:, inner: inner + GN], u[:, inner + GN:], dtr, self.dt_bias, self.a_log, self.S, ctx.ent_slot, ctx.ent_row0,
                   ctx.ent_count, ctx.max_count, self.H, self.G, self.N, self.P)
        yn = so.gate_group_rmsnorm(y, z, self.norm, ctx.eps, self.H, self.P, self.norm_groups, x=u, skip=self.skip,
                                   out=ctx.act_buffer(inner))
        return so.linear(yn, self.o, math=ctx.math)


class SideBySide:
    """two mixers that read the same input: coef * (rms_norm(left) * w_left + rms_norm(right) * w_right), norms over the width"""

    def __init__(self, left, right, w_left, w_right, coef=0.5):
        self.left, self.right, self.coef = left, right, float(coef)
        self.w_left, self.w_right = w_left.contiguous(), w_right.contiguous()

    def __call__(self, ctx, h, h16=None):
        return so.rmsnorm_pair(self.left(ctx, h, h16), self.w_left, self.right(ctx, h, h16), self.w_right, self.coef, ctx.eps)


class GatedMlp:
    def __init__(self, gate, up, down, act):
        self.gate, self.up, self.down, self.act = gate.contiguous(), up.contiguous(), down.contiguous(), act

    def __call__(self, ctx, h, h16=None):
        x = h16 if h16 is not None else h
        u = so.linear(x, self.up, math=ctx.math)
        g = so.linear(x, self.gate, act=self.act, mul=u, math=ctx.math, out=ctx.act_buffer(self.gate.shape[0]))   # act(gate h) * (up h)
        return so.linear(g, self.down, math=ctx.math)


class ExpertMlp:
    GLU_SLOPE = 1.702    # g * sigmoid(1.702 g): the sigmoid form of gelu

    def __init__(self, router, router_b, gates, ups, downs, top, limit=0.0, unit="clamped", scoring="chosen_softmax", correction=None,
                 identity=0, shared=None, groups=None):
        """gates / ups [ff, width] and downs [width, ff] per expert.  unit "clamped": an expert is
        down(glu(min(gate h, limit), clamp(up h, +-limit))); "silu": down(silu(gate h) * (up h)).
        scoring "chosen_softmax": the `top` largest router logits, weights = softmax over them alone; "scores": scores = softmax over
        all router outputs, the choice by score + correction [experts + identity] (None: the score alone), weights = the chosen
        scores over their sum.  identity: the last `identity` router outputs have no tensors: such an expert returns its input.
        shared: a feed-forward (GatedMlp) that runs for every token and is added, or None.
        groups: None or (count, keep): the router outputs form `count` equal groups of neighbours, a group counts by its largest score
        (logit), and only experts of the `keep` best groups can be chosen."""
        self.groups = (int(groups[0]), int(groups[1])) if groups else (1, 1)
        self.E, self.top, self.limit = len(gates), int(top), float(limit)
        self.unit = {"clamped": so.UNIT_CLAMPED, "silu": so.UNIT_SILU}[unit]
        self.scoring = {"chosen_softmax": so.ROUTE_CHOSEN_SOFTMAX, "scores": so.ROUTE_SCORES}[scoring]
        self.identity, self.shared = int(identity), shared
        self.router, self.router_b = router.contiguous(), router_b.contiguous() if router_b is not None else None
        self.correction = correction.contiguous() if correction is not None else None
        self.F = gates[0].shape[0]
        self.w_gu = torch.stack([torch.cat([g, u], 0) for g, u in zip(gates, ups)]).contiguous()    # [E, 2 ff, width]
        self.w_down = torch.stack(list(downs)).contiguous()                                          # [E, width, ff]
        assert self.router.shape[0] == self.E + self.identity and 0 < self.top <= self.E + self.identity
        assert self.correction is None or (self.scoring == so.ROUTE_SCORES and self.correction.shape == (self.E + self.identity,))

    def __call__(self, ctx, h, h16=None):
        x = h16 if h16 is not None else h
        T, R = ctx.T, ctx.T * self.top
        logits = so.linear(x, self.router, self.router_b, math=so.MATH_F32 if ctx.math == so.MATH_F32 else so.MATH_F32_STREAM)
        ids, wts, seg, src_row, dst = so.moe_route(logits, self.top, self.scoring, self.correction, self.groups)
        # the pairs of the identity experts sort behind those of the real ones: the expert products never see their rows
        gu = so.linear_segmented(x, self.w_gu, seg, src_row, T, R, math=ctx.math)
        y = so.moe_glu(gu, self.F, self.limit, self.GLU_SLOPE, ctx_rows(ctx, R, self.F), unit=self.unit)
        d = so.linear_segmented(y, self.w_down, seg, None, T, R, math=ctx.math)
        add = self.shared(ctx, h, h16) if self.shared is not None else None
        return so.moe_combine(d, dst, wts, T, self.top, ids=ids if self.identity else None, n_real=self.E, own=x, add=add)


def ctx_rows(ctx, rows, n):
    """[rows, n] for an activation that only a product reads (see StepContext.act_buffer)"""
    return torch.empty(rows, n, dtype=torch.bfloat16 if ctx.math == so.MATH_BF16 else torch.float32, device=ctx.ids.device)
