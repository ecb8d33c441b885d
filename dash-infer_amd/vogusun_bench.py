"""bench.py --workload vogusun_layers: prefill and decode throughput of the sequence engine on random Vogusun models of layer
sizes that resemble real models', per-operator times against their rooflines, and Modanex models of equal width / heads /
feed-forward size (the closest design the engine serves) with their like operators beside them."""
import math

import torch

from .seq_bench import HBM_BW, MFMA_BF16, VALU_F32, SIZES as MODANEX_SIZES, _time, engine_throughput, operator_table as modanex_operator_table, \
    random_model as random_modanex

SIZES = {
    # attention: heads / kv heads of dim = vdim = 128; gated linear attention: heads of 64 key and 128 value channels, decay rank 64;
    # experts: 8 of which 2 per token, each half the dense feed-forward (the same active parameters)
    "2k": dict(width=2048, heads=16, kv_heads=4, dim=128, vdim=128, gla_heads=16, gla_dim=64, gla_vdim=128, gla_rank=64, ff=8192, experts=8, top=2,
               expert_ff=4096, vocab=32000),
    "4k": dict(width=4096, heads=32, kv_heads=8, dim=128, vdim=128, gla_heads=32, gla_dim=64, gla_vdim=128, gla_rank=64, ff=14336, experts=8, top=2,
               expert_ff=7168, vocab=32000),
}
PATTERN = ("attention+dense", "gla+moe", "attention_2+dense", "attention+moe", "gla+dense", "attention_2+moe")


def random_model(size, device="cuda", seed=0, pattern=PATTERN):
    """config + bf16 tensors on the device (torch generator: nothing of it is trained or loaded); pattern: the layers' kinds"""
    s = SIZES[size] if isinstance(size, str) else size
    g = torch.Generator(device=device).manual_seed(seed)
    W = s["width"]

    def r(*shape, sd=None):
        sd = sd if sd is not None else 1.0 / math.sqrt(shape[-1])
        return (torch.randn(*shape, generator=g, device=device) * sd).to(torch.bfloat16)

    def one(n):
        return (1 + 0.1 * torch.randn(n, generator=g, device=device)).to(torch.bfloat16)

    def norm(name):
        t[name], t[name + ".b"], t[name + ".alpha"] = one(W), r(W, sd=0.1), torch.tensor(0.75, dtype=torch.bfloat16, device=device)
    cfg = {"architecture": "Vogusun", "width": W, "vocab": s["vocab"], "norm": {"eps": 1e-6}, "layers": []}
    t = {"embed": r(s["vocab"], W, sd=1.0), "head": r(s["vocab"], W)}
    norm("final.norm")
    H, G, D, V = s["heads"], s["kv_heads"], s["dim"], s["vdim"]
    for i, spec in enumerate(pattern):
        kind, _, ff = spec.partition("+")
        p = f"l{i}."
        norm(p + "norm1")
        if kind == "gla":
            h, d, v, rk = s["gla_heads"], s["gla_dim"], s["gla_vdim"], s["gla_rank"]
            m = {"heads": h, "dim": d, "vdim": v, "tau": 8.0}
            t[p + "mix.q"], t[p + "mix.k"], t[p + "mix.v"], t[p + "mix.g"] = r(h * d, W), r(h * d, W), r(h * v, W), r(h * v, W)
            t[p + "mix.o"], t[p + "mix.norm"] = r(W, h * v), one(v)
            t[p + "mix.a1"], t[p + "mix.a2"], t[p + "mix.a2.b"] = r(rk, W), r(h * d, rk), r(h * d, sd=1.0)
        else:
            m = {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "scale": 1.0 / math.sqrt(D), "v_mix": True,
                 "rot": {"base": 1000000.0, "dims": D}}
            t[p + "mix.q"], t[p + "mix.k"], t[p + "mix.v"], t[p + "mix.o"] = r(H * D, W), r(G * D, W), r(G * V, W), r(W, H * V)
            t[p + "mix.vmix"] = torch.tensor(0.25, dtype=torch.bfloat16, device=device)
            if kind == "attention":
                t[p + "mix.q.norm"], t[p + "mix.k.norm"], t[p + "mix.g"] = one(D), one(D), r(H, W)
            else:
                t[p + "mix.q.b"], t[p + "mix.k.b"], t[p + "mix.v.b"] = r(H * D, sd=0.1), r(G * D, sd=0.1), r(G * V, sd=0.1)
                m["softcap"] = 50.0
                m["rot"]["scaling"] = {"factor": 4.0, "original": 4096, "fast": 16.0, "slow": 2.0}
        layer = {"type": kind, "mixer": m, "mlp": None}
        if ff == "dense":
            layer["mlp"] = {"kind": "dense", "ff": s["ff"]}
            t[p + "mlp.gate"], t[p + "mlp.up"], t[p + "mlp.down"] = r(s["ff"], W), r(s["ff"], W), r(W, s["ff"])
        else:
            E, F = s["experts"], s["expert_ff"]
            layer["mlp"] = {"kind": "moe", "expert": {"ff": F, "limit": 7.0}, "router": {"experts": E, "top": s["top"]}}
            for e in range(E):
                t[p + f"mlp.e{e}.gate"], t[p + f"mlp.e{e}.up"], t[p + f"mlp.e{e}.down"] = r(F, W), r(F, W), r(W, F)
            t[p + "mlp.router"], t[p + "mlp.router.b"] = r(E, W), r(E, sd=0.1)
        cfg["layers"].append(layer)
    return cfg, t


def operator_table(size, prompt_len):
    """the design's own operators alone, at the prompt's row count and at one row: seconds and the fraction of their bound
    (matrix-core work: the bf16 peak; f32 recurrences: the vector units' peak; everything else: 8 TB/s over the bytes moved)"""
    from . import seq_ops as so
    from .seq_state import SequenceStateManager
    s = SIZES[size]
    W, H, G, D, V = s["width"], s["heads"], s["kv_heads"], s["dim"], s["vdim"]
    gh, gd, gv = s["gla_heads"], s["gla_dim"], s["gla_vdim"]
    E, top, F = s["experts"], s["top"], s["expert_ff"]
    dev = "cuda"
    rows = []
    bf = lambda *sh: (torch.randn(*sh, device=dev) * 0.05).to(torch.bfloat16)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
    for T in (prompt_len, 1):
        # -- attention over the pages: prompt rows at positions 0 .. T-1, or one row at position prompt_len - 1
        st = SequenceStateManager(prompt_len + 64, 1, 64, dev)
        kt, vt = st.add_span_cache("k", G * D, torch.bfloat16), st.add_span_cache("v", G * V, torch.bfloat16)
        st.admit("a")
        st.reserve("a", prompt_len)
        st.upload()
        for tab in (kt, vt):
            tab.pool.pool.view(torch.bfloat16).normal_(0, 0.3)
        pos = torch.arange(T, dtype=torch.int32, device=dev) if T > 1 else i32([prompt_len - 1])
        slot = torch.zeros(T, dtype=torch.int32, device=dev)
        n_in = (H + G) * D + G * V + H
        a = torch.randn(T, n_in, device=dev) * 0.3
        gate = torch.rand(T, H, device=dev)
        o = torch.empty(T, H * V, device=dev)
        qn, freq = bf(D) + 1, torch.rand(D // 2, device=dev)
        vf = torch.randn(T, G * V, device=dev)
        sec = _time(lambda: so.qkv_prep_append(a, 0, H * D, (H + G) * D, H, G, D, V, qn, qn, 1e-6, freq, D, 0, 1.0, 0.25, vf, None, kt, vt, slot, pos), 3)
        by = 8.0 * T * (H + G) * D + 4.0 * T * G * V * 2 + 2.0 * T * G * (D + V)
        rows.append({"op": f"q/k norm + rotation + value mix + page append T={T}", "us": round(sec * 1e6, 1), "of_bound": round(by / HBM_BW / sec, 3)})
        e_slot, e_row0, e_cnt = i32([0]), i32([0]), i32([T])
        for name, kw in (("sink + gate", dict(sink_mode=so.SINK_ZERO, gate=gate)), ("capped scores", dict(softcap=50.0))):
            sec = _time(lambda: so.gqa_attn_mc(a, kt, vt, pos, e_slot, e_row0, e_cnt, T, int(pos[-1]), H, G, D, V, 0.09, out=o, **kw), 3)
            keys = sum(int(p) + 1 for p in pos.tolist())
            fl = 2.0 * keys * H * (D + V)
            by = 2.0 * G * (D + V) * prompt_len + 4.0 * T * H * (D + V)
            bound = max(fl / MFMA_BF16, by / HBM_BW)
            rows.append({"op": f"grouped-query attention ({name}) T={T} H={H} G={G} D={D} V={V} keys<={prompt_len}", "us": round(sec * 1e6, 1),
                         "tflops": round(fl / sec / 1e12, 2), "of_bound": round(bound / sec, 3)})
        # -- gated linear attention
        es, er, ec = i32([0]), i32([0]), i32([T])
        qkvz = torch.randn(T, 3 * gh * gd + gh * gv, device=dev) * 0.3
        state = torch.zeros(1, gh, gd, gv, device=dev)
        og = torch.empty(T, gh * gv, device=dev)
        sec = _time(lambda: so.gla(qkvz, qkvz[:, gh * gd:], qkvz[:, 3 * gh * gd:], qkvz[:, 2 * gh * gd:], 0.125, 8.0, state, es, er, ec, T, gh, gd, gv, out=og), 3)
        fl = 4.0 * T * gh * gd * gv * (2 if T >= so.CHUNKED_GLA_ROWS else 1)       # the chunked form runs every row twice
        by = 4.0 * T * (3 * gh * gd + 2 * gh * gv) + 8.0 * gh * gd * gv
        bound = max(fl / VALU_F32, by / HBM_BW)
        rows.append({"op": f"gated linear attention T={T} heads={gh} D={gd} V={gv}", "us": round(sec * 1e6, 1), "tflops_f32": round(fl / sec / 1e12, 2),
                     "of_bound": round(bound / sec, 3)})
        gam, mul, on = bf(gv) + 1, torch.rand(T, gh * gv, device=dev), torch.empty(T, gh * gv, dtype=torch.bfloat16, device=dev)
        sec = _time(lambda: so.head_rmsnorm_mul(og, gam, 1e-6, gh, gv, mul=mul, out=on), 3)
        rows.append({"op": f"per-head norm x gate T={T}", "us": round(sec * 1e6, 1), "of_bound": round(10.0 * T * gh * gv / HBM_BW / sec, 3)})
        # -- norm + parallel residual
        x, m1, m2 = (torch.randn(T, W, device=dev) for _ in range(3))
        nw = (0.75, bf(W) + 1, bf(W))
        sec = _time(lambda: so.add_dyt(x, m1, m2, norm=nw, x_out=x, want16=True), 3)
        rows.append({"op": f"residual of two sublayers + dyt norm T={T}", "us": round(sec * 1e6, 1), "of_bound": round(18.0 * T * W / HBM_BW / sec, 3)})
        # -- dense gated feed-forward and the routed experts
        h16 = (torch.randn(T, W, device=dev) * 0.5).to(torch.bfloat16)
        wg, wu = bf(s["ff"], W), bf(s["ff"], W)
        up, act = torch.empty(T, s["ff"], device=dev), torch.empty(T, s["ff"], dtype=torch.bfloat16, device=dev)
        def gated():
            so.linear(h16, wu, out=up, math=so.MATH_BF16)
            so.linear(h16, wg, act="gelu_tanh", mul=up, out=act, math=so.MATH_BF16)
        sec = _time(gated, 3)
        fl, by = 4.0 * T * s["ff"] * W, 4.0 * s["ff"] * W + 10.0 * T * s["ff"] + 4.0 * T * W
        rows.append({"op": f"linear gate (gelu) x up [{T}x{W}]x[2x{s['ff']}]", "us": round(sec * 1e6, 1), "tflops": round(fl / sec / 1e12, 1),
                     "of_bound": round(max(fl / MFMA_BF16, by / HBM_BW) / sec, 3)})
        router, rb = bf(E, W), bf(E)
        w_gu, w_dn = bf(E, 2 * F, W), bf(E, W, F)
        logits = so.linear(h16, router, rb, math=so.MATH_F32_STREAM)
        sec = _time(lambda: so.moe_route(logits, top), 3)
        rows.append({"op": f"routing: top-{top} of {E}, softmax, grouping by expert T={T}", "us": round(sec * 1e6, 1)})
        _, wts, seg, src, dst = so.moe_route(logits, top)
        R = T * top
        gu, y, dn = torch.empty(R, 2 * F, device=dev), torch.empty(R, F, dtype=torch.bfloat16, device=dev), torch.empty(R, W, device=dev)
        used = min(E, R)
        sec = _time(lambda: so.linear_segmented(h16, w_gu, seg, src, T, R, out=gu, math=so.MATH_BF16), 3)
        fl, by = 4.0 * R * F * W, 4.0 * used * F * W + 8.0 * R * F + 2.0 * R * W
        rows.append({"op": f"experts' gate | up, rows grouped by expert [{R}x{W}]x[{E}x{2 * F}]", "us": round(sec * 1e6, 1), "tflops": round(fl / sec / 1e12, 1),
                     "of_bound": round(max(fl / MFMA_BF16, by / HBM_BW) / sec, 3)})
        sec = _time(lambda: so.moe_glu(gu, F, 7.0, 1.702, y), 3)
        rows.append({"op": f"experts' clamped gated unit [{R}x{F}]", "us": round(sec * 1e6, 1), "of_bound": round(10.0 * R * F / HBM_BW / sec, 3)})
        sec = _time(lambda: so.linear_segmented(y, w_dn, seg, None, T, R, out=dn, math=so.MATH_BF16), 3)
        fl, by = 2.0 * R * F * W, 2.0 * used * F * W + 2.0 * R * F + 4.0 * R * W
        rows.append({"op": f"experts' down, rows grouped by expert [{R}x{F}]x[{E}x{W}]", "us": round(sec * 1e6, 1), "tflops": round(fl / sec / 1e12, 1),
                     "of_bound": round(max(fl / MFMA_BF16, by / HBM_BW) / sec, 3)})
        sec = _time(lambda: so.moe_combine(dn, dst, wts, T, top), 3)
        rows.append({"op": f"weighted sum of the chosen experts T={T}", "us": round(sec * 1e6, 1), "of_bound": round(4.0 * (R + T) * W / HBM_BW / sec, 3)})
    return rows


def run(args):
    from . import models
    from .engine import SeqEngine
    prompt_len = 2048
    res = {"metric": "prefill / decode throughput of the sequence engine (random Vogusun models) beside Modanex models of equal size",
           "unit": "tokens/s", "n_gpus": 1, "dtype": "bf16", "data": "synthetic", "prompt_len": prompt_len, "sizes": {}}
    for size in SIZES:
        entry = {"layers": list(PATTERN), **SIZES[size]}
        for name, make in (("engine", random_model), ("modanex_equal_size", random_modanex)):
            cfg, t = make(size)
            eng = SeqEngine(models.resolve(cfg), cfg, t, dtype=torch.bfloat16, max_tokens=4 * (prompt_len + 128), max_slots=4)
            entry[name] = engine_throughput(eng, cfg["vocab"], prompt_len)
            entry[name]["weight_bytes"] = int(sum(v.numel() * v.element_size() for k, v in t.items() if k != "embed"))
            del eng, t
            torch.cuda.empty_cache()
        entry["modanex_equal_size"]["layers"] = {k: MODANEX_SIZES[size][k] for k in ("width", "heads", "kv_rank", "window", "rec_width", "ff")}
        entry["operators"] = operator_table(size, prompt_len)
        entry["modanex_operators"] = [r for r in modanex_operator_table(size, prompt_len)
                                      if any(k in r["op"] for k in ("latent window attention", "gated recurrence", "norm + residual", "mlp up", "mlp down"))]
        res["sizes"][size] = entry
    res["value"] = res["sizes"]["4k"]["engine"]["prefill_tokens_per_s"]
    return res
