"""bench.py --workload filipel_layers: prefill and decode throughput of the sequence engine on random Filipel models of layer sizes
that resemble real models', per-operator times of the design's own kernels against their rooflines, and Vogusun models of equal
width / heads / feed-forward sizes (the closest design the engine serves: layers whose mixer and feed-forward run side by side,
grouped-query attention, a linear-attention mixer with a matrix state, routed experts) with their like operators beside them."""
import math

import torch

from . import vogusun_bench
from .seq_bench import HBM_BW, MFMA_BF16, VALU_F32, _time, engine_throughput

SIZES = {
    # windowed attention with mixed softmax maps: heads of 128, a window of 1024; state-space mixer: heads of 64 value channels over the
    # model width, 128 state channels; latent attention: latent 448 + 64 rotated (one 512-element page row); experts: 8 in 4 groups of
    # which 2 are kept, 2 per token, each half the dense feed-forward
    "2k": dict(width=2048, heads=16, kv_heads=4, dim=128, vdim=128, window=1024, ssm_heads=32, ssm_vdim=64, ssm_state=128, ssm_groups=1,
               lat_heads=16, lat_dim=128, lat_rot=64, lat_vdim=128, kv_rank=448, q_rank=768, ff=8192, experts=8, top=2, expert_ff=4096, vocab=32000),
    "4k": dict(width=4096, heads=32, kv_heads=8, dim=128, vdim=128, window=1024, ssm_heads=64, ssm_vdim=64, ssm_state=128, ssm_groups=1,
               lat_heads=32, lat_dim=128, lat_rot=64, lat_vdim=128, kv_rank=448, q_rank=1536, ff=14336, experts=8, top=2, expert_ff=7168, vocab=32000),
}
PATTERN = ("parallel+dense", "parallel+moe", "latent+moe", "parallel+moe", "latent_from_2+moe", "parallel+moe")
LIKE_PATTERN = ("attention+dense", "gla+moe", "attention_2+moe", "attention+moe", "gla+moe", "attention_2+moe")


def random_model(size, device="cuda", seed=0, pattern=PATTERN):
    """config + bf16 tensors on the device (torch generator: nothing of it is trained or loaded)"""
    s = SIZES[size]
    g = torch.Generator(device=device).manual_seed(seed)
    W = s["width"]

    def r(*shape, sd=None):
        sd = sd if sd is not None else 1.0 / math.sqrt(shape[-1])
        return (torch.randn(*shape, generator=g, device=device) * sd).to(torch.bfloat16)

    def one(*shape):
        return (1 + 0.1 * torch.randn(*shape, generator=g, device=device)).to(torch.bfloat16)
    cfg = {"architecture": "Filipel", "width": W, "vocab": s["vocab"], "norm": {"eps": 1e-6}, "residual_mult": 0.5, "layers": []}
    t = {"embed": r(s["vocab"], W, sd=1.0), "head": r(s["vocab"], W), "final.norm": one(W)}
    H, G, D, V = s["heads"], s["kv_heads"], s["dim"], s["vdim"]
    SH, SP, SN, SG = s["ssm_heads"], s["ssm_vdim"], s["ssm_state"], s["ssm_groups"]
    LH, LD, LR, LV, R, Q = s["lat_heads"], s["lat_dim"], s["lat_rot"], s["lat_vdim"], s["kv_rank"], s["q_rank"]
    for i, spec in enumerate(pattern):
        kind, _, ff = spec.partition("+")
        p = f"l{i}."
        t[p + "norm1"] = one(W)
        if kind == "parallel":
            m = {"left": {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "mask": {"size": s["window"]}, "rot": {"base": 10000.0, "dims": D // 2},
                          "scale": 1.0 / math.sqrt(D)},
                 "right": {"heads": SH, "vdim": SP, "state": SN, "groups": SG, "conv": 4, "norm_groups": SG}}
            q = p + "mix.left."
            t[q + "q"], t[q + "k"], t[q + "v"], t[q + "g"], t[q + "o"] = r(H * D, W), r(G * D, W), r(G * V, W), r(H * V, W), r(W, H * V)
            t[q + "talk"] = (torch.eye(H, device=device) + 0.1 * torch.randn(H, H, generator=g, device=device)).to(torch.bfloat16)
            t[q + "temp"], t[q + "out"] = one(H), one(W)
            q = p + "mix.right."
            inner, ch = SH * SP, SH * SP + 2 * SG * SN
            t[q + "in"], t[q + "conv"], t[q + "conv.b"] = r(2 * inner + 2 * SG * SN + SH, W), r(ch, 4, sd=0.5), r(ch, sd=0.1)
            t[q + "dt_bias"], t[q + "A_log"], t[q + "D"] = r(SH, sd=1.0) - 2.0, r(SH, sd=0.5), one(SH)
            t[q + "norm"], t[q + "o"], t[q + "out"] = one(inner), r(W, inner), one(W)
            kind = "parallel"
        else:
            m = {"heads": LH, "dim": LD, "rot_dim": LR, "vdim": LV, "kv_rank": R, "q_rank": Q, "rot": {"base": 500000.0, "dims": LR},
                 "scale": 1.0 / math.sqrt(LD + LR)}
            q = p + "mix."
            t[q + "dq"], t[q + "dq.norm"], t[q + "uq"] = r(Q, W), one(Q), r(LH * (LD + LR), Q)
            t[q + "uk"], t[q + "uv"], t[q + "g"], t[q + "o"] = r(LH * LD, R), r(LH * LV, R), r(LH * LV, W), r(W, LH * LV)
            if kind.startswith("latent_from_"):
                m["kv_from"] = int(kind.rsplit("_", 1)[1])
            else:
                t[q + "dkv"], t[q + "dkv.norm"] = r(R + LR, W), one(R)
            kind = "latent_attention"
        layer = {"type": kind, "mixer": m, "mlp": None}
        if ff == "dense":
            layer["mlp"] = {"kind": "dense", "ff": s["ff"]}
            t[p + "mlp.up"], t[p + "mlp.down"] = r(s["ff"], W), r(W, s["ff"])
            t[p + "mlp.act"] = torch.tensor([0.7, 0.3, 0.2, 0.05], dtype=torch.bfloat16, device=device)
        elif ff == "moe":
            E, F = s["experts"], s["expert_ff"]
            layer["mlp"] = {"kind": "moe", "expert": {"ff": F}, "router": {"experts": E, "top": s["top"], "groups": {"count": 4, "keep": 2}}}
            for e in range(E):
                t[p + f"mlp.e{e}.gate"], t[p + f"mlp.e{e}.up"], t[p + f"mlp.e{e}.down"] = r(F, W), r(F, W), r(W, F)
            t[p + "mlp.router"] = r(E, W)
        cfg["layers"].append(layer)
    return cfg, t


def vogusun_equal_size(size):
    """the closest served design at equal size: as many layers, grouped-query attention of the same heads, a linear-attention mixer with
    a matrix state in place of the state-space mixer, the same dense and routed feed-forwards"""
    s = SIZES[size]
    v = dict(width=s["width"], heads=s["heads"], kv_heads=s["kv_heads"], dim=s["dim"], vdim=s["vdim"], gla_heads=s["heads"], gla_dim=64, gla_vdim=128,
             gla_rank=64, ff=s["ff"], experts=s["experts"], top=s["top"], expert_ff=s["expert_ff"], vocab=s["vocab"])
    return vogusun_bench.random_model(v, pattern=LIKE_PATTERN)


def operator_table(size, prompt_len):
    """the design's own kernels alone, at the prompt's row count and at one row: seconds and the fraction of their bound (matrix-core
    work: the bf16 peak; f32 work on the vector units: their peak; everything else: 8 TB/s over the bytes moved)"""
    from . import seq_ops as so
    from .seq_state import SequenceStateManager
    s = SIZES[size]
    W, H, G, D, V, win = s["width"], s["heads"], s["kv_heads"], s["dim"], s["vdim"], s["window"]
    SH, SP, SN, SG = s["ssm_heads"], s["ssm_vdim"], s["ssm_state"], s["ssm_groups"]
    LH, LD, LR, LV, R = s["lat_heads"], s["lat_dim"], s["lat_rot"], s["lat_vdim"], s["kv_rank"]
    Rp = -(-(R + LR) // 32) * 32
    E, top, F, ff = s["experts"], s["top"], s["expert_ff"], s["ff"]
    dev = "cuda"
    rows = []
    bf = lambda *sh: (torch.randn(*sh, device=dev) * 0.05).to(torch.bfloat16)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
    for T in (prompt_len, 1):
        st = SequenceStateManager(prompt_len + 64, 1, 64, dev)
        kt, vt = st.add_span_cache("k", G * D, torch.bfloat16), st.add_span_cache("v", G * V, torch.bfloat16)
        lt = st.add_span_cache("c", Rp, torch.bfloat16)
        S = st.add_state("S", (SH, SN, SP))
        st.admit("a")
        st.reserve("a", prompt_len)
        st.upload()
        for tab in (kt, vt, lt):
            tab.pool.pool.view(torch.bfloat16).normal_(0, 0.3)
        pos = torch.arange(T, dtype=torch.int32, device=dev) if T > 1 else i32([prompt_len - 1])
        slot = torch.zeros(T, dtype=torch.int32, device=dev)
        e_slot, e_row0, e_cnt = i32([0]), i32([0]), i32([T])
        max_pos = int(pos[-1])
        # windowed attention with mixed maps
        a = torch.randn(T, (H + 2 * G) * D + H * V, device=dev) * 0.3
        talk, temp = bf(H, H), bf(H)
        o16 = torch.empty(T, H * V, dtype=torch.bfloat16, device=dev)
        gate = a[:, (H + 2 * G) * D:]
        if T >= so.TALK_MC_MIN_ROWS and so.talk_attn_mc_supported(H, G, D, V, kt):      # as the mixer chooses: matrix cores for portions, the split row kernel for few rows
            talk32 = talk.float()
            sec = _time(lambda: so.talk_attn_mc(a, kt, vt, pos, e_slot, e_row0, e_cnt, T, H, G, D, V, 0.09, talk32, temp=temp, gate=gate, window=win, out=o16), 3)
        else:
            sec = _time(lambda: so.talk_attn(a, kt, vt, slot, pos, max_pos, H, G, D, V, 0.09, talk, temp=temp, gate=gate, window=win, out=o16), 3)
        keys = sum(min(int(p) + 1, win) for p in pos.tolist())
        fl_mm, fl_mix = 2.0 * keys * H * (2 * D + V), 2.0 * keys * H * H      # two score passes + values on the matrix cores; the mix in f32
        by = 2.0 * G * (D + V) * min(prompt_len, win + T) + 4.0 * T * H * (D + 2 * V)
        bound = max(fl_mm / MFMA_BF16 + fl_mix / VALU_F32, by / HBM_BW)
        rows.append({"op": f"windowed attention, softmax maps mixed between {H} heads (window {win}) T={T} G={G} D={D} V={V} keys<={prompt_len}",
                     "us": round(sec * 1e6, 1), "tflops": round((fl_mm + fl_mix) / sec / 1e12, 2), "of_bound": round(bound / sec, 4)})
        # latent attention with a rotated part: the rotation + append, then the shared attention kernel at the padded width
        ckv, qrot, ql = torch.randn(T, R + LR, device=dev), torch.randn(T, LH * LR, device=dev), torch.randn(T, LH * Rp, device=dev) * 0.1
        gam, freq = bf(R), torch.rand(LR // 2, device=dev)
        sec = _time(lambda: so.latent_rope_append(lt, ckv, gam, 1e-6, R, LR, freq, qrot, ql, LH, slot, pos), 3)
        by = 4.0 * T * (R + LR) + 2.0 * T * Rp + 8.0 * T * LH * LR
        rows.append({"op": f"latent norm + rotated key part -> page, rotated query parts T={T}", "us": round(sec * 1e6, 1), "of_bound": round(by / HBM_BW / sec, 3)})
        sec = _time(lambda: so.latent_window_attn_mc(ql, lt, None, pos, e_slot, e_row0, e_cnt, T, max_pos, LH, 0, 0.07), 3)
        keys = sum(int(p) + 1 for p in pos.tolist())
        fl = 4.0 * keys * LH * Rp
        by = 2.0 * Rp * prompt_len + 8.0 * T * LH * Rp
        rows.append({"op": f"latent attention, all keys, row width {Rp} (latent {R} + rotated {LR}) T={T} H={LH}", "us": round(sec * 1e6, 1),
                     "tflops": round(fl / sec / 1e12, 2), "of_bound": round(max(fl / MFMA_BF16, by / HBM_BW) / sec, 4)})
        # state-space mixer
        inner, ch = SH * SP, SH * SP + 2 * SG * SN
        u, dtr = torch.randn(T, ch, device=dev) * 0.3, torch.randn(T, SH, device=dev)
        dtb, alog = bf(SH), bf(SH)
        sec = _time(lambda: so.ssd(u, u[:, inner: inner + SG * SN], u[:, inner + SG * SN:], dtr, dtb, alog, S, e_slot, e_row0, e_cnt, T, SH, SG, SN, SP), 3)
        fl = 4.0 * T * SH * SN * SP * (2 if T >= so.CHUNKED_GLA_ROWS else 1)
        by = 4.0 * T * (ch + inner) + 8.0 * SH * SN * SP
        rows.append({"op": f"state-space scan T={T} heads={SH} state={SN} x {SP} (f32, vector units)", "us": round(sec * 1e6, 1),
                     "tflops": round(fl / sec / 1e12, 2), "of_bound": round(max(fl / VALU_F32, by / HBM_BW) / sec, 3)})
        xb = torch.randn(T, ch, device=dev)
        cw, cb, tail = bf(ch, 4), bf(ch), torch.zeros(1, 3, ch, device=dev)
        off = torch.arange(T, dtype=torch.int32, device=dev)
        sec = _time(lambda: so.causal_conv_state(xb, cw, cb, tail, slot, off, act="silu"), 3)
        rows.append({"op": f"causal convolution (4 taps) + silu T={T} x {ch}", "us": round(sec * 1e6, 1), "of_bound": round(8.0 * T * ch / HBM_BW / sec, 3)})
        y, z = torch.randn(T, inner, device=dev), torch.randn(T, inner, device=dev)
        gw, dsk = bf(inner), bf(SH)
        yn = torch.empty(T, inner, dtype=torch.bfloat16, device=dev)
        sec = _time(lambda: so.gate_group_rmsnorm(y, z, gw, 1e-6, SH, SP, SG, x=u, skip=dsk, out=yn), 3)
        rows.append({"op": f"skip + silu gate + grouped norm T={T} x {inner}", "us": round(sec * 1e6, 1), "of_bound": round(14.0 * T * inner / HBM_BW / sec, 3)})
        # norms and joins
        x, m1, m2 = torch.randn(T, W, device=dev), torch.randn(T, W, device=dev), torch.randn(T, W, device=dev)
        nw = bf(W)
        sec = _time(lambda: so.residual_layernorm(x, nw, a=m1, b=m2, mult=0.5, eps=1e-6, x_out=x, out_dtype=torch.bfloat16), 3)
        rows.append({"op": f"residual of two sublayers + layer norm T={T}", "us": round(sec * 1e6, 1), "of_bound": round(18.0 * T * W / HBM_BW / sec, 3)})
        sec = _time(lambda: so.rmsnorm_pair(m1, nw, m2, nw, 0.5, 1e-6), 3)
        rows.append({"op": f"two normed branches joined T={T}", "us": round(sec * 1e6, 1), "of_bound": round(12.0 * T * W / HBM_BW / sec, 3)})
        zz, coef = torch.randn(T, ff, device=dev), bf(4)
        pa = torch.empty(T, ff, dtype=torch.bfloat16, device=dev)
        sec = _time(lambda: so.polynorm(zz, coef, 1e-6, pa), 3)
        rows.append({"op": f"cubic of normalised powers T={T} x {ff}", "us": round(sec * 1e6, 1), "of_bound": round(6.0 * T * ff / HBM_BW / sec, 3)})
        hin = (torch.randn(T, W, device=dev) * 0.5).to(torch.bfloat16)
        logits = so.linear(hin, bf(E, W), None, math=so.MATH_F32_STREAM)
        sec = _time(lambda: so.moe_route(logits, top, so.ROUTE_SCORES, None, (4, 2)), 3)
        rows.append({"op": f"routing: softmax over {E}, best 2 of 4 groups, top-{top}, grouping by expert T={T}", "us": round(sec * 1e6, 1)})
    return rows


LIKE_OPERATORS = ("grouped-query attention", "gated linear attention", "residual of two sublayers", "per-head norm", "routing", "page append")


def run(args):
    from . import models
    from .engine import SeqEngine
    prompt_len = 2048
    res = {"metric": "prefill / decode throughput of the sequence engine (random Filipel models) beside Vogusun models of equal size",
           "unit": "tokens/s", "n_gpus": 1, "dtype": "bf16", "data": "synthetic", "prompt_len": prompt_len, "sizes": {}}
    for size in SIZES:
        entry = {"layers": list(PATTERN), **SIZES[size]}
        for name, make in (("engine", random_model), ("vogusun_equal_size", vogusun_equal_size)):
            cfg, t = make(size)
            eng = SeqEngine(models.resolve(cfg), cfg, t, dtype=torch.bfloat16, max_tokens=4 * (prompt_len + 128), max_slots=4)
            entry[name] = engine_throughput(eng, cfg["vocab"], prompt_len)
            entry[name]["weight_bytes"] = int(sum(v.numel() * v.element_size() for k, v in t.items() if k != "embed"))
            del eng, t
            torch.cuda.empty_cache()
        entry["vogusun_equal_size"]["layers"] = list(LIKE_PATTERN)
        entry["operators"] = operator_table(size, prompt_len)
        vs = dict(SIZES[size], gla_heads=SIZES[size]["heads"], gla_dim=64, gla_vdim=128, gla_rank=64)
        saved = vogusun_bench.SIZES.get(size)
        vogusun_bench.SIZES[size] = vs
        try:
            entry["vogusun_operators"] = [r for r in vogusun_bench.operator_table(size, prompt_len) if any(k in r["op"] for k in LIKE_OPERATORS)]
        finally:
            vogusun_bench.SIZES[size] = saved
        res["sizes"][size] = entry
    res["value"] = res["sizes"]["4k"]["engine"]["prefill_tokens_per_s"]
    return res
