"""bench.py --workload tobilorn_layers: prefill and decode throughput of the sequence engine on random Tobilorn models of layer
sizes that resemble real models', per-operator times of the design's own kernels against their rooflines, and Vogusun models of
equal width / heads / experts (the closest design the engine serves: grouped-query attention with routed experts) with their like
operators beside them."""
import math

import torch

from . import vogusun_bench
from .seq_bench import HBM_BW, MFMA_BF16, _time, engine_throughput

SIZES = {
    # attention: heads of two maps of 64 (as many query and key channels as a plain head of 128), values of 128, a window of 1024 keys
    # plus 64 kept ones; experts: 8 + 1 identity of which 2 per token, a shared expert of a quarter of their size; 6 layers of which the
    # two in the middle run twice (8 layer runs)
    "2k": dict(width=2048, heads=16, kv_heads=4, dim=64, vdim=128, window=1024, keep_first=64, experts=8, identity=1, top=2, expert_ff=4096,
               shared_ff=1024, side_dim=256, vocab=32000),
    "4k": dict(width=4096, heads=32, kv_heads=8, dim=64, vdim=128, window=1024, keep_first=64, experts=8, identity=1, top=2, expert_ff=7168,
               shared_ff=1792, side_dim=256, vocab=32000),
}
LAYERS, LOOP = 6, {"start": 2, "stop": 4, "times": 2}
RUNS = LAYERS + (LOOP["stop"] - LOOP["start"]) * (LOOP["times"] - 1)


def random_model(size, device="cuda", seed=0):
    """config + bf16 tensors on the device (torch generator: nothing of it is trained or loaded)"""
    s = SIZES[size]
    g = torch.Generator(device=device).manual_seed(seed)
    W, H, G, D, V = s["width"], s["heads"], s["kv_heads"], s["dim"], s["vdim"]

    def r(*shape, sd=None):
        sd = sd if sd is not None else 1.0 / math.sqrt(shape[-1])
        return (torch.randn(*shape, generator=g, device=device) * sd).to(torch.bfloat16)
    cfg = {"architecture": "Tobilorn", "width": W, "vocab": s["vocab"], "norm": {"eps": 1e-6}, "embedding": {"scale": math.sqrt(W)},
           "logit_scale": 0.25, "loop": dict(LOOP), "token_side": {"dim": s["side_dim"]}, "layers": []}
    t = {"embed": r(s["vocab"], W, sd=1.0), "head": r(s["vocab"], W), "final.norm": r(W, sd=0.1), "loop.in": r(W, 2 * W), "loop.step": r(LOOP["times"], W, sd=0.1),
         "side.embed": r(s["vocab"], LAYERS * s["side_dim"], sd=1.0)}
    E, I, F, S = s["experts"], s["identity"], s["expert_ff"], s["shared_ff"]
    for i in range(LAYERS):
        p = f"l{i}."
        for nm in ("norm1", "norm1b", "norm2", "norm2b"):
            t[p + nm] = r(W, sd=0.1)
        t[p + "mix.q"], t[p + "mix.k"], t[p + "mix.v"], t[p + "mix.o"] = r(H * 2 * D, W), r(G * 2 * D, W), r(G * V, W), r(W, H * V)
        t[p + "mix.q.b"], t[p + "mix.k.b"], t[p + "mix.v.b"], t[p + "mix.o.b"] = r(H * 2 * D, sd=0.1), r(G * 2 * D, sd=0.1), r(G * V, sd=0.1), r(W, sd=0.1)
        for nm in ("lq1", "lk1", "lq2", "lk2"):
            t[p + "mix." + nm] = r(D, sd=0.1)
        for e in range(E):
            t[p + f"mlp.e{e}.gate"], t[p + f"mlp.e{e}.up"], t[p + f"mlp.e{e}.down"] = r(F, W), r(F, W), r(W, F)
        t[p + "mlp.router"], t[p + "mlp.correction"] = r(E + I, W), r(E + I, sd=0.01)
        t[p + "mlp.shared.gate"], t[p + "mlp.shared.up"], t[p + "mlp.shared.down"] = r(S, W), r(S, W), r(W, S)
        t[p + "side.gate"], t[p + "side.proj"], t[p + "side.norm"] = r(s["side_dim"], W), r(W, s["side_dim"]), r(W, sd=0.1)
        cfg["layers"].append({"type": "attention",
                              "mixer": {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "diff": 0.2, "scale": 1.0 / math.sqrt(D),
                                        "mask": {"size": s["window"], "keep_first": s["keep_first"]}, "rot": {"base": 1000000.0, "dims": D}},
                              "mlp": {"kind": "moe", "expert": {"ff": F}, "router": {"experts": E, "identity": I, "top": s["top"]}, "shared": {"ff": S}}})
    return cfg, t


def vogusun_equal_size(size):
    """the closest served design at equal size: as many layer runs of capped grouped-query attention (heads of 128) + routed experts"""
    s = SIZES[size]
    v = dict(width=s["width"], heads=s["heads"], kv_heads=s["kv_heads"], dim=2 * s["dim"], vdim=s["vdim"], ff=0, experts=s["experts"], top=s["top"],
             expert_ff=s["expert_ff"], vocab=s["vocab"], gla_heads=0, gla_dim=0, gla_vdim=0, gla_rank=0)
    return vogusun_bench.random_model(v, pattern=("attention_2+moe",) * RUNS)


def operator_table(size, prompt_len):
    """the design's own kernels alone, at the prompt's row count and at one row: seconds and the fraction of their bound (matrix-core
    work: the bf16 peak; everything else: 8 TB/s over the bytes moved)"""
    from . import seq_ops as so
    from .seq_state import SequenceStateManager
    s = SIZES[size]
    W, H, G, D, V = s["width"], s["heads"], s["kv_heads"], s["dim"], s["vdim"]
    win, keep = s["window"], s["keep_first"]
    E, I, top, F = s["experts"], s["identity"], s["top"], s["expert_ff"]
    dev = "cuda"
    rows = []
    bf = lambda *sh: (torch.randn(*sh, device=dev) * 0.05).to(torch.bfloat16)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
    for T in (prompt_len, 1):
        st = SequenceStateManager(prompt_len + 64, 1, 64, dev)
        kt, vt = st.add_span_cache("k", G * 2 * D, torch.bfloat16), st.add_span_cache("v", G * V, torch.bfloat16)
        st.admit("a")
        st.reserve("a", prompt_len)
        st.upload()
        for tab in (kt, vt):
            tab.pool.pool.view(torch.bfloat16).normal_(0, 0.3)
        pos = torch.arange(T, dtype=torch.int32, device=dev) if T > 1 else i32([prompt_len - 1])
        slot = torch.zeros(T, dtype=torch.int32, device=dev)
        n_in = (H + G) * 2 * D + G * V
        a = torch.randn(T, n_in, device=dev) * 0.3
        freq = torch.rand(D // 2, device=dev)
        sec = _time(lambda: so.qkv_prep_append(a, 0, H * 2 * D, (H + G) * 2 * D, H, G, D, V, None, None, 1e-6, freq, D, 1, 1.0, 0.0, None, None, kt, vt,
                                               slot, pos, maps=2), 3)
        by = 8.0 * T * (H + G) * 2 * D + 4.0 * T * G * V + 2.0 * T * G * (2 * D + V)
        rows.append({"op": f"rotation of two maps + page append T={T}", "us": round(sec * 1e6, 1), "of_bound": round(by / HBM_BW / sec, 3)})
        e_slot, e_row0, e_cnt = i32([0]), i32([0]), i32([T])
        o = torch.empty(T, H * 2 * V, device=dev)
        sec = _time(lambda: so.gqa_attn_mc(a, kt, vt, pos, e_slot, e_row0, e_cnt, T, int(pos[-1]), H, G, D, V, 0.125, out=o, maps=2, window=win,
                                           keep_first=keep), 3)
        keys = sum(min(int(p) + 1, win + keep) for p in pos.tolist())
        fl = 2.0 * keys * H * 2 * (D + V)
        by = 2.0 * G * (2 * D + V) * min(prompt_len, win + keep + T) + 4.0 * T * H * 2 * (D + V)
        bound = max(fl / MFMA_BF16, by / HBM_BW)
        rows.append({"op": f"differential attention (2 maps, window {win} + {keep} kept) T={T} H={H} G={G} D={D} V={V} keys<={prompt_len}",
                     "us": round(sec * 1e6, 1), "tflops": round(fl / sec / 1e12, 2), "of_bound": round(bound / sec, 3)})
        on = torch.empty(T, H * V, dtype=torch.bfloat16, device=dev)
        sec = _time(lambda: so.maps_diff_norm(o, 0.3, 0.8, 1e-6, H, V, out=on), 3)
        rows.append({"op": f"difference of the maps + per-head norm T={T}", "us": round(sec * 1e6, 1), "of_bound": round(10.0 * T * H * V / HBM_BW / sec, 3)})
        x, m1 = torch.randn(T, W, device=dev), torch.randn(T, W, device=dev)
        gm, gh = bf(W), bf(W)
        h16 = torch.empty(T, W, dtype=torch.bfloat16, device=dev)
        sec = _time(lambda: so.residual_norm_step(x, 1e-6, m=m1, gamma_m=gm, add_m=1.0, gamma_h=gh, add_h=1.0, h=h16), 3)
        rows.append({"op": f"residual of a normed sublayer + next norm T={T}", "us": round(sec * 1e6, 1), "of_bound": round(14.0 * T * W / HBM_BW / sec, 3)})
        ids = torch.randint(0, s["vocab"], (T,), dtype=torch.int32, device=dev)
        table = bf(s["vocab"], W)
        sec = _time(lambda: so.embed_rows(ids, table, scale=3.0, out=x), 3)
        rows.append({"op": f"embedding rows x scale T={T}", "us": round(sec * 1e6, 1), "of_bound": round(6.0 * T * W / HBM_BW / sec, 3)})
        hin = (torch.randn(T, W, device=dev) * 0.5).to(torch.bfloat16)
        router, corr = bf(E + I, W), bf(E + I)
        logits = so.linear(hin, router, None, math=so.MATH_F32_STREAM)
        sec = _time(lambda: so.moe_route(logits, top, so.ROUTE_SCORES, corr), 3)
        rows.append({"op": f"routing: softmax over {E + I}, top-{top} of corrected scores, grouping by expert T={T}", "us": round(sec * 1e6, 1)})
        ids_, wts, seg, src, dst = so.moe_route(logits, top, so.ROUTE_SCORES, corr)
        R = T * top
        gu, y, dn = torch.randn(R, 2 * F, device=dev), torch.empty(R, F, dtype=torch.bfloat16, device=dev), torch.randn(R, W, device=dev)
        sec = _time(lambda: so.moe_glu(gu, F, 0.0, 0.0, y, unit=so.UNIT_SILU), 3)
        rows.append({"op": f"experts' silu unit [{R}x{F}]", "us": round(sec * 1e6, 1), "of_bound": round(10.0 * R * F / HBM_BW / sec, 3)})
        shared = torch.randn(T, W, device=dev)
        sec = _time(lambda: so.moe_combine(dn, dst, wts, T, top, ids=ids_, n_real=E, own=hin, add=shared), 3)
        rows.append({"op": f"weighted sum of the chosen experts (identity experts, shared expert added) T={T}", "us": round(sec * 1e6, 1),
                     "of_bound": round((4.0 * (R + 2 * T) * W + 2.0 * T * W) / HBM_BW / sec, 3)})
        cat, w_in, step = (torch.randn(T, 2 * W, device=dev) * 0.5).to(torch.bfloat16), bf(W, 2 * W), bf(W)
        xo = torch.empty(T, W, device=dev)
        sec = _time(lambda: so.linear(cat, w_in, step, out=xo, math=so.MATH_BF16), 3)
        fl, by = 4.0 * T * W * W, 4.0 * W * W + 8.0 * T * W
        rows.append({"op": f"loop entry [{T}x{2 * W}]x[{W}] + step vector", "us": round(sec * 1e6, 1), "tflops": round(fl / sec / 1e12, 1),
                     "of_bound": round(max(fl / MFMA_BF16, by / HBM_BW) / sec, 3)})
    return rows


LIKE_OPERATORS = ("page append", "grouped-query attention (capped", "per-head norm", "residual of two sublayers", "routing:", "clamped gated unit",
                  "weighted sum")


def run(args):
    from . import models
    from .engine import SeqEngine
    prompt_len = 2048
    res = {"metric": "prefill / decode throughput of the sequence engine (random Tobilorn models) beside Vogusun models of equal size",
           "unit": "tokens/s", "n_gpus": 1, "dtype": "bf16", "data": "synthetic", "prompt_len": prompt_len, "sizes": {}}
    for size in SIZES:
        entry = {"layers": LAYERS, "loop": dict(LOOP), "layer_runs": RUNS, **SIZES[size]}
        for name, make in (("engine", random_model), ("vogusun_equal_size", vogusun_equal_size)):
            cfg, t = make(size)
            eng = SeqEngine(models.resolve(cfg), cfg, t, dtype=torch.bfloat16, max_tokens=4 * (prompt_len + 128), max_slots=4)
            entry[name] = engine_throughput(eng, cfg["vocab"], prompt_len)
            entry[name]["weight_bytes"] = int(sum(v.numel() * v.element_size() for k, v in t.items() if k not in ("embed", "side.embed")))
            del eng, t
            torch.cuda.empty_cache()
        entry["vogusun_equal_size"]["layers"] = f"{RUNS} x (capped grouped-query attention with heads of {2 * SIZES[size]['dim']} + routed experts)"
        entry["operators"] = operator_table(size, prompt_len)
        vs = dict(SIZES[size], dim=2 * SIZES[size]["dim"], ff=SIZES[size]["expert_ff"], gla_heads=SIZES[size]["heads"], gla_dim=64, gla_vdim=128, gla_rank=64)
        saved = vogusun_bench.SIZES.get(size)
        vogusun_bench.SIZES[size] = vs
        try:
            entry["vogusun_operators"] = [r for r in vogusun_bench.operator_table(size, prompt_len) if any(k in r["op"] for k in LIKE_OPERATORS)]
        finally:
            vogusun_bench.SIZES[size] = saved
        res["sizes"][size] = entry
    res["value"] = res["sizes"]["4k"]["engine"]["prefill_tokens_per_s"]
    return res
