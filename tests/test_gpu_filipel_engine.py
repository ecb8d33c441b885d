"""The sequence engine on small random Filipel models against oracle/filipel.py: whole prompts with the stream after every layer,
decoding through the caches and the recurrent state, portions, mixed batches, reuse of pages and slots, the first tokens, a far
token that decides the logits pages later, long decoding past every window, generation through the scheduler, graph replays."""
import numpy as np
import pytest
import torch

from oracle import filipel as of
from tests.seq_helpers import make_engine, rel_err, rows_close, run_portions, run_whole

pytestmark = pytest.mark.gpu

CONFIGS = {
    # both kinds of layer and all three kinds of feed-forward, a layer that reads an earlier layer's latent cache
    "mixed": dict(layers=[("parallel", None, ("dense", 50)), ("latent_attention", None, ("moe",)), ("parallel", None, ("moe",)),
                          ("latent_attention", {"kv_from": 1}, None), ("parallel", {"right": {"groups": 3}}, None)]),
    # sizes that are no multiples of 4 or 8, one head, one key/value head, the whole head rotated, one group of everything, two taps,
    # every expert chosen, the latent layer first, a residual multiplier of one
    "odd": dict(width=50, vocab=61, eps=1e-3, residual_mult=1.0,
                layers=[("latent_attention", dict(heads=1, dim=12, rot_dim=4, vdim=9, kv_rank=10, q_rank=6), ("moe", dict(experts=4, count=1, keep=1, top=4, ff=10))),
                        ("parallel", {"left": dict(heads=3, kv_heads=1, dim=20, vdim=12, rot_dims=20, window=17, scale=0.4),
                                      "right": dict(heads=2, vdim=7, state=5, groups=2, conv=2, norm_groups=1)}, ("dense", 33)),
                        ("parallel", {"left": dict(heads=2, kv_heads=2, dim=6, vdim=10, rot_dims=2, window=1),
                                      "right": dict(heads=1, vdim=9, state=3, groups=1, conv=1, norm_groups=3)}, None),
                        ("latent_attention", dict(heads=1, dim=12, rot_dim=4, vdim=5, kv_rank=10, q_rank=9, kv_from=0), ("moe", dict(experts=2, count=2, keep=1, top=1, ff=6)))]),
    # sizes of the matrix-core tiles: latent + rotated part of exactly one 64-element row, as many key/value heads as query heads, a
    # window of one page and one that never binds, groups of the state-space mixer as many as heads, a choice that fills its groups
    "tiles": dict(width=64, vocab=130, residual_mult=0.25,
                  layers=[("parallel", {"left": dict(heads=4, kv_heads=4, dim=32, vdim=64, rot_dims=32, window=64),
                                        "right": dict(heads=4, vdim=32, state=16, groups=4, conv=4, norm_groups=4)}, ("moe", dict(experts=8, count=4, keep=2, top=4, ff=32))),
                          ("latent_attention", dict(heads=4, dim=32, rot_dim=16, vdim=32, kv_rank=48, q_rank=32, base=100.0), ("dense", 96)),
                          ("parallel", {"left": dict(heads=8, kv_heads=2, dim=16, vdim=32, rot_dims=8, window=1000, base=300.0),
                                        "right": dict(heads=2, vdim=64, state=32, groups=1, conv=3, norm_groups=1)}, ("moe", dict(experts=4, count=2, keep=1, top=2, ff=16))),
                          ("latent_attention", dict(heads=2, dim=16, rot_dim=16, vdim=64, kv_rank=48, q_rank=16, base=100.0, kv_from=1), None)]),
}

# rows of a 16-bit engine that must lie within the tolerance: a rounding can tip a narrow choice of experts, which swaps the
# feed-forward output of that row (and, weakly, of the rows that read it)
SHARE = {"odd": 0.8}


def model(name, seed=0):
    rng = np.random.default_rng(seed)
    cfg, t = of.random_filipel(rng, **CONFIGS[name])
    return cfg, t, rng


@pytest.mark.parametrize("name", list(CONFIGS))
def test_whole_prompt_f32_and_bf16(name):
    cfg, t, rng = model(name)
    tokens = rng.integers(0, cfg["vocab"], 150).tolist()
    streams = []
    want = of.forward(cfg, t, tokens, streams)
    assert len(streams) == len(cfg["layers"])
    eng = make_engine(cfg, t, torch.float32)
    taps = {}
    got = eng.step([("a", tokens, list(range(len(tokens))))], taps=taps).cpu().numpy()
    for i, s in enumerate(streams):
        assert rel_err(taps[i].cpu().numpy(), s) < 2e-5, f"layer {i}"
    assert rel_err(got, want) < 5e-5
    eng.release("a")
    eng16 = make_engine(cfg, t, torch.bfloat16)
    assert rows_close(run_whole(eng16, "a", tokens), want, 0.08, SHARE.get(name, 0.95))


@pytest.mark.parametrize("name", list(CONFIGS))
def test_prefill_against_token_by_token_decoding(name):
    cfg, t, rng = model(name, 1)
    tokens = rng.integers(0, cfg["vocab"], 200).tolist()      # decoding runs over three pages and past the windows
    want = of.forward(cfg, t, tokens)
    eng = make_engine(cfg, t, torch.float32)
    whole = run_whole(eng, "w", tokens)                        # the state-space scan runs in chunks side by side
    dec = run_portions(eng, "d", tokens, [1])
    assert rel_err(whole, want) < 5e-5 and rel_err(dec, want) < 5e-5
    mixed = run_portions(eng, "m", tokens, [70, 1])           # a prompt, then its last tokens one by one
    assert rel_err(mixed, dec) < 2e-5
    eng16 = make_engine(cfg, t, torch.bfloat16)
    w16 = run_whole(eng16, "w", tokens)
    d16 = run_portions(eng16, "d", tokens, [120, 1])          # decode steps replay graphs; the key walks are split
    assert rows_close(d16, w16, 0.04, SHARE.get(name, 0.95)) and rows_close(d16, want, 0.08, SHARE.get(name, 0.95))


@pytest.mark.parametrize("sizes", [[2], [3, 2, 64, 1, 5, 63, 2], [64], [65, 2, 2, 1, 127], [1, 2, 128, 2], [130, 2]])
def test_portions_of_any_size(sizes):
    cfg, t, rng = model("mixed", 2)
    tokens = rng.integers(0, cfg["vocab"], 201).tolist()
    eng = make_engine(cfg, t, torch.float32)
    whole = run_whole(eng, "w", tokens)
    assert rel_err(run_portions(eng, "p", tokens, sizes), whole) < 2e-5
    eng16 = make_engine(cfg, t, torch.bfloat16)
    w16 = run_whole(eng16, "w", tokens)
    assert rows_close(run_portions(eng16, "p", tokens, sizes), w16, 0.04)


@pytest.mark.parametrize("name", ["mixed", "tiles"])
def test_batches_of_unequal_requests_against_each_alone(name):
    cfg, t, rng = model(name, 3)
    lens = [1, 23, 97, 190]
    toks = [rng.integers(0, cfg["vocab"], n).tolist() for n in lens]
    for dtype, tol in ((torch.float32, 2e-5), (torch.bfloat16, None)):
        eng = make_engine(cfg, t, dtype, max_tokens=1024)
        alone = [run_whole(eng, ("a", i), tk) for i, tk in enumerate(toks)]
        got = [[] for _ in toks]
        at = [0] * len(toks)
        plan = [[20, 20, 20, 20], [0, 1, 40, 2], [0, 1, 1, 64], [0, 1, 36, 1], [0, 0, 0, 103]]
        for step in plan:
            ent, who = [], []
            for i, n in enumerate(step):
                n = min(n, lens[i] - at[i])
                if n > 0:
                    ent.append((("b", i), toks[i][at[i]:at[i] + n], list(range(n))))
                    who.append((i, n))
            out = eng.step(ent).cpu().numpy()
            o = 0
            for i, n in who:
                got[i].append(out[o:o + n])
                o, at[i] = o + n, at[i] + n
        for i in range(len(toks)):
            assert at[i] == lens[i]
            if tol is None:
                assert rows_close(np.concatenate(got[i]), alone[i], 0.04), f"request {i}"
            else:
                assert rel_err(np.concatenate(got[i]), alone[i]) < tol, f"request {i}"


def test_pages_and_slots_that_are_freed_and_used_again():
    cfg, t, rng = model("odd", 4)
    toks = [rng.integers(0, cfg["vocab"], n).tolist() for n in (150, 100, 120, 64, 30)]
    fresh = [run_whole(make_engine(cfg, t, torch.float32, max_tokens=256, max_slots=2), "f", tk) for tk in toks]
    eng = make_engine(cfg, t, torch.float32, max_tokens=320, max_slots=2)      # 5 pages, 2 slots
    assert eng.state.num_pages == 5
    a = run_portions(eng, "a", toks[0], [64, 1, 85])                           # 3 pages, released
    assert eng.state.used_pages() == 0
    b = eng.step([("b", toks[1][:90], list(range(90))), ("c", toks[2][:40], list(range(40)))]).cpu().numpy()
    b2 = eng.step([("b", toks[1][90:], list(range(10))), ("c", toks[2][40:], list(range(80)))]).cpu().numpy()
    assert eng.state.used_pages() == 4
    with pytest.raises(RuntimeError):
        eng.step([("d", toks[3], [])])                                         # no slot left
    eng.release("b")
    d = eng.step([("d", toks[3], list(range(64))), ("c", [], [])]).cpu().numpy()   # b's slot (state, convolution tail) and pages, dirty from b
    eng.release("c")
    e = run_whole(eng, "e", toks[4])
    eng.release("d")
    assert eng.state.used_pages() == 0 and len(eng.state.free_slots) == 2
    assert rel_err(a, fresh[0]) < 2e-5 and rel_err(np.concatenate([b[:90], b2[:10]]), fresh[1]) < 2e-5
    assert rel_err(np.concatenate([b[90:], b2[10:]]), fresh[2]) < 2e-5
    assert rel_err(d, fresh[3]) < 2e-5 and rel_err(e, fresh[4]) < 2e-5


def test_the_first_tokens_of_a_sequence():
    cfg, t, rng = model("tiles", 5)
    tokens = rng.integers(0, cfg["vocab"], 6).tolist()
    want = of.forward(cfg, t, tokens)
    for dtype, tol in ((torch.float32, 5e-5), (torch.bfloat16, 0.08)):
        eng = make_engine(cfg, t, dtype)
        assert rel_err(run_whole(eng, "a", tokens[:1]), want[:1]) < tol      # one key, an empty state, a convolution over zeros
        got = run_portions(eng, "b", tokens, [1, 2, 3])
        assert rel_err(got, want) < tol if dtype == torch.float32 else rows_close(got, want, tol, 0.8)
    second = run_whole(eng, "c", tokens[1:2])
    assert rel_err(got[1:2], second) > 1e-3                                  # a token at position 1 is not that token at position 0


def test_far_tokens_decide_the_logits_pages_later():
    """sharp scores in the latent attention, which reads every earlier position: the logits of the last rows change visibly when
    tokens more than 230 positions (three pages and more) back are others, through the layer's own cache and through a borrowed one"""
    rng = np.random.default_rng(8)
    cfg, t = of.random_filipel(rng, [("latent_attention", {"scale": 1.5}, None), ("parallel", {"left": {"window": 30}}, ("moe",)),
                                     ("latent_attention", {"kv_from": 0, "heads": 2, "vdim": 8, "scale": 1.5}, None)])
    a = [int(x) for x in rng.integers(0, cfg["vocab"], 330)]
    b = [int(x) for x in rng.integers(0, cfg["vocab"], 100)] + a[100:]
    wa, wb = of.forward(cfg, t, a)[-20:], of.forward(cfg, t, b)[-20:]
    assert rel_err(wa, wb) > 1e-2
    eng = make_engine(cfg, t, torch.float32)
    ga = run_portions(eng, "a", a, [310, 1])[-20:]                            # the last 20 tokens decoded alone, 5 pages on
    gb = run_portions(eng, "b", b, [2, 150, 158, 1])[-20:]
    assert rel_err(ga, wa) < 5e-5 and rel_err(gb, wb) < 5e-5
    eng16 = make_engine(cfg, t, torch.bfloat16)
    assert rows_close(run_portions(eng16, "a", a, [310, 1])[-20:], wa, 0.08, 0.8)


def test_long_decoding_past_the_window():
    cfg, t, rng = model("mixed", 10)
    tokens = rng.integers(0, cfg["vocab"], 170).tolist()
    want = of.forward(cfg, t, tokens)
    eng16 = make_engine(cfg, t, torch.bfloat16)
    got = run_portions(eng16, "d", tokens, [10, 1])                           # 160 decoded tokens: windows of decoded keys only, three pages
    assert rows_close(got, want, 0.08)
    eng = make_engine(cfg, t, torch.float32)
    assert rel_err(run_portions(eng, "d", tokens, [10, 1]), want) < 5e-5


def test_greedy_generation_through_the_scheduler():
    cfg, t, rng = model("mixed", 6)
    prompts = [rng.integers(0, cfg["vocab"], n).tolist() for n in (5, 41, 18)]
    new = 12
    want = []
    for p in prompts:
        seq = list(p)
        for _ in range(new):
            seq.append(int(np.argmax(of.forward(cfg, t, seq)[-1])))
        want.append(seq[len(p):])
    eng = make_engine(cfg, t, torch.float32, max_tokens=192, max_slots=2)      # the third prompt waits for a slot
    got = eng.generate(prompts, max_new_tokens=new, token_budget=24, max_chunk=16)
    assert got == want
    assert eng.state.used_pages() == 0 and not eng.state.live
    sampled = eng.generate(prompts[:2], max_new_tokens=4, sampling={"top_k": 5, "top_p": 0.9, "temperature": 0.8, "seed": 3})
    assert all(len(s) == 4 and all(0 <= x < cfg["vocab"] for x in s) for s in sampled)


def test_decode_steps_replayed_as_graphs_equal_eager_steps(monkeypatch):
    cfg, t, rng = model("tiles", 7)
    toks = [rng.integers(0, cfg["vocab"], n).tolist() for n in (90, 150, 40)]
    def run(eng):
        out = []
        eng.step([("a", toks[0][:50], []), ("b", toks[1][:100], [])])
        for i in range(25):
            out.append(eng.step([("a", [toks[0][50 + i]], [0]), ("b", [toks[1][100 + i]], [0])]).cpu().numpy().copy())
            if i == 10:
                torch.cuda.synchronize()
                eng.step([("c", toks[2][:30], [])])      # a prompt's portion between two replays
        for i in range(10):
            out.append(eng.step([("a", [toks[0][75 + i]], [0]), ("b", [toks[1][125 + i]], [0]), ("c", [toks[2][30 + i]], [0])]).cpu().numpy().copy())
        return out
    graphed = make_engine(cfg, t, torch.bfloat16)
    assert graphed.use_graphs
    got = run(graphed)
    assert any(g["graph"] is not None for g in graphed._graphs.values())
    monkeypatch.setenv("DIHIP_SEQ_GRAPH", "0")
    eager = make_engine(cfg, t, torch.bfloat16)
    assert not eager.use_graphs
    want = run(eager)
    for a, b in zip(got, want):
        assert np.array_equal(a, b)
