"""The sequence engine on small random Tobilorn models against oracle/tobilorn.py: whole prompts with the stream after every layer
run, decoding through the caches (a cache per pass of the looped layers), portions, mixed batches, reuse of pages and slots, the
first tokens, keys far back that the mask keeps, long decoding past the window, generation through the scheduler, graph replays."""
import numpy as np
import pytest
import torch

from oracle import tobilorn as ot
from tests.seq_helpers import make_engine, rel_err, rows_close, run_portions, run_whole

pytestmark = pytest.mark.gpu

CONFIGS = {
    "looped": dict(),
    # the loop covers every layer and starts the model, sizes that are no multiples of 8 (no matrix-core attention), one key/value
    # head, part of a map rotated, no kept keys, one expert per token and no identity or shared expert, a layer without feed-forward,
    # no token side input, scales of one
    "odd": dict(width=100, vocab=61, layers=3, loop=(0, 3, 2), heads=3, kv_heads=1, dim=20, vdim=12, rot_dims=8, scale=0.4, window=17,
                keep_first=0, experts=3, identity=0, top=1, expert_ff=10, shared_ff=0, side_dim=0, embed_scale=1.0, logit_scale=1.0,
                eps=1e-3, no_mlp=(1,), diff=0.5),
    # no loop, head sizes of the matrix-core tiles, as many key/value heads as query heads, windows and kept keys of whole pages, every
    # router output chosen, more identity experts than one, layers that differ from each other
    "tiles": dict(width=64, vocab=130, layers=4, loop=None, heads=4, kv_heads=4, dim=32, vdim=64, window=64, keep_first=64, experts=4,
                  identity=3, top=7, expert_ff=32, shared_ff=64, side_dim=8, base=500.0,
                  per_layer={1: dict(window=1, keep_first=1, heads=2, kv_heads=1, top=2), 2: dict(window=1000, keep_first=0, vdim=16, dim=16),
                             3: dict(window=30, keep_first=70, identity=0, top=1, diff=0.1)}),
    # one pass only, the loop at the end; a width that is no multiple of 4 (no vector loads, no rows in registers)
    "once": dict(width=50, layers=3, loop=(2, 3, 1), window=25, keep_first=2, heads=2, kv_heads=2, top=2, side_dim=6),
}


# rows of a 16-bit engine that must lie within the tolerance: where one expert serves a token alone, a rounding that tips a narrow
# choice swaps the whole feed-forward output of that row (and, weakly, of the rows that read it)
SHARE = {"odd": 0.7}


def model(name, seed=0):
    rng = np.random.default_rng(seed)
    cfg, t = ot.random_tobilorn(rng, **CONFIGS[name])
    return cfg, t, rng


@pytest.mark.parametrize("name", list(CONFIGS))
def test_whole_prompt_f32_and_bf16(name):
    cfg, t, rng = model(name)
    tokens = rng.integers(0, cfg["vocab"], 150).tolist()
    streams = []
    want = ot.tobilorn_forward(cfg, t, tokens, streams)
    assert len(streams) == len(ot.layer_runs(cfg))
    eng = make_engine(cfg, t, torch.float32)
    taps = {}
    got = eng.step([("a", tokens, list(range(len(tokens))))], taps=taps).cpu().numpy()
    for i, s in enumerate(streams):
        assert rel_err(taps[i].cpu().numpy(), s) < 2e-5, f"layer run {i}"
    assert rel_err(got, want) < 5e-5
    eng.release("a")
    assert rel_err(run_whole(eng, "b", tokens), got) < 1e-6                  # without the taps the residual steps run fused
    eng16 = make_engine(cfg, t, torch.bfloat16)
    assert rows_close(run_whole(eng16, "a", tokens), want, 0.08, SHARE.get(name, 0.95))


@pytest.mark.parametrize("name", list(CONFIGS))
def test_prefill_against_token_by_token_decoding(name):
    cfg, t, rng = model(name, 1)
    tokens = rng.integers(0, cfg["vocab"], 200).tolist()      # decoding runs over three pages and past every window
    want = ot.tobilorn_forward(cfg, t, tokens)
    eng = make_engine(cfg, t, torch.float32)
    whole = run_whole(eng, "w", tokens)
    dec = run_portions(eng, "d", tokens, [1])
    assert rel_err(whole, want) < 5e-5 and rel_err(dec, want) < 5e-5
    mixed = run_portions(eng, "m", tokens, [70, 1])           # a prompt, then its last tokens one by one
    assert rel_err(mixed, dec) < 2e-6
    eng16 = make_engine(cfg, t, torch.bfloat16)
    w16 = run_whole(eng16, "w", tokens)
    d16 = run_portions(eng16, "d", tokens, [120, 1])          # decode steps replay graphs; the key walk is split
    assert rows_close(d16, w16, 0.04, SHARE.get(name, 0.95)) and rows_close(d16, want, 0.08, SHARE.get(name, 0.95))


@pytest.mark.parametrize("sizes", [[2], [3, 2, 64, 1, 5, 63, 2], [64], [65, 2, 2, 1, 127], [1, 2, 128, 2], [130, 2]])
def test_portions_of_any_size(sizes):
    cfg, t, rng = model("looped", 2)
    tokens = rng.integers(0, cfg["vocab"], 201).tolist()
    eng = make_engine(cfg, t, torch.float32)
    whole = run_whole(eng, "w", tokens)
    assert rel_err(run_portions(eng, "p", tokens, sizes), whole) < 2e-6
    eng16 = make_engine(cfg, t, torch.bfloat16)
    w16 = run_whole(eng16, "w", tokens)
    assert rows_close(run_portions(eng16, "p", tokens, sizes), w16, 0.04)


def test_batches_of_unequal_requests_against_each_alone():
    cfg, t, rng = model("looped", 3)
    lens = [1, 23, 97, 190]
    toks = [rng.integers(0, cfg["vocab"], n).tolist() for n in lens]
    for dtype, tol in ((torch.float32, 2e-6), (torch.bfloat16, None)):
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
    d = eng.step([("d", toks[3], list(range(64))), ("c", [], [])]).cpu().numpy()   # b's slot and pages, dirty from b, in every pass's cache
    eng.release("c")
    e = run_whole(eng, "e", toks[4])
    eng.release("d")
    assert eng.state.used_pages() == 0 and len(eng.state.free_slots) == 2
    assert rel_err(a, fresh[0]) < 2e-6 and rel_err(np.concatenate([b[:90], b2[:10]]), fresh[1]) < 2e-6
    assert rel_err(np.concatenate([b[90:], b2[10:]]), fresh[2]) < 2e-6
    assert rel_err(d, fresh[3]) < 2e-6 and rel_err(e, fresh[4]) < 2e-6


def test_the_first_tokens_of_a_sequence():
    cfg, t, rng = model("tiles", 5)
    tokens = rng.integers(0, cfg["vocab"], 6).tolist()
    want = ot.tobilorn_forward(cfg, t, tokens)
    for dtype, tol in ((torch.float32, 5e-5), (torch.bfloat16, 0.08)):
        eng = make_engine(cfg, t, dtype)
        assert rel_err(run_whole(eng, "a", tokens[:1]), want[:1]) < tol      # one key: both maps return its value, the norm sees (1 - lambda) v
        got = run_portions(eng, "b", tokens, [1, 2, 3])
        assert rel_err(got, want) < tol if dtype == torch.float32 else rows_close(got, want, tol, 0.8)
    # (the same token twice gives the same logits twice: every key then carries the same value)
    second = run_whole(eng, "c", tokens[1:2])
    assert rel_err(got[1:2], second) > 1e-3                                  # a token at position 1 is not that token at position 0


def test_a_kept_first_key_decides_the_logits_far_later():
    """the embedding of one token is scaled up, so that where it stands among the kept first keys its key and value reach every
    later position, however far: the logits change visibly when it stands one position further, outside the kept keys"""
    cfg, t = ot.random_tobilorn(np.random.default_rng(8), layers=3, loop=(1, 2, 2), window=30, keep_first=4, side_dim=0)
    rng = np.random.default_rng(9)
    t = dict(t)
    t["embed"] = t["embed"].copy()
    t["embed"][7] *= 4.0                                                     # (a power of two: the values stay 16-bit ones)
    base = [int(x) for x in rng.integers(8, cfg["vocab"], 330)]
    a, b = list(base), list(base)
    a[3], b[4] = 7, 7                                                        # kept / not kept, and out of every later window
    wa, wb = ot.tobilorn_forward(cfg, t, a)[-20:], ot.tobilorn_forward(cfg, t, b)[-20:]
    wc = ot.tobilorn_forward(cfg, t, base)[-20:]
    assert rel_err(wa, wc) > 1e-2 and rel_err(wa, wb) > 1e-2
    eng = make_engine(cfg, t, torch.float32)
    ga = run_portions(eng, "a", a, [310, 1])[-20:]                            # the last 20 tokens decoded alone, 5 pages on
    gb = run_portions(eng, "b", b, [2, 150, 158, 1])[-20:]
    assert rel_err(ga, wa) < 5e-5 and rel_err(gb, wb) < 5e-5
    eng16 = make_engine(cfg, t, torch.bfloat16)
    assert rows_close(run_portions(eng16, "a", a, [310, 1])[-20:], wa, 0.08, 0.8)


def test_long_decoding_past_the_window():
    cfg, t, rng = model("once", 10)
    tokens = rng.integers(0, cfg["vocab"], 170).tolist()
    want = ot.tobilorn_forward(cfg, t, tokens)
    eng16 = make_engine(cfg, t, torch.bfloat16)
    got = run_portions(eng16, "d", tokens, [10, 1])                           # 160 decoded tokens: windows of decoded keys only, three pages
    assert rows_close(got, want, 0.08)
    eng = make_engine(cfg, t, torch.float32)
    assert rel_err(run_portions(eng, "d", tokens, [10, 1]), want) < 5e-5


def test_greedy_generation_through_the_scheduler():
    cfg, t, rng = model("looped", 6)
    prompts = [rng.integers(0, cfg["vocab"], n).tolist() for n in (5, 41, 18)]
    new = 12
    want = []
    for p in prompts:
        seq = list(p)
        for _ in range(new):
            seq.append(int(np.argmax(ot.tobilorn_forward(cfg, t, seq)[-1])))
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
