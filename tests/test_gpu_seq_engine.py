"""The sequence engine on small random Modanex models against oracle/seq_model.py: whole prompts, decoding through the cache
and the state, portions, mixed batches, reuse of pages and slots, generation through the scheduler."""
import numpy as np
import pytest
import torch

from oracle import seq_model as om
from tests.seq_helpers import make_engine, rel_err, run_portions, run_whole

pytestmark = pytest.mark.gpu

CONFIGS = {
    "mixed": dict(),
    # sizes that are no multiples of 8, one head, one block, two taps, equal ranks, a window longer than any prompt, no bigram
    "odd": dict(width=100, vocab=61, layers=("latent_attention+mlp", "rglru", "latent_attention:share"), heads=1, dim=20, vdim=20, kv_rank=36,
                q_rank=36, window=1000, scale=1.0, rec_width=52, blocks=1, taps=2, ff=44, bigram=False, eps=1e-3),
    # attention first and last, a window of one page exactly, a recurrent layer with a feed-forward, a single tap
    "page": dict(width=64, vocab=130, layers=("latent_attention", "rglru+mlp", "rglru", "latent_attention+mlp"), heads=4, dim=16, vdim=8,
                 kv_rank=32, q_rank=24, window=64, scale=0.25, rec_width=64, blocks=4, taps=1, ff=64, buckets=7),
}


def model(name, seed=0):
    rng = np.random.default_rng(seed)
    cfg, t = om.random_modanex(rng, **CONFIGS[name])
    return cfg, t, rng


@pytest.mark.parametrize("name", list(CONFIGS))
def test_whole_prompt_f32_and_bf16(name):
    cfg, t, rng = model(name)
    tokens = rng.integers(0, cfg["vocab"], 150).tolist()
    streams = []
    want = om.modanex_forward(cfg, t, tokens, streams)
    eng = make_engine(cfg, t, torch.float32)
    taps = {}
    got = eng.step([("a", tokens, list(range(len(tokens))))], taps=taps).cpu().numpy()
    for i, s in enumerate(streams):
        assert rel_err(taps[i].cpu().numpy(), s) < 2e-5, f"layer {i}"
    assert rel_err(got, want) < 5e-5
    eng16 = make_engine(cfg, t, torch.bfloat16)
    assert rel_err(run_whole(eng16, "a", tokens), want) < 0.08


@pytest.mark.parametrize("name", list(CONFIGS))
def test_prefill_against_token_by_token_decoding(name):
    cfg, t, rng = model(name, 1)
    tokens = rng.integers(0, cfg["vocab"], 210).tolist()     # decoding runs past every window, page and convolution tail
    want = om.modanex_forward(cfg, t, tokens)
    eng = make_engine(cfg, t, torch.float32)
    whole = run_whole(eng, "w", tokens)
    dec = run_portions(eng, "d", tokens, [1])
    assert rel_err(whole, want) < 5e-5 and rel_err(dec, want) < 5e-5
    assert rel_err(dec, whole) < 1e-6
    mixed = run_portions(eng, "m", tokens, [70, 1])           # a prompt, then its last tokens one by one
    assert rel_err(mixed, whole) < 1e-6


@pytest.mark.parametrize("sizes", [[2], [3, 2, 64, 1, 5, 63, 2], [64], [65, 2, 2, 1, 127], [1, 2, 128, 2]])
def test_portions_of_any_size(sizes):
    cfg, t, rng = model("mixed", 2)
    tokens = rng.integers(0, cfg["vocab"], 201).tolist()
    eng = make_engine(cfg, t, torch.float32)
    whole = run_whole(eng, "w", tokens)
    assert rel_err(run_portions(eng, "p", tokens, sizes), whole) < 1e-6
    eng16 = make_engine(cfg, t, torch.bfloat16)
    w16 = run_whole(eng16, "w", tokens)
    assert rel_err(run_portions(eng16, "p", tokens, sizes), w16) < 0.03    # rounding only: other kernels for short portions


def test_batches_of_unequal_requests_against_each_alone():
    cfg, t, rng = model("mixed", 3)
    lens = [1, 23, 97, 160]
    toks = [rng.integers(0, cfg["vocab"], n).tolist() for n in lens]
    eng = make_engine(cfg, t, torch.float32, max_tokens=1024)
    alone = [run_whole(eng, ("a", i), tk) for i, tk in enumerate(toks)]
    # step 1: the first 20 tokens of each (or all it has); then portions of some beside single tokens of others
    got = [[] for _ in toks]
    at = [0] * len(toks)
    plan = [[20, 20, 20, 20], [0, 1, 40, 2], [0, 1, 1, 64], [0, 1, 36, 1], [0, 0, 0, 73]]
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
        assert rel_err(np.concatenate(got[i]), alone[i]) < 1e-6, f"request {i}"


def test_pages_and_slots_that_are_freed_and_used_again():
    cfg, t, rng = model("mixed", 4)
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
    d = eng.step([("d", toks[3], list(range(64))), ("c", [], [])]).cpu().numpy()   # b's slot and pages, dirty from b
    eng.release("c")
    e = run_whole(eng, "e", toks[4])
    eng.release("d")
    assert eng.state.used_pages() == 0 and len(eng.state.free_slots) == 2
    assert rel_err(a, fresh[0]) < 1e-6 and rel_err(np.concatenate([b[:90], b2[:10]]), fresh[1]) < 1e-6
    assert rel_err(np.concatenate([b[90:], b2[10:]]), fresh[2]) < 1e-6
    assert rel_err(d, fresh[3]) < 1e-6 and rel_err(e, fresh[4]) < 1e-6


def test_the_first_tokens_of_a_sequence():
    cfg, t, rng = model("page", 5)
    tokens = rng.integers(0, cfg["vocab"], 6).tolist()
    want = om.modanex_forward(cfg, t, tokens)
    eng = make_engine(cfg, t, torch.float32)
    assert rel_err(run_whole(eng, "a", tokens[:1]), want[:1]) < 5e-5
    assert rel_err(run_portions(eng, "b", tokens, [1, 2, 3]), want) < 5e-5
    # the same token again as a sequence's first and as its second token: the second table and the state make the difference
    two = run_whole(eng, "c", [tokens[0], tokens[0]])
    assert rel_err(two[:1], want[:1]) < 5e-5 and rel_err(two[1:], two[:1]) > 1e-3


def test_greedy_generation_through_the_scheduler():
    cfg, t, rng = model("mixed", 6)
    prompts = [rng.integers(0, cfg["vocab"], n).tolist() for n in (5, 41, 18)]
    new = 12
    want = []
    for p in prompts:
        seq = list(p)
        for _ in range(new):
            seq.append(int(np.argmax(om.modanex_forward(cfg, t, seq)[-1])))
        want.append(seq[len(p):])
    eng = make_engine(cfg, t, torch.float32, max_tokens=192, max_slots=2)      # the third prompt waits for a slot
    got = eng.generate(prompts, max_new_tokens=new, token_budget=24, max_chunk=16)
    assert got == want
    assert eng.state.used_pages() == 0 and not eng.state.live
    sampled = eng.generate(prompts[:2], max_new_tokens=4, sampling={"top_k": 5, "top_p": 0.9, "temperature": 0.8, "seed": 3})
    assert all(len(s) == 4 and all(0 <= x < cfg["vocab"] for x in s) for s in sampled)


def test_decode_steps_replayed_as_graphs_equal_eager_steps(monkeypatch):
    """bf16 decode steps of two requests: captured and replayed (several replays, eager work and synchronisation between
    them) against the same steps launched eagerly, and a request that joins later (another graph)"""
    cfg, t, rng = model("page", 7)
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
