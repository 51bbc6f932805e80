"""The engine above the step function: greedy generation through the entry point against the plain
implementation, seeded sampling, long decoding, the first tokens of a sequence, decode steps as
captured graphs against eager steps, preemption under a tiny pool, and the replay program itself."""
import json
import os
import subprocess
import sys

import pytest
import torch

import plain_minicpm4 as P
from helpers import CONFIGS, TOL, Driver, make_model_dir, random_tokens, rel_err

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name in ("A", "B", "C"):
        for dtype in ("float32", "bfloat16"):
            cfg = CONFIGS[name]()
            d = str(tmp_path_factory.mktemp(f"eng_{name}_{dtype}"))
            out[(name, dtype)] = (cfg, d, make_model_dir(d, cfg, seed=40 + ord(name), store=dtype))
    return out


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_greedy_generation_through_the_entry_point(models, name):
    """Batch of prompts of lengths 1..40, cut into portions under a small token budget and decoded
    beside each other: the tokens equal the plain implementation's greedy tokens."""
    from infinilm_amd import LLM, SamplingParams

    cfg, d, W = models[(name, "float32")]
    prompts = [random_tokens(cfg, n, 300 + n) for n in (1, 2, 17, 40, 9)]
    llm = LLM(d, dtype="float32", num_blocks=24, block_size=8, max_batch_size=3, max_num_batched_tokens=11, chunk_size=7)
    outs = llm.generate(prompt_token_ids=prompts, sampling_params=SamplingParams(top_k=1, max_tokens=16))
    for p, o in zip(prompts, outs):
        assert o.finished and o.finish_reason.value == "length"
        assert o.outputs[0].token_ids == P.plain_greedy(cfg, W, p, 16), f"prompt of {len(p)} tokens"
    assert llm.engine.runner.cache.free_pages() == 24
    log = llm.engine.scheduler.log
    assert any(s["decode"] > 0 and s["portions"] for s in log), "no step mixed decoded tokens with a prompt's portion"
    llm.close()


@pytest.mark.parametrize("name", ["A", "B"])
def test_requests_that_share_a_beginning_share_its_pages(models, name):
    """One prompt, then the same prompt with other endings, the prompt again, and a request that is
    preempted and finds its own pages: with the published pages taken over, the tokens are the
    plain implementation's (float32: the shared keys are bit for bit what the request would have
    computed), and fewer tokens run."""
    from infinilm_amd import LLM, SamplingParams

    cfg, d, W = models[(name, "float32")]
    stem = random_tokens(cfg, 37, 900)
    prompts = [stem, stem + random_tokens(cfg, 6, 901), stem[:30] + random_tokens(cfg, 9, 902), stem, stem[:8]]
    sp = SamplingParams(top_k=1, max_tokens=10)
    ran = {}
    for sharing in (True, False):
        llm = LLM(d, dtype="float32", num_blocks=40, block_size=8, max_batch_size=2, chunk_size=16,
                  enable_prefix_caching=sharing)
        assert llm.engine.runner.cache.prefix_caching == sharing
        first = llm.generate(prompt_token_ids=[prompts[0]], sampling_params=sp)
        rest = llm.generate(prompt_token_ids=prompts[1:], sampling_params=sp)
        for p, o in zip(prompts, first + rest):
            assert o.outputs[0].token_ids == P.plain_greedy(cfg, W, p, 10), f"sharing {sharing}, prompt of {len(p)}"
        st = llm.engine.stats()
        ran[sharing] = st["prompt_tokens"]
        if sharing:
            # whole pages of 8 below the last token: 32 of 37+6, 24 of 30+9, 32 of 37 and 0 of 8
            assert st["cache"]["prefix_hit_tokens"] == 32 + 24 + 32
            reqs = list(llm.engine.requests.values())
            assert [r.num_cached_tokens for r in reqs] == [0, 32, 24, 32, 0]
        else:
            assert st["cache"]["prefix_hit_tokens"] == 0
        assert llm.engine.runner.cache.free_pages() == 40
        llm.engine.runner.cache.check()
        llm.close()
    assert ran[False] - ran[True] == 32 + 24 + 32


@pytest.mark.parametrize("name,dtype,graph,policy,page", [("A", "float32", True, "optimistic", 8), ("B", "bfloat16", True, "optimistic", 16),
                                                          ("C", "bfloat16", True, "reserve_full", 16),
                                                          ("C", "bfloat16", True, "optimistic", 64)])
def test_random_load_with_shared_beginnings_preemptions_and_graphs(models, name, dtype, graph, policy, page):
    """Sixty requests that trickle in, with prompts cut from three stems, greedy and sampled, into a
    pool of a few pages: after every step the cache manager's books agree; at the end everything
    is finished and free, pages were shared, requests were preempted (optimistic admission), and in
    float32 the greedy ones equal the plain implementation."""
    import random
    from infinilm_amd import LLM, SamplingParams

    cfg, d, W = models[(name, dtype)]
    V = cfg["vocab_size"]
    rng = random.Random(5)
    # (bfloat16 with pages of 16 and 64: the matrix-core attention kernels serve the load)
    llm = LLM(d, dtype=dtype, num_blocks=12, block_size=page, max_batch_size=4, max_num_batched_tokens=8 * page,
              chunk_size=2 * page, enable_graph=graph, admission=policy, seed=3)
    eng = llm.engine
    stems = [[rng.randrange(V) for _ in range(5 * page)] for _ in range(3)]
    reqs, pending, steps = [], 60, 0
    while pending or eng.has_unfinished():
        while pending and rng.random() < 0.3:
            ids = rng.choice(stems)[:rng.randrange(1, 5 * page + 1)] + [rng.randrange(V) for _ in range(rng.randrange(0, 6))]
            greedy = rng.random() < 0.6
            sp = SamplingParams(top_k=1 if greedy else rng.choice([0, 5, 50]), top_p=1.0 if greedy else rng.choice([1.0, 0.9]),
                                temperature=1.0 if greedy else rng.choice([0.7, 1.3]), max_tokens=rng.randrange(1, 30),
                                ignore_eos=rng.random() < 0.5)
            reqs.append((eng.add_request(ids, sp), ids, greedy))
            pending -= 1
        if eng.has_unfinished():
            eng.step()
            steps += 1
            eng.runner.cache.check()
        assert steps < 5000
    assert all(r.is_finished() for r, _, _ in reqs)
    assert all("no_capacity" in r.error for r, _, _ in reqs if r.error)
    cache = eng.runner.cache
    assert cache.free_pages() == 12 and not cache.requests
    st = eng.stats()["cache"]
    assert st["prefix_hit_tokens"] > 0
    if policy == "optimistic":
        assert st["preemptions"] > 0
    if dtype == "float32":
        checked = 0
        for r, ids, greedy in reqs:
            if greedy and not r.error and r.sampling_params.ignore_eos and checked < 6:
                assert r.output_token_ids == P.plain_greedy(cfg, W, ids, r.sampling_params.max_tokens)
                checked += 1
        assert checked > 0
    llm.close()


@pytest.mark.parametrize("name", ["A", "B"])
def test_decode_steps_launched_ahead_give_the_same_tokens(models, name):
    """With recorded decode steps the engine launches a step before the tokens of the one before it
    are back; the tokens fed on the device, the requests that end meanwhile (an end-of-sequence
    token, a length) and the seeded sampling give what the step-by-step loop gives, token for token."""
    from infinilm_amd import LLM, SamplingParams

    cfg, d, W = models[(name, "bfloat16")]
    V = cfg["vocab_size"]
    prompts = [random_tokens(cfg, n, 700 + n) for n in (5, 21, 12, 40, 3, 17)]
    ran = {}
    for ahead in (False, True):
        llm = LLM(d, dtype="float32", num_blocks=64, block_size=16, max_batch_size=4, enable_graph=True, look_ahead=ahead, seed=11)
        eos = llm.engine.eos_token_ids
        sps = [SamplingParams(top_k=1, max_tokens=30), SamplingParams(top_k=0, temperature=1.5, max_tokens=25),
               SamplingParams(top_k=1, max_tokens=7, ignore_eos=True), SamplingParams(top_k=20, top_p=0.9, temperature=0.8, max_tokens=40),
               SamplingParams(top_k=1, max_tokens=1), SamplingParams(top_k=0, temperature=2.0, max_tokens=33)]
        # ends that no length foretells: every request stops at tokens that random sampling meets soon
        for sp in sps[1::2]:
            sp.stop_token_ids = list(range(0, V, 7))
        outs = llm.generate(prompt_token_ids=prompts, sampling_params=sps)
        ran[ahead] = [(o.outputs[0].token_ids, o.finish_reason) for o in outs]
        st = llm.engine.stats()
        assert (st["ahead_steps"] > 0) == ahead
        assert llm.engine.runner.cache.free_pages() == 64
        llm.engine.runner.cache.check()
        llm.close()
    assert ran[True] == ran[False]
    assert any(r.value == "stop" for _, r in ran[True]), "no request ended on a stop token: the test does not test that"


@pytest.mark.parametrize("page", [16, 256])
def test_greedy_generation_bfloat16_with_graphs(models, page):
    """bfloat16 with decode steps replayed from captured graphs gives the same tokens as eager
    bfloat16 steps, and the plain implementation's up to near ties (pages of 16, and of 256, the
    entry point's default)."""
    from infinilm_amd import LLM, SamplingParams

    cfg, d, W = models[("B", "bfloat16")]
    prompts = [random_tokens(cfg, n, 500 + n) for n in (5, 33, 12, 70)]
    sp = SamplingParams(top_k=1, max_tokens=40)
    toks = {}
    for graph in (False, True):
        llm = LLM(d, dtype="bfloat16", num_blocks=40 if page == 16 else 5, block_size=page, max_batch_size=4, enable_graph=graph)
        toks[graph] = [o.outputs[0].token_ids for o in llm.generate(prompt_token_ids=prompts, sampling_params=sp)]
        if graph:
            assert llm.engine.runner._graphs, "no graph was captured"
        llm.close()
    assert toks[True] == toks[False]
    # Against the plain implementation: up to the first token that differs the sequences are equal;
    # where they part, the engine's token must be an argmax within the bfloat16 tolerance (a near tie).
    for p, t in zip(prompts, toks[True]):
        want = P.plain_greedy(cfg, W, p, 40)
        k = next((i for i in range(40) if t[i] != want[i]), None)
        if k is None:
            continue
        row = P.plain_forward(cfg, W, p + want[:k])[-1]
        gap = float(row.max() - row[t[k]])
        assert gap <= TOL["bfloat16"] * max(1.0, float(row.abs().max())), \
            f"token {k}: the engine chose {t[k]}, {gap:.3f} below the plain implementation's maximum"


def test_graph_replays_equal_eager_steps(models):
    """Every replay is checked against an eager step on the same state, with eager work and
    synchronisation between the replays."""
    from infinilm_amd.engine.loading import load_model, make_runner
    from infinilm_amd.engine.step import StepEntry

    cfg, d, W = models[("C", "bfloat16")]
    model = load_model(d, "bfloat16", "cuda:0")
    eager = make_runner(model, num_pages=32, page_size=16, max_requests=4)
    graph = make_runner(model, num_pages=32, page_size=16, max_requests=4, enable_graph=True)
    prompts = {"a": random_tokens(cfg, 37, 1), "b": random_tokens(cfg, 5, 2), "c": random_tokens(cfg, 40, 3)}
    for r in (eager, graph):
        for rid, p in prompts.items():
            r.cache.admit(rid)
            r.step([StepEntry(rid, p, [])])
    nxt = {rid: 7 + i for i, rid in enumerate(prompts)}
    for step in range(40):   # crosses page edges and the first block-table width
        entries = [StepEntry(rid, [t], [0]) for rid, t in nxt.items()]
        le = eager.step(entries).clone()
        torch.cuda.synchronize()
        lg = graph.step(entries)
        assert torch.equal(le.cpu(), lg.cpu()), f"replay {step} differs from the eager step"
        nxt = {rid: int(torch.argmax(le[i])) for i, rid in enumerate(prompts)}
    assert len(graph._graphs) >= 2   # the context outgrew the first graph's block-table width


def test_graph_steps_with_a_changing_set_of_requests(models):
    """The next decode step's metadata is prepared while the device runs the current one; it must be
    dropped when a request ends, another joins, a step of another kind comes between, or the order
    changes.  Replays must still equal eager steps bit for bit."""
    from infinilm_amd.engine.loading import load_model, make_runner
    from infinilm_amd.engine.step import StepEntry

    cfg, d, W = models[("C", "bfloat16")]
    model = load_model(d, "bfloat16", "cuda:0")
    eager = make_runner(model, num_pages=48, page_size=16, max_requests=6)
    graph = make_runner(model, num_pages=48, page_size=16, max_requests=6, enable_graph=True)
    graph.graph_after = 1

    def both(entries):
        le = eager.step(entries).clone()
        torch.cuda.synchronize()
        lg = graph.step(entries)
        assert torch.equal(le.cpu(), lg.cpu())
        return le

    def admit(rid, n, seed):
        for r in (eager, graph):
            r.cache.admit(rid)
        both([StepEntry(rid, random_tokens(cfg, n, seed), [n - 1])])

    admit("a", 20, 1), admit("b", 33, 2), admit("c", 7, 3)
    live = ["a", "b", "c"]
    nxt = {rid: 5 + i for i, rid in enumerate(live)}
    used = 0
    for step in range(30):
        if step == 6:     # a request ends
            for r in (eager, graph):
                r.cache.release("b")
            live.remove("b")
        if step == 11:    # another joins (a step of another kind in between)
            admit("d", 15, 4)
            live.append("d")
            nxt["d"] = 9
            admit("p", 10, 5)   # a prompt that goes on in portions later, beside the decoding set
        if step == 26:    # two steps of another request between two decode steps of the same set, nobody
            #               admitted or released: what was prepared for the set is two staging buffers old
            more = random_tokens(cfg, 5, 6)
            both([StepEntry("p", more[:3], [2])])
            both([StepEntry("p", more[3:], [1])])
        if step == 17:    # the same requests in another order
            live = live[::-1]
        if step == 22:    # one of them is served alone for a step
            l = both([StepEntry("a", [nxt["a"]], [0])])
            nxt["a"] = int(torch.argmax(l[0]))
        prepared = graph._prepared is not None
        l = both([StepEntry(rid, [nxt[rid]], [0]) for rid in live])
        used += prepared and graph._prepared is not None
        nxt.update({rid: int(torch.argmax(l[i])) for i, rid in enumerate(live)})
    assert used > 10      # the prepared path did run in the quiet stretches
    for r in (eager, graph):
        for rid in live + ["p"]:
            r.cache.release(rid)
        r.cache.check()
        assert r.cache.free_pages() == 48


def test_recorded_steps_filled_up_with_rows_of_no_request(models):
    """A recorded decode step has 1, 2, 4, 8, 16, 24, ... rows; fewer requests are served by it with the rest
    of the rows belonging to no request.  Requests leave one by one: every step must equal the eager
    step bit for bit, few recordings are made, and the cache's books and pages stay right."""
    from infinilm_amd.engine.loading import load_model, make_runner
    from infinilm_amd.engine.step import StepEntry

    cfg, d, W = models[("C", "bfloat16")]
    model = load_model(d, "bfloat16", "cuda:0")
    n = 11
    eager = make_runner(model, num_pages=48, page_size=16, max_requests=n)
    graph = make_runner(model, num_pages=48, page_size=16, max_requests=n, enable_graph=True)
    graph.graph_after = 1
    prompts = {f"r{i}": random_tokens(cfg, 4 + 3 * i, 80 + i) for i in range(n)}
    for r in (eager, graph):
        for rid, p in prompts.items():
            r.cache.admit(rid)
        r.step([StepEntry(rid, p, []) for rid, p in prompts.items()])
    live = list(prompts)
    nxt = {rid: 3 + i for i, rid in enumerate(live)}
    sizes = set()
    for step in range(2 * n):
        entries = [StepEntry(rid, [nxt[rid]], [0]) for rid in live]
        le = eager.step(entries).clone()
        torch.cuda.synchronize()
        lg = graph.step(entries)
        assert lg.shape == le.shape and torch.equal(le.cpu(), lg.cpu()), f"{len(live)} requests: replay differs from the eager step"
        sizes.add(len(live))
        nxt = {rid: int(torch.argmax(le[i])) for i, rid in enumerate(live)}
        if step % 2 == 1 and len(live) > 1:    # a request leaves every other step
            gone = live.pop(step % len(live))
            for r in (eager, graph):
                r.cache.release(gone)
                r.cache.check()
    assert sizes == set(range(1, n + 1))
    assert {k[0] for k in graph._graphs if k[0] != "mixed"} == {1, 2, 4, 8, 16}   # five recordings served eleven sizes
    # the rows of no request wrote to the cache's spare page only: every page a request can hold equals the eager runner's
    for e in eager.cache.k:
        assert torch.equal(eager.cache.k[e][:48], graph.cache.k[e][:48]) and torch.equal(eager.cache.v[e][:48], graph.cache.v[e][:48])
    for r in (eager, graph):
        for rid in live:
            r.cache.release(rid)
        assert r.cache.free_pages() == 48


@pytest.mark.parametrize("n,rows", [(17, 24), (33, 48), (65, 96), (129, 160), (161, 208)])
def test_recorded_steps_filled_up_in_every_range_of_the_products(models, n, rows):
    """17 requests run as 24 rows, 33 as 48, 65 as 96, 129 as 160, 161 as 208: one size in each range of rows in
    which the products take another kernel (few rows with X in registers, 17 to 64, the medium-rows product up
    to 208).  The recording, filled up with rows of no request, equals the eager step of the requests alone
    bit for bit wherever the two run the same kernels, and within rounding where the filled-up step crosses
    into the next kernel's range (the eager step of 17 rows and the recording of 24 both lie in one range)."""
    from infinilm_amd import kernels
    from infinilm_amd.engine.loading import load_model, make_runner
    from infinilm_amd.engine.step import StepEntry

    assert kernels.bound_rows(n) == rows
    cfg, d, W = models[("B", "bfloat16")]
    model = load_model(d, "bfloat16", "cuda:0")
    eager = make_runner(model, num_pages=n + 8, page_size=16, max_requests=n)
    graph = make_runner(model, num_pages=n + 8, page_size=16, max_requests=n, enable_graph=True)
    graph.graph_after = 1
    prompts = {f"r{i}": random_tokens(cfg, 1 + i % 7, 500 + i) for i in range(n)}
    for r in (eager, graph):
        for rid in prompts:
            r.cache.admit(rid)
        r.step([StepEntry(rid, p, []) for rid, p in prompts.items()])
    nxt = {rid: 3 + i % 50 for i, rid in enumerate(prompts)}
    for step in range(3):
        entries = [StepEntry(rid, [nxt[rid]], [0]) for rid in prompts]
        le = eager.step(entries).clone()
        torch.cuda.synchronize()
        lg = graph.step(entries)
        assert lg.shape == le.shape
        assert torch.equal(le.cpu(), lg.cpu()), f"{n} requests as {rows} rows, step {step}: replay differs from the eager step"
        nxt = {rid: int(torch.argmax(le[i])) for i, rid in enumerate(prompts)}
    assert {k[0] for k in graph._graphs if k[0] != "mixed"} == {rows}


def test_decode_steps_recorded_before_the_first_request(models):
    """`record_graphs_at_start`: every decode step size that the batch limit, the model's positions and the pool
    allow is recorded from rows of no request when the engine is built; the requests that come later find
    their recordings (none is added), replay them with their own rows first, and generate what the plain
    implementation generates.  Nothing of the cache is held or written outside the page for such rows."""
    from infinilm_amd import LLM, SamplingParams

    cfg, d, W = models[("A", "float32")]
    llm = LLM(d, dtype="float32", num_blocks=16, block_size=16, max_batch_size=5, enable_graph=True,
              record_graphs_at_start=True, enable_prefix_caching=False)
    runner = llm.engine.runner
    # rows 1, 2, 4, 8 (five requests run as eight rows); widths 4, 6, 8 pages (128 positions: 8 pages of 16)
    assert set(runner._graphs) == {(r, w) for r in (1, 2, 4, 8) for w in (4, 6, 8)}
    assert llm.graphs_recorded_at_start == 12
    assert runner.cache.free_pages() == 16 and not runner.cache.requests
    prompts = [random_tokens(cfg, n, 300 + n) for n in (3, 40, 17, 9, 1)]
    outs = llm.generate(prompt_token_ids=prompts, sampling_params=SamplingParams(top_k=1, max_tokens=20, ignore_eos=True))
    assert len([k for k in runner._graphs if k[0] != "mixed"]) == 12   # no decode step had to record
    assert runner.cache.free_pages() == 16
    for p, o in zip(prompts, outs):
        assert o.outputs[0].token_ids == P.plain_greedy(cfg, W, p, 20)
    llm.close()


def test_graph_with_many_requests_replays_like_eager(models):
    """More than 16 decoded tokens a step: the projections go to the vendor library inside the
    captured graph; replays must still equal eager steps, several times over."""
    from infinilm_amd.engine.loading import load_model, make_runner
    from infinilm_amd.engine.step import StepEntry

    cfg, d, W = models[("A", "bfloat16")]
    model = load_model(d, "bfloat16", "cuda:0")
    n = 20
    eager = make_runner(model, num_pages=64, page_size=16, max_requests=n)
    graph = make_runner(model, num_pages=64, page_size=16, max_requests=n, enable_graph=True)
    prompts = {f"r{i}": random_tokens(cfg, 3 + i, 50 + i) for i in range(n)}
    for r in (eager, graph):
        for rid, p in prompts.items():
            r.cache.admit(rid)
        r.step([StepEntry(rid, p, []) for rid, p in prompts.items()])
    nxt = {rid: 11 + i for i, rid in enumerate(prompts)}
    for step in range(12):
        entries = [StepEntry(rid, [t], [0]) for rid, t in nxt.items()]
        le = eager.step(entries).clone()
        torch.cuda.synchronize()
        lg = graph.step(entries)
        assert rel_err(lg, le) < 1e-6, f"replay {step} differs from the eager step"
        nxt = {rid: int(torch.argmax(le[i])) for i, rid in enumerate(prompts)}


def test_seeded_sampling_is_reproducible_and_independent_of_the_batch(models):
    from infinilm_amd import LLM, SamplingParams

    cfg, d, W = models[("B", "float32")]
    prompts = [random_tokens(cfg, n, 900 + n) for n in (3, 50, 120, 8)]
    sp = SamplingParams(temperature=0.8, top_k=0, top_p=0.9, max_tokens=12)
    runs = []
    for batch, budget, chunk in ((4, 256, None), (2, 17, 17), (1, 256, None)):
        llm = LLM(d, dtype="float32", num_blocks=64, block_size=8, max_batch_size=batch, max_num_batched_tokens=budget,
                  chunk_size=chunk, seed=123)
        runs.append([o.outputs[0].token_ids for o in llm.generate(prompt_token_ids=prompts, sampling_params=sp)])
        llm.close()
    assert runs[0] == runs[1] == runs[2]
    llm = LLM(d, dtype="float32", num_blocks=64, block_size=8, max_batch_size=4, seed=124)
    other = [o.outputs[0].token_ids for o in llm.generate(prompt_token_ids=prompts, sampling_params=sp)]
    llm.close()
    assert other != runs[0]
    greedy_like = [P.plain_greedy(cfg, W, p, 12) for p in prompts]
    assert runs[0] != greedy_like   # it does sample


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(models, dtype):
    """A short prompt, then every further token one by one to the end of the position table."""
    cfg, d, W = models[("C", dtype)]
    toks = random_tokens(cfg, 400, 77)
    drv = Driver(d, dtype, num_pages=16, page_size=32)
    drv.step([("r", toks[:3])])
    for i in range(3, 400):
        drv.step([("r", toks[i:i + 1])])
    err = rel_err(drv.request_logits("r", 400), P.plain_forward(cfg, W, toks))
    assert err < TOL[dtype], f"error {err:.3e}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens_of_a_sequence(models, dtype):
    """Prompts of one and two tokens, alone and batched, and a sequence fed from its very first
    token one token a step."""
    cfg, d, W = models[("B", dtype)]
    drv = Driver(d, dtype, num_pages=8, page_size=16)
    one, two, seq = [5], [9, 300], random_tokens(cfg, 6, 3)
    drv.step([("one", one), ("two", two)], end=["one", "two"])
    for i, t in enumerate(seq):
        drv.step([("seq", [t])])
    for rid, t in (("one", one), ("two", two), ("seq", seq)):
        err = rel_err(drv.request_logits(rid, len(t)), P.plain_forward(cfg, W, t))
        assert err < TOL[dtype], f"{rid}: error {err:.3e}"


def test_preemption_recomputes_and_gives_the_same_tokens(models):
    from infinilm_amd import LLM, SamplingParams

    cfg, d, W = models[("A", "float32")]
    prompts = [random_tokens(cfg, n, 40 + n) for n in (20, 22, 18)]
    sp = SamplingParams(top_k=1, max_tokens=30)
    llm = LLM(d, dtype="float32", num_blocks=14, block_size=8, max_batch_size=3, admission="optimistic")
    outs = llm.generate(prompt_token_ids=prompts, sampling_params=sp)
    assert llm.engine.scheduler.num_preemptions > 0, "the pool was meant to run out"
    for p, o in zip(prompts, outs):
        assert o.outputs[0].token_ids == P.plain_greedy(cfg, W, p, 30)
    assert llm.engine.runner.cache.free_pages() == 14
    llm.close()
    # the reference's admission never preempts and gives the same tokens
    llm = LLM(d, dtype="float32", num_blocks=14, block_size=8, max_batch_size=3, admission="reserve_full")
    outs2 = llm.generate(prompt_token_ids=prompts, sampling_params=sp)
    assert llm.engine.scheduler.num_preemptions == 0
    assert [o.outputs[0].token_ids for o in outs2] == [o.outputs[0].token_ids for o in outs]
    llm.close()


def test_step_errors_are_loud(models):
    from infinilm_amd.engine.loading import load_model, make_runner
    from infinilm_amd.engine.step import StepEntry
    from infinilm_amd.cache import OutOfPages

    cfg, d, W = models[("A", "float32")]
    model = load_model(d, "float32", "cuda:0")
    r = make_runner(model, num_pages=2, page_size=8, max_requests=2)
    r.cache.admit("a")
    with pytest.raises(ValueError, match="outside the vocabulary"):
        r.step([StepEntry("a", [cfg["vocab_size"]], [0])])
    with pytest.raises(ValueError, match="outside its"):
        r.step([StepEntry("a", [1, 2], [2])])
    with pytest.raises(OutOfPages):
        r.step([StepEntry("a", list(range(17)), [])])
    with pytest.raises(ValueError, match="exceed the model's"):
        r.step([StepEntry("a", [1] * (cfg["max_position_embeddings"] + 1), [])])
    with pytest.raises(ValueError, match="twice"):
        r.step([StepEntry("a", [1], [0]), StepEntry("a", [2], [0])])
    assert r.cache.length("a") == 0
    with pytest.raises(RuntimeError, match="GPU only"):
        from infinilm_amd.engine.loading import require_gpu
        require_gpu("cpu")


def test_trace_run_program(models, tmp_path):
    """bin/trace_run as a user runs it: steps on stdin, logits files out, `done <step>` lines."""
    cfg, d, W = models[("B", "float32")]
    a, b = random_tokens(cfg, 70, 1), random_tokens(cfg, 30, 2)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:40], "want": [0, 39]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[40:42], "want": []}, {"id": "b", "tokens": b[:29], "want": [28]}], "end": []},
        {"step": 2, "entries": [{"id": "b", "tokens": b[29:], "want": [0]}], "end": ["b"]},
        {"step": 3, "entries": [{"id": "a", "tokens": a[42:], "want": list(range(28))}], "end": ["a"]},
        {"step": 4, "entries": [{"id": "c", "tokens": b, "want": [29]}], "end": ["c"]},
    ]
    out = tmp_path / "out"
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", d, "--dtype", "float32",
                           "--out", str(out), "--max-tokens", "192"],
                          input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(5)]
    import numpy as np
    V = cfg["vocab_size"]
    la, lb = P.plain_forward(cfg, W, a), P.plain_forward(cfg, W, b)
    read = lambda i: torch.from_numpy(np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, V))
    assert not (out / "1.f32").exists() or read(1).shape[0] == 1
    assert rel_err(read(0), la[[0, 39]]) < TOL["float32"]
    assert rel_err(read(1), lb[[28]]) < TOL["float32"]
    assert rel_err(read(2), lb[[29]]) < TOL["float32"]
    assert rel_err(read(3), la[42:]) < TOL["float32"]
    assert rel_err(read(4), lb[[29]]) < TOL["float32"]


def test_command_line(models):
    """examples/test_infer.py with the reference's option names, token ids in place of a tokenizer."""
    cfg, d, W = models[("A", "float32")]
    prompt = random_tokens(cfg, 9, 5)
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "examples", "test_infer.py"), "--model", d, "--dtype", "float32",
                           "--batch-size", "2", "--prompt-ids", ",".join(map(str, prompt)), "--max-new-tokens", "7",
                           "--top-k", "1", "--num-blocks", "16", "--block-size", "16", "--enable-paged-attn"],
                          capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    want = str(P.plain_greedy(cfg, W, prompt, 7))
    assert proc.stdout.count(want) == 2, proc.stdout[-1500:]
    assert "total_time:" in proc.stdout


def test_kernel_timers_and_engine_counters(models):
    """The per-entry-point timers behind a flag, and the loop's counters."""
    from infinilm_amd import LLM, SamplingParams, kernels

    cfg, d, W = models[("A", "bfloat16")]
    llm = LLM(d, dtype="bfloat16", num_blocks=16, block_size=16, max_batch_size=2)
    kernels.enable_timing(True)
    try:
        prompts = [random_tokens(cfg, 9, 1), random_tokens(cfg, 20, 2)]
        llm.generate(prompt_token_ids=prompts, sampling_params=SamplingParams(max_tokens=5, top_k=1, ignore_eos=True))
        rep = kernels.timing_report()
    finally:
        kernels.enable_timing(False)
    L = cfg["num_hidden_layers"]
    assert rep["ilm_embed"]["calls"] == 5                       # one step of prompts, four of decoded tokens
    assert rep["ilm_rope_kvwrite"]["calls"] == 5 * L
    # the step of prompts runs both norms of every layer and the final one; in the four steps of decoded tokens the
    # second norm of a layer is folded into the projections around it
    assert rep["ilm_add_rmsnorm"]["calls"] == (2 * L + 1) + 4 * (L + 1)
    assert rep["ilm_gemm_tail"]["calls"] == 4 * L
    assert all(v["total_ms"] > 0 for v in rep.values())
    assert kernels.timing_report() == {}                        # switched off again
    st = llm.engine.stats()
    assert st["steps"] == 5 and st["prompt_tokens"] == 29 and st["generated_tokens"] == 10
    assert st["cache"]["running"] == 0 and st["cache"]["groups"][0]["free"] == 16
    llm.close()


class _ToyTokenizer:
    """Words 'w<id>' separated by blanks: enough of a tokenizer's face for the entry point."""
    chat_template = "toy"

    def encode(self, text, add_special_tokens=False):
        return [int(w[1:]) for w in text.split()]

    def decode(self, ids, skip_special_tokens=True):
        return " ".join(f"w{i}" for i in ids)

    def apply_chat_template(self, messages, tokenize=False, add_generation_prompt=True):
        return " ".join(m["content"] for m in messages) + (" w1" if add_generation_prompt else "")


def test_text_prompts_chat_and_stops(models):
    """Text in and out through a tokenizer object; chat; a stop string cuts the text and ends the
    request; a stop token id ends it; ignore_eos runs on."""
    from infinilm_amd import LLM, SamplingParams
    from infinilm_amd.engine.request import FinishReason

    cfg, d, W = models[("A", "float32")]
    llm = LLM(d, dtype="float32", num_blocks=32, block_size=16, max_batch_size=4, tokenizer=_ToyTokenizer())
    prompt = random_tokens(cfg, 6, 77)
    want = P.plain_greedy(cfg, W, prompt, 10)
    text = " ".join(f"w{i}" for i in prompt)
    sp = SamplingParams(top_k=1, max_tokens=10, ignore_eos=True)
    out = llm.generate([text], sampling_params=sp)[0]
    assert out.outputs[0].token_ids == want and out.outputs[0].text == " ".join(f"w{i}" for i in want)
    assert out.prompt == text and out.finish_reason == FinishReason.LENGTH
    # chat: the template's text is encoded; here it appends the token 1 to the user's words
    chat = llm.chat([{"role": "user", "content": text}], sampling_params=sp)[0]
    assert chat.outputs[0].token_ids == P.plain_greedy(cfg, W, prompt + [1], 10)
    # a stop string: the text ends before it, the request is finished with that reason
    stop = f"w{want[3]} w{want[4]}"
    cut = llm.generate([text], sampling_params=SamplingParams(top_k=1, max_tokens=10, stop=[stop]))[0]
    assert cut.finish_reason == FinishReason.STOP_STRING
    assert cut.outputs[0].text == " ".join(f"w{i}" for i in want[:3]) + " " and len(cut.outputs[0].token_ids) == 5
    # a stop token id
    st = llm.generate([text], sampling_params=SamplingParams(top_k=1, max_tokens=10, stop_token_ids=[want[2]]))[0]
    first = want.index(want[2])
    assert st.finish_reason == FinishReason.STOP and st.outputs[0].token_ids == want[:first + 1]
    assert llm.engine.stats()["cache"]["running"] == 0 and llm.engine.stats()["cache"]["groups"][0]["free"] == 32
    llm.close()


def test_cache_sized_from_free_memory(models):
    """`num_pages=None`: the pool takes a fraction of what is free, counted in pages of every layer."""
    from infinilm_amd.engine.loading import fragment_copy_bytes, load_model, pages_that_fit

    cfg, d, W = models[("B", "bfloat16")]
    model = load_model(d, "bfloat16", "cuda:0")
    free, _ = torch.cuda.mem_get_info()
    per_page = cfg["num_hidden_layers"] * 2 * cfg["num_key_value_heads"] * P.plain_head_dim(cfg) * 64 * 2
    n = pages_that_fit(model, 64, memory_fraction=0.5, reserve_bytes=1 << 30)
    # the projections' copies in fragment order, made at their first use with many rows, have their room kept
    copies = fragment_copy_bytes(model)
    H, I = cfg["hidden_size"], cfg["intermediate_size"]
    qkv_rows = (cfg["num_attention_heads"] + 2 * cfg["num_key_value_heads"]) * P.plain_head_dim(cfg)
    o_in = cfg["num_attention_heads"] * P.plain_head_dim(cfg)
    assert copies == cfg["num_hidden_layers"] * 2 * (qkv_rows * H + H * o_in + 2 * I * H + H * I)
    assert abs(n - (int(free * 0.5) - (1 << 30) - copies) // per_page) <= max(2, n // 100)   # free memory moves a little
    with pytest.raises(RuntimeError, match="no room for a cache"):
        pages_that_fit(model, 64, memory_fraction=0.5, reserve_bytes=1 << 50)


def test_benchmark_example(models):
    """examples/bench.py: the case grid in order of cache size, one JSON line a case."""
    import json
    cfg, d, W = models[("B", "bfloat16")]
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "examples", "bench.py"), "--model", d, "--batch-size", "3,1",
                           "--input-len", "40,7", "--output-len", "5", "--block-size", "16", "--enable-graph", "--warmup"],
                          capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    rows = [json.loads(l) for l in proc.stdout.splitlines() if l.startswith("{")]
    assert [(r["batch_size"], r["input_len"]) for r in rows] == [(1, 7), (3, 7), (1, 40), (3, 40)]
    assert all("error" not in r and r["decode_tok_s"] > 0 and r["ttft_ms"] > 0 for r in rows)


def _real_shape(name):
    base = {"architectures": ["MiniCPMForCausalLM"], "model_type": "minicpm", "num_hidden_layers": 2, "scale_emb": 12,
            "scale_depth": 1.4, "dim_model_base": 256, "rope_theta": 10000.0, "max_position_embeddings": 4096}
    if name == "8b":      # 32 heads in 2 groups of 16, head 128, untied head
        return dict(base, hidden_size=4096, num_attention_heads=32, num_key_value_heads=2, head_dim=128,
                    intermediate_size=16384, vocab_size=73448, rms_norm_eps=1e-6,
                    rope_scaling={"type": "longrope", "short_factor": [1.0 + i / 64 for i in range(64)],
                                  "long_factor": [2.0] * 64, "original_max_position_embeddings": 4096})
    if name == "0.5b":    # head 64, 16 heads in 2 groups of 8, tied head
        return dict(base, hidden_size=1024, num_attention_heads=16, num_key_value_heads=2, head_dim=64,
                    intermediate_size=4096, vocab_size=73448, rms_norm_eps=1e-6, tie_word_embeddings=True,
                    rope_scaling={"type": "longrope", "short_factor": [1.0 + i / 32 for i in range(32)],
                                  "long_factor": [3.0] * 32, "original_max_position_embeddings": 4096})
    if name == "2b":      # every head its own keys (36 of 64), widths that are no power of two, odd vocabulary
        return dict(base, hidden_size=2304, num_attention_heads=36, num_key_value_heads=36, head_dim=64,
                    intermediate_size=5760, vocab_size=122753, rms_norm_eps=1e-5, tie_word_embeddings=True)
    raise KeyError(name)


@pytest.mark.parametrize("shape", ["8b", "0.5b", "2b"])
def test_layers_of_real_size_against_the_plain_implementation(shape):
    """Two layers of a real shape (the 8B, the 0.5B and the 2B-family sizes): the float32 path and the
    bfloat16 kernels that serving uses at that size (resident and K-split few-rows products, tile
    and chunked attention over pages of 64, graph replay), each against the plain implementation in
    float64 on the same weights (the plain formulas run on the GPU's tensors here: on the CPU this
    size takes minutes): a 600-token prompt in portions, then decoded tokens."""
    from infinilm_amd.engine.loading import build_model, make_runner
    from infinilm_amd.engine.step import StepEntry
    from infinilm_amd.weights import fill_random_

    cfg = _real_shape(shape)
    tied = bool(cfg.get("tie_word_embeddings"))
    g = torch.Generator().manual_seed(5)
    prompt = torch.randint(0, cfg["vocab_size"], (600,), generator=g).tolist()
    logits, fed, oracle = {}, [], None
    for dtype, graph in (("float32", False), ("bfloat16", True)):
        model = build_model(cfg, dtype, "cuda:0")
        fill_random_(model, seed=1, std=0.02, norm_init="one_plus", tie=tied)
        if dtype == "float32":   # the same values the bfloat16 model holds
            for p in model.named_parameters().values():
                p.tensor.copy_(p.tensor.to(torch.bfloat16).to(torch.float32))
        r = make_runner(model, num_pages=16, page_size=64, max_requests=2, enable_graph=graph)
        r.cache.admit("a")
        rows = [r.step([StepEntry("a", prompt[:300], [0, 299])]).cpu().clone()]
        rows.append(r.step([StepEntry("a", prompt[300:599], [298])]).cpu().clone())
        tok = prompt[599]
        for i in range(6):
            l = r.step([StepEntry("a", [tok], [0])]).cpu().clone()
            rows.append(l)
            if dtype == "float32":
                fed.append(int(torch.argmax(l[0])))
            tok = fed[i]   # both runs are fed the float32 run's greedy tokens
        logits[dtype] = torch.cat(rows)
        if dtype == "float32":
            W = {n: p.tensor for n, p in model.named_parameters().items() if not (tied and n == "lm_head.weight")}
            full = P.plain_forward(cfg, W, prompt[:600] + fed[:5])
            oracle = full[[0, 299, 598] + list(range(599, 605))].cpu()
            del W, full
        del r, model
        torch.cuda.empty_cache()
    err32 = rel_err(logits["float32"], oracle)
    err16 = rel_err(logits["bfloat16"], oracle)
    print(f"[err] real size {shape}: float32 {err32:.3e}, bfloat16 {err16:.3e}")
    assert err32 < 1e-4, f"float32 against the plain implementation at real size: {err32:.3e}"
    assert err16 < TOL["bfloat16"], f"bfloat16 against the plain implementation at real size: {err16:.3e}"


def _both_dtypes(cfg, num_pages, _unused=None):
    """Builds the configuration's model with the same (bfloat16-representable) random weights in float32 (eager
    steps) and in bfloat16 (decode steps recorded as graphs) and yields (dtype, runner, weights for the plain implementation) for each."""
    from infinilm_amd.engine.loading import build_model, make_runner
    from infinilm_amd.weights import fill_random_

    tied = bool(cfg.get("tie_word_embeddings"))
    for dtype, graph in (("float32", False), ("bfloat16", True)):
        model = build_model(cfg, dtype, "cuda:0")
        fill_random_(model, seed=1, std=0.02, norm_init="one_plus", tie=tied)
        if dtype == "float32":   # the same values the bfloat16 model holds
            for p in model.named_parameters().values():
                p.tensor.copy_(p.tensor.to(torch.bfloat16).to(torch.float32))
        r = make_runner(model, num_pages=num_pages, page_size=64, max_requests=4, enable_graph=graph)
        W = {n: p.tensor for n, p in model.named_parameters().items() if not (tied and n == "lm_head.weight")}
        yield dtype, r, W
        del r, model, W
        torch.cuda.empty_cache()


@pytest.mark.parametrize("requests", [20, 40, 100, 150])
def test_decode_steps_of_many_requests_at_the_8b_shape(requests):
    """Two layers of the 8B shape in bfloat16 with 20 to 150 live requests of different lengths: their prompts in one
    step, then decode steps that replay a recording of 24, 48, 128 or 160 rows (the products that keep chunks of X in
    LDS with 2, 3, 8 and 10 groups of rows, the fragment-order q/k/v product up to 64 rows, the add+RMSNorm over many
    float parts, attention chunks chosen by rounds of workgroups).  The decoded tokens' logits of a sample of the
    requests against the plain implementation in float64 on the same weights."""
    from infinilm_amd.engine.loading import build_model, make_runner
    from infinilm_amd.engine.step import StepEntry
    from infinilm_amd.weights import fill_random_

    cfg = _real_shape("8b")
    model = build_model(cfg, "bfloat16", "cuda:0")
    fill_random_(model, seed=1, std=0.02, norm_init="one_plus")
    r = make_runner(model, num_pages=2 * requests + 4, page_size=64, max_requests=requests, enable_graph=True)
    r.graph_after = 1
    g = torch.Generator().manual_seed(11 + requests)
    lens = torch.randint(20, 90, (requests,), generator=g).tolist()
    toks = [torch.randint(0, cfg["vocab_size"], (n + 3,), generator=g).tolist() for n in lens]
    ids = [f"q{i}" for i in range(requests)]
    for rid in ids:
        r.cache.admit(rid)
    r.step([StepEntry(rid, t[:n], []) for rid, t, n in zip(ids, toks, lens)])
    got = []
    for k in range(3):
        got.append(r.step([StepEntry(rid, [t[n + k]], [0]) for rid, t, n in zip(ids, toks, lens)]).float().cpu().clone())
    assert any(key[0] != "mixed" and key[0] == kernels_bound_rows(requests) for key in r._graphs), list(r._graphs)
    W = {n: p.tensor.to(torch.float32) for n, p in model.named_parameters().items()}
    sample = sorted(set([0, 1, requests // 2, requests - 2, requests - 1] + [int(i) for i in torch.randint(0, requests, (3,), generator=g)]))
    worst = 0.0
    for i in sample:
        full = P.plain_forward(cfg, W, toks[i])
        for k in range(3):
            worst = max(worst, rel_err(got[k][i][None], full[lens[i] + k][None].cpu()))
    print(f"[err] {requests} requests at the 8B shape: {worst:.3e}")
    assert worst < TOL["bfloat16"], f"{requests} requests: {worst:.3e}"
    for rid in ids:
        r.cache.release(rid)
    r.cache.check()


def kernels_bound_rows(n):
    from infinilm_amd import kernels
    return kernels.bound_rows(n)


def test_mixed_steps_at_the_8b_head_shape_with_recorded_steps_and_pages_used_again():
    """Two layers of the 8B shape (heads of 128 in groups of 16, pages of 64): five requests over a pool of 13
    pages, up to four live.  One step holds a portion with history, two decoded tokens and a fresh prompt
    (the tile attention's direct loads beside the chunked kernel, the library's products); one holds
    the same mix in 12 rows (the few-rows products with rotation, cache write, residual sum and half a norm in
    their epilogues); the steps of four decoded tokens replay a recording in bfloat16; the last request gets
    pages that two finished ones gave back.  Every logit of every request against the plain implementation
    in float64, in 32-bit and in bfloat16."""
    from infinilm_amd.engine.step import StepEntry

    cfg = _real_shape("8b")
    g = torch.Generator().manual_seed(11)
    lens = {"a": 340, "b": 140, "c": 70, "d": 150, "e": 100}
    toks = {r: torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist() for r, n in lens.items()}
    steps = [([("b", 130), ("c", 60)], []),
             ([("a", 200), ("b", 1), ("c", 1)], []),
             ([("a", 90), ("b", 1), ("c", 1), ("d", 140)], [])]        # a portion with history, two decoded tokens, a fresh prompt
    steps += [([("a", 1), ("b", 1), ("c", 1), ("d", 1)], [])] * 7
    steps += [([("a", 1), ("b", 1), ("c", 1), ("d", 1)], ["b", "c"])]
    steps += [([("a", 5), ("d", 1), ("e", 6)], []),                     # the same mix in 12 rows
              ([("a", 1), ("d", 1), ("e", 60)], ["d"]),
              ([("a", 36), ("e", 1)], ["a"]),
              ([("e", 2)], [])]
    steps += [([("e", 1)], [])] * 31
    oracle = None
    for dtype, r, W in _both_dtypes(cfg, 13, None):
        if oracle is None:
            oracle = {q: P.plain_forward(cfg, W, t).cpu() for q, t in toks.items()}
        fed = {q: 0 for q in toks}
        got = {q: [] for q in toks}
        old_pages, replays = set(), 0
        for entries, end in steps:
            es = []
            for q, n in entries:
                if not r.cache.has(q):
                    r.cache.admit(q)
                es.append(StepEntry(q, toks[q][fed[q]:fed[q] + n], list(range(n))))
            before = len(r._graphs)
            singles = all(n == 1 for _, n in entries)
            out = r.step(es).cpu().clone()
            replays += int(singles and r.enable_graph and len(r._graphs) == before and bool(r._graphs))
            row = 0
            for q, n in entries:
                got[q].append(out[row:row + n])
                row += n
                fed[q] += n
            for q in end:
                old_pages |= set(r.cache.table(q, 0))
                r.cache.release(q)
            r.cache.check()
            if entries[-1] == ("e", 6):
                assert set(r.cache.table("e", 0)) <= old_pages, "the last request's pages were not used before"
        assert fed == lens
        r.cache.release("e")
        assert r.cache.free_pages() == 13
        if r.enable_graph:
            assert replays >= 6, "the decode steps did not replay a recording"
        tol = 1e-4 if dtype == "float32" else TOL["bfloat16"]
        for q in toks:
            err = rel_err(torch.cat(got[q]), oracle[q])
            print(f"[err] mixed steps at the 8B head shape, {dtype}, request {q}: {err:.3e}")
            assert err < tol, f"{dtype}, request {q}: {err:.3e}"


def test_a_context_beyond_9000_tokens_at_the_benchmark_configuration():
    """Two layers of the configuration the benchmark times (examples/shapes.py: 32,768 positions, LongRoPE with
    64 factors): a prompt of 9,100 tokens in portions of 2,048, then decoded tokens, against the plain
    implementation in float64 on the same weights: positions far beyond a page table's first entries, the
    long tiles of the portion attention and 142 pages under one decoded token."""
    from infinilm_amd.engine.step import StepEntry

    sys.path.insert(0, os.path.join(ROOT, "examples"))
    from shapes import shape_config

    cfg = shape_config("8b", 2)
    N = 9100
    g = torch.Generator().manual_seed(5)
    prompt = torch.randint(0, cfg["vocab_size"], (N,), generator=g).tolist()
    want_rows, i = [], 0
    while i < N - 1:
        k = min(2048, N - 1 - i)
        want_rows += [i, i + k // 2, i + k - 1]
        i += k
    want_rows += list(range(N - 1, N + 4))
    fed, oracle = [], None
    for dtype, r, W in _both_dtypes(cfg, N // 64 + 4, None):
        r.cache.admit("a")
        rows, i = [], 0
        while i < N - 1:
            k = min(2048, N - 1 - i)
            rows.append(r.step([StepEntry("a", prompt[i:i + k], [0, k // 2, k - 1])]).cpu().clone())
            i += k
        tok = prompt[N - 1]
        for s in range(5):
            l = r.step([StepEntry("a", [tok], [0])]).cpu().clone()
            rows.append(l)
            if dtype == "float32":
                fed.append(int(torch.argmax(l[0])))
            tok = fed[s]   # both runs are fed the float32 run's greedy tokens
        logits = torch.cat(rows)
        if oracle is None:
            oracle = P.plain_forward(cfg, W, prompt + fed[:4])[want_rows].cpu()
        err = rel_err(logits, oracle)
        print(f"[err] context of {N} tokens, {dtype}: {err:.3e}")
        assert err < (1e-4 if dtype == "float32" else TOL["bfloat16"]), f"{dtype}: {err:.3e}"


@pytest.mark.parametrize("name,dtype", [("B", "float32"), ("E", "float32"), ("B", "bfloat16"), ("A", "bfloat16")])
def test_recorded_steps_with_portions_of_prompts(models_de, name, dtype):
    """Steps that hold portions of prompts beside decoded tokens are recorded by their bounded shape (tokens,
    requests, wanted rows, block-table width, each rounded up) and replayed with the lists filled up by entries that
    do nothing.  The same steps through an eager runner: in 32-bit the same bits
    (every sum has one order whatever the number of rows), in bfloat16 within the tolerance of the plain
    implementation's; few recordings serve many different steps, and the cache's books and pages agree."""
    from infinilm_amd.engine.loading import load_model, make_runner
    from infinilm_amd.engine.step import StepEntry
    import random

    cfg, d, W = models_de[(name, dtype)]
    model = load_model(d, dtype, "cuda:0")
    eager = make_runner(model, num_pages=32, page_size=64, max_requests=8)
    graph = make_runner(model, num_pages=32, page_size=64, max_requests=8, enable_graph=True)
    graph.graph_after = 1
    graph.graph_mixed_pad_share = 0   # these small steps are recorded however many rows fill their shapes up
    rng = random.Random(3)
    n_max = min(cfg["max_position_embeddings"], 200)
    toks = {f"r{i}": random_tokens(cfg, rng.randint(30, n_max), 700 + i) for i in range(7)}
    fed = {r: 0 for r in toks}
    logits = {r: [] for r in toks}
    waiting, live, replays, steps = list(toks), [], 0, 0
    while waiting or live:
        while waiting and len(live) < 4:
            live.append(waiting.pop(0))
        entries = []
        for r in live:
            left = len(toks[r]) - fed[r]
            n = 1 if left <= 6 else min(left - 6, rng.choice([17, 17, 17, 9, 30]))   # portions first, the last six tokens one by one
            entries.append((r, toks[r][fed[r]:fed[r] + n]))
        if all(len(t) == 1 for _, t in entries) and rng.random() < 0.5 and waiting:
            continue
        es = [StepEntry(r, t, [len(t) - 1]) for r, t in entries]
        for run in (eager, graph):
            for r, _ in entries:
                if not run.cache.has(r):
                    run.cache.admit(r)
        before = len(graph._graphs)
        le = eager.step(es).clone()
        torch.cuda.synchronize()
        lg = graph.step(es).clone()
        replays += int(len(graph._graphs) == before and any(len(t) > 1 for _, t in entries))
        steps += int(any(len(t) > 1 for _, t in entries))
        assert lg.shape == le.shape
        if dtype == "float32":
            assert torch.equal(le.cpu(), lg.cpu()), f"step {steps}: the recorded step differs from the eager one"
        for i, (r, t) in enumerate(entries):
            logits[r].append((fed[r] + len(t) - 1, lg[i].cpu()))
            fed[r] += len(t)
            if fed[r] == len(toks[r]):
                live.remove(r)
                for run in (eager, graph):
                    run.cache.release(r)
        for run in (eager, graph):
            run.cache.check()
    mixed = [k for k in graph._graphs if k[0] == "mixed"]
    assert steps >= 12 and replays >= steps - len(mixed) and replays >= 4, (steps, replays, len(mixed))   # shapes came again and were replayed
    for r, t in toks.items():
        want = P.plain_forward(cfg, W, t)
        for pos, row in logits[r]:
            assert rel_err(row[None], want[pos][None]) < TOL[dtype] * (1 if dtype == "bfloat16" else 5), f"{r} position {pos}"
    assert eager.cache.free_pages() == graph.cache.free_pages() == 32
    # by default a step whose shape would be filled up by more than an eighth runs eagerly: 36 tokens would run as 48 rows
    graph.graph_mixed_pad_share = 8
    n_before = len(graph._graphs)
    late = random_tokens(cfg, 66, 999)
    assert cfg["max_position_embeddings"] >= 66
    for run in (eager, graph):
        run.cache.admit("late")
    es = [StepEntry("late", late[:36], [35])]
    assert torch.equal(eager.step(es), graph.step(es)) or dtype == "bfloat16"
    assert len(graph._graphs) == n_before
    es = [StepEntry("late", late[36:], [29])]      # 30 tokens run as 32 rows
    graph.step(es)
    assert len(graph._graphs) == n_before + 1


@pytest.fixture(scope="module")
def models_de(tmp_path_factory):
    out = {}
    for name, dtype in (("B", "float32"), ("E", "float32"), ("B", "bfloat16"), ("A", "bfloat16")):
        cfg = CONFIGS[name]()
        d = str(tmp_path_factory.mktemp(f"mix_{name}_{dtype}"))
        out[(name, dtype)] = (cfg, d, make_model_dir(d, cfg, seed=60 + ord(name), store=dtype))
    return out
