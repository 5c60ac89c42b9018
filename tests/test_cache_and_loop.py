"""The cache's bookkeeping and the generation loop's decisions.  No GPU: the cache is built without a device and
the loop runs on stand-ins for the kernels."""
import random

import pytest
import torch

import emulated_kernels
from tiny_configs import TINY, TINY_A, TINY_B
from turboquant_cpp_amd.cache import CacheError, CacheFull, PagedCache, PagePool
from turboquant_cpp_amd.engine.generate import (GenerationOptions, LoopDetector, SequenceTrack, generate,
                                                plan_batches)
from turboquant_cpp_amd.engine.model import load_model
from turboquant_cpp_amd.engine.step import Engine, StepError
from turboquant_cpp_amd.parts import CacheNeed, StateNeed
from turboquant_cpp_amd.sampling.rng import XorShift64Star, stream_seed


# ------------------------------------------------------------------------------------------------ pages and slots
def test_page_pool_never_loses_or_doubles_a_page():
    pool = PagePool(10)
    a, b = pool.take(4), pool.take(6)
    assert sorted(a + b) == list(range(10)) and pool.n_free == 0
    with pytest.raises(CacheFull):
        pool.take(1)
    pool.give_back(a)
    with pytest.raises(CacheError, match="not held"):
        pool.give_back([a[0]])                       # freed twice
    with pytest.raises(CacheError, match="not held"):
        pool.give_back([99])
    assert sorted(pool.take(4)) == sorted(a)


def two_group_cache(max_tokens=64 * 8, **kw):
    needs = [(CacheNeed(2, 16, None), None, None), (CacheNeed(2, 16, 100), None, None), (CacheNeed(2, 16, 100), None, None),
             (CacheNeed(2, 16, None), StateNeed((3,)), 0)]
    return PagedCache(needs, max_tokens, torch.float32, None, page_size=64, **kw)


def held(cache):
    """Every page of every group is either free or in exactly one live slot's table."""
    for g in cache.groups:
        in_tables = g.host_table[g.host_table >= 0].tolist()
        assert len(in_tables) == len(set(in_tables)), "a page is held twice"
        assert len(in_tables) + g.pool.n_free == g.pool.n_pages, "a page is lost"
        dead = [s.index for s in cache.slots if not s.live]
        assert (g.host_table[dead] < 0).all(), "a closed slot still holds pages"


def test_groups_by_need_and_views():
    c = two_group_cache()
    assert len(c.groups) == 2
    full, win = c.groups
    assert full.entries == [0] and win.entries == [1, 2] and win.page_stride == 2 * 2 * 64 * 16
    assert c.kv(2).layer_offset == 2 * 64 * 16 and c.kv(2).owns and c.kv(2).window == 100
    shared = c.kv(3)
    assert not shared.owns and shared.layer_offset == c.kv(0).layer_offset and shared.page_stride == full.page_stride
    with pytest.raises(CacheError, match="keeps none of its own"):
        PagedCache([(CacheNeed(1, 16), None, None), (CacheNeed(1, 16), None, 0), (CacheNeed(1, 16), None, 1)], 64,
                   torch.float32, None)
    with pytest.raises(CacheError, match="looks further back"):
        PagedCache([(CacheNeed(1, 16, 8), None, None), (CacheNeed(1, 16, None), None, 0)], 64, torch.float32, None)


def test_slots_and_pages_through_random_batches():
    rng = random.Random(0)
    c = two_group_cache(max_tokens=64 * 12, max_slots=5)
    for _ in range(60):
        n = rng.randint(1, 4)
        slots = [c.open() for _ in range(min(n, c.max_slots - c.n_live))]
        lens = {s: rng.randint(1, 150) for s in slots}
        ok = []
        for s in slots:
            try:
                assert c.reserve(s, lens[s]) == 0
                c.commit(s)
                ok.append(s)
            except CacheFull:
                pass
            held(c)
        for _ in range(rng.randint(0, 80)):
            for s in list(ok):
                if rng.random() < 0.05:
                    c.close(s)
                    ok.remove(s)
                    continue
                try:
                    pos = c.reserve(s, 1)
                    assert pos == c.length(s)
                    c.commit(s)
                except CacheFull:
                    c.close(s)
                    ok.remove(s)
            held(c)
        for s in slots:
            if c.slots[s].live:
                c.close(s)
        held(c)
        assert c.n_live == 0 and all(g.pool.n_free == g.pool.n_pages for g in c.groups)


def test_slot_errors_and_reuse():
    c = two_group_cache(max_slots=2)
    a, b = c.open(), c.open()
    with pytest.raises(CacheFull, match="slots"):
        c.open()
    c.close(a)
    with pytest.raises(CacheError, match="no live sequence"):
        c.close(a)                                   # closed twice
    with pytest.raises(CacheError, match="no live sequence"):
        c.reserve(a, 1)
    assert c.open() == a and c.length(a) == 0        # the slot is handed out again, empty
    c.reserve(b, 3)
    with pytest.raises(CacheError, match="already has positions reserved"):
        c.reserve(b, 1)


def test_window_group_gives_back_pages_that_no_later_token_reaches():
    c = two_group_cache(max_tokens=64 * 20)
    full, win = c.groups
    s = c.open()
    c.reserve(s, 300)
    assert (win.host_table[s] >= 0).sum() == 5       # a whole prompt needs all its pages while it runs
    c.commit(s)
    # the next token, at position 300, reaches back to 201: pages 0..2 (positions < 192) are gone
    assert (win.host_table[s][:3] < 0).all() and (win.host_table[s][3:5] >= 0).all()
    assert (full.host_table[s] >= 0).sum() == 5
    for _ in range(200):
        c.reserve(s, 1)
        c.commit(s)
        assert (win.host_table[s] >= 0).sum() <= 3   # window 100 over pages of 64: at most 3 pages
    assert (full.host_table[s] >= 0).sum() == 8
    held(c)


def test_a_group_with_a_window_has_pages_for_its_windows_only():
    """With few slots, the pool of a group that keeps a window holds what the windows and one step's new positions
    need (window 100 + 128 new positions: 4 pages of 64, and two for where they begin and end) and no more; the
    group that keeps everything has all pages.  Sequences that grow in steps of that length never find it empty."""
    c = two_group_cache(max_tokens=64 * 200, max_slots=3, window_step=128)
    full, win = c.groups
    assert full.pool.n_pages == 200 and win.pool.n_pages == 3 * (4 + 2) and c.step_limit == 128
    slots = [c.open() for _ in range(3)]
    for step in range(30):
        for s in slots:
            c.reserve(s, 128 if step % 3 else 1)
        for s in slots:
            c.commit(s)
        held(c)
    assert all(c.length(s) == 20 * 128 + 10 for s in slots)
    # a step of more positions is for the caller to cut: the whole of it has room or not, before anything runs
    c.room_for(slots, [1000, 1000, 1000])
    with pytest.raises(CacheFull):
        c.room_for(slots, [5000, 3000, 3000])
    for s in slots:
        c.close(s)
    held(c)
    # with many slots the windows would take more than every page there is: the pool is no smaller then, no limit
    many = two_group_cache(max_tokens=64 * 20)
    assert many.step_limit is None and all(g.pool.n_pages == 20 for g in many.groups)


def test_a_sequence_that_outgrows_the_cache_is_refused_and_nothing_leaks():
    c = two_group_cache(max_tokens=64 * 3)
    s, t = c.open(), c.open()
    c.reserve(s, 100)
    c.commit(s)
    with pytest.raises(CacheFull):
        c.reserve(t, 129)                            # needs 3 pages, 1 is left
    held(c)
    assert c.groups[0].pool.n_free == 1 and c.slots[t].reserved == 0
    c.reserve(t, 10)
    c.commit(t)
    capped = PagedCache([(CacheNeed(1, 16), None, None)], 64 * 100, torch.float32, None, max_positions=128)
    with pytest.raises(CacheFull, match="per sequence"):
        capped.reserve(capped.open(), 129)


# ------------------------------------------------------------------------------------------------ decisions of the loop
def test_plan_batches():
    assert plan_batches(5, 2) == [[0, 1], [2, 3], [4]] and plan_batches(0, 3) == []
    with pytest.raises(ValueError):
        plan_batches(3, 0)


def track(**kw):
    o = GenerationOptions(**{**dict(max_tokens=5, stop_tokens=(9,), loop_detection=False), **kw})
    return SequenceTrack(0, prompt_len=3, options=o, max_positions=100)


def test_a_stop_token_ends_the_sequence_and_is_not_emitted():
    t = track()
    assert t.accept(4) and t.accept(5)
    assert not t.accept(9) and t.finish_reason == "stop" and t.out == [4, 5]


def test_max_tokens_and_context_end_the_sequence():
    t = track(max_tokens=3)
    assert t.accept(1) and t.accept(2) and not t.accept(3)
    assert t.finish_reason == "length" and t.out == [1, 2, 3]
    t = SequenceTrack(0, prompt_len=3, options=GenerationOptions(max_tokens=50, loop_detection=False), max_positions=5)
    assert t.accept(1) and not t.accept(2) and t.finish_reason == "context" and t.out == [1, 2]


def test_loop_detector_counts_a_four_gram_seen_three_times_before():
    """/root/reference/src/engine/tq_generate.c:611-629."""
    d, hist, fired = LoopDetector(), [], []
    for tok in [1, 2, 3, 4] * 6:
        hist.append(tok)
        fired.append(d.push(hist))
    assert fired.index(True) == 15                   # the 4th full repetition of (1,2,3,4) ends at token 16
    t = track(max_tokens=100, loop_detection=True)
    n = 0
    for tok in [1, 2, 3, 4] * 10:
        n += 1
        if not t.accept(tok):
            break
    assert t.finish_reason == "loop" and n == 16
    assert LoopDetector().push([1, 2, 3]) is False


def test_callback_sees_every_emitted_token():
    seen = []
    t = track(on_token=lambda r, tok: seen.append((r, tok)))
    for tok in (4, 5, 9):
        t.accept(tok)
    assert seen == [(0, 4), (0, 5)]


def test_rng_is_the_reference_xorshift():
    """First values of xorshift64* seeded with 42 (/root/reference/src/engine/tq_generate.c:53-58), computed by hand."""
    r = XorShift64Star(42)
    s = 42
    s ^= s >> 12
    s ^= (s << 25) & (2 ** 64 - 1)
    s ^= s >> 27
    want = float(((s * 0x2545F4914F6CDD1D) & (2 ** 64 - 1)) >> 33) / float(1 << 31)
    assert r.next_float() == want and 0.0 <= want < 1.0
    assert XorShift64Star(0).state == 42                          # seed 0 stands for 42 (:407)
    assert stream_seed(7, 0) == 7 and stream_seed(7, 1) != stream_seed(7, 2) != 7


# ------------------------------------------------------------------------------------------------ the loop on stand-in kernels
@pytest.fixture
def cpu_engine(monkeypatch, model_dirs):
    emulated_kernels.install(monkeypatch)

    def make(name, max_tokens=1024, **kw):
        return Engine(load_model(model_dirs(name), act="float32", device="cpu"), max_tokens=max_tokens, **kw)
    return make


def test_step_logits_equal_the_plain_model_whole_split_and_batched(cpu_engine, model_dirs):
    from plain_qwen2moe import PlainQwen2Moe
    for name in ("A", "B"):
        eng = cpu_engine(name)
        plain = PlainQwen2Moe(model_dirs(name))
        V = TINY[name][0]["vocab_size"]
        g = torch.Generator().manual_seed(5)
        prompts = [torch.randint(0, V, (n,), generator=g).tolist() for n in (1, 9, 40, 70)]
        ref = [plain.logits(p).float() for p in prompts]
        slots = eng.open(4)
        lg = eng.step(slots, prompts, [list(range(len(p))) for p in prompts])
        assert (lg - torch.cat(ref)).abs().max() < 1e-4
        eng.close(slots)
        # the last tokens one by one, in a batch whose shorter members end first
        slots = eng.open(4)
        cut = [max(1, len(p) - 8) for p in prompts]
        eng.step(slots, [p[:c] for p, c in zip(prompts, cut)], [[] for _ in prompts])
        pos = list(cut)
        eng.close([slots[i] for i in range(4) if pos[i] == len(prompts[i])])
        while True:
            live = [i for i in range(4) if pos[i] < len(prompts[i])]
            if not live:
                break
            lg = eng.step([slots[i] for i in live], [[prompts[i][pos[i]]] for i in live])
            for j, i in enumerate(live):
                assert (lg[j] - ref[i][pos[i]]).abs().max() < 1e-4
                pos[i] += 1
                if pos[i] == len(prompts[i]):
                    eng.close([slots[i]])
        assert eng.cache.n_live == 0 and all(g.pool.n_free == g.pool.n_pages for g in eng.cache.groups)


def test_a_long_prompt_runs_in_cuts_where_a_window_has_few_pages(cpu_engine, model_dirs):
    """Configuration B keeps a window of 24 on two layers.  With three slots their group has pages for three windows and
    a step of 64 positions, so prompts of 150 and 70 tokens go through in cuts of 64; the logits, asked for in an
    order of their own, are the plain model's.  A step that the other group has no room for is refused whole."""
    from plain_qwen2moe import PlainQwen2Moe
    eng = cpu_engine("B", max_tokens=64 * 20, max_slots=3, window_step=64)
    win = [g for g in eng.cache.groups if g.key.window is not None][0]
    assert eng.cache.step_limit == 64 and win.pool.n_pages == 3 * (2 + 2) and eng.cache.n_pages == 20
    plain = PlainQwen2Moe(model_dirs("B"))
    g = torch.Generator().manual_seed(9)
    prompts = [torch.randint(0, 384, (n,), generator=g).tolist() for n in (150, 20, 70)]
    wants = [[149, 0, 64, 63, 100], [], [69, 5]]
    slots = eng.open(3)
    lg = eng.step(slots, prompts, wants)
    ref = torch.cat([plain.logits(p).float()[w] for p, w in zip(prompts, wants) if w])
    assert lg.shape == ref.shape and (lg - ref).abs().max() < 1e-4
    assert [eng.length(s) for s in slots] == [150, 20, 70]
    # one more position each, then a step that does not fit: nothing of it has run
    eng.step(slots, [[1], [2], [3]])
    with pytest.raises(CacheFull):
        eng.step(slots, [[1] * 600, [2] * 600, [3] * 600])
    assert [eng.length(s) for s in slots] == [151, 21, 71]
    eng.close(slots)
    assert all(g.pool.n_free == g.pool.n_pages for g in eng.cache.groups)


def test_step_refuses_bad_input(cpu_engine):
    eng = cpu_engine("A")
    s = eng.open(2)
    with pytest.raises(StepError, match="outside the vocabulary"):
        eng.step(s, [[1, 2], [256]])
    with pytest.raises(StepError, match="twice"):
        eng.step([s[0], s[0]], [[1], [2]])
    with pytest.raises(StepError, match="no token"):
        eng.step(s, [[1], []])
    with pytest.raises(ValueError, match="outside the"):
        eng.step(s, [[1], [2]], [[0], [1]])
    assert eng.length(s[0]) == 0                      # nothing was run


def test_generate_matches_the_plain_loop_for_unequal_prompts_in_several_batches(cpu_engine, model_dirs):
    from plain_qwen2moe import PlainQwen2Moe, generate as plain_generate
    eng = cpu_engine("B", max_tokens=64 * 3, max_slots=3)
    plain = PlainQwen2Moe(model_dirs("B"))
    g = torch.Generator().manual_seed(6)
    prompts = [torch.randint(0, 384, (n,), generator=g).tolist() for n in (3, 11, 1, 6, 20)]
    for opts in (dict(temperature=0.0, rep_penalty=1.0), dict(temperature=0.0, rep_penalty=1.3),
                 dict(temperature=0.9, top_p=0.8, rep_penalty=1.0, seed=5)):
        stop = (7, 11)
        lens = [4, 9, 2, 7, 5]
        res = []
        for i, (p, n) in enumerate(zip(prompts, lens)):     # one request at a time: its own max_tokens
            o = GenerationOptions(max_tokens=n, stop_tokens=stop, loop_detection=False, max_batch=2, **opts)
            res.append(generate(eng, [p], o)[0])
            want = plain_generate(plain, p, max_tokens=n, stop_tokens=stop, **opts)
            assert res[-1].tokens == want
        # all at once, two at a time: the same tokens whatever shares the batch (random streams are per request,
        # so only the greedy runs can be compared across batchings)
        if opts["temperature"] == 0.0:
            o = GenerationOptions(max_tokens=9, stop_tokens=stop, loop_detection=False, max_batch=2, **opts)
            together = generate(eng, prompts, o)
            for r, p in zip(together, prompts):
                assert r.tokens == plain_generate(plain, p, max_tokens=9, stop_tokens=stop, **opts)
                assert r.finish_reason in ("length", "stop")
                assert (r.finish_reason == "stop") == (len(r.tokens) < 9)
        assert eng.cache.n_live == 0


def test_generate_runs_ahead_only_where_a_page_is_free(cpu_engine):
    """Two pages, two sequences: after the prompts one sequence fills its page and the next step of both is
    issued before their tokens are known, which finds no page free.  The loop then waits for the tokens; the
    full sequence ends on its first token (an end token), gives its page back, and the other goes on into it."""
    eng = cpu_engine("A", max_tokens=128, max_slots=2)
    a, b = [3] * 60, [5] * 64
    greedy = dict(temperature=0.0, rep_penalty=1.0, loop_detection=False)
    first_of_b = generate(eng, [b], GenerationOptions(max_tokens=1, **greedy))[0].tokens[0]
    alone = generate(eng, [a], GenerationOptions(max_tokens=12, **greedy))[0]
    if first_of_b in alone.tokens:
        pytest.skip("the end token chosen for this test also ends the other sequence")
    both = generate(eng, [a, b], GenerationOptions(max_tokens=12, stop_tokens=(first_of_b,), **greedy))
    assert both[1].tokens == [] and both[1].finish_reason == "stop"
    assert both[0].tokens == alone.tokens and len(alone.tokens) == 12       # positions 60..71: into the second page
    assert eng.cache.n_live == 0 and all(g.pool.n_free == g.pool.n_pages for g in eng.cache.groups)


def test_generate_ends_a_sequence_when_the_cache_is_full(cpu_engine):
    eng = cpu_engine("A", max_tokens=64, max_slots=1)
    r = generate(eng, [[1] * 60], GenerationOptions(max_tokens=50, temperature=0.0, rep_penalty=1.0, loop_detection=False))[0]
    assert r.finish_reason == "context" and len(r.tokens) == 4 and eng.cache.n_live == 0
    r = generate(eng, [[1] * 65], GenerationOptions(max_tokens=5))[0]
    assert r.finish_reason == "context" and r.tokens == []


def test_a_refused_step_leaves_its_slots_usable(cpu_engine):
    eng = cpu_engine("A", max_tokens=128, max_slots=2)
    s = eng.open(2)
    with pytest.raises(StepError, match="wanted place"):
        eng.step(s, [[1, 2], [3]], [[0], [1]])
    with pytest.raises(CacheFull):
        eng.step(s, [[1] * 70, [2] * 70])              # three pages would be needed, two exist
    assert all(g.pool.n_free == g.pool.n_pages for g in eng.cache.groups)
    lg = eng.step(s, [[1, 2], [3]])                    # the same slots step as if nothing had happened
    assert lg.shape == (2, 256) and eng.length(s[0]) == 2 and eng.length(s[1]) == 1
    eng.close(s)


def test_generate_survives_a_full_pool(cpu_engine):
    """Two pages, two sequences of 60 tokens: at position 64 both need a page and none is free.  One ends with
    reason "context" (with the token that found no room as its last), its page lets the other go on, and the
    other's tokens are what it generates alone."""
    eng = cpu_engine("A", max_tokens=128, max_slots=2)
    greedy = dict(temperature=0.0, rep_penalty=1.0, loop_detection=False)
    a, b = [3] * 60, [5, 9] * 30
    alone = [generate(eng, [p], GenerationOptions(max_tokens=12, **greedy))[0] for p in (a, b)]
    both = generate(eng, [a, b], GenerationOptions(max_tokens=12, **greedy))
    assert [r.finish_reason for r in both] == ["context", "length"]
    assert both[0].tokens == alone[0].tokens[:5] and both[1].tokens == alone[1].tokens and len(both[1].tokens) == 12
    assert eng.cache.n_live == 0 and all(g.pool.n_free == g.pool.n_pages for g in eng.cache.groups)


def test_prompts_that_do_not_fit_together_run_one_after_the_other(cpu_engine):
    eng = cpu_engine("A", max_tokens=192, max_slots=2)
    greedy = dict(temperature=0.0, rep_penalty=1.0, loop_detection=False)
    a, b, c = [3] * 100, [5, 9] * 50, [7] * 300
    alone = [generate(eng, [p], GenerationOptions(max_tokens=6, **greedy))[0] for p in (a, b)]
    res = generate(eng, [a, b, c], GenerationOptions(max_tokens=6, max_batch=2, **greedy))
    assert [r.tokens for r in res[:2]] == [r.tokens for r in alone] and all(len(r.tokens) == 6 for r in res[:2])
    assert res[2].tokens == [] and res[2].finish_reason == "context"        # four pages are needed, three exist
    assert eng.cache.n_live == 0


def test_a_limit_of_positions_per_sequence_binds(cpu_engine):
    eng = cpu_engine("A", max_tokens=1024, max_slots=2, max_positions=100)
    assert eng.cache.max_positions == 100
    r = generate(eng, [[1] * 90, [2] * 101], GenerationOptions(max_tokens=50, temperature=0.0, rep_penalty=1.0,
                                                               loop_detection=False))
    assert r[0].finish_reason == "context" and len(r[0].tokens) == 10
    assert r[1].finish_reason == "context" and r[1].tokens == []


def test_generate_with_the_default_options_matches_the_plain_loop(cpu_engine, model_dirs):
    """Loop detection, repetition penalty and sampling as the options default to them; greedy decoding of a
    tiny model soon repeats itself, so the 4-gram stop fires."""
    from plain_qwen2moe import PlainQwen2Moe, generate as plain_generate
    eng = cpu_engine("A")
    plain = PlainQwen2Moe(model_dirs("A"))
    reasons = []
    for prompt, opts in (([3, 3, 3, 3, 3, 3], dict(temperature=0.0, rep_penalty=1.0)),
                         ([1, 2, 3, 4] * 4, dict(temperature=0.0, rep_penalty=1.0)),
                         ([9, 8, 7], dict())):
        o = GenerationOptions(max_tokens=40, **opts)
        assert o.loop_detection
        got = generate(eng, [prompt], o)[0]
        want = plain_generate(plain, prompt, max_tokens=40, loop_detection=True,
                              **{**dict(temperature=0.7, top_p=0.9, rep_penalty=1.1), **opts})
        assert got.tokens == want
        reasons.append(got.finish_reason)
    assert "loop" in reasons


def test_a_sequence_that_outlives_its_request(cpu_engine):
    """``continue_in_slot``: the slot's cache holds the beginning of a history, the rest is run as one prompt step and
    a continuation is generated; what comes out is what ``generate`` gives for the whole history, turn after turn,
    and the cache then holds all but a token that ended the turn by its number.  A cache that runs full ends the turn
    with reason "context" and keeps what it holds."""
    from turboquant_cpp_amd.engine.generate import continue_in_slot
    eng = cpu_engine("A", max_tokens=64 * 6, max_slots=2)
    greedy = dict(temperature=0.0, rep_penalty=1.0, loop_detection=False)
    (slot,) = eng.open(1)
    history = [3, 9, 4, 1, 7]
    brought = []
    step = eng.step
    eng.step = lambda slots, toks, *a, **k: (brought.append(len(toks[0])), step(slots, toks, *a, **k))[1]
    for turn, more in enumerate(([], [8, 8, 2], [5])):
        history = history + more
        before = eng.length(slot)
        del brought[:]
        res = continue_in_slot(eng, slot, history, GenerationOptions(max_tokens=4, **greedy))
        assert brought[0] == len(history) - before and brought[1:] == [1] * 3
        eng.step = step
        want = generate(eng, [history], GenerationOptions(max_tokens=4, **greedy))[0]
        eng.step = lambda slots, toks, *a, **k: (brought.append(len(toks[0])), step(slots, toks, *a, **k))[1]
        assert res.tokens == want.tokens and res.finish_reason == "length"
        assert eng.length(slot) == len(history) + 3            # the fourth token ended the turn and was never run
        history = history + res.tokens
    with pytest.raises(ValueError, match="at least one"):
        continue_in_slot(eng, slot, history[:eng.length(slot)], GenerationOptions(max_tokens=4, **greedy))
    assert continue_in_slot(eng, slot, history, GenerationOptions(max_tokens=0, **greedy)).finish_reason == "length"
    eng.step = step
    eng.close([slot])
    small = cpu_engine("A", max_tokens=64, max_slots=1)
    (slot,) = small.open(1)
    res = continue_in_slot(small, slot, [3] * 60, GenerationOptions(max_tokens=12, **greedy))
    assert res.finish_reason == "context" and len(res.tokens) == 4 and small.length(slot) == 63
    small.close([slot])


def test_a_sequence_goes_back_to_an_earlier_position():
    """``truncate`` forgets the positions from a point on and gives their pages back; it refuses where a window has
    dropped pages that the earlier position would look at, and where the model keeps fixed-size state."""
    from turboquant_cpp_amd.cache.paged import CacheError, PagedCache
    from turboquant_cpp_amd.parts.base import CacheNeed, StateNeed
    cache = PagedCache([(CacheNeed(2, 16), None, None), (CacheNeed(2, 16, window=100), None, None)], 64 * 10, torch.float32,
                       None, page_size=64, max_slots=2)
    s = cache.open()
    cache.reserve(s, 200)
    cache.commit(s)
    assert cache.pages_held() == {0: 4, 1: 3}              # the window of 100 has let page 0 go
    with pytest.raises(CacheError, match="window"):
        cache.truncate(s, 120)                             # position 120 looks back to 21: page 0
    cache.truncate(s, 170)                                 # looks back to 71: page 1
    assert cache.length(s) == 170 and cache.pages_held() == {0: 3, 1: 2}
    cache.truncate(s, 170)
    with pytest.raises(CacheError):
        cache.truncate(s, 171)
    assert cache.reserve(s, 30) == 170
    cache.commit(s)
    assert cache.length(s) == 200 and cache.pages_held() == {0: 4, 1: 3}
    cache.close(s)
    assert cache.pages_held() == {0: 0, 1: 0}
    plain = PagedCache([(CacheNeed(2, 16), None, None)], 64 * 4, torch.float32, None, page_size=64, max_slots=1)
    s = plain.open()
    plain.reserve(s, 130)
    with pytest.raises(CacheError, match="reserved"):
        plain.truncate(s, 10)
    plain.commit(s)
    plain.truncate(s, 0)
    assert plain.length(s) == 0 and plain.pages_held() == {0: 0}
    stateful = PagedCache([(None, StateNeed((4,)), None)], 64, torch.float32, None, page_size=64, max_slots=1)
    s = stateful.open()
    stateful.reserve(s, 5)
    stateful.commit(s)
    with pytest.raises(CacheError, match="state"):
        stateful.truncate(s, 2)
