"""The engine above the step function: generation through the entry points, sampling,
what happens when pages run out, failure of a step."""
import json
import os
import subprocess
import sys

import pytest
import torch

from conftest import ROOT, TINY, seeded_tokens
from plain.gpt2_plain import PlainGPT2
from plain import sampler_plain as SP


def options_for(dtype, device, **kw):
    from denno_beta_amd.config import EngineOptions
    opts = dict(dtype=dtype, device=device, page_size=16, cache_tokens=1024, max_live=4)
    opts.update(kw)
    return EngineOptions(**opts)


def engine_for(folder, dtype, device, **kw):
    from denno_beta_amd.engine import Engine
    return Engine.from_folder(folder, options_for(dtype, device, **kw))


def test_greedy_generation_matches_plain(backend, model_folders):
    """Tiny A's workload: prompts of 7, 19 and 33 tokens, 16 greedy tokens each, prompts cut
    into portions of 5 beside the decoding of earlier requests."""
    from denno_beta_amd.engine import SamplingParams
    folder = model_folders("A", "float32")
    plain = PlainGPT2.from_folder(folder)
    prompts = [seeded_tokens(i, n, 512) for i, n in enumerate((7, 19, 33))]
    want = [plain.greedy(p, 16) for p in prompts]
    e = engine_for(folder, "float32", backend, prefill_chunk=5, max_batch_tokens=12)
    assert e.generate(prompts, SamplingParams(max_tokens=16, temperature=0.0)) == want
    assert any(r.decode_rows and r.prefill_rows for r in e.records), "no step mixed decoding with a prompt"
    assert e.runner.cache.manager.live() == 0
    assert [e.finish_reason(i) for i in range(3)] == ["length"] * 3


@pytest.mark.parametrize("policy,cache_tokens", [("preempt", 96), ("reserve", 128)])
def test_few_pages(backend, model_folders, policy, cache_tokens):
    """With too few pages for all requests at once the result is the same: under "preempt" the
    youngest request is recomputed, under "reserve" requests wait their turn."""
    from denno_beta_amd.engine import SamplingParams
    folder = model_folders("A", "float32")
    plain = PlainGPT2.from_folder(folder)
    prompts = [seeded_tokens(i, n, 512) for i, n in enumerate((7, 19, 33))]
    want = [plain.greedy(p, 16) for p in prompts]
    e = engine_for(folder, "float32", backend, cache_tokens=cache_tokens, kv_policy=policy, prefill_chunk=8)
    assert e.generate(prompts, SamplingParams(max_tokens=16, temperature=0.0)) == want
    pre = sum(r.preemptions for r in e.requests.values())
    assert (pre > 0) if policy == "preempt" else (pre == 0)
    e.runner.cache.manager.check()
    assert e.runner.cache.manager.free_pages(0) == cache_tokens // 16


def test_temperature_sampling_is_seeded_and_independent_of_the_batch(backend, model_folders):
    """Tiny B's workload, shortened on the host: temperature 0.8, seeded, prompts admitted into
    a running batch.  A request's tokens are those it gets alone."""
    from denno_beta_amd.engine import SamplingParams
    folder = model_folders("B", "float32")
    lengths = (1, 50, 120, 200) if backend != "cpu" else (1, 20, 45)
    prompts = [seeded_tokens(20 + i, n, 1000) for i, n in enumerate(lengths)]
    params = [SamplingParams(max_tokens=24, temperature=0.8, seed=100 + i) for i in range(len(prompts))]
    alone = []
    for p, sp in zip(prompts, params):
        e = engine_for(folder, "float32", backend, prefill_chunk=32)
        alone.append(e.generate([p], sp)[0])
    e = engine_for(folder, "float32", backend, prefill_chunk=32, max_batch_tokens=48)
    rids = [e.add_request(prompts[0], params[0])]
    for _ in range(3):
        e.step()
    rids += [e.add_request(p, sp) for p, sp in zip(prompts[1:], params[1:])]    # into a running batch
    while e.has_unfinished():
        e.step()
    together = [e.requests[r].generated for r in rids]
    assert together == alone
    assert len(set(map(tuple, alone))) > 1 and all(len(t) == 24 for t in alone)
    # and the tokens are what the plain sampler picks from the plain logits with the same numbers
    from denno_beta_amd.sampling import uniform
    plain = PlainGPT2.from_folder(folder)
    seq = list(prompts[1])
    for n, tok in enumerate(alone[1][:6]):
        row = plain.logits(seq)[-1]
        assert SP.temperature_walk(row.tolist(), 0.8, uniform(101, n)) == tok
        seq.append(tok)


def test_top_k_top_p_and_penalties_follow_the_plain_sampler(backend, model_folders):
    from denno_beta_amd.engine import SamplingParams
    from denno_beta_amd.sampling import uniform
    folder = model_folders("A", "float32")
    plain = PlainGPT2.from_folder(folder)
    prompt = seeded_tokens(9, 12, 512)
    sp = SamplingParams(max_tokens=8, temperature=0.9, top_k=5, top_p=0.8, seed=7, repetition_penalty=1.3,
                        frequency_penalty=0.2, presence_penalty=0.1, no_repeat_ngram_size=2)
    got = engine_for(folder, "float32", backend).generate([prompt], sp)[0]
    seq = list(prompt)
    for n, tok in enumerate(got):
        row = plain.logits(seq)[-1].tolist()
        row = SP.repetition_penalty(row, seq, 1.3)
        row = SP.frequency_presence(row, seq, 0.2, 0.1)
        row = SP.no_repeat_ngram(row, seq, 2)
        assert SP.top_k_top_p(row, 0.9, 5, 0.8, uniform(7, n)) == tok, n
        seq.append(tok)


def test_eos_and_max_tokens(backend, model_folders, tmp_path):
    from denno_beta_amd.engine import SamplingParams
    from denno_beta_amd.weights import write_model_folder
    cfg, seed = TINY["A"]
    folder = model_folders("A", "float32")
    prompt = seeded_tokens(1, 10, 512)
    first = engine_for(folder, "float32", backend).generate([prompt], SamplingParams(max_tokens=4, temperature=0.0))[0]
    # the same weights with the third generated token declared end-of-sequence
    d = write_model_folder(str(tmp_path / "eos"), dict(cfg, eos_token_id=first[2]), seed)
    e = engine_for(d, "float32", backend)
    out = e.generate([prompt], SamplingParams(max_tokens=10, temperature=0.0))[0]
    stop = first.index(first[2])
    assert out == first[:stop + 1] and e.finish_reason(0) == "eos"      # the stop token is kept (engine.rs:1125-1129)
    e = engine_for(d, "float32", backend)
    assert len(e.generate([prompt], SamplingParams(max_tokens=10, temperature=0.0, ignore_eos=True))[0]) == 10
    # max_tokens is clamped to the positions left; 0 computes the prompt only
    e = engine_for(folder, "float32", backend)
    long_prompt = seeded_tokens(2, 120, 512)
    assert len(e.generate([long_prompt], SamplingParams(max_tokens=50, temperature=0.0))[0]) == 8
    assert e.generate([prompt], SamplingParams(max_tokens=0))[0] == [] and e.finish_reason(1) == "length"
    assert e.runner.cache.manager.live() == 0
    # the end-of-sequence token as the very last token that max_tokens allows: the scheduler has let the
    # request go when its last token was launched, and the end-of-sequence rule finds nothing left to give back
    e = engine_for(d, "float32", backend)
    out = e.generate([prompt], SamplingParams(max_tokens=stop + 1, temperature=0.0))[0]
    assert out == first[:stop + 1] and e.finish_reason(0) == "eos" and e.runner.cache.manager.live() == 0
    e.runner.cache.manager.check()
    # a request given up while its last token is on its way (steps are launched ahead where they can be)
    e = engine_for(folder, "float32", backend)
    rid = e.add_request(prompt, SamplingParams(max_tokens=6, temperature=0.0, ignore_eos=True))
    while len(e.requests[rid].generated) < 5:
        e.step()
    e.abort(rid)
    assert e.finish_reason(rid) == "aborted"
    while e.has_unfinished():
        e.step()
    assert e.runner.cache.manager.live() == 0
    e.runner.cache.manager.check()


def test_stop_sequences(backend, model_folders):
    """crates/denno-engine/src/engine.rs:2214-2236 (stop_sequence_truncates_at_first_occurrence): the text is cut
    where the first stop sequence begins and does not hold it, the reason and the sequence are told; a sequence
    that never appears changes nothing.  The detokenizer is the caller's: here token t reads "t<t>"."""
    from denno_beta_amd.engine import Engine, ModelRunner, SamplingParams
    folder = model_folders("A", "float32")
    words = lambda ids: " ".join(f"t{t}" for t in ids)                          # noqa: E731

    def engine(**kw):
        return Engine(ModelRunner.from_folder(folder, options_for("float32", backend, **kw)), detokenize=words)
    prompts = [seeded_tokens(i, n, 512) for i, n in enumerate((9, 30, 4))]
    free = SamplingParams(max_tokens=20, temperature=0.0, ignore_eos=True)
    e = engine()
    full = e.generate(prompts, free)
    assert [e.requests[i].text for i in range(3)] == [words(t) for t in full] and e.finish_reason(0) == "length"
    # each request stops at its own seventh token's text, or at its twelfth's if that comes first in the text
    for i, toks in enumerate(full):
        stops = (f"t{toks[11]} ", f"t{toks[6]} ")
        at = min(words(toks).find(x) for x in stops)
        first = min(stops, key=lambda x: words(toks).find(x))
        e = engine()
        rid = e.add_request(prompts[i], SamplingParams(max_tokens=20, temperature=0.0, ignore_eos=True, stop_sequences=stops))
        while e.has_unfinished():
            e.step()
        r = e.requests[rid]
        assert r.finish_reason == "stop_sequence" and r.stop_sequence == first
        assert r.text == words(toks)[:at] and first not in r.text and words(toks).startswith(r.text)
        assert r.generated == toks[:len(r.generated)] and len(r.generated) < 20
        assert e.runner.cache.manager.live() == 0
    # a sequence that never appears, and an empty one: nothing changes
    e = engine()
    same = e.generate(prompts, SamplingParams(max_tokens=20, temperature=0.0, ignore_eos=True, stop_sequences=("t9999", "")))
    assert same == full and e.finish_reason(1) == "length"
    # all three together, each with its own sequence, beside each other in the batch
    e = engine()
    rids = [e.add_request(p, SamplingParams(max_tokens=20, temperature=0.0, ignore_eos=True,
                                            stop_sequences=(f"t{toks[8]} ",))) for p, toks in zip(prompts, full)]
    while e.has_unfinished():
        e.step()
    for rid, toks in zip(rids, full):
        assert e.requests[rid].text == words(toks)[:words(toks).find(f"t{toks[8]} ")]
    # an unfinished character at the end of the text waits for the token that finishes it
    halves = lambda ids: "".join("\u00e9" if t % 2 else "x" for t in ids[:len(ids) - len(ids) % 2]) + ("\ufffd" if len(ids) % 2 else "")   # noqa: E731
    e = Engine(ModelRunner.from_folder(folder, options_for("float32", backend)), detokenize=halves)
    e.generate([prompts[0]], SamplingParams(max_tokens=5, temperature=0.0, ignore_eos=True))
    assert "\ufffd" not in e.requests[0].text and len(e.requests[0].text) == 4
    # texts need a detokenizer
    with pytest.raises(ValueError, match="detokenizer"):
        Engine(ModelRunner.from_folder(folder, options_for("float32", backend))).add_request([1], SamplingParams(stop_sequences=("a",)))
    with pytest.raises(ValueError, match="list of strings"):
        SamplingParams(stop_sequences="ab").validate()


def test_a_sampler_alone_takes_any_contexts(backend):
    """A Sampler that serves no engine keeps its own table of histories: a later call with more rows or longer
    contexts than the first gets a larger one."""
    from denno_beta_amd.sampling import Sampler, SamplingParams
    dev = torch.device(backend)
    s = Sampler(dev)
    g = torch.Generator().manual_seed(5)
    V = 97
    sp = SamplingParams(temperature=0.0, repetition_penalty=1.5, presence_penalty=0.4)
    for rows, n in ((2, 5), (3, 40), (1, 7), (5, 41)):
        logits = torch.randn(rows, V, generator=g)
        ctxs = [torch.randint(0, V, (n + r,), generator=g).tolist() for r in range(rows)]
        got = s.sample(logits.clone().to(dev), [sp] * rows, [1] * rows, [0] * rows, ctxs)
        for r in range(rows):
            row = SP.repetition_penalty(logits[r].tolist(), ctxs[r], 1.5)
            row = SP.frequency_presence(row, ctxs[r], 0.0, 0.4)
            assert got[r] == SP.greedy(row), (rows, n, r)


def test_refused_requests(backend, model_folders):
    from denno_beta_amd.engine import SamplingParams, SchedulerError
    e = engine_for(model_folders("A", "float32"), "float32", backend, cache_tokens=64)
    with pytest.raises(SchedulerError, match="empty"):
        e.add_request([])
    with pytest.raises(SchedulerError, match="longer"):
        e.add_request([1] * 129)
    with pytest.raises(ValueError, match="vocabulary"):
        e.add_request([1, 999])
    with pytest.raises(SchedulerError, match="even alone"):
        e.add_request([1] * 60, SamplingParams(max_tokens=30))
    with pytest.raises(ValueError, match="no_repeat_ngram_size"):
        e.add_request([1], SamplingParams(no_repeat_ngram_size=1))
    assert not e.has_unfinished()


def test_a_failed_step_gives_everything_back(backend, model_folders):
    """crates/denno-engine/src/engine.rs:3395-3438: a failed prefill releases what it took and the
    next request runs as on a clean engine."""
    from denno_beta_amd.engine import SamplingParams
    folder = model_folders("A", "float32")
    prompt = seeded_tokens(4, 20, 512)
    sp = SamplingParams(max_tokens=6, temperature=0.0)
    clean = engine_for(folder, "float32", backend).generate([prompt], sp)[0]
    e = engine_for(folder, "float32", backend)
    rid = e.add_request(prompt, sp)
    e.fail_next_step = True
    with pytest.raises(RuntimeError, match="injected"):
        e.step()
    assert e.finish_reason(rid) == "error" and not e.has_unfinished()
    assert e.runner.cache.manager.live() == 0 and e.runner.cache.manager.free_pages(0) == 64
    e.runner.cache.manager.check()
    assert e.generate([prompt], sp)[0] == clean


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_step_that_fails_between_its_kernels(model_folders, dtype):
    """A step that fails after some of its kernels have run (crates/denno-engine/src/engine.rs:3354-3438:
    the reference's failing model errors after it has written the cache): keys and values of some
    layers stand in pages that go back to the pool.  Whatever the kernel it fails at (the first of layer
    0, one in the middle, the head's), every page and slot comes back, the other requests' error is
    reported, and the next requests, which get those pages, give a clean engine's tokens bit for bit."""
    from denno_beta_amd.engine import SamplingParams
    from denno_beta_amd.kernels import ops
    folder = model_folders("B", dtype)
    prompts = [seeded_tokens(50 + i, n, 1000) for i, n in enumerate((40, 9, 75))]
    sp = SamplingParams(max_tokens=6, temperature=0.0)
    mk = lambda: engine_for(folder, dtype, "cuda:0", cache_tokens=256, use_graphs=False)   # noqa: E731
    clean = mk().generate(prompts, sp)
    e = mk()
    for p in prompts:
        e.add_request(p, sp)
    e.step()
    before = ops.launches
    e.step()
    per_step = ops.launches - before              # launches of the step that will fail, the sampling kernel last
    assert per_step > 3 * 4
    for n in (0, 3, per_step // 2, per_step - 3, per_step - 1):
        e = mk()
        rids = [e.add_request(p, sp) for p in prompts]
        e.step()                                   # the prompts are in the cache, a token each is sampled
        ops.fail_after_launches(n)
        with pytest.raises(ops.KernelError, match="injected"):
            e.step()
        assert ops._fail_after is None
        assert all(e.finish_reason(r) == "error" for r in rids) and not e.has_unfinished()
        m = e.runner.cache.manager
        assert m.live() == 0 and m.free_pages(0) == 16
        m.check()
        assert e.generate(prompts, sp) == clean, f"after a failure at launch {n}"
        assert m.reuse_count(0) > 0
    ops.fail_after_launches(None)


def test_the_slot_record_holds_position_and_generator(backend, model_folders):
    """A live request's slot record (position, generator, last token) follows what the engine does, is
    zero for the next request that gets the slot, and carries a preempted request's generator on."""
    from denno_beta_amd.engine import SamplingParams
    from denno_beta_amd.sampling import uniform
    e = engine_for(model_folders("A", "float32"), "float32", backend, cache_tokens=256, max_live=1,
                   run_ahead=False)      # (step by step: nothing is launched before the last step's tokens are read)
    m = e.runner.cache.manager
    prompt = seeded_tokens(3, 11, 512)
    rid = e.add_request(prompt, SamplingParams(max_tokens=3, temperature=0.7, seed=99))
    e.step()
    st = m.state(rid)
    tok = e.requests[rid].generated[0]
    assert (st.num_computed, st.last_token, st.rng_seed, st.rng_drawn) == (11, tok, 99, 1)
    e.step()
    st = m.state(rid)
    assert (st.num_computed, st.last_token, st.rng_drawn) == (12, e.requests[rid].generated[1], 2)
    while e.has_unfinished():
        e.step()
    other = e.add_request(prompt[:4], SamplingParams(max_tokens=2, temperature=0.0, seed=5))
    e.step()
    st = m.state(other)
    assert m.slot(other) == 0 and (st.num_computed, st.rng_seed, st.rng_drawn) == (4, 5, 1)
    assert uniform(99, 0) != uniform(99, 1)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_running_ahead_changes_no_token(model_folders, tmp_path, dtype):
    """In steady decoding the next step is launched before the host has read this step's tokens, which it takes
    from the device.  Greedy and seeded temperature sampling, requests of different lengths that end by length
    and by an end-of-sequence token, so few pages that requests are put back, more requests than may live at
    once: every token is what the engine gives without running ahead."""
    from denno_beta_amd.engine import SamplingParams
    from denno_beta_amd.weights import write_model_folder
    cfg, seed = TINY["B"]
    prompts = [seeded_tokens(80 + i, n, 1000) for i, n in enumerate((5, 40, 9, 75, 21, 33, 2))]
    greedy = [SamplingParams(max_tokens=m, temperature=0.0) for m in (30, 7, 45, 12, 1, 60, 25)]
    # an end-of-sequence token that greedy decoding does meet: what request 0 generates tenth
    first = engine_for(model_folders("B", dtype), dtype, "cuda:0", run_ahead=False).generate(prompts[:1], greedy[:1])[0]
    folder = write_model_folder(str(tmp_path / "eos"), dict(cfg, eos_token_id=first[9]), seed, dtype)
    warm = [SamplingParams(max_tokens=m, temperature=0.9, seed=5 + i) for i, m in enumerate((30, 7, 45, 12, 1, 60, 25))]
    # top-k and top-p, among them top-p alone (whose rows a second kernel may have to finish: on the device, without
    # the host in between, so that these steps run ahead as well)
    cut = [SamplingParams(max_tokens=m, temperature=1.1, seed=9 + i, top_k=(None, 5, 40)[i % 3], top_p=(0.9, None, 0.7)[i % 3])
           for i, m in enumerate((30, 7, 45, 12, 1, 60, 25))]
    # penalties over the request's own tokens, which lie on the device beside the sampler: a step that runs ahead
    # counts the token of the step before, which the host has not seen.  Some rows with, some without
    punished = [SamplingParams(max_tokens=m, temperature=(0.0, 0.9, 1.2)[i % 3], seed=20 + i, top_k=(None, None, 30)[i % 3],
                               repetition_penalty=(1.4, None, 1.1, None)[i % 4], frequency_penalty=(None, 0.3)[i % 2],
                               presence_penalty=(0.2, None, None)[i % 3], no_repeat_ngram_size=(None, 2, 3, None)[i % 4])
                for i, m in enumerate((30, 7, 45, 12, 1, 60, 25))]
    for params in (greedy, warm, cut, punished):
        for kw in (dict(cache_tokens=1024, max_live=8), dict(cache_tokens=192, max_live=3)):
            want_engine = engine_for(folder, dtype, "cuda:0", run_ahead=False, **kw)
            want = want_engine.generate(prompts, params)
            e = engine_for(folder, dtype, "cuda:0", run_ahead=True, **kw)
            got = e.generate(prompts, params)
            assert got == want, (params is greedy, kw)
            assert [e.finish_reason(i) for i in range(7)] == [want_engine.finish_reason(i) for i in range(7)]
            assert sum(r.ran_ahead for r in e.records) > 10 and not any(r.ran_ahead for r in want_engine.records)
            m = e.runner.cache.manager
            assert m.live() == 0 and not e.has_unfinished()
            m.check()
    assert "eos" in [e.finish_reason(i) for i in range(7)]
    # one request alone, step by step: every step but the first of its decoding runs ahead
    e = engine_for(folder, dtype, "cuda:0", run_ahead=True)
    rid = e.add_request(prompts[3], SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True))
    outs = []
    while e.has_unfinished():
        outs += [o.token for o in e.step() if o.token is not None]
    assert outs == e.requests[rid].generated and len(outs) == 12
    assert [r.ran_ahead for r in e.records] == [False] + [True] * 11


@pytest.mark.gpu
@pytest.mark.parametrize("how", ["flag", "launch"])
def test_a_step_launched_ahead_that_fails(model_folders, how):
    """The step that is launched before the last one's tokens are read fails (in the engine, or at a kernel
    launch of its sampling).  The step before is told whole: its tokens are the requests' own and its outputs say
    that the requests ended with an error; the error reaches whoever calls `step` next, `generate` included
    (`has_unfinished` stays true until then); nothing stale is raised later; pages and slots come back and the
    next requests give a clean engine's tokens."""
    from denno_beta_amd.engine import SamplingParams
    from denno_beta_amd.kernels import ops
    folder = model_folders("B", "float32")
    prompts = [seeded_tokens(60 + i, n, 1000) for i, n in enumerate((12, 30, 5))]
    sp = SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True)
    mk = lambda: engine_for(folder, "float32", "cuda:0", cache_tokens=512, run_ahead=True)   # noqa: E731
    clean = mk().generate(prompts, sp)

    def fail(e):
        if how == "flag":
            e.fail_next_step = True
        else:
            ops.fail_after_launches(0)      # a replayed graph launches nothing through ops: the sampling kernel is next
    e = mk()
    rids = [e.add_request(p, sp) for p in prompts]
    while not (e.records and e.records[-1].ran_ahead):
        e.step()
    n_before = [len(e.requests[r].generated) for r in rids]
    fail(e)
    outs = e.step()          # reads the step launched ahead; the step launched from here fails
    ops.fail_after_launches(None)
    assert sorted(o.rid for o in outs) == rids and all(o.finished and o.finish_reason == "error" for o in outs)
    assert all(o.token == e.requests[o.rid].generated[-1] for o in outs)
    assert [len(e.requests[r].generated) for r in rids] == [n + 1 for n in n_before]
    assert [e.requests[r].generated for r in rids] == [c[:n + 1] for c, n in zip(clean, n_before)]
    assert e.has_unfinished()
    with pytest.raises((RuntimeError, ops.KernelError), match="injected"):
        e.step()
    assert not e.has_unfinished() and e.step() == []
    m = e.runner.cache.manager
    assert m.live() == 0 and m.free_pages(0) == 32
    m.check()
    assert e.generate(prompts, sp) == clean
    # through generate: the error is the caller's, and the engine goes on afterwards
    e = mk()
    launch = e.sampler.launch

    def failing(*a, **kw):
        if sum(r.ran_ahead for r in e.records) >= 3:       # (the step that asks now is launched ahead as well)
            raise RuntimeError("injected: the sampler")
        return launch(*a, **kw)
    e.sampler.launch = failing
    with pytest.raises(RuntimeError, match="injected"):
        e.generate(prompts, sp)
    e.sampler.launch = launch
    assert all(e.finish_reason(r) == "error" for r in range(3))
    assert [e.requests[r].generated for r in range(3)] == [c[:len(e.requests[r].generated)] for r, c in enumerate(clean)]
    assert all(len(e.requests[r].generated) >= 4 for r in range(3))
    assert not e.has_unfinished() and e.runner.cache.manager.live() == 0
    e.runner.cache.manager.check()
    assert e.generate(prompts, sp) == clean


@pytest.mark.gpu
def test_abort_and_stop_sequence_while_a_step_is_ahead(model_folders):
    """A request is aborted, and another ends by a stop sequence, while the step after is already launched with
    them in it: their pages and slots go back behind that step on the stream, the other requests' tokens are what
    they are without running ahead, and nothing is lost or held twice."""
    from denno_beta_amd.engine import Engine, ModelRunner, SamplingParams
    folder = model_folders("B", "float32")
    words = lambda ids: " ".join(f"t{t}" for t in ids)                          # noqa: E731
    prompts = [seeded_tokens(70 + i, n, 1000) for i, n in enumerate((9, 33, 17, 4))]
    free = SamplingParams(max_tokens=24, temperature=0.0, ignore_eos=True)

    def engine(run_ahead):
        return Engine(ModelRunner.from_folder(folder, options_for("float32", "cuda:0", cache_tokens=512, run_ahead=run_ahead)),
                      detokenize=words)
    full = engine(False).generate(prompts, free)
    stop = f"t{full[1][10]} "
    # (the text of a token ends with a space only once the next token stands behind it)
    k = full[1].index(full[1][10]) + 1      # the token with which the stop sequence first stands in the text
    got = {}
    for run_ahead in (False, True):
        e = engine(run_ahead)
        rids = [e.add_request(p, SamplingParams(max_tokens=24, temperature=0.0, ignore_eos=True,
                                                stop_sequences=(stop,) if i == 1 else ())) for i, p in enumerate(prompts)]
        while e.has_unfinished():
            e.step()
            if len(e.requests[rids[2]].generated) == 6 and not e.requests[rids[2]].finished:
                e.abort(rids[2])            # (with run_ahead the step that holds its seventh token is in flight)
        got[run_ahead] = [(e.requests[r].generated, e.requests[r].finish_reason, e.requests[r].text) for r in rids]
        m = e.runner.cache.manager
        m.check()
        assert m.live() == 0 and m.free_pages(0) == 32
        if run_ahead:
            assert sum(r.ran_ahead for r in e.records) > 10
        # the engine goes on: the same prompts again, nothing stopped, give the full tokens
        assert e.generate(prompts, free) == full
    assert got[True] == got[False]
    assert got[True][1][1] == "stop_sequence" and got[True][1][0] == full[1][:k + 1] and 1 <= k < 23
    assert got[True][2][1] == "aborted" and got[True][2][0] == full[2][:6]
    assert got[True][0][0] == full[0] and got[True][3][0] == full[3]


@pytest.mark.gpu
def test_no_collection_runs_while_a_step_is_captured(model_folders):
    """What of an engine sits in a cycle of references is freed by Python's cyclic collector, whenever its turn
    comes; the finalizers give pinned and device memory back and destroy graphs, which must not happen while
    another engine's stream records a step.  With the collector made eager (a collection at every allocation
    or so), engines are let go one after the other and the next one captures its steps: no collection may
    start during a capture, every engine gives the same tokens, and the collector is left as it was found."""
    import gc
    from denno_beta_amd.engine import SamplingParams
    folder = model_folders("A", "bfloat16")
    prompts = [seeded_tokens(300 + i, n, TINY["A"][0]["vocab_size"]) for i, n in enumerate((9, 30))]
    params = [SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True)] * 2
    during = []

    def watch(phase, info):
        if phase == "start" and torch.cuda.is_current_stream_capturing():
            during.append(info)
    old = gc.get_threshold()
    gc.callbacks.append(watch)
    gc.set_threshold(20, 3, 3)
    try:
        assert gc.isenabled()
        first = None
        for _ in range(3):
            e = engine_for(folder, "bfloat16", "cuda:0")      # graphs are on by default
            got = e.generate(prompts, params)
            assert len(e.runner.graphs.graphs) > 0, "no step was captured"
            first = first or got
            assert got == first
            del e      # garbage now: the next engine's captures run while it waits for the collector
        assert gc.isenabled()
    finally:
        gc.set_threshold(*old)
        gc.callbacks.remove(watch)
    assert during == []


@pytest.mark.gpu
def test_serving_at_large_layer_sizes_gives_each_request_its_solo_tokens(tmp_path):
    """Two layers of GPT-2 Large's sizes, 24 requests with prompts of 16 to 300 tokens admitted into a
    running batch, portions of 64, 200 tokens a step, so few pages that requests are put back: in 32-bit
    every request's tokens are those of its run alone, as interleaved sessions equal solo ones in the
    reference (crates/denno-engine/src/engine.rs:2449-2542)."""
    import torch
    from denno_beta_amd.config import EngineOptions
    from denno_beta_amd.engine import Engine, SamplingParams
    from denno_beta_amd.weights import write_model_folder
    cfg = dict(architectures=["GPT2LMHeadModel"], n_layer=2, n_embd=1280, n_head=20, n_inner=5120, vocab_size=50257,
               n_positions=1024, layer_norm_epsilon=1e-5, activation_function="gelu_new")
    folder = write_model_folder(str(tmp_path), cfg, 3, "float32")
    g = torch.Generator().manual_seed(4)
    lengths = torch.randint(16, 301, (24,), generator=g).tolist()
    prompts = [torch.randint(0, 50257, (n,), generator=g).tolist() for n in lengths]
    sp = SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True)
    mk = lambda **kw: Engine.from_folder(folder, EngineOptions(dtype="float32", page_size=16, **kw))   # noqa: E731
    solo = mk(max_live=1, cache_tokens=1024)
    want = [solo.generate([p], sp)[0] for p in prompts]
    e = mk(max_live=8, cache_tokens=800, prefill_chunk=64, max_batch_tokens=200)
    got = e.generate(prompts, sp)
    assert got == want
    assert sum(1 for r in e.records if r.decode_rows and r.prefill_rows) > 10, "few steps mixed prompts and decoding"
    assert sum(r.preempted for r in e.records) > 0, "the pool was too large: nobody was put back"
    e.runner.cache.manager.check()
    assert e.runner.cache.manager.live() == 0


def test_command_line(backend, model_folders):
    """`denno generate` with the reference's option names; greedy, against the plain implementation."""
    if backend == "cpu":
        pytest.skip("the command line runs the HIP kernels")
    folder = model_folders("A", "float32")
    prompt = seeded_tokens(6, 9, 512)
    want = PlainGPT2.from_folder(folder).greedy(prompt, 8)
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "denno"), "generate", folder, "--prompt-ids",
                          ",".join(map(str, prompt)), "--max-tokens", "8", "--temperature", "0", "--quant", "fp32",
                          "--raw"], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr
    assert [int(t) for t in out.stdout.strip().split(",")] == want


def test_command_line_with_several_prompts(backend, model_folders, tmp_path):
    """`denno generate --prompt-file`: five prompts through the scheduler at once, with three live
    requests, portions of 8 tokens, 20 tokens a step and so few pages that requests wait or are put
    back: every line equals the prompt's run alone."""
    if backend == "cpu":
        pytest.skip("the command line runs the HIP kernels")
    folder = model_folders("A", "float32")
    prompts = [seeded_tokens(30 + i, n, 512) for i, n in enumerate((9, 40, 17, 3, 60))]
    plain = PlainGPT2.from_folder(folder)
    want = [plain.greedy(p, 6) for p in prompts]
    path = tmp_path / "prompts.txt"
    path.write_text("".join((", " if i % 2 else " ").join(map(str, p)) + "\n" for i, p in enumerate(prompts)))
    for policy in ("preempt", "reserve"):
        out = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "denno"), "generate", folder, "--prompt-file",
                              str(path), "--max-tokens", "6", "--temperature", "0", "--quant", "fp32", "--raw",
                              "--max-live", "3", "--page-size", "16", "--cache-tokens", "128", "--prefill-chunk", "8",
                              "--max-batch-tokens", "20", "--kv-policy", policy], capture_output=True, text=True,
                             timeout=300)
        assert out.returncode == 0, out.stderr
        got = [[int(t) for t in line.split(",")] for line in out.stdout.strip().splitlines()]
        assert got == want, policy


def test_command_line_with_text(backend, model_folders, tmp_path):
    """`denno generate <model> --prompt TEXT`: the folder's tokenizer.json, the reference's fallback
    template for models without one ("user: ..\\n\\nassistant:", crates/denno-engine/src/tokenizer.rs:226-236),
    and `--raw` without it."""
    if backend == "cpu":
        pytest.skip("the command line runs the HIP kernels")
    import shutil
    from tokenizers import Tokenizer
    from tokenizers.models import WordLevel
    from tokenizers.pre_tokenizers import WhitespaceSplit
    from denno_beta_amd.cli import fallback_template
    folder = str(tmp_path / "with_tokenizer")
    shutil.copytree(model_folders("A", "float32"), folder)
    words = ["[UNK]", "user:", "assistant:", "system:", "hello", "world", "be", "nice"] + [f"w{i}" for i in range(504)]
    tok = Tokenizer(WordLevel({w: i for i, w in enumerate(words)}, unk_token="[UNK]"))
    tok.pre_tokenizer = WhitespaceSplit()
    tok.save(os.path.join(folder, "tokenizer.json"))
    plain = PlainGPT2.from_folder(folder)
    run = lambda *extra: subprocess.run(   # noqa: E731
        [sys.executable, os.path.join(ROOT, "bin", "denno"), "generate", folder, "--prompt", "hello world",
         "--max-tokens", "5", "--temperature", "0", "--quant", "fp32", *extra], capture_output=True, text=True, timeout=300)
    for extra, text in (((), fallback_template(None, "hello world")), (("--raw",), "hello world"),
                        (("--system", "be nice"), fallback_template("be nice", "hello world"))):
        out = run(*extra)
        assert out.returncode == 0, out.stderr
        ids = tok.encode(text).ids
        assert out.stdout.strip() == tok.decode(plain.greedy(ids, 5)), extra
    # --stop: the text ends where the stop sequence begins
    whole = tok.decode(plain.greedy(tok.encode("hello world").ids, 5))
    third = whole.split()[2]
    out = run("--raw", "--stop", third, "--stop", "never")
    assert out.returncode == 0, out.stderr
    assert out.stdout.strip() == whole[:whole.find(third)].strip() and third not in out.stdout
    assert fallback_template(None, "hello") == "user: hello\n\nassistant:"          # tokenizer.rs:319-324
    assert fallback_template("be nice", "hi") == "system: be nice\n\nuser: hi\n\nassistant:"
