"""The same requests replayed in every way of cutting the work, compared with the plain
implementation: whole; most in one step and the last 32 tokens one by one; portions of
changing size down to two tokens; mixed, up to four live requests with so few pages that
they are used again.  In 32-bit and in bfloat16.

Backend "gpu" runs the HIP kernels; backend "host" runs the same engine code on the CPU with
the kernels' plain references in their place, so the cache and batch logic is tested where
there is no GPU.
"""
import pytest
import torch

import replay_util as U
from conftest import TINY, seeded_tokens
from plain.gpt2_plain import PlainGPT2

def runner_for(folder, dtype, device, cache_tokens, page_size=16, max_live=4):
    from denno_beta_amd.config import EngineOptions
    from denno_beta_amd.engine import ModelRunner
    return ModelRunner.from_folder(folder, EngineOptions(dtype=dtype, device=device, page_size=page_size,
                                                         cache_tokens=cache_tokens, max_live=max_live))


_plain_cache = {}


def plain_logits(folder, seqs):
    out = []
    for s in seqs:
        key = (folder, tuple(s))
        if key not in _plain_cache:
            _plain_cache[key] = PlainGPT2.from_folder(folder).logits(s)
        out.append(_plain_cache[key])
    return out


def sequences(name, lengths, seed=11):
    vocab = TINY[name][0]["vocab_size"]
    return [seeded_tokens(seed + i, n, vocab) for i, n in enumerate(lengths)]


CASES = [("A", "float32", (7, 19, 33, 100)), ("B", "float32", (1, 50, 120, 200)),
         ("A", "bfloat16", (7, 19, 33, 100)), ("B", "bfloat16", (1, 50, 120, 200))]


@pytest.mark.parametrize("name,dtype,lengths", CASES)
def test_every_cutting_matches_the_plain_implementation(backend, model_folders, name, dtype, lengths):
    if backend == "cpu" and (dtype == "bfloat16" or name == "B"):
        lengths = lengths[:3] if name == "A" else (1, 50, 70)    # the host backend is slow
    folder = model_folders(name, dtype)
    seqs = sequences(name, lengths)
    want = plain_logits(folder, seqs)
    traces = {"whole": U.whole_trace(seqs), "tail": U.tail_decode_trace(seqs, 32),
              "chunks": U.chunk_trace(seqs), "mixed": U.mixed_trace(seqs, seed=5)}
    results = {}
    for kind, steps in traces.items():
        tokens = U.max_live_tokens(steps)
        r = runner_for(folder, dtype, backend, cache_tokens=tokens)
        got = U.replay(r, steps)
        r.cache.manager.check()
        assert r.cache.manager.live() == 0 and r.cache.manager.free_pages(0) == -(-tokens // 16)
        if kind == "mixed":
            assert r.cache.manager.reuse_count(0) > 0, "the pool was too large: no page was used again"
        for i in range(len(seqs)):
            U.assert_close(got[f"r{i}"], want[i], dtype, f"{name} {dtype} {kind} request {i}")
        results[kind] = got
    # the same (request, position) agrees across the cuttings: in 32-bit to the last bit, since a
    # row's sums have one order whatever else is in the batch
    for kind in ("tail", "chunks", "mixed"):
        for i in range(len(seqs)):
            a, b = results["whole"][f"r{i}"], results[kind][f"r{i}"]
            if dtype == "float32" and backend != "cpu":
                assert torch.equal(a, b), f"{name} {kind} request {i}: 32-bit logits depend on the cutting"
            else:
                U.assert_close(b, a, dtype, f"{name} {dtype} {kind} vs whole, request {i}")


def _cfg(L, E, H, I, V, P, eps=1e-5, act="gelu_new", inv=False):
    return dict(architectures=["GPT2LMHeadModel"], model_type="gpt2", n_layer=L, n_embd=E, n_head=H, n_inner=I,
                vocab_size=V, n_positions=P, layer_norm_epsilon=eps, activation_function=act,
                scale_attn_by_inverse_layer_idx=inv)


OTHER_SIZES = {
    "one head of 80": _cfg(1, 80, 1, 320, 101, 160, 1e-3),                        # a key on 10 of the decode kernel's 16 lanes
    "three heads of 112": _cfg(2, 336, 3, 1000, 777, 200, 1e-6, "gelu", True),    # on 14 of 16; widths no multiple of 32
    "two heads of 208": _cfg(1, 416, 2, 800, 500, 200),                           # on 26 of 32; the portions' kernel with a CU to itself
    "three heads of 16": _cfg(4, 48, 3, 64, 50, 130),                             # a feed-forward narrower than 4 E
    "two heads of 256": _cfg(1, 512, 2, 2048, 1000, 300),                         # the largest head size
    "five heads of 48": _cfg(2, 240, 5, 960, 333, 260, 1e-5, "gelu", True),
}


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(OTHER_SIZES))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_other_head_sizes_and_widths(tmp_path, name, dtype):
    """Every head size in steps of 16 has its kernels (in bfloat16 the MFMA kernel for portions and the split
    kernel for decode steps, whose lanes a head size that is no power of two does not fill), and widths need be
    no multiple of 32: four cuttings of four requests each, one of them to the last position but two."""
    from denno_beta_amd.weights import write_model_folder
    cfg = OTHER_SIZES[name]
    folder = str(tmp_path)
    write_model_folder(folder, cfg, 7, "float32")
    P = cfg["n_positions"]
    seqs = [seeded_tokens(20 + i, n, cfg["vocab_size"]) for i, n in enumerate((7, 70, P - 3, 40))]
    want = plain_logits(folder, seqs)
    for kind, steps in (("whole", U.whole_trace(seqs)), ("tail", U.tail_decode_trace(seqs, 32)),
                        ("chunks", U.chunk_trace(seqs)), ("mixed", U.mixed_trace(seqs, seed=5))):
        r = runner_for(folder, dtype, "cuda:0", cache_tokens=U.max_live_tokens(steps))
        got = U.replay(r, steps)
        r.cache.manager.check()
        for i in range(len(seqs)):
            U.assert_close(got[f"r{i}"], want[i], dtype, f"{name} {dtype} {kind} request {i}")


ODD_SIZES = {
    "four heads of 15": _cfg(2, 60, 4, 100, 301, 96),                       # nothing a multiple of 8
    "three heads of 22": _cfg(3, 66, 3, 150, 77, 80, 1e-6, "gelu", True),   # an inner size that no 4 divides
    "one head of 100": _cfg(1, 100, 1, 36, 129, 72),                        # padded to 112 in the kernel, a narrow feed-forward
}


@pytest.mark.parametrize("name", list(ODD_SIZES))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sizes_that_are_multiples_of_nothing(backend, tmp_path, name, dtype):
    """The architecture's forward runs any width, inner size and head size (gpt2.rs:138, the plain loops
    :170-202): so do the plain kernels, which both engines fall to for sizes that the matrix-core kernels do
    not take (a head size that is no multiple of 16, an inner size of a product that is no multiple of 8).
    Four cuttings; 32-bit logits equal bit for bit across them."""
    from denno_beta_amd.weights import write_model_folder
    cfg = ODD_SIZES[name]
    folder = str(tmp_path)
    write_model_folder(folder, cfg, 9, dtype)
    P = cfg["n_positions"]
    seqs = [seeded_tokens(40 + i, n, cfg["vocab_size"]) for i, n in enumerate((5, 50, P - 2, 33))]
    if backend == "cpu":
        seqs = seqs[:3]
    want = plain_logits(folder, seqs)
    whole = None
    for kind, steps in (("whole", U.whole_trace(seqs)), ("tail", U.tail_decode_trace(seqs, 32)),
                        ("chunks", U.chunk_trace(seqs)), ("mixed", U.mixed_trace(seqs, seed=5))):
        r = runner_for(folder, dtype, backend, cache_tokens=U.max_live_tokens(steps))
        got = U.replay(r, steps)
        r.cache.manager.check()
        for i in range(len(seqs)):
            U.assert_close(got[f"r{i}"], want[i], dtype, f"{name} {dtype} {kind} request {i}")
            if dtype == "float32" and backend != "cpu" and whole is not None:
                assert torch.equal(got[f"r{i}"], whole[f"r{i}"]), f"{name} {kind} request {i}: 32-bit logits depend on the cutting"
        if whole is None:
            whole = got


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_and_first_tokens(backend, model_folders, dtype):
    """A sequence decoded token by token from its first token on, across many pages."""
    n = 60 if backend == "cpu" else 600
    folder = model_folders("C", dtype)
    seq = sequences("C", (n,))[0]
    want = plain_logits(folder, [seq])[0]
    steps = [{"step": i, "entries": [{"id": "a", "tokens": [t], "want": [0]}], "end": []} for i, t in enumerate(seq)]
    r = runner_for(folder, dtype, backend, cache_tokens=-(-n // 64) * 64)
    got = U.replay(r, steps)["a"]
    U.assert_close(got[:4], want[:4], dtype, "the first tokens")
    U.assert_close(got, want, dtype, "long decoding")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("page_size", [16, 32, 64])
def test_page_sizes(backend, model_folders, page_size, dtype):
    """Pages of 32 and 64 tokens through the whole engine, in both precisions: a mixed trace (portions and
    single tokens: in bfloat16 the kernel for portions and the kernel for single rows), and the last tokens
    one by one."""
    if backend == "cpu" and dtype == "bfloat16":
        pytest.skip("the host backend is slow; bfloat16 pages are a matter of the GPU kernels")
    folder = model_folders("A", dtype)
    seqs = sequences("A", (70, 45, 128))
    want = plain_logits(folder, seqs)
    for steps in (U.mixed_trace(seqs, seed=2), U.tail_decode_trace(seqs, 20)):
        tokens = -(-U.max_live_tokens(steps) // page_size) * page_size
        r = runner_for(folder, dtype, backend, cache_tokens=tokens, page_size=page_size)
        got = U.replay(r, steps)
        r.cache.manager.check()
        for i in range(len(seqs)):
            U.assert_close(got[f"r{i}"], want[i], dtype, f"page size {page_size} {dtype} request {i}")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("page_size", [8, 48])
def test_pages_that_do_not_divide_the_positions(tmp_path, page_size, dtype):
    """130 positions in pages of 8 or 48 tokens: a request's block table holds whole pages (136 or 144 keys), and the
    bucket of contexts that a captured decode step is made for stays within them.  Requests decoded to their last
    position."""
    from denno_beta_amd.weights import write_model_folder
    cfg = _cfg(2, 64, 4, 128, 97, 130)
    folder = write_model_folder(str(tmp_path), cfg, 3, dtype)
    seqs = [seeded_tokens(60 + i, n, 97) for i, n in enumerate((130, 77, 129))]
    want = plain_logits(folder, seqs)
    for steps in (U.tail_decode_trace(seqs, 40), U.mixed_trace(seqs, seed=4)):
        tokens = -(-U.max_live_tokens(steps) // page_size) * page_size
        r = runner_for(folder, dtype, "cuda:0", cache_tokens=tokens + 2 * page_size, page_size=page_size)
        got = U.replay(r, steps)
        r.cache.manager.check()
        for i in range(len(seqs)):
            U.assert_close(got[f"r{i}"], want[i], dtype, f"page size {page_size} {dtype} request {i}")


def test_step_refuses_what_it_cannot_run(backend, model_folders):
    from denno_beta_amd.cache import OutOfPages
    from denno_beta_amd.engine import BatchError, StepEntry
    r = runner_for(model_folders("A", "float32"), "float32", backend, cache_tokens=64)
    r.start_request(0)
    with pytest.raises(BatchError, match="vocabulary"):
        r.step([StepEntry(0, [5, 512], [0])])
    with pytest.raises(BatchError, match="positions"):
        r.step([StepEntry(0, [1] * 129, [])])
    with pytest.raises(BatchError, match="twice"):
        r.step([StepEntry(0, [1], []), StepEntry(0, [2], [])])
    with pytest.raises(BatchError, match="wanted place"):
        r.step([StepEntry(0, [1, 2], [2])])
    with pytest.raises(OutOfPages):
        r.step([StepEntry(0, [1] * 65, [])])
    # nothing of the refused steps has stayed: the request is still empty and runs
    assert r.cache.manager.length(0) == 0
    assert r.step([StepEntry(0, [1, 2, 3], [2])]).shape == (1, 512)
    assert r.cache.manager.length(0) == 3


def test_a_refused_step_leaves_nothing_of_the_requests_it_started(backend, model_folders):
    """A replayed step that cannot run (a token outside the vocabulary, a request named twice, no pages
    left) gives back the slots of the requests that it started; requests that were live before stay."""
    from denno_beta_amd.cache import OutOfPages
    from denno_beta_amd.engine import BatchError
    from denno_beta_amd.engine.replay import TraceReplayer
    r = runner_for(model_folders("A", "float32"), "float32", backend, cache_tokens=64, max_live=2)
    rp = TraceReplayer(r)
    rp.run_step({"step": 0, "entries": [{"id": "old", "tokens": [1, 2, 3], "want": []}], "end": []})
    for bad, error in (([{"id": "new", "tokens": [5, 512], "want": []}], BatchError),
                       ([{"id": "new", "tokens": [5], "want": []}, {"id": "new", "tokens": [6], "want": []}], BatchError),
                       ([{"id": "new", "tokens": [1] * 60, "want": []}], OutOfPages)):
        with pytest.raises(error):
            rp.run_step({"step": 1, "entries": bad, "end": []})
        assert rp.live() == ["old"] and r.cache.manager.live() == 1
        r.cache.manager.check()
    # the slot that the refused requests took and gave back serves the next one
    out = rp.run_step({"step": 2, "entries": [{"id": "new", "tokens": [7, 8], "want": [1]},
                                              {"id": "old", "tokens": [4], "want": [0]}], "end": ["new", "old"]})
    assert out.shape == (2, 512) and rp.live() == [] and r.cache.manager.live() == 0
    r.cache.manager.check()


def test_an_entry_without_tokens_is_a_request_left_out(backend, model_folders):
    from denno_beta_amd.engine.replay import TraceReplayer
    r = runner_for(model_folders("A", "float32"), "float32", backend, cache_tokens=64, max_live=2)
    rp = TraceReplayer(r)
    a = rp.run_step({"step": 0, "entries": [{"id": "a", "tokens": [1, 2, 3], "want": [2]},
                                            {"id": "b", "tokens": [], "want": []}], "end": []})
    assert a.shape == (1, 512) and rp.live() == ["a"]          # "b" has not begun
    assert rp.run_step({"step": 1, "entries": [{"id": "a", "tokens": [], "want": []}], "end": []}) is None
    assert r.cache.manager.length(0) == 3
    with pytest.raises(ValueError, match="does not bring"):
        rp.run_step({"step": 2, "entries": [{"id": "a", "tokens": [], "want": [0]}], "end": []})
    b = rp.run_step({"step": 3, "entries": [{"id": "a", "tokens": [4], "want": [0]}], "end": ["a"]})
    assert b.shape == (1, 512) and rp.live() == [] and r.cache.manager.live() == 0


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_graphs_replay_what_eager_steps_compute(model_folders, dtype):
    """Decode steps come from captured HIP graphs.  Every replay is checked against the same step
    run kernel by kernel, over several batch sizes and context lengths, with eager steps (prompts
    of other requests) and synchronisations between the replays."""
    from denno_beta_amd.config import EngineOptions
    from denno_beta_amd.engine import ModelRunner, StepEntry
    folder = model_folders("C", dtype)
    vocab = TINY["C"][0]["vocab_size"]
    mk = lambda graphs: ModelRunner.from_folder(folder, EngineOptions(   # noqa: E731
        dtype=dtype, page_size=16, cache_tokens=4096, max_live=8, use_graphs=graphs))
    a, b = mk(True), mk(False)
    assert a.graphs is not None and b.graphs is None
    seqs = [seeded_tokens(70 + i, n, vocab) for i, n in enumerate((300, 5, 250, 40, 90))]
    fed = [0] * len(seqs)
    live = []
    for step in range(70):
        if step % 12 == 0 and len(live) < len(seqs):          # a new request: its prompt runs eagerly in both
            i = len(live)
            live.append(i)
            n = max(1, min(len(seqs[i]) - 60, 260))
            for r in (a, b):
                r.start_request(i)
                r.step([StepEntry(i, seqs[i][:n], [])])
            fed[i] = n
        entries = [StepEntry(i, seqs[i][fed[i]:fed[i] + 1], [0]) for i in live if fed[i] < len(seqs[i]) and (step + i) % 5]
        if not entries:
            continue
        la, lb = a.step(entries).cpu(), b.step(entries).cpu()
        for e in entries:
            fed[e.rid] += 1
        assert torch.equal(la, lb), f"step {step}: a replayed graph differs from the eager step"
        if step % 7 == 0:
            torch.cuda.synchronize()
    assert len(a.graphs.graphs) >= 3, "several batch and context buckets were to be captured"


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_context_with_heads_of_64(model_folders, dtype):
    """The head size and context length of the large models: a 1,000-token request in portions, with
    decoding at the end, beside a second request, so that the keys of a row span dozens of pages."""
    folder = model_folders("D", dtype)
    seqs = sequences("D", (1000, 300))
    want = plain_logits(folder, seqs)
    steps = U.mixed_trace(seqs, seed=4, sizes=(1, 1, 2, 64, 200, 333))
    r = runner_for(folder, dtype, "cuda:0", cache_tokens=U.max_live_tokens(steps))
    got = U.replay(r, steps)
    for i in range(2):
        U.assert_close(got[f"r{i}"], want[i], dtype, f"long context {dtype} request {i}")


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["C", "D"])
@pytest.mark.parametrize("graphs", [False, True])
def test_twenty_requests_decode_together(model_folders, name, graphs):
    """Steps of 17 to 64 rows hand their bfloat16 rows from kernel to kernel in the packed layout
    (LayerNorm, the decode attention and the first feed-forward product write it, the few-rows
    product reads it).  C's feed-forward width is no multiple of 32, so its second product takes
    ordinary rows; D packs all of them."""
    from denno_beta_amd.config import EngineOptions
    from denno_beta_amd.engine import ModelRunner, StepEntry
    folder = model_folders(name, "bfloat16")
    seqs = sequences(name, (40, 25, 70, 33, 90, 21, 58, 64, 30, 47, 36, 81, 22, 55, 73, 38, 61, 27, 44, 66), seed=40)
    n = len(seqs)
    want = plain_logits(folder, seqs)
    r = ModelRunner.from_folder(folder, EngineOptions(dtype="bfloat16", page_size=16, cache_tokens=n * 96,
                                                      max_live=n, use_graphs=graphs))
    assert r.model.blocks[0].mixer.packed_input(n) and not r.model.blocks[0].mixer.packed_input(16)
    assert r.model.blocks[0].ffn.down.packed_input(n) == (name == "D")
    for i in range(n):
        r.start_request(i)
    tail = 20
    got = r.step([StepEntry(i, s[:-tail], list(range(len(s) - tail))) for i, s in enumerate(seqs)]).cpu()
    at = 0
    for i, s in enumerate(seqs):
        U.assert_close(got[at:at + len(s) - tail], want[i][:len(s) - tail], "bfloat16", f"prompt of request {i}")
        at += len(s) - tail
    for j in range(tail, 0, -1):
        got = r.step([StepEntry(i, [s[len(s) - j]], [0]) for i, s in enumerate(seqs)]).cpu()
        for i, s in enumerate(seqs):
            U.assert_close(got[i:i + 1], want[i][len(s) - j:len(s) - j + 1], "bfloat16", f"request {i}, {j} from its end")


@pytest.mark.gpu
@pytest.mark.parametrize("name,n", [("E", 20), ("E", 64), ("F", 17), ("F", 40), ("F", 64)])
def test_up_to_64_requests_on_wide_layers(model_folders, name, n):
    """Steps of 17 to 64 rows of models whose layers are 1,024 columns wide or more: the norms between
    the products run inside them (counted: two a layer, less the first layer's first), the rows travel
    packed.  Every request decodes from its second token on; at the end some requests have ended."""
    from denno_beta_amd.config import EngineOptions
    from denno_beta_amd.engine import ModelRunner, StepEntry
    from denno_beta_amd.kernels import ops
    folder = model_folders(name, "bfloat16")
    layers = TINY[name][0]["n_layer"]
    seqs = sequences(name, [7] * n, seed=70)
    want = plain_logits(folder, seqs)
    calls = []
    real = ops.linear_norm_in
    ops.linear_norm_in = lambda *a, **k: (calls.append(a[0].shape[0]), real(*a, **k))[1]
    try:
        r = ModelRunner.from_folder(folder, EngineOptions(dtype="bfloat16", page_size=16, cache_tokens=n * 16,
                                                          max_live=n, use_graphs=False))
        for i in range(n):
            r.start_request(i)
        for i in range(0, n, 8):       # the first tokens, eight requests to a step
            got = r.step([StepEntry(k, seqs[k][:1], [0]) for k in range(i, min(i + 8, n))]).cpu()
            for k in range(i, min(i + 8, n)):
                U.assert_close(got[k - i:k - i + 1], want[k][:1], "bfloat16", f"first token of request {k}")
        alive = list(range(n))
        for j in range(1, 7):
            calls.clear()
            got = r.step([StepEntry(i, [seqs[i][j]], [0]) for i in alive]).cpu()
            assert calls == [len(alive)] * (2 * layers - 1), calls
            for row, i in enumerate(alive):
                U.assert_close(got[row:row + 1], want[i][j:j + 1], "bfloat16", f"request {i}, token {j}")
            if j == 3:                 # a third of them ends: fewer rows, another kernel shape
                for i in alive[::3]:
                    r.end_request(i)
                alive = [i for i in alive if i % 3 != 0]
    finally:
        ops.linear_norm_in = real


@pytest.mark.gpu
@pytest.mark.parametrize("n", [150, 230])
def test_many_requests_on_a_wide_layer(model_folders, n):
    """Steps of 129 to 256 rows of a model whose products are wide: the rows stay packed from kernel to
    kernel, the two products with many columns go to the many-rows kernel (the projection with its
    cache write among them), the other two to the few-rows kernel.  The prompts run in one step of
    three rows each (more than 256 rows: ordinary rows), then every request decodes."""
    from denno_beta_amd.config import EngineOptions
    from denno_beta_amd.engine import ModelRunner, StepEntry
    folder = model_folders("E", "bfloat16")
    seqs = sequences("E", [7] * n, seed=90)
    want = plain_logits(folder, seqs)
    r = ModelRunner.from_folder(folder, EngineOptions(dtype="bfloat16", page_size=16, cache_tokens=n * 16,
                                                      max_live=n, use_graphs=False))
    assert r.model.blocks[0].mixer.packed_input(n) and r.model.blocks[0].ffn.down.packed_input(n)
    for i in range(n):
        r.start_request(i)
    got = r.step([StepEntry(i, s[:3], [0, 1, 2]) for i, s in enumerate(seqs)]).cpu()
    for i in range(n):
        U.assert_close(got[3 * i:3 * i + 3], want[i][:3], "bfloat16", f"prompt of request {i}")
    for j in range(3, 7):
        got = r.step([StepEntry(i, [s[j]], [0]) for i, s in enumerate(seqs)]).cpu()
        for i in range(n):
            U.assert_close(got[i:i + 1], want[i][j:j + 1], "bfloat16", f"request {i}, token {j}")


def test_weights_stored_in_32_bit_stay_so_in_a_bfloat16_engine(backend, model_folders):
    """A folder stored in 32-bit, run with --dtype bfloat16: the matrices stay 32-bit and their
    products run in 32-bit on widened activations; the result is at least as close to the plain
    implementation as with bfloat16 weights."""
    folder = model_folders("A", "float32")
    seqs = sequences("A", (40, 23))
    want = plain_logits(folder, seqs)
    steps = U.mixed_trace(seqs, seed=6)
    r = runner_for(folder, "bfloat16", backend, cache_tokens=U.max_live_tokens(steps))
    assert r.notes and r.model.blocks[0].mixer.qkv.weight.dtype == torch.float32
    got = U.replay(r, steps)
    for i in range(2):
        U.assert_close(got[f"r{i}"], want[i], "bfloat16", f"32-bit weights in a bfloat16 engine, request {i}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sharp_attention_shows_a_wrong_key(backend, model_folders, tmp_path, dtype):
    """Random weights give nearly flat attention, which hides a key read from the wrong place.  With
    the query and key weights scaled up each row attends to a few keys only, so one misplaced
    key (a page's edge, a reused page, the start of a portion) changes the logits visibly."""
    from safetensors.torch import load_file, save_file
    import shutil
    src = model_folders("A", dtype)
    dst = str(tmp_path / "sharp")
    shutil.copytree(src, dst)
    t = load_file(dst + "/model.safetensors")
    for i in range(2):
        w = t[f"h.{i}.attn.c_attn.weight"].float()
        w[:, :128] *= 12.0          # the query and key columns of the fused projection
        t[f"h.{i}.attn.c_attn.weight"] = w.to(t[f"h.{i}.attn.c_attn.weight"].dtype)
    save_file(t, dst + "/model.safetensors")
    lengths = (90, 33, 128, 64, 50) if backend != "cpu" else (40, 33, 50)
    seqs = sequences("A", lengths, seed=31)
    plain = PlainGPT2.from_folder(dst)
    want = [plain.logits(s) for s in seqs]
    # attention is sharp indeed: some row of the first layer puts most of its weight on one key
    steps = U.mixed_trace(seqs, seed=8)
    r = runner_for(dst, dtype, backend, cache_tokens=U.max_live_tokens(steps))
    got = U.replay(r, steps)
    assert r.cache.manager.reuse_count(0) > 0
    for i in range(len(seqs)):
        U.assert_close(got[f"r{i}"], want[i], dtype, f"sharp attention {dtype} request {i}")
    # and the logits do depend on a far token: changing token 3 changes the last row
    changed = list(seqs[0])
    changed[3] = (changed[3] + 1) % 512
    assert (plain.logits(changed)[-1] - want[0][-1]).abs().max() > 1e-3


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_steps_with_portions_are_replayed_from_graphs(model_folders, dtype):
    """A step that holds portions is captured as a graph when its bucket (rows, requests, wanted rows) comes a
    second time, over buffers of the bucket's size with padding rows, requests and tiles.  The same traces with
    and without: 32-bit logits equal bit for bit, bfloat16 within rounding (a bucket's rows may choose another
    kernel than the real rows would); every graph replayed several times over other requests, other pages and
    other positions, with steps that run kernel by kernel in between."""
    from denno_beta_amd.config import EngineOptions
    from denno_beta_amd.engine import ModelRunner
    name = "B"
    folder = model_folders(name, dtype)
    seqs = sequences(name, (60, 200, 33, 120, 97, 250), seed=31)
    want = plain_logits(folder, seqs)
    traces = {"chunks": U.chunk_trace(seqs, sizes=(17, 2, 40, 17, 3, 64, 40, 2, 17)),
              "mixed": U.mixed_trace(seqs, seed=8, sizes=(1, 1, 2, 17, 17, 40))}
    for kind, steps in traces.items():
        got = {}
        for on in (True, False):
            r = ModelRunner.from_folder(folder, EngineOptions(dtype=dtype, page_size=16, max_live=4, graph_portions=on,
                                                              cache_tokens=U.max_live_tokens(steps)))
            got[on] = U.replay(r, steps)
            r.cache.manager.check()
            assert r.cache.manager.live() == 0
            if on:
                assert len(r.graphs.portions) >= 3, sorted(r.graphs.portions)
                replayed = sum(n - 1 for key, n in r.graphs.seen.items() if key in r.graphs.portions)
                assert replayed >= len(r.graphs.portions) + 5
                # (every bucket's first step ran kernel by kernel, between the replays of the buckets before it)
                if kind == "mixed":
                    assert r.cache.manager.reuse_count(0) > 0
            else:
                assert not r.graphs.portions
        for i in range(len(seqs)):
            U.assert_close(got[True][f"r{i}"], want[i], dtype, f"portions from graphs, {dtype}, {kind}, request {i}")
            if dtype == "float32":
                assert torch.equal(got[True][f"r{i}"], got[False][f"r{i}"]), (kind, i)
            else:
                U.assert_close(got[True][f"r{i}"], got[False][f"r{i}"], dtype, f"graphs against kernel by kernel, {kind}, request {i}")
