"""The four cuttings at the layer sizes that the measurements run, against the plain implementation:
two layers of GPT-2 XL's sizes (1,600 wide, 25 heads, a feed-forward of 6,400, a vocabulary of 50,257,
1,024 positions) and two of GPT-2 Medium's (1,024 wide, 16 heads, the same vocabulary).  The tiny models are too narrow for
some of the kernels that serve these widths: steps of 17 to 64 rows whose norms run inside the products
beside them, steps of 65 to 256 rows whose rows travel packed between kernels, the many-rows kernels
beyond that.  A mixed trace here holds portions of prompts beside decoded tokens in steps of every one
of those sizes, with so few pages that they are used again; a sequence fills all 1,024 positions.
"""
import pytest
import torch

import replay_util as U
from conftest import seeded_tokens
from plain.gpt2_plain import PlainGPT2

pytestmark = pytest.mark.gpu


def _cfg(L, E, H, V, P=1024):
    return dict(architectures=["GPT2LMHeadModel"], model_type="gpt2", n_layer=L, n_embd=E, n_head=H,
                vocab_size=V, n_positions=P, layer_norm_epsilon=1e-5, activation_function="gelu_new")


SHAPES = {"xl": (_cfg(2, 1600, 25, 50257), 21, (1024, 600, 257, 130, 64)),
          "medium": (_cfg(2, 1024, 16, 50257), 22, (1024, 333, 600, 96, 150))}

_made = {}


@pytest.fixture(scope="module")
def real_folder(tmp_path_factory):
    from denno_beta_amd.weights import write_model_folder

    def get(shape, dtype):
        if (shape, dtype) not in _made:
            d = str(tmp_path_factory.mktemp(f"{shape}_{dtype}"))
            write_model_folder(d, SHAPES[shape][0], SHAPES[shape][1], dtype)
            _made[(shape, dtype)] = d
        return _made[(shape, dtype)]
    return get


_plain = {}


def plain_logits(folder, shape, dtype, seqs):
    key = (shape, dtype)
    if key not in _plain:
        model = PlainGPT2.from_folder(folder)
        _plain[key] = [model.logits(s) for s in seqs]
    return _plain[key]


def rows_of(step):
    return sum(len(e["tokens"]) for e in step["entries"])


def is_mixed(step):
    """A portion of a prompt beside a decoded token."""
    return any(len(e["tokens"]) == 1 for e in step["entries"]) and any(len(e["tokens"]) > 1 for e in step["entries"])


def wide_mixed_trace(seqs):
    """Up to four live requests; the sizes make steps of 17 to 64 rows, of 65 to 256 rows and of more,
    with portions beside single tokens in each."""
    return U.mixed_trace(seqs, seed=9, sizes=(1, 1, 1, 2, 9, 20, 33, 70, 140, 300))


def runner_for(folder, dtype, cache_tokens, graphs=True):
    from denno_beta_amd.config import EngineOptions
    from denno_beta_amd.engine import ModelRunner
    return ModelRunner.from_folder(folder, EngineOptions(dtype=dtype, page_size=16, cache_tokens=cache_tokens,
                                                         max_live=4, use_graphs=graphs))


# What bfloat16 may differ by at these sizes.  Logits here have a spread (standard deviation over a
# row) of about 0.8 (XL) and 0.64 (Medium); every activation between kernels is rounded to 8 bits of
# mantissa, which measured 0.028 of a row's spread at worst over all logits of all cuttings and 0.0039
# of it on average.  The bound is on the worst logit, relative to the row's spread, and on the mean.
BF16_WORST, BF16_MEAN = 0.035, 0.006


def check(got, want, dtype, what):
    if dtype == "float32":
        U.assert_close(got, want, "float32", what)
        return
    spread = want.std(dim=1, keepdim=True)
    diff = (got - want).abs() / spread
    worst, mean = diff.max().item(), diff.mean().item()
    assert worst <= BF16_WORST and mean <= BF16_MEAN, (
        f"{what}: bfloat16 logits differ from the plain ones by {worst:.4f} of a row's spread at worst "
        f"(position {int(diff.max(dim=1).values.argmax())}), {mean:.5f} on average")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", ["xl", "medium"])
def test_every_cutting_at_real_layer_sizes(real_folder, shape, dtype):
    cfg, _, lengths = SHAPES[shape]
    folder = real_folder(shape, dtype)
    seqs = [seeded_tokens(300 + i, n, cfg["vocab_size"]) for i, n in enumerate(lengths)]
    want = plain_logits(folder, shape, dtype, seqs)
    traces = {"whole": U.whole_trace(seqs), "tail": U.tail_decode_trace(seqs, 32),
              "chunks": U.chunk_trace(seqs, sizes=(2, 128, 3, 17, 2, 64, 128, 7, 40, 128, 2, 31)),
              "mixed": wide_mixed_trace(seqs)}
    mixed = traces["mixed"]
    for lo, hi in ((17, 64), (65, 256), (257, 4096)):
        assert any(lo <= rows_of(st) <= hi and is_mixed(st) for st in mixed), f"no mixed step of {lo} to {hi} rows"
    whole = None
    for kind, steps in traces.items():
        tokens = U.max_live_tokens(steps)
        r = runner_for(folder, dtype, tokens)
        got = U.replay(r, steps)
        r.cache.manager.check()
        assert r.cache.manager.live() == 0 and r.cache.manager.free_pages(0) == tokens // 16
        if kind == "mixed":
            assert r.cache.manager.reuse_count(0) > 0, "the pool was too large: no page was used again"
        for i in range(len(seqs)):
            check(got[f"r{i}"], want[i], dtype, f"{shape} {dtype} {kind} request {i}")
        if kind == "whole":
            whole = got
        else:
            for i in range(len(seqs)):
                a, b = whole[f"r{i}"], got[f"r{i}"]
                if dtype == "float32":
                    assert torch.equal(a, b), f"{shape} {kind} request {i}: 32-bit logits depend on the cutting"
                else:
                    # the plain implementation's greedy token, wherever its lead over the runner-up is
                    # clear of the rounding, is the engine's in every cutting
                    top2 = want[i].topk(2, dim=1).values
                    clear = (top2[:, 0] - top2[:, 1]) > 2 * BF16_WORST * want[i].std(dim=1)
                    assert bool((b.argmax(dim=1) == want[i].argmax(dim=1))[clear].all()), (shape, kind, i)
                    assert int(clear.sum()) > len(seqs[i]) // 3
        del got


# All 24 layers of the Medium shape: what rounding adds up to over a model's whole depth.  Measured over eight
# sequences of 1,024 tokens in four cuttings: 0.047 of a row's spread at worst and 0.0060 on average (the 48 layers of
# the XL shape: 0.051 and 0.0061), where two layers give 0.028 and 0.0039; the 32-bit engine stays within 3.5e-6.
DEEP_BF16_WORST, DEEP_BF16_MEAN = 0.06, 0.008
DEEP = (_cfg(24, 1024, 16, 50257), 23, (1024, 310))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_all_layers_of_the_medium_shape(tmp_path, dtype):
    from denno_beta_amd.weights import write_model_folder
    cfg, seed, lengths = DEEP
    folder = str(tmp_path / "medium24")
    write_model_folder(folder, cfg, seed, dtype)
    seqs = [seeded_tokens(500 + i, n, cfg["vocab_size"]) for i, n in enumerate(lengths)]
    plain = PlainGPT2.from_folder(folder)
    want = [plain.logits(s) for s in seqs]
    del plain
    whole = None
    for kind, steps in (("whole", U.whole_trace(seqs)), ("mixed", wide_mixed_trace(seqs)),
                        ("tail", U.tail_decode_trace(seqs, 32))):
        tokens = U.max_live_tokens(steps)
        r = runner_for(folder, dtype, tokens)
        got = U.replay(r, steps)
        r.cache.manager.check()
        assert r.cache.manager.live() == 0 and r.cache.manager.free_pages(0) == tokens // 16
        for i in range(len(seqs)):
            what = f"medium, 24 layers, {dtype}, {kind}, request {i}"
            if dtype == "float32":
                U.assert_close(got[f"r{i}"], want[i], "float32", what)
                if whole is not None:
                    assert torch.equal(whole[f"r{i}"], got[f"r{i}"]), f"{what}: 32-bit logits depend on the cutting"
            else:
                spread = want[i].std(dim=1, keepdim=True)
                diff = (got[f"r{i}"] - want[i]).abs() / spread
                assert diff.max().item() <= DEEP_BF16_WORST and diff.mean().item() <= DEEP_BF16_MEAN, (
                    f"{what}: {diff.max().item():.4f} of a row's spread at worst, {diff.mean().item():.5f} on average")
                top2 = want[i].topk(2, dim=1).values
                clear = (top2[:, 0] - top2[:, 1]) > 2 * DEEP_BF16_WORST * want[i].std(dim=1)
                assert bool((got[f"r{i}"].argmax(dim=1) == want[i].argmax(dim=1))[clear].all()), what
        if kind == "whole":
            whole = got
        del r
