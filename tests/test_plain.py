"""The plain implementation, pinned by what fixes it beside the reference's text: vectors that
the reference's own tests hold, special cases that reduce to a library routine, invariants.
Each pin is chosen so that a plausible mistake fails it."""
import math

import pytest
import torch
import torch.nn.functional as F

from conftest import TINY, TINY_A, TINY_B, seeded_tokens
from plain import gpt2_plain as P
from plain import sampler_plain as S


def rnd(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed))


# -- vectors from crates/denno-engine/src/tensor.rs tests -------------------------------------
def test_layer_norm_known_values():
    # tensor.rs:1706-1718
    x = torch.tensor([0.0, 2.0])
    out = P.layer_norm(x, torch.ones(2), torch.zeros(2), 0.0)
    assert torch.allclose(out, torch.tensor([-1.0, 1.0]), atol=1e-6)
    out = P.layer_norm(x, torch.full((2,), 2.0), torch.ones(2), 0.0)
    assert torch.allclose(out, torch.tensor([-1.0, 3.0]), atol=1e-6)


def test_layer_norm_rows_are_normalised():
    # tensor.rs:1721-1733
    out = P.layer_norm(rnd(6, 8, seed=7), torch.ones(8), torch.zeros(8), 1e-5)
    assert out.mean(dim=-1).abs().max() < 1e-4
    assert ((out * out).mean(dim=-1) - 1).abs().max() < 1e-3


def test_layer_norm_is_the_library_routine():
    x, g, b = rnd(5, 96, seed=1) * 3 + 1, rnd(96, seed=2), rnd(96, seed=3)
    for eps in (1e-5, 1e-6, 1e-2):    # a wrong place for eps (outside the root) fails at 1e-2
        assert torch.allclose(P.layer_norm(x, g, b, eps), F.layer_norm(x, (96,), g, b, eps), atol=1e-5)


def test_bias_add_per_row():
    # tensor.rs:1699-1703
    x = torch.tensor([[1.0, 2.0], [3.0, 4.0]])
    y = P.linear_in_out(x, torch.eye(2), torch.tensor([0.5, -0.5]))
    assert y.flatten().tolist() == [1.5, 1.5, 3.5, 3.5]


def test_linear_keeps_in_out_layout():
    # x @ W with W stored [in, out], not transposed (gpt2.rs:155, tensor.rs:1263-1275)
    x, w = rnd(3, 4, seed=1), rnd(4, 6, seed=2)
    want = torch.zeros(3, 6)
    for i in range(3):
        for j in range(6):
            for k in range(4):
                want[i, j] += x[i, k] * w[k, j]
    assert torch.allclose(P.linear_in_out(x, w, None), want, atol=1e-6)


def test_softmax_values_and_stability():
    # tensor.rs:1766-1782
    p = P.softmax_rows(torch.tensor([[1.0, 2.0, 3.0]]))[0]
    assert abs(p.sum().item() - 1) < 1e-6 and p[2] > p[1] > p[0]
    denom = math.exp(-2) + math.exp(-1) + 1
    assert abs(p[0].item() - math.exp(-2) / denom) < 1e-6
    big = P.softmax_rows(torch.tensor([[1e9, 1e9 + 1, 1e9 + 2]]))
    assert torch.isfinite(big).all() and abs(big.sum().item() - 1) < 1e-6
    x = rnd(4, 33, seed=5) * 4
    assert torch.allclose(P.softmax_rows(x), torch.softmax(x, dim=-1), atol=1e-6)


def test_gelu_values_and_library_forms():
    # tensor.rs:1785-1790
    y = P.gelu_tanh(torch.tensor([0.0, 1.0]))
    assert y[0].item() == 0.0 and abs(y[1].item() - 0.8412) < 1e-3
    x = rnd(1000, seed=3) * 3
    assert torch.allclose(P.gelu_tanh(x), F.gelu(x, approximate="tanh"), atol=1e-6)
    assert torch.allclose(P.gelu_erf(x), F.gelu(x), atol=1e-6)
    # the two forms differ: a swap of them is seen
    assert (P.gelu_tanh(x) - P.gelu_erf(x)).abs().max() > 1e-4


# -- attention --------------------------------------------------------------------------------
@pytest.mark.parametrize("n_head,dh", [(1, 16), (4, 16), (2, 48)])
def test_attention_is_the_library_routine(n_head, dh):
    n, e = 9, n_head * dh
    q, k, v = rnd(n, e, seed=1), rnd(n, e, seed=2), rnd(n, e, seed=3)
    scale = 0.37
    got = P.causal_attention(q, k, v, n_head, scale)
    sp = lambda t: t.view(n, n_head, dh).transpose(0, 1)   # noqa: E731
    want = F.scaled_dot_product_attention(sp(q), sp(k), sp(v), is_causal=True, scale=scale)
    assert torch.allclose(got, want.transpose(0, 1).reshape(n, e), atol=1e-5)


def test_attention_by_head_is_the_loop(model_folders):
    """The matrix form that long sequences use gives what the loop over queries gives."""
    n, n_head, dh = 70, 3, 32
    q, k, v = rnd(n, n_head * dh, seed=4), rnd(n, n_head * dh, seed=5), rnd(n, n_head * dh, seed=6)
    assert torch.allclose(P.causal_attention_by_head(q, k, v, n_head, 0.4), P.causal_attention(q, k, v, n_head, 0.4),
                          atol=2e-6)
    plain = P.PlainGPT2.from_folder(model_folders("B", "float32"))
    seq = seeded_tokens(1, 90, 1000)
    assert torch.allclose(plain.logits(seq, by_head=True), plain.logits(seq), atol=2e-6)


def test_attention_first_position_returns_value():
    q, k, v = rnd(1, 32, seed=1), rnd(1, 32, seed=2), rnd(1, 32, seed=3)
    assert torch.equal(P.causal_attention(q, k, v, 2, 1.0), v)


def test_attention_heads_are_side_by_side():
    # only head 1's keys carry a signal: the output changes in head 1's columns only
    n, dh = 5, 16
    q, k, v = rnd(n, 2 * dh, seed=1), rnd(n, 2 * dh, seed=2), rnd(n, 2 * dh, seed=3)
    base = P.causal_attention(q, k, v, 2, 0.25)
    k2 = k.clone()
    k2[:, dh:] *= 3
    out = P.causal_attention(q, k2, v, 2, 0.25)
    assert torch.equal(out[:, :dh], base[:, :dh]) and not torch.allclose(out[:, dh:], base[:, dh:])


def test_attention_window_and_offset():
    n, e = 12, 16
    q, k, v = rnd(n, e, seed=1), rnd(n, e, seed=2), rnd(n, e, seed=3)
    full = P.causal_attention(q, k, v, 1, 0.3)
    # a window as long as the sequence changes nothing; the rows of a later portion are the same rows
    assert torch.allclose(P.causal_attention(q, k, v, 1, 0.3, window=n), full)
    assert torch.allclose(P.causal_attention(q[7:], k, v, 1, 0.3, first_position=7), full[7:], atol=1e-6)
    w = P.causal_attention(q, k, v, 1, 0.3, window=3)
    assert torch.allclose(w[:3], full[:3], atol=1e-6) and not torch.allclose(w[5], full[5])
    # window 1: each position sees itself only
    assert torch.allclose(P.causal_attention(q, k, v, 1, 0.3, window=1), v, atol=1e-6)


def test_attention_scale_options():
    assert P.attention_scale(64, 0) == pytest.approx(0.125)
    assert P.attention_scale(64, 0, scale_attn_by_inverse_layer_idx=True) == pytest.approx(0.125)   # layer 0: / 1
    assert P.attention_scale(64, 2, scale_attn_by_inverse_layer_idx=True) == pytest.approx(0.125 / 3)
    assert P.attention_scale(64, 2, scale_attn_weights=False) == 1.0


# -- the whole model ---------------------------------------------------------------------------
def tiny(name, dtype=torch.float32):
    import tempfile
    from denno_beta_amd.weights import write_model_folder
    cfg, seed = TINY[name]
    with tempfile.TemporaryDirectory() as d:
        write_model_folder(d, cfg, seed, "float32")
        return cfg, P.PlainGPT2.from_folder(d, dtype)


def test_causality_and_position_offset():
    cfg, m = tiny("A")
    a = seeded_tokens(1, 12, cfg["vocab_size"])
    b = list(a)
    b[8:] = seeded_tokens(2, 4, cfg["vocab_size"])
    la, lb = m.logits(a), m.logits(b)
    assert torch.allclose(la[:8], lb[:8], atol=1e-6) and not torch.allclose(la[8:], lb[8:])
    # a token's row depends on its position: the same token at two places gives two rows (gpt2.rs:146)
    c = [a[0]] * 3
    lc = m.logits(c)
    assert not torch.allclose(lc[0], lc[1])


def test_block_is_pre_norm():
    # with both output projections zero a block leaves x as it is: only a pre-norm block does
    cfg, m = tiny("A")
    p = dict(m.layer_params(0))
    for n in ("attn.c_proj.weight", "attn.c_proj.bias", "mlp.c_proj.weight", "mlp.c_proj.bias"):
        p[n] = torch.zeros_like(p[n])
    x = rnd(5, cfg["n_embd"], seed=4)
    assert torch.equal(P.block(x, p, cfg["n_head"], 0.25, 1e-5, P.gelu_tanh), x)


def test_head_is_tied_and_without_bias():
    cfg, m = tiny("A")
    toks = seeded_tokens(3, 6, cfg["vocab_size"])
    unused = next(t for t in range(cfg["vocab_size"]) if t not in toks)
    m.t["wte.weight"][unused] = 0
    assert m.logits(toks)[:, unused].abs().max().item() == 0.0


def test_tiny_b_uses_its_options():
    # exact GELU, eps 1e-6, n_inner != 4E and the per-layer scale all enter: switching one changes the logits
    cfg, m = tiny("B")
    toks = seeded_tokens(4, 10, cfg["vocab_size"])
    base = m.logits(toks)
    for key, val in (("activation_function", "gelu_new"), ("layer_norm_epsilon", 1e-2),
                     ("scale_attn_by_inverse_layer_idx", False)):
        c2 = dict(cfg)
        c2[key] = val
        m2 = P.PlainGPT2(c2, m.t)
        assert not torch.allclose(m2.logits(toks), base, atol=1e-7), key


def test_score_scale_options_are_a_scaling_of_the_queries():
    """The two score options are not in the reference (it fixes 1/sqrt(head), gpt2.rs:174); their meaning
    here is the architecture's config keys': scores divided by (layer index + 1), counted from 0, and no
    1/sqrt(head) at all.  Parity unpinned by any vector of the reference; what pins the plain model is the
    invariant that both are a scaling of a layer's query columns: a model with an option set equals the
    model without it whose query weights and biases of layer l are multiplied by that layer's factor
    (a wrong layer count, a factor applied twice or to the keys as well, would fail this)."""
    cfg, m = tiny("B")
    E, dh = cfg["n_embd"], cfg["n_embd"] // cfg["n_head"]
    toks = seeded_tokens(6, 14, cfg["vocab_size"])
    for option, factor in (("scale_attn_by_inverse_layer_idx", lambda l: 1.0 / (l + 1)),
                           ("scale_attn_weights", lambda l: math.sqrt(dh))):
        on = dict(cfg, scale_attn_by_inverse_layer_idx=False, scale_attn_weights=True)
        on[option] = option == "scale_attn_by_inverse_layer_idx"
        off = dict(cfg, scale_attn_by_inverse_layer_idx=False, scale_attn_weights=True)
        scaled = dict(m.t)
        for l in range(cfg["n_layer"]):
            w, b = scaled[f"h.{l}.attn.c_attn.weight"].clone(), scaled[f"h.{l}.attn.c_attn.bias"].clone()
            w[:, :E] *= factor(l)
            b[:E] *= factor(l)
            scaled[f"h.{l}.attn.c_attn.weight"], scaled[f"h.{l}.attn.c_attn.bias"] = w, b
        want = P.PlainGPT2(off, scaled).logits(toks)
        got = P.PlainGPT2(on, m.t).logits(toks)
        assert torch.allclose(got, want, atol=2e-6), option
        assert not torch.allclose(got, P.PlainGPT2(off, m.t).logits(toks), atol=1e-5), option


def test_the_first_layer_is_divided_by_one():
    """`scale_attn_by_inverse_layer_idx` divides a layer's scores by its index counted so that the first layer
    keeps its scores: a count from 0 as it stands would divide the first layer by zero, and any other start
    changes a model of one layer.  So in a model of one layer the option changes nothing, to the last bit, and
    in a model of two layers it changes the second layer alone: the first layer's output is the same with and
    without it.  (What the option means is still this build's reading of the key's name: the reference has no
    such option and no vector for it, and model code of installed packages is not consulted.)"""
    cfg, m = tiny("B")
    toks = seeded_tokens(7, 12, cfg["vocab_size"])
    one = dict(cfg, n_layer=1)
    on = P.PlainGPT2(dict(one, scale_attn_by_inverse_layer_idx=True), m.t).logits(toks)
    off = P.PlainGPT2(dict(one, scale_attn_by_inverse_layer_idx=False), m.t).logits(toks)
    assert torch.isfinite(on).all() and torch.equal(on, off)
    assert P.attention_scale(48, 0, True, True) == P.attention_scale(48, 0, True, False) == 1 / math.sqrt(48)
    assert P.attention_scale(48, 1, True, True) == 1 / math.sqrt(48) / 2 and P.attention_scale(48, 2, False, True) == 1 / 3
    two = dict(cfg, n_layer=2)
    assert not torch.equal(P.PlainGPT2(dict(two, scale_attn_by_inverse_layer_idx=True), m.t).logits(toks),
                           P.PlainGPT2(dict(two, scale_attn_by_inverse_layer_idx=False), m.t).logits(toks))
    # and the engine's own factor is the plain one's, layer by layer
    from denno_beta_amd.models.gpt2 import GPT2Config, attention_scale
    for inv in (False, True):
        for sw in (False, True):
            c = GPT2Config.from_dict(dict(cfg, scale_attn_by_inverse_layer_idx=inv, scale_attn_weights=sw))
            for l in range(3):
                assert attention_scale(c, l) == pytest.approx(P.attention_scale(c.head_dim, l, sw, inv), rel=1e-7)


def test_float64_agrees_with_float32():
    cfg, m32 = tiny("B")
    _, m64 = tiny("B", torch.float64)
    toks = seeded_tokens(5, 40, cfg["vocab_size"])
    assert (m32.logits(toks).double() - m64.logits(toks)).abs().max() < 2e-5


# -- samplers (crates/denno-engine/src/sampler.rs tests) -----------------------------------------
def test_greedy_first_maximum_nan_ignored():
    assert S.greedy([1.0, 5.0, 5.0, 2.0]) == 1            # sampler.rs:569-582
    assert S.greedy([float("nan"), 1.0, 3.0]) == 2          # sampler.rs:1222-1224
    assert P.argmax_first(torch.tensor([2.0, 7.0, 7.0])) == 1


def test_temperature_walk_frequencies():
    # [0, 4] at T = 1 picks index 1 with probability e^4/(1+e^4) = 0.982 (sampler.rs:686-704)
    from denno_beta_amd.sampling import uniform
    n = 10000
    hits = sum(S.temperature_walk([0.0, 4.0], 1.0, uniform(42, i)) for i in range(n))
    assert abs(hits / n - 0.982) < 0.02
    picks = {S.temperature_walk([2.0, 1.5], 1.0, uniform(7, i)) for i in range(200)}
    assert picks == {0, 1}                                   # sampler.rs:718-726
    assert S.temperature_walk([1.0, 2.0, 3.0], 1.0, 0.0) == 0


def test_top_k_and_top_p():
    logits = [1.0, 3.0, 2.0, 3.0, 0.0]
    # k = 1: the first of the two maxima, whatever u is
    assert {S.top_k_top_p(logits, 1.0, 1, None, u / 10) for u in range(10)} == {1}
    # k = 2: both maxima, the lower index first in the walk
    assert S.top_k_top_p(logits, 1.0, 2, None, 0.0) == 1 and S.top_k_top_p(logits, 1.0, 2, None, 0.99) == 3
    # a small p keeps the head of the sorted list only
    assert {S.top_k_top_p(logits, 1.0, None, 0.1, u / 10) for u in range(10)} == {1}


def test_top_p_alone_falls_back_to_the_whole_vocabulary():
    """sampler.rs:387-435: over more than 2,048 tokens the cut is looked for among the 2,048 largest, with
    probabilities relative to their sum: a row is decided there unless the cut falls on the last of them
    (a flat row with p near 1), which needs the whole vocabulary, and then tokens beyond the 2,048 largest
    are drawn.  Up to 2,048 tokens there is the whole vocabulary only."""
    n = 3000
    peaked = [0.0] * n
    peaked[5], peaked[9] = 12.0, 11.0
    tok, whole = S.top_p_alone(peaked, 1.0, 0.9, 0.99)
    assert not whole and tok == 9 and S.top_p_alone(peaked, 1.0, 0.5, 0.99) == (5, False)
    flat = [0.001 * ((i * 7919) % n) / n for i in range(n)]
    order = sorted(range(n), key=lambda i: (-flat[i], i))
    draws = [S.top_p_alone(flat, 1.0, 0.9, u / 50) for u in range(50)]
    assert not any(whole for _, whole in draws)             # 0.9 of the 2,048 largest's mass lies among them
    assert all(order.index(tok) < 0.9 * 2048 + 2 for tok, _ in draws)
    draws = [S.top_p_alone(flat, 1.0, 0.9999, u / 50) for u in range(50)]
    assert all(whole for _, whole in draws)
    assert any(order.index(tok) >= 2048 for tok, _ in draws)
    assert S.top_p_alone([1.0, 3.0, 2.0], 1.0, 0.1, 0.5) == (1, False)


def test_penalties():
    l = [2.0, -2.0, 1.0, 0.5]
    assert S.repetition_penalty(l, [0, 1, 0], 2.0) == [1.0, -4.0, 1.0, 0.5]      # each distinct token once
    assert S.repetition_penalty(l, [0, 1], 1.0) == l
    out = S.frequency_presence(l, [0, 0, 2], 0.5, 0.25)
    assert out == [2.0 - 1.0 - 0.25, -2.0, 1.0 - 0.5 - 0.25, 0.5]
    # context 5 6 7 5 6: with n = 3 the token after "5 6" earlier, 7, is banned
    out = S.no_repeat_ngram([0.0] * 10, [5, 6, 7, 5, 6], 3)
    assert out[7] == float("-inf") and sum(1 for v in out if v == float("-inf")) == 1
    assert S.no_repeat_ngram([0.0] * 10, [5, 6], 3) == [0.0] * 10
