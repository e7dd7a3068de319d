"""The parts alone, and what the assembly allows: a layer named twice, a layer that reads
another layer's cache, and a mixer with state of its own that is defined here, registered,
built and stepped without a change to the framework's files."""
import json
import math

import pytest
import torch

import replay_util as U
from conftest import TINY, seeded_tokens
from plain import gpt2_plain as P


def options(device, dtype="float32", **kw):
    from denno_beta_amd.config import EngineOptions
    o = dict(dtype=dtype, device=device, page_size=16, cache_tokens=256, max_live=4)
    o.update(kw)
    return EngineOptions(**o)


def gpt2_spec(name, **changes):
    from denno_beta_amd.models.gpt2 import GPT2Config, build_gpt2
    cfg = dict(TINY[name][0])
    cfg.update(changes)
    return cfg, build_gpt2(GPT2Config.from_dict(cfg))


def stored(tensors, spec):
    """{name: tensor in checkpoint layout, CPU 32-bit} from bound tensors (held [out, in])."""
    out = {}
    for s in spec.param_specs():
        t = tensors[s.name].detach().float().cpu()
        out[s.name] = t.t().contiguous() if s.transpose else t
    return out


def draw(spec, device, seed=3, dtype="float32"):
    from denno_beta_amd.weights import draw_all
    return draw_all(spec.param_specs(), seed, engine_dtype=dtype, device=torch.device(device), stored=dtype)


# -- each part alone --------------------------------------------------------------------------
def test_norm_part(backend):
    from denno_beta_amd.parts import NORMS, Runtime
    dev = torch.device(backend)
    n = NORMS.make(("layernorm", dict(width=96, eps=1e-3, weight_name="g", bias_name="b")))
    assert [(s.name, s.shape, s.role) for s in n.param_specs()] == [("g", (96,), "vector"), ("b", (96,), "vector")]
    g, b = torch.randn(96, device=dev), torch.randn(96, device=dev)
    n.bind({"g": g, "b": b}, Runtime(torch.float32, dev))
    x = torch.randn(7, 96, device=dev) * 2 + 0.5
    want = P.layer_norm(x.cpu(), g.cpu(), b.cpu(), 1e-3)
    assert torch.allclose(n.forward(x, torch.float32).cpu(), want, atol=1e-5)
    rows = torch.tensor([5, 0], dtype=torch.int32, device=dev)
    assert torch.allclose(n.forward(x, torch.float32, rows=rows).cpu(), want[[5, 0]], atol=1e-5)
    assert n.forward(x, torch.bfloat16).dtype == torch.bfloat16


def test_embedding_and_position_parts(backend):
    """Token rows plus position rows, by the positions of the step, not by the rows' order."""
    from denno_beta_amd.kernels import ops
    from denno_beta_amd.parts import POSITIONS, Runtime
    from denno_beta_amd.parts.positions import TokenEmbedding
    dev = torch.device(backend)
    emb, pos = TokenEmbedding(37, 24, "tok"), POSITIONS.make(("learned_absolute", dict(n_positions=50, width=24, name="pos")))
    assert [(s.name, s.shape, s.role) for s in emb.param_specs() + pos.param_specs()] == [
        ("tok", (37, 24), "table"), ("pos", (50, 24), "table")]
    t = {"tok": torch.randn(37, 24, device=dev), "pos": torch.randn(50, 24, device=dev)}
    emb.bind(t, Runtime(torch.float32, dev)), pos.bind(t, Runtime(torch.float32, dev))
    tokens = torch.tensor([5, 5, 36, 0], dtype=torch.int32, device=dev)
    positions = torch.tensor([49, 0, 7, 7], dtype=torch.int32, device=dev)
    x = torch.empty(4, 24, device=dev)
    ops.embed(tokens, positions, emb.weight, pos.table(), x)
    want = P.embed(tokens.long().cpu(), positions.long().cpu(), t["tok"].cpu(), t["pos"].cpu())
    assert torch.equal(x.cpu(), want)
    none = POSITIONS.make(("none", {}))
    ops.embed(tokens, positions, emb.weight, none.table(), x)
    assert torch.equal(x.cpu(), t["tok"].cpu()[tokens.long().cpu()])


@pytest.mark.parametrize("act", ["gelu_tanh", "gelu_erf"])
def test_feed_forward_part(backend, act):
    from denno_beta_amd.parts import FEED_FORWARDS, Runtime
    dev = torch.device(backend)
    f = FEED_FORWARDS.make(("dense_mlp", dict(width=48, inner=136, activation=act, up_weight="u.w", up_bias="u.b",
                                              down_weight="d.w", down_bias="d.b", stored_in_out=True)))
    specs = {s.name: s for s in f.param_specs()}
    assert specs["u.w"].shape == (48, 136) and specs["u.w"].transpose and specs["d.w"].shape == (136, 48)
    t = {"u.w": torch.randn(136, 48, device=dev) * 0.2, "u.b": torch.randn(136, device=dev) * 0.1,
         "d.w": torch.randn(48, 136, device=dev) * 0.2, "d.b": torch.randn(48, device=dev) * 0.1}
    f.bind(t, Runtime(torch.float32, dev))
    h = torch.randn(9, 48, device=dev)
    x = torch.randn(9, 48, device=dev)
    want = x.cpu() + P.mlp_block(h.cpu(), {"mlp.c_fc.weight": t["u.w"].t().cpu(), "mlp.c_fc.bias": t["u.b"].cpu(),
                                           "mlp.c_proj.weight": t["d.w"].t().cpu(), "mlp.c_proj.bias": t["d.b"].cpu()},
                                 P.gelu_tanh if act == "gelu_tanh" else P.gelu_erf)
    f.forward(h, None, accumulate_into=x)
    assert torch.allclose(x.cpu(), want, atol=2e-5)


@pytest.mark.parametrize("heads,kv_heads,dh,window", [(4, 4, 16, 0), (6, 2, 32, 0), (3, 1, 16, 5)])
def test_attention_mixer_part(backend, heads, kv_heads, dh, window):
    """The mixer over a real cache, in two portions, against plain attention; grouped key heads
    and a window are options of the part although GPT-2 uses neither."""
    from denno_beta_amd.cache import CacheStorage
    from denno_beta_amd.engine.batch import StepEntry, build_context
    from denno_beta_amd.parts import MIXERS, Runtime
    dev = torch.device(backend)
    E = 64
    m = MIXERS.make(("causal_attention", dict(width=E, n_heads=heads, n_kv_heads=kv_heads, head_dim=dh, scale=0.3,
                                              qkv_weight="qkv.w", qkv_bias="qkv.b", out_weight="o.w", out_bias=None,
                                              window=window)))
    qw, kw = heads * dh, kv_heads * dh
    # (weights of a size that keeps the scores within a few units: with scores of tens, exp turns the last bit
    # of a 32-bit score into more than this test allows)
    t = {"qkv.w": torch.randn(qw + 2 * kw, E, device=dev) * 0.12, "qkv.b": torch.randn(qw + 2 * kw, device=dev) * 0.1,
         "o.w": torch.randn(E, qw, device=dev) * 0.2}
    m.bind(t, Runtime(torch.float32, dev))
    cache = CacheStorage([m.cache_spec()], kv_dtype=torch.float32, page_size=16, cache_tokens=64, max_live=2,
                         device=dev)
    cache.start_request(0)
    n = 23
    h = torch.randn(n, E, device=dev)
    got = torch.zeros(n, E, device=dev)
    for a, b in ((0, 14), (14, n)):
        ctx = build_context([StepEntry(0, [0] * (b - a), [])], cache, 10, 64, dev)
        m.forward(h[a:b].contiguous(), ctx, cache.view(0, True), accumulate_into=got[a:b])
        cache.manager.commit(0, b)
    # (the plain side in 64-bit: the outputs reach 15, where 32-bit sums in another order differ by as much as
    # the bound allows the mixer itself)
    qkv = h.cpu().double() @ t["qkv.w"].t().cpu().double() + t["qkv.b"].cpu().double()
    q, k, v = qkv[:, :qw], qkv[:, qw:qw + kw], qkv[:, qw + kw:]
    rep = heads // kv_heads      # query head i reads key head i // rep
    kx = k.view(n, kv_heads, dh).repeat_interleave(rep, dim=1).reshape(n, qw)
    vx = v.view(n, kv_heads, dh).repeat_interleave(rep, dim=1).reshape(n, qw)
    want = P.causal_attention(q, kx, vx, heads, 0.3, window=window or None) @ t["o.w"].t().cpu().double()
    assert torch.allclose(got.cpu().double(), want, atol=2e-5), (got.cpu().double() - want).abs().max().item()


def test_a_cache_group_holds_the_dtype_that_its_mixers_ask_for():
    """Pages hold the engine's activation dtype unless the mixer's PagedKV names one; caches that differ
    in it are groups of their own."""
    from denno_beta_amd.cache import CacheStorage
    from denno_beta_amd.parts import PagedKV
    c = CacheStorage([PagedKV(2, 16), PagedKV(2, 16, dtype="float32"), PagedKV(2, 16)], kv_dtype=torch.bfloat16,
                     page_size=16, cache_tokens=64, max_live=2, device=torch.device("cpu"))
    assert c.n_groups == 2 and c.k[0].dtype == torch.bfloat16 and c.k[1].dtype == torch.float32
    assert c.k[0].shape[0] == 2 and c.v[1].shape == (1, 4, 2, 16, 16)
    assert c.bytes_per_token() == 2 * 2 * 2 * 16 * 2 + 2 * 2 * 16 * 4


def test_a_cache_group_may_hold_values_of_another_width_than_its_keys():
    """PagedKV names a width for values where it is not the keys': the pools are laid out for both and are a
    group of their own."""
    from denno_beta_amd.cache import CacheStorage
    from denno_beta_amd.parts import PagedKV
    assert PagedKV(2, 32).v_dim == 32 and PagedKV(2, 32, value_dim=48).v_dim == 48
    c = CacheStorage([PagedKV(2, 32), PagedKV(2, 32, value_dim=48)], kv_dtype=torch.float32, page_size=16,
                     cache_tokens=64, max_live=2, device=torch.device("cpu"))
    assert c.n_groups == 2 and c.k[1].shape == (1, 4, 2, 16, 32) and c.v[1].shape == (1, 4, 2, 48, 16)
    assert c.bytes_per_token() == 2 * (32 + 32) * 4 + 2 * (32 + 48) * 4


@pytest.mark.gpu
def test_the_attention_kernels_refuse_values_of_another_width():
    """The package's attention kernels take keys and values of one width; asked for others they say so."""
    from denno_beta_amd.kernels import ops
    dev = "cuda:0"
    q = torch.zeros(4, 64, device=dev)
    k = torch.zeros(2, 2, 16, 32, device=dev)
    v = torch.zeros(2, 2, 48, 16, device=dev)
    bt = torch.zeros(1, 2, dtype=torch.int32, device=dev)
    tiles = torch.tensor([[0], [0], [4], [0]], dtype=torch.int32, device=dev)
    with pytest.raises(ops.KernelError, match="one width"):
        ops.attention(q, torch.empty(4, 64, device=dev), k, v, bt, tiles, 2, 0.5)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_further_embedding_tables_are_added_in_the_embedding_kernel(backend, dtype):
    """A description may list further tables whose rows are added to the token and position rows: here a second
    table over the tokens (times a half) and a second one over the positions.  Since every later part is linear
    in nothing, the check is against the plain GPT-2 run on a token table and a position table that hold the
    sums, which exist because each further table is indexed like one of the two."""
    from denno_beta_amd.engine import ModelRunner
    from denno_beta_amd.parts import EmbeddingTable
    cfg, spec = gpt2_spec("A")
    spec.extra_embeddings = [EmbeddingTable("tok2.weight", cfg["vocab_size"], "tokens", 0.5),
                             EmbeddingTable("pos2.weight", cfg["n_positions"], "positions")]
    assert [s.name for s in spec.param_specs() if s.role == "table"] == ["wte.weight", "wpe.weight", "tok2.weight", "pos2.weight"]
    tensors = draw(spec, backend, dtype=dtype)
    r = ModelRunner(spec, tensors, options(backend, dtype))
    seq = seeded_tokens(2, 50, cfg["vocab_size"])
    got = U.replay(r, U.chunk_trace([seq], sizes=(9, 2, 20)))["r0"]
    st = stored(tensors, spec)
    # the head is tied to the first token table alone: the plain model gets the summed table for its input rows
    # and the first table for its head
    plain = P.PlainGPT2(cfg, {**st, "wpe.weight": st["wpe.weight"] + st["pos2.weight"]})
    want = plain.logits(seq, input_table=st["wte.weight"] + 0.5 * st["tok2.weight"])
    U.assert_close(got, want, dtype, "further embedding tables")
    # one table too many for the kernel, and an index that a step does not have
    spec.extra_embeddings = [EmbeddingTable(f"t{i}", 8) for i in range(3)]
    with pytest.raises(ValueError, match="in all"):
        spec.instantiate()
    spec.extra_embeddings = [EmbeddingTable("t", 8, "token_types")]
    with pytest.raises(ValueError, match="token_types"):
        spec.instantiate()


# -- the order in which layers run is data -----------------------------------------------------
def test_a_layer_named_twice(backend):
    from denno_beta_amd.engine import ModelRunner
    from denno_beta_amd.parts import LayerCall
    cfg, spec = gpt2_spec("A", n_layer=1)
    spec.run_order = [LayerCall(0, 0), LayerCall(0, 1)]      # one layer's weights, run twice, a cache each
    tensors = draw(spec, backend)
    r = ModelRunner(spec, tensors, options(backend))
    st = stored(tensors, spec)
    twice = dict(st)
    twice.update({k.replace("h.0.", "h.1."): v for k, v in st.items() if k.startswith("h.0.")})
    plain = P.PlainGPT2(dict(cfg, n_layer=2), twice)
    seq = seeded_tokens(1, 40, cfg["vocab_size"])
    got = U.replay(r, U.chunk_trace([seq], sizes=(7, 2, 13)))["r0"]
    U.assert_close(got, plain.logits(seq), "float32", "a layer run twice")
    assert len(r.cache.k[0]) == 2       # two caches although there is one layer


def test_a_layer_that_reads_another_layers_cache(backend):
    from denno_beta_amd.engine import ModelRunner
    from denno_beta_amd.parts import LayerCall
    cfg, spec = gpt2_spec("A")
    spec.run_order = [LayerCall(0, 0), LayerCall(1, 0, writes_cache=False)]
    tensors = draw(spec, backend)
    r = ModelRunner(spec, tensors, options(backend))
    assert len(r.cache.k[0]) == 1
    st = stored(tensors, spec)
    seq = seeded_tokens(2, 37, cfg["vocab_size"])
    # plain: layer 1 attends with its own queries over layer 0's keys and values
    E, H = cfg["n_embd"], cfg["n_head"]
    scale = 1 / math.sqrt(E // H)
    lp = lambda i: {k[len(f"h.{i}."):]: v for k, v in st.items() if k.startswith(f"h.{i}.")}   # noqa: E731
    x = P.embed(torch.tensor(seq), torch.arange(len(seq)), st["wte.weight"], st["wpe.weight"])
    p0, p1 = lp(0), lp(1)
    h = P.layer_norm(x, p0["ln_1.weight"], p0["ln_1.bias"], 1e-5)
    qkv0 = P.linear_in_out(h, p0["attn.c_attn.weight"], p0["attn.c_attn.bias"])
    k0, v0 = qkv0[:, E:2 * E], qkv0[:, 2 * E:]
    x = P.block(x, p0, H, scale, 1e-5, P.gelu_tanh)
    h = P.layer_norm(x, p1["ln_1.weight"], p1["ln_1.bias"], 1e-5)
    q1 = P.linear_in_out(h, p1["attn.c_attn.weight"], p1["attn.c_attn.bias"])[:, :E]
    x = x + P.linear_in_out(P.causal_attention(q1, k0, v0, H, scale), p1["attn.c_proj.weight"], p1["attn.c_proj.bias"])
    x = x + P.mlp_block(P.layer_norm(x, p1["ln_2.weight"], p1["ln_2.bias"], 1e-5), p1, P.gelu_tanh)
    want = P.head(x, st["ln_f.weight"], st["ln_f.bias"], 1e-5, st["wte.weight"])
    got = U.replay(r, U.tail_decode_trace([seq], 9))["r0"]
    U.assert_close(got, want, "float32", "a layer reading another layer's cache")


def test_run_order_is_checked():
    from denno_beta_amd.parts import LayerCall
    _, spec = gpt2_spec("A")
    spec.run_order = [LayerCall(0, 0), LayerCall(1, 1, writes_cache=False)]
    with pytest.raises(ValueError, match="before any call has written"):
        spec.instantiate()
    spec.run_order = [LayerCall(0, 0), LayerCall(1, 0)]
    with pytest.raises(ValueError, match="writes cache 0"):
        spec.instantiate()
    spec.run_order = [LayerCall(0, 0), LayerCall(5, 1)]
    with pytest.raises(ValueError, match="names layer 5"):
        spec.instantiate()


# -- a toy mixer with state of its own ---------------------------------------------------------
def toy_model(device, mixers):
    """A decoder whose layers use the given mixer kinds: 'toy_decay' (defined below) or 'attn'."""
    from denno_beta_amd.parts import DecoderSpec, LayerCall, LayerSpec
    E = 32
    layers = []
    for i, kind in enumerate(mixers):
        p = f"L{i}."
        mixer = ("toy_decay", dict(width=E, decay=0.5 + 0.1 * i, weight_name=p + "mix.w")) if kind == "toy_decay" else \
            ("causal_attention", dict(width=E, n_heads=2, n_kv_heads=2, head_dim=16, scale=0.25, qkv_weight=p + "qkv.w",
                                      qkv_bias=None, out_weight=p + "o.w", out_bias=None))
        layers.append(LayerSpec("pre_norm", dict(
            norm1=("layernorm", dict(width=E, eps=1e-5, weight_name=p + "n1.g", bias_name=None)), mixer=mixer,
            norm2=("layernorm", dict(width=E, eps=1e-5, weight_name=p + "n2.g", bias_name=None)),
            ffn=("dense_mlp", dict(width=E, inner=64, activation="gelu_tanh", up_weight=p + "up.w", up_bias=None,
                                   down_weight=p + "down.w", down_bias=None)))))
    return DecoderSpec(vocab=50, width=E, max_positions=128, token_table="tok", position=("none", {}), layers=layers,
                       run_order=[LayerCall(i, i) for i in range(len(layers))],
                       final_norm=("layernorm", dict(width=E, eps=1e-5, weight_name="nf.g", bias_name=None)))


def register_toy_mixer():
    from denno_beta_amd.parts import MIXERS, FixedState, Part
    from denno_beta_amd.weights import ParamSpec
    if "toy_decay" in MIXERS:
        return

    @MIXERS.register("toy_decay")
    class ToyDecayMixer(Part):
        """s_t = decay * s_(t-1) + h_t ;  out_t = s_t W^T.  Its state is one vector per request,
        which a portion of a prompt carries on in token order."""

        def __init__(self, width, decay, weight_name):
            self.width, self.decay, self.weight_name = width, decay, weight_name

        def param_specs(self):
            return [ParamSpec(self.weight_name, (self.width, self.width), "matrix", ("normal", 0.0, 0.2))]

        def cache_spec(self):
            return FixedState((self.width,), "float32")

        def bind(self, tensors, runtime):
            super().bind(tensors, runtime)
            self.w = tensors[self.weight_name].float()

        def forward(self, h, ctx, cache, accumulate_into):
            for s, slot in enumerate(ctx.host_slots):
                a, b = ctx.host_row_start[s], ctx.host_row_start[s + 1]
                state = cache.state[slot]
                for t in range(a, b):
                    state.mul_(self.decay).add_(h[t].float())
                    accumulate_into[t] += state @ self.w.t()


def toy_plain(spec, st, seq):
    """The toy model on one whole sequence, written out with the plain functions."""
    x = st["tok"][torch.tensor(seq)]
    for i, ls in enumerate(spec.layers):
        p = f"L{i}."
        h = P.layer_norm(x, st[p + "n1.g"], 0.0, 1e-5)
        if ls.parts["mixer"][0] == "toy_decay":
            s, out = torch.zeros(x.shape[1]), []
            for t in range(len(seq)):
                s = ls.parts["mixer"][1]["decay"] * s + h[t]
                out.append(s @ st[p + "mix.w"].t())
            x = x + torch.stack(out)
        else:
            qkv = h @ st[p + "qkv.w"].t()
            a = P.causal_attention(qkv[:, :32], qkv[:, 32:64], qkv[:, 64:], 2, 0.25)
            x = x + a @ st[p + "o.w"].t()
        h = P.layer_norm(x, st[p + "n2.g"], 0.0, 1e-5)
        x = x + P.gelu_tanh(h @ st[p + "up.w"].t()) @ st[p + "down.w"].t()
    return P.layer_norm(x, st["nf.g"], 0.0, spec.final_norm[1]["eps"]) @ st["tok"].t()


def test_a_toy_mixer_with_state_is_registered_built_and_stepped(backend):
    from denno_beta_amd.engine import ModelRunner
    register_toy_mixer()
    # different mixers in different layers: state, attention, state
    spec = toy_model(backend, ["toy_decay", "attn", "toy_decay"])
    tensors = draw(spec, backend)
    r = ModelRunner(spec, tensors, options(backend, cache_tokens=192))
    assert r.cache.n_groups == 2 and r.cache.state[0].shape == (2, 4, 32)     # two state caches, four slots
    st = {k: v.float().cpu() for k, v in tensors.items()}
    seqs = [seeded_tokens(i, n, 50) for i, n in enumerate((30, 11, 47, 25, 40))]
    want = [toy_plain(spec, st, s) for s in seqs]
    for kind, steps in (("whole", U.whole_trace(seqs)), ("mixed", U.mixed_trace(seqs, seed=3))):
        got = U.replay(r, steps)       # five requests over four slots: a slot is used again and starts at zero
        for i in range(len(seqs)):
            U.assert_close(got[f"r{i}"], want[i], "float32", f"toy model, {kind}, request {i}")
    r.cache.manager.check()


# -- a toy position encoding that turns queries and keys, a toy feed-forward with routing --------
def register_toy_rotation_and_experts():
    from denno_beta_amd.parts import FEED_FORWARDS, POSITIONS, Part
    from denno_beta_amd.weights import ParamSpec
    if "toy_rotation" in POSITIONS:
        return

    @POSITIONS.register("toy_rotation")
    class ToyRotation(Part):
        """Pairs (2i, 2i + 1) of every head of q and k are turned by the angle position * base^(-2i/dh)."""
        rotates = True

        def __init__(self, head_dim, base):
            self.head_dim, self.base = head_dim, base

        def table(self):
            return None

        def rotate(self, q, k, ctx):
            for t in (q, k):
                turn_pairs(t, ctx.positions.to(torch.float32), self.head_dim, self.base)
            return q, k

    @FEED_FORWARDS.register("toy_experts")
    class ToyExperts(Part):
        """A router picks one expert per row (the first maximum of h R^T, in 32-bit); that expert's
        two products with a tanh GELU between them are added into the residual stream."""

        def __init__(self, width, inner, n_experts, prefix):
            self.width, self.inner, self.n, self.prefix = width, inner, n_experts, prefix

        def param_specs(self):
            specs = [ParamSpec(self.prefix + "router", (self.n, self.width), "matrix", ("normal", 0.0, 0.5))]
            for e in range(self.n):
                specs += [ParamSpec(f"{self.prefix}e{e}.up", (self.inner, self.width), "matrix", ("normal", 0.0, 0.2)),
                          ParamSpec(f"{self.prefix}e{e}.down", (self.width, self.inner), "matrix", ("normal", 0.0, 0.2))]
            return specs

        def bind(self, tensors, runtime):
            super().bind(tensors, runtime)
            self.router = tensors[self.prefix + "router"].float()
            self.up = [tensors[f"{self.prefix}e{e}.up"].float() for e in range(self.n)]
            self.down = [tensors[f"{self.prefix}e{e}.down"].float() for e in range(self.n)]

        def forward(self, h, ctx, accumulate_into):
            h = h.float()
            choice = first_max(h @ self.router.t())
            for e in range(self.n):
                rows = (choice == e).nonzero().flatten()
                if len(rows):
                    accumulate_into[rows] += P.gelu_tanh(h[rows] @ self.up[e].t()) @ self.down[e].t()


def first_max(scores):
    """Index of each row's first maximum."""
    best = scores.max(dim=-1, keepdim=True).values
    return (scores == best).float().argmax(dim=-1)


def turn_pairs(t, positions, head_dim, base):
    """In place: in every head of t [T, heads * head_dim], the pair (2i, 2i + 1) turned by
    positions[row] * base^(-2i / head_dim); angles, sines and the products in 32-bit."""
    T, W = t.shape
    x = t.float().reshape(T, W // head_dim, head_dim // 2, 2)
    i = torch.arange(head_dim // 2, device=t.device, dtype=torch.float32)
    angle = positions.to(t.device)[:, None, None] * base ** (-2.0 * i / head_dim)[None, None, :]
    c, s = torch.cos(angle), torch.sin(angle)
    a, b = x[..., 0], x[..., 1]
    t.copy_(torch.stack([a * c - b * s, a * s + b * c], dim=-1).reshape(T, W).to(t.dtype))


ROTATION_BASES = (50.0, 50.0, 7.0)     # the third layer turns by a base of its own, the others by the model's


def rotation_model():
    """Three layers; the model's position encoding turns queries and keys by a base of 50, the third
    layer names one of its own with a base of 7."""
    from denno_beta_amd.parts import DecoderSpec, LayerCall, LayerSpec
    E = 32
    layers = []
    for i, (heads, kv_heads) in enumerate(((2, 2), (4, 2), (2, 1))):
        p = f"L{i}."
        own = dict(position=("toy_rotation", dict(head_dim=16, base=ROTATION_BASES[i]))) if i == 2 else {}
        layers.append(LayerSpec("pre_norm", dict(
            norm1=("layernorm", dict(width=E, eps=1e-5, weight_name=p + "n1.g", bias_name=None)),
            mixer=("causal_attention", dict(width=E, n_heads=heads, n_kv_heads=kv_heads, head_dim=16, scale=0.25,
                                            qkv_weight=p + "qkv.w", qkv_bias=None, out_weight=p + "o.w", out_bias=None,
                                            **own)),
            norm2=("layernorm", dict(width=E, eps=1e-5, weight_name=p + "n2.g", bias_name=None)),
            ffn=("toy_experts", dict(width=E, inner=48, n_experts=3, prefix=p + "ffn.")))))
    return DecoderSpec(vocab=50, width=E, max_positions=128, token_table="tok",
                       position=("toy_rotation", dict(head_dim=16, base=50.0)), layers=layers,
                       run_order=[LayerCall(i, i) for i in range(len(layers))],
                       final_norm=("layernorm", dict(width=E, eps=1e-5, weight_name="nf.g", bias_name=None)))


def rotation_plain(spec, st, seq, positions=None):
    """The same model on one whole sequence with the plain functions; `positions` other than
    0, 1, 2, ... shift every token."""
    T = len(seq)
    pos = torch.arange(T, dtype=torch.float32) if positions is None else positions
    x = st["tok"][torch.tensor(seq)]
    for i, ls in enumerate(spec.layers):
        p = f"L{i}."
        a = ls.parts["mixer"][1]
        H, Hkv, dh = a["n_heads"], a["n_kv_heads"], a["head_dim"]
        h = P.layer_norm(x, st[p + "n1.g"], 0.0, ls.parts["norm1"][1]["eps"])
        qkv = h @ st[p + "qkv.w"].t()
        q, k, v = qkv[:, :H * dh].clone(), qkv[:, H * dh:(H + Hkv) * dh].clone(), qkv[:, (H + Hkv) * dh:]
        turn_pairs(q, pos, dh, ROTATION_BASES[i])
        turn_pairs(k, pos, dh, ROTATION_BASES[i])
        # query head hd reads key head hd // (H / Hkv): spread keys and values out to H heads
        spread = lambda t: t.reshape(T, Hkv, 1, dh).expand(T, Hkv, H // Hkv, dh).reshape(T, H * dh)   # noqa: E731
        x = x + P.causal_attention(q, spread(k), spread(v), H, a["scale"]) @ st[p + "o.w"].t()
        h = P.layer_norm(x, st[p + "n2.g"], 0.0, ls.parts["norm2"][1]["eps"])
        f = ls.parts["ffn"][1]
        choice = first_max(h @ st[f["prefix"] + "router"].t())
        out = torch.zeros_like(x)
        for t in range(T):
            e = int(choice[t])
            out[t] = P.gelu_tanh(h[t] @ st[f"{f['prefix']}e{e}.up"].t()) @ st[f"{f['prefix']}e{e}.down"].t()
        x = x + out
    return P.layer_norm(x, st["nf.g"], 0.0, spec.final_norm[1]["eps"]) @ st["tok"].t()


def test_toy_rotation_and_toy_experts_are_registered_built_and_stepped(backend):
    """A position encoding that turns queries and keys before the keys go to the cache (with fewer
    key heads than query heads in one layer) and a feed-forward that routes rows to experts, both
    defined here; the framework's files do not change."""
    from denno_beta_amd.engine import ModelRunner
    register_toy_rotation_and_experts()
    spec = rotation_model()
    tensors = draw(spec, backend)
    for name in tensors:              # sharp attention, so that a wrong turn of a query or key shows in the logits
        if name.endswith("qkv.w"):
            tensors[name] *= 25.0
    r = ModelRunner(spec, tensors, options(backend, cache_tokens=192))
    st = {k: v.float().cpu() for k, v in tensors.items()}
    seqs = [seeded_tokens(i, n, 50) for i, n in enumerate((30, 11, 47, 25, 40))]
    want = [rotation_plain(spec, st, s) for s in seqs]
    for kind, steps in (("whole", U.whole_trace(seqs)), ("tail", U.tail_decode_trace(seqs, 8)),
                        ("mixed", U.mixed_trace(seqs, seed=3))):
        got = U.replay(r, steps)
        for i in range(len(seqs)):
            U.assert_close(got[f"r{i}"], want[i], "float32", f"rotation and experts, {kind}, request {i}")
    r.cache.manager.check()
    # the plain model is pinned by what a rotation must keep: only distances between positions
    # count, so shifting every position by the same amount changes nothing; and the rotation does
    # act (without it the logits differ)
    shifted = rotation_plain(spec, st, seqs[0], positions=torch.arange(len(seqs[0]), dtype=torch.float32) + 7.0)
    assert torch.allclose(shifted, want[0], atol=2e-4)
    still = rotation_plain(spec, st, seqs[0], positions=torch.zeros(len(seqs[0])))
    assert (still - want[0]).abs().max() > 0.05
    # the third layer's own base acts: with the model's base there too the logits differ
    global ROTATION_BASES
    kept, ROTATION_BASES = ROTATION_BASES, (50.0, 50.0, 50.0)
    try:
        assert (rotation_plain(spec, st, seqs[0]) - want[0]).abs().max() > 0.05
    finally:
        ROTATION_BASES = kept


# -- a whole toy architecture: its own config.json keys, registered here, written, loaded, served -----------
def register_toy_architecture():
    """`ToyTurnLM`: the toy rotation and the toy experts as an architecture of their own, with a configuration
    class that reads its own keys from config.json.  Nothing of the framework's files changes."""
    from dataclasses import asdict, dataclass
    from denno_beta_amd.config import ConfigError, known_architectures, register_architecture
    from denno_beta_amd.parts import DecoderSpec, LayerCall, LayerSpec
    register_toy_rotation_and_experts()
    if "ToyTurnLM" in known_architectures():
        return

    @dataclass(frozen=True)
    class ToyTurnConfig:
        toy_width: int
        toy_heads: tuple          # per layer: (query heads, key heads)
        toy_head_size: int
        toy_inner: int
        toy_experts: int
        toy_vocab: int
        toy_positions: int
        toy_base: float
        toy_last_base: float      # the last layer turns by a base of its own
        toy_eps: float
        toy_end: int              # the token that ends a request

        @classmethod
        def from_dict(cls, d):
            missing = [k for k in cls.__dataclass_fields__ if k not in d]
            if missing:
                raise ConfigError(f"config.json of a ToyTurnLM lacks {missing}")
            c = cls(**{k: d[k] for k in cls.__dataclass_fields__})
            if c.toy_head_size % 16 != 0:
                raise ConfigError(f"toy_head_size {c.toy_head_size}: heads come in steps of 16")
            return cls(**{**asdict(c), "toy_heads": tuple(tuple(h) for h in c.toy_heads)})

        def to_dict(self):
            return {**asdict(self), "toy_heads": [list(h) for h in self.toy_heads]}

    def build(cfg):
        E, dh, layers = cfg.toy_width, cfg.toy_head_size, []
        for i, (heads, kv_heads) in enumerate(cfg.toy_heads):
            p = f"L{i}."
            last = i == len(cfg.toy_heads) - 1
            own = dict(position=("toy_rotation", dict(head_dim=dh, base=cfg.toy_last_base))) if last else {}
            layers.append(LayerSpec("pre_norm", dict(
                norm1=("layernorm", dict(width=E, eps=cfg.toy_eps, weight_name=p + "n1.g", bias_name=None)),
                mixer=("causal_attention", dict(width=E, n_heads=heads, n_kv_heads=kv_heads, head_dim=dh, scale=dh ** -0.5,
                                                qkv_weight=p + "qkv.w", qkv_bias=None, out_weight=p + "o.w", out_bias=None,
                                                **own)),
                norm2=("layernorm", dict(width=E, eps=cfg.toy_eps, weight_name=p + "n2.g", bias_name=None)),
                ffn=("toy_experts", dict(width=E, inner=cfg.toy_inner, n_experts=cfg.toy_experts, prefix=p + "ffn.")))))
        return DecoderSpec(vocab=cfg.toy_vocab, width=E, max_positions=cfg.toy_positions, token_table="tok",
                           position=("toy_rotation", dict(head_dim=dh, base=cfg.toy_base)), layers=layers,
                           run_order=[LayerCall(i, i) for i in range(len(layers))],
                           final_norm=("layernorm", dict(width=E, eps=cfg.toy_eps, weight_name="nf.g", bias_name=None)),
                           eos_token_ids=(cfg.toy_end,))

    register_architecture(["ToyTurnLM", "toy_turn"], ToyTurnConfig, build)


TOY_TURN = dict(architectures=["ToyTurnLM"], toy_width=48, toy_heads=[[3, 3], [3, 1]], toy_head_size=16, toy_inner=40,
                toy_experts=2, toy_vocab=61, toy_positions=96, toy_base=30.0, toy_last_base=5.0, toy_eps=1e-6, toy_end=60)


def test_a_whole_architecture_is_registered_written_loaded_and_served(backend, tmp_path):
    """An architecture that the framework does not know: its configuration class, its builder and its parts are
    defined in this file and registered by name; a model folder is written from a configuration and a seed,
    read back through the registry by what its config.json says, and served by the engine (scheduler, portions,
    sampling): every request's greedy tokens equal those of its run alone, and the logits of every way of cutting
    the work agree with the plain functions of this file."""
    from denno_beta_amd.config import ConfigError, load_config
    from denno_beta_amd.engine import Engine, ModelRunner, SamplingParams
    from denno_beta_amd.weights import write_model_folder
    register_toy_architecture()
    folder = write_model_folder(str(tmp_path / "toy"), TOY_TURN, seed=4, dtype="float32")
    arch, cfg = load_config(folder)
    assert arch.name == "ToyTurnLM" and cfg.toy_heads == ((3, 3), (3, 1)) and cfg.to_dict()["toy_inner"] == 40
    with pytest.raises(ConfigError, match="toy_experts"):
        arch.config_cls.from_dict({k: v for k, v in TOY_TURN.items() if k != "toy_experts"})
    # the replay: whole, the tail token by token, portions, mixed with pages used again
    r = ModelRunner.from_folder(folder, options(backend, cache_tokens=160))
    seqs = [seeded_tokens(20 + i, n, 60) for i, n in enumerate((33, 9, 50, 21))]
    # against the plain functions of this file (the toy parts multiply with the library, whose sums depend on
    # the rows beside them: close, not equal)
    from denno_beta_amd.weights.safetensors_io import SafetensorsFile
    sf = SafetensorsFile(folder + "/model.safetensors")
    st = {k: sf.tensor(k).float().clone() for k in sf.entries}
    sf.close()
    global ROTATION_BASES
    kept, ROTATION_BASES = ROTATION_BASES, (30.0, 5.0)
    try:
        want = [rotation_plain(r.spec, st, s) for s in seqs]
    finally:
        ROTATION_BASES = kept
    for kind, steps in (("whole", U.whole_trace(seqs)), ("tail", U.tail_decode_trace(seqs, 8)),
                        ("portions", U.chunk_trace(seqs)), ("mixed", U.mixed_trace(seqs, seed=9))):
        got = U.replay(r, steps)
        for i in range(len(seqs)):
            U.assert_close(got[f"r{i}"], want[i], "float32", f"the toy architecture, {kind}, request {i}")
    r.cache.manager.check()
    assert r.cache.manager.reuse_count(0) > 0
    # served: six requests through the scheduler, portions of 16 tokens, three live at a time
    def engine():
        return Engine.from_folder(folder, options(backend, max_live=3, prefill_chunk=16, max_batch_tokens=40))
    prompts = [seeded_tokens(40 + i, n, 60) for i, n in enumerate((5, 37, 18, 2, 44, 11))]
    params = SamplingParams(temperature=0.0, max_tokens=12)
    together = engine().generate(prompts, params)
    for p, toks in zip(prompts, together):
        assert engine().generate([p], params)[0] == toks
        assert len(toks) == 12 or toks[-1] == 60


# -- an arrangement with four norms, a head with a bias and a scale -------------------------------
def register_sandwich_arrangement():
    from denno_beta_amd.parts import ARRANGEMENTS
    if "toy_sandwich" in ARRANGEMENTS:
        return

    @ARRANGEMENTS.register("toy_sandwich")
    class SandwichBlock:
        """x += post1(mixer(pre1(x))); x += post2(ffn(pre2(x))): a norm before and a norm after each part, so
        the parts' results pass through a norm before they are added.  The parts add into a stream of zeros
        that stands in for the residual stream."""
        SLOTS = {"pre1": "norm", "mixer": "mixer", "post1": "norm", "pre2": "norm", "ffn": "feed_forward",
                 "post2": "norm"}

        def __init__(self, pre1, mixer, post1, pre2, ffn, post2):
            self.pre1, self.mixer, self.post1, self.pre2, self.ffn, self.post2 = pre1, mixer, post1, pre2, ffn, post2

        def parts(self):
            return [self.pre1, self.mixer, self.post1, self.pre2, self.ffn, self.post2]

        def mixers(self):
            return [self.mixer]

        def forward(self, x, ctx, caches, runtime):
            runtime.stream_stats = None            # nothing is left for a norm of these rows
            out = torch.zeros_like(x)
            self.mixer.forward(self.pre1.forward(x, runtime.act_dtype), ctx, caches[0], accumulate_into=out)
            x += self.post1.forward(out, torch.float32)
            out.zero_()
            self.ffn.forward(self.pre2.forward(x, runtime.act_dtype), ctx, accumulate_into=out)
            x += self.post2.forward(out, torch.float32)


def sandwich_model():
    from denno_beta_amd.parts import DecoderSpec, LayerCall, LayerSpec
    E = 32
    norm = lambda name, eps: ("layernorm", dict(width=E, eps=eps, weight_name=name + ".g", bias_name=name + ".b"))   # noqa: E731
    layers = []
    for i in range(2):
        p = f"L{i}."
        layers.append(LayerSpec("toy_sandwich", dict(
            pre1=norm(p + "pre1", 1e-5), post1=norm(p + "post1", 1e-3), pre2=norm(p + "pre2", 1e-5),
            post2=norm(p + "post2", 1e-2),
            mixer=("causal_attention", dict(width=E, n_heads=2, n_kv_heads=2, head_dim=16, scale=0.25,
                                            qkv_weight=p + "qkv.w", qkv_bias=None, out_weight=p + "o.w", out_bias=None)),
            ffn=("dense_mlp", dict(width=E, inner=64, activation="gelu_tanh", up_weight=p + "up.w", up_bias=None,
                                   down_weight=p + "down.w", down_bias=None)))))
    return DecoderSpec(vocab=50, width=E, max_positions=128, token_table="tok",
                       position=("learned_absolute", dict(n_positions=128, width=E, name="pos")), layers=layers,
                       run_order=[LayerCall(i, i) for i in range(2)], final_norm=norm("nf", 1e-5),
                       head_weight="head.w", head_bias="head.b", logit_scale=0.5, logit_softcap=3.0,
                       embedding_scale=E ** 0.5)


def sandwich_plain(st, seq):
    E = 32
    ln = lambda x, name, eps: P.layer_norm(x, st[name + ".g"], st[name + ".b"], eps)   # noqa: E731
    x = st["tok"][torch.tensor(seq)] * E ** 0.5 + st["pos"][:len(seq)]
    for i in range(2):
        p = f"L{i}."
        qkv = ln(x, p + "pre1", 1e-5) @ st[p + "qkv.w"].t()
        a = P.causal_attention(qkv[:, :E], qkv[:, E:2 * E], qkv[:, 2 * E:], 2, 0.25) @ st[p + "o.w"].t()
        x = x + ln(a, p + "post1", 1e-3)
        f = P.gelu_tanh(ln(x, p + "pre2", 1e-5) @ st[p + "up.w"].t()) @ st[p + "down.w"].t()
        x = x + ln(f, p + "post2", 1e-2)
    logits = (ln(x, "nf", 1e-5) @ st["head.w"].t() + st["head.b"]) * 0.5
    return 3.0 * torch.tanh(logits / 3.0)


def test_a_four_norm_arrangement_and_a_head_with_bias_scale_and_cap(backend):
    """An arrangement with other parts than the framework's own (four norms around a mixer and a
    feed-forward) is registered here and described by name; the head is a matrix of its own with a
    bias, its logits are scaled and capped, the token rows are multiplied.  The framework's files do not
    change."""
    from denno_beta_amd.engine import ModelRunner
    from denno_beta_amd.parts import LayerSpec
    register_sandwich_arrangement()
    spec = sandwich_model()
    names = {s.name for s in spec.param_specs()}
    assert {"head.w", "head.b", "L1.post2.g", "L0.pre1.b"} <= names
    tensors = draw(spec, backend)
    tensors["head.w"] *= 40.0          # logits large enough for the cap to bend them
    r = ModelRunner(spec, tensors, options(backend, cache_tokens=192))
    st = {k: v.float().cpu() for k, v in tensors.items()}
    seqs = [seeded_tokens(i, n, 50) for i, n in enumerate((30, 11, 47, 25))]
    want = [sandwich_plain(st, s) for s in seqs]
    assert max(w.abs().max().item() for w in want) > 2.0
    for kind, steps in (("whole", U.whole_trace(seqs)), ("tail", U.tail_decode_trace(seqs, 8)),
                        ("mixed", U.mixed_trace(seqs, seed=3))):
        got = U.replay(r, steps)
        for i in range(len(seqs)):
            U.assert_close(got[f"r{i}"], want[i], "float32", f"four norms, {kind}, request {i}")
    # a description that does not give the arrangement's parts is refused with their names
    bad = sandwich_model()
    bad.layers[0] = LayerSpec("toy_sandwich", {k: v for k, v in bad.layers[0].parts.items() if k != "post2"})
    with pytest.raises(ValueError, match="post2"):
        bad.instantiate()


@pytest.mark.gpu
@pytest.mark.parametrize("name,rows", [("A", 1), ("B", 7), ("D", 16)])
def test_norms_that_run_inside_the_products_beside_them(model_folders, name, rows):
    """In a step of at most 16 rows the block's norms are no kernels of their own: the product
    before a norm leaves what it needs, the product after it applies it.  The same steps with every
    norm as a kernel: logits agree to bfloat16 rounding, the cache holds the same keys but for
    roundings, and the products with a norm inside did run (two a layer, less the first layer's
    first, whose rows come from the embedding)."""
    from denno_beta_amd.engine import ModelRunner, StepEntry
    from denno_beta_amd.kernels import ops
    cfg = TINY[name][0]
    folder = model_folders(name, "bfloat16")
    seq = seeded_tokens(5, 40 + rows, cfg["vocab_size"])
    calls = {"in": 0, "out": 0}
    real_in, real_out = ops.linear_norm_in, ops.linear_norm_out

    def count_in(*a, **k):
        calls["in"] += 1
        return real_in(*a, **k)

    def count_out(*a, **k):
        calls["out"] += 1
        return real_out(*a, **k)
    got = {}
    try:
        ops.linear_norm_in, ops.linear_norm_out = count_in, count_out
        for inside in (True, False):
            r = ModelRunner.from_folder(folder, options("cuda:0", "bfloat16", use_graphs=False, norms_inside_products=inside))
            r.start_request(0)
            r.step([StepEntry(0, seq[:40], [])])
            before = dict(calls)
            got[inside] = r.step([StepEntry(0, seq[40:], list(range(rows)))]).float().cpu()
            if inside:
                assert calls["in"] - before["in"] == 2 * cfg["n_layer"] - 1
                assert calls["out"] - before["out"] == 2 * cfg["n_layer"] - 1
            else:
                assert calls == before
    finally:
        ops.linear_norm_in, ops.linear_norm_out = real_in, real_out
    U.assert_close(got[True], got[False], "bfloat16", f"{name}: norms inside the products against norms as kernels")
    want = P.PlainGPT2.from_folder(folder).logits(seq)[40:]
    U.assert_close(got[True], want, "bfloat16", f"{name}: norms inside the products against the plain implementation")


# -- a checkpoint that stores q, k and v apart still runs the fused projection ---------------------------
def register_split_qkv_architecture():
    """`ToySplitQKV`: GPT-2's own parts and configuration keys, but its checkpoints hold the three projections of
    a layer as tensors of their own (`attn.q.weight`, `attn.k.weight`, `attn.v.weight` and their biases).  The
    description names them as the sources of the attention mixer's one fused weight; nothing of the framework's
    files changes."""
    import copy
    from denno_beta_amd.config import known_architectures, register_architecture
    from denno_beta_amd.models.gpt2 import GPT2Config, build_gpt2
    if "ToySplitQKV" in known_architectures():
        return

    def build(cfg):
        spec = copy.deepcopy(build_gpt2(cfg))
        E = cfg.n_embd
        for i, layer in enumerate(spec.layers):
            kind, args = layer.parts["mixer"]
            p = f"h.{i}.attn."
            args = dict(args, qkv_weight=p + "qkv_joined.weight", qkv_bias=p + "qkv_joined.bias",
                        qkv_weight_sources=((p + "q.weight", E), (p + "k.weight", E), (p + "v.weight", E)),
                        qkv_bias_sources=((p + "q.bias", E), (p + "k.bias", E), (p + "v.bias", E)))
            layer.parts["mixer"] = (kind, args)
        return spec
    register_architecture(["ToySplitQKV"], GPT2Config, build)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_checkpoint_with_q_k_v_apart_feeds_the_fused_projection(backend, tmp_path, dtype):
    """The folder holds q, k and v as tensors of their own and no fused one; the loader joins them once; the mixer
    runs its one fused projection with the cache write (the same kernel as for a checkpoint that stores them
    fused); the logits are those of the plain GPT-2 on the joined tensors, in every cutting."""
    from safetensors.torch import load_file, save_file
    from denno_beta_amd.engine import ModelRunner
    from denno_beta_amd.kernels import ops
    from denno_beta_amd.weights import write_model_folder
    register_split_qkv_architecture()
    cfg = dict(TINY["B"][0], architectures=["ToySplitQKV"])
    folder = write_model_folder(str(tmp_path / "split"), cfg, seed=8, dtype=dtype)
    t = load_file(folder + "/model.safetensors")
    assert "h.0.attn.q.weight" in t and tuple(t["h.1.attn.k.weight"].shape) == (96, 96) and "h.2.attn.v.bias" in t
    assert not any("qkv_joined" in n or "c_attn" in n for n in t)
    assert not torch.equal(t["h.0.attn.q.weight"], t["h.0.attn.k.weight"])
    # the same weights as a GPT-2 folder, for the plain implementation
    joined = {n: x for n, x in t.items() if ".attn.q." not in n and ".attn.k." not in n and ".attn.v." not in n}
    for i in range(cfg["n_layer"]):
        p = f"h.{i}.attn."
        joined[p + "c_attn.weight"] = torch.cat([t[p + f"{x}.weight"] for x in "qkv"], dim=1).contiguous()
        joined[p + "c_attn.bias"] = torch.cat([t[p + f"{x}.bias"] for x in "qkv"]).contiguous()
    plain_dir = tmp_path / "joined"
    plain_dir.mkdir()
    save_file(joined, str(plain_dir / "model.safetensors"))
    (plain_dir / "config.json").write_text(json.dumps(dict(cfg, architectures=["GPT2LMHeadModel"])))
    plain = P.PlainGPT2.from_folder(str(plain_dir))
    seqs = [seeded_tokens(90 + i, n, cfg["vocab_size"]) for i, n in enumerate((40, 9, 70))]
    want = [plain.logits(s) for s in seqs]
    calls = {"fused": 0}
    real = ops.linear_qkv

    def counting(*a, **k):
        calls["fused"] += 1
        return real(*a, **k)
    try:
        ops.linear_qkv = counting
        r = ModelRunner.from_folder(folder, options(backend, dtype, cache_tokens=256, use_graphs=False,
                                                    norms_inside_products=False))
        for kind, steps in (("whole", U.whole_trace(seqs)), ("tail", U.tail_decode_trace(seqs, 8)),
                            ("portions", U.chunk_trace(seqs)), ("mixed", U.mixed_trace(seqs, seed=3))):
            before = calls["fused"]
            got = U.replay(r, steps)
            assert calls["fused"] - before == cfg["n_layer"] * len(steps)
            for i in range(len(seqs)):
                U.assert_close(got[f"r{i}"], want[i], dtype, f"q, k, v apart, {dtype}, {kind}, request {i}")
    finally:
        ops.linear_qkv = real
    r.cache.manager.check()


# -- a norm without a mean, defined here, runs inside the products beside it -----------------------------
def register_toy_rms_norm():
    from denno_beta_amd.parts import NORMS, Part
    from denno_beta_amd.weights import ParamSpec
    if "toy_rms" in NORMS:
        return

    @NORMS.register("toy_rms")
    class ToyRMSNorm(Part):
        """x / sqrt(mean(x^2) + eps) * weight, with the library; `fused_params` says what a product's kernel needs to
        run it itself."""
        graph_safe = True

        def __init__(self, width, eps, weight_name):
            self.width, self.eps, self.weight_name = width, eps, weight_name

        def param_specs(self):
            return [ParamSpec(self.weight_name, (self.width,), "vector", ("normal", 1.0, 0.1))]

        def bind(self, tensors, runtime):
            super().bind(tensors, runtime)
            self.weight = tensors[self.weight_name]

        def fused_params(self):
            return ("rmsnorm", self.weight, None, self.eps)

        def forward(self, x, out_dtype, rows=None, packed=False):
            src = x if rows is None else x[rows.long()]
            y = src * torch.rsqrt((src * src).mean(dim=1, keepdim=True) + self.eps) * self.weight
            return y.to(out_dtype)


@pytest.mark.gpu
@pytest.mark.parametrize("rows", [3, 16, 40])
def test_a_norm_without_a_mean_runs_inside_the_products(rows):
    """GPT-2's layers with a toy norm that takes no mean off in place of the layer norms: in steps of few rows the
    products beside it run it (the calls are counted), and the logits are those of the same steps with the norm
    run by its own forward, and of the plain formulas."""
    import copy
    from denno_beta_amd.engine import ModelRunner, StepEntry
    from denno_beta_amd.kernels import ops
    register_toy_rms_norm()
    cfg, spec = gpt2_spec("F")
    spec = copy.deepcopy(spec)
    for i, layer in enumerate(spec.layers):
        for slot in ("norm1", "norm2"):
            layer.parts[slot] = ("toy_rms", dict(width=cfg["n_embd"], eps=1e-6, weight_name=f"h.{i}.{slot}.g"))
    tensors = draw(spec, "cuda:0", dtype="bfloat16")
    seq = seeded_tokens(6, 20 + rows, cfg["vocab_size"])
    calls = {"in": 0}
    real_in = ops.linear_norm_in

    def count_in(*a, **k):
        assert k.get("no_mean") is True
        calls["in"] += 1
        return real_in(*a, **k)
    got = {}
    try:
        ops.linear_norm_in = count_in
        for inside in (True, False):
            r = ModelRunner(spec, dict(tensors), options("cuda:0", "bfloat16", use_graphs=False, norms_inside_products=inside))
            r.start_request(0)
            r.step([StepEntry(0, seq[:20], [])])
            before = calls["in"]
            got[inside] = r.step([StepEntry(0, seq[20:], list(range(rows)))]).float().cpu()
            assert calls["in"] - before == (2 * cfg["n_layer"] - 1 if inside else 0)
    finally:
        ops.linear_norm_in = real_in
    U.assert_close(got[True], got[False], "bfloat16", "a norm without a mean inside the products against its own forward")
    # the plain formulas: GPT-2's functions with this norm in the two places
    st = stored(tensors, spec)
    x = P.embed(torch.tensor(seq), torch.arange(len(seq)), st["wte.weight"], st["wpe.weight"]).double()
    rms = lambda v, g: v / torch.sqrt((v * v).mean(dim=1, keepdim=True) + 1e-6) * g.double()       # noqa: E731
    dh = cfg["n_embd"] // cfg["n_head"]
    for i in range(cfg["n_layer"]):
        p = f"h.{i}."
        qkv = rms(x, st[p + "norm1.g"]) @ st[p + "attn.c_attn.weight"].double() + st[p + "attn.c_attn.bias"].double()
        q, k, v = qkv.split(cfg["n_embd"], dim=1)
        o = P.causal_attention(q, k, v, cfg["n_head"], dh ** -0.5)
        x = x + o @ st[p + "attn.c_proj.weight"].double() + st[p + "attn.c_proj.bias"].double()
        f = torch.nn.functional.gelu(rms(x, st[p + "norm2.g"]) @ st[p + "mlp.c_fc.weight"].double() + st[p + "mlp.c_fc.bias"].double())
        x = x + f @ st[p + "mlp.c_proj.weight"].double() + st[p + "mlp.c_proj.bias"].double()
    want = P.head(x.float(), st["ln_f.weight"], st["ln_f.bias"], cfg["layer_norm_epsilon"], st["wte.weight"])[20:]
    U.assert_close(got[True], want, "bfloat16", "a norm without a mean inside the products against the plain formulas")


@pytest.mark.gpu
@pytest.mark.parametrize("name,rows", [("E", 40), ("F", 33)])
def test_a_sum_left_for_the_next_norm(model_folders, name, rows):
    """Steps of 65 to 256 rows: the attention's output projection and the feed-forward's second product leave their
    sums for the norms behind them, whose kernels add them (the calls are counted: in a model of L layers every norm
    but the first of the first layer; the last layer's feed-forward adds into the stream itself, since the final
    norm reads chosen rows only).  The logits are those of the same steps with every product adding its own sum."""
    from denno_beta_amd.engine import ModelRunner, StepEntry
    from denno_beta_amd.kernels import ops
    cfg = TINY[name][0]
    folder = model_folders(name, "bfloat16")
    seqs = [seeded_tokens(50 + i, rows, cfg["vocab_size"]) for i in range(3)]      # three requests: 99 to 120 rows a step
    calls = {"join": 0, "flush": 0}
    real_lj, real_j = ops.layernorm_join, ops.join

    def count_lj(*a, **k):
        calls["join"] += 1
        return real_lj(*a, **k)

    def count_j(*a, **k):
        calls["flush"] += 1
        return real_j(*a, **k)
    got = {}
    try:
        ops.layernorm_join, ops.join = count_lj, count_j
        for on in (True, False):
            r = ModelRunner.from_folder(folder, options("cuda:0", "bfloat16", use_graphs=False, deferred_sums=on))
            for i in range(3):
                r.start_request(i)
            before = dict(calls)
            got[on] = r.step([StepEntry(i, s, list(range(rows))) for i, s in enumerate(seqs)]).float().cpu()
            if on:
                assert calls["join"] - before["join"] == 2 * cfg["n_layer"] - 1 and calls["flush"] == before["flush"]
            else:
                assert calls == before
    finally:
        ops.layernorm_join, ops.join = real_lj, real_j
    U.assert_close(got[True], got[False], "bfloat16", f"{name}: sums left for the next norm against sums added at once")
    want = torch.cat([P.PlainGPT2.from_folder(folder).logits(s) for s in seqs])
    U.assert_close(got[True], want, "bfloat16", f"{name}: sums left for the next norm against the plain implementation")
