"""A key that stands out, through the whole engine.

Random weights give nearly flat attention: a key lost for one row moves a logit by less than bfloat16
rounds.  The model here is made so that the last token of a sequence attends to one far token and to
nothing else: keys are the normed rows with a fixed pattern of signs, queries the normed rows
themselves, both times 1.5, and the last token's row in the token table is the far token's row with
that pattern of signs.  Its score with the far key is then about 18 where every other key, its own
among them, scores like noise (about +-2), so nearly all of the output of attention is the far key's
value.  If that key is not found (a page's edge, a split's edge, a table that is off by one), the logits
of the last row change by what `effect` measures with the plain implementation: the same sequence
with another token in the far place.  The engine must be closer to the plain logits than a twentieth of
that, whichever kernel serves the row: the whole prompt in one step, portions, a decoded token (eager
and from a captured graph), and a decoded token beside another request's portion.
"""
import json
import os

import pytest
import torch

from plain.gpt2_plain import PlainGPT2

E, H, V, P = 128, 2, 1201, 1100
A_TOKEN, B_TOKEN, OTHER = 1199, 1200, 1198       # the far token, the last token, what stands in the far place otherwise


def write_lookup_model(folder, dtype):
    from safetensors.torch import save_file
    g = torch.Generator().manual_seed(5)
    n = lambda *shape, std=1.0: torch.randn(*shape, generator=g) * std   # noqa: E731
    signs = (torch.randint(0, 2, (E,), generator=g) * 2 - 1).float()
    wte = n(V, E)
    wte[B_TOKEN] = wte[A_TOKEN] * signs
    c_attn = torch.zeros(E, 3 * E)
    c_attn[:, :E] = 1.5 * torch.eye(E)                     # q = 1.5 h
    c_attn[:, E:2 * E] = 1.5 * torch.diag(signs)           # k = 1.5 signs * h
    c_attn[:, 2 * E:] = n(E, E, std=E ** -0.5)
    t = {"wte.weight": wte, "wpe.weight": n(P, E, std=0.05),
         "h.0.ln_1.weight": torch.ones(E), "h.0.ln_1.bias": torch.zeros(E),
         "h.0.attn.c_attn.weight": c_attn, "h.0.attn.c_attn.bias": torch.zeros(3 * E),
         "h.0.attn.c_proj.weight": n(E, E, std=E ** -0.5), "h.0.attn.c_proj.bias": torch.zeros(E),
         "h.0.ln_2.weight": torch.ones(E), "h.0.ln_2.bias": torch.zeros(E),
         "h.0.mlp.c_fc.weight": n(E, 4 * E, std=0.02), "h.0.mlp.c_fc.bias": torch.zeros(4 * E),
         "h.0.mlp.c_proj.weight": n(4 * E, E, std=0.02), "h.0.mlp.c_proj.bias": torch.zeros(E),
         "ln_f.weight": torch.ones(E), "ln_f.bias": torch.zeros(E)}
    dt = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype]
    save_file({k: v.to(dt).contiguous() for k, v in t.items()}, os.path.join(folder, "model.safetensors"))
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(dict(architectures=["GPT2LMHeadModel"], model_type="gpt2", n_layer=1, n_embd=E, n_head=H,
                       vocab_size=V, n_positions=P, layer_norm_epsilon=1e-5, activation_function="gelu_new"), f)


def sequence(n, far, planted=True):
    """n distinct tokens, the far token (or another) in place `far`, the last token at the end."""
    g = torch.Generator().manual_seed(1000 + n)
    seq = torch.randperm(OTHER, generator=g)[:n].tolist()
    seq[far] = A_TOKEN if planted else OTHER
    seq[-1] = B_TOKEN
    return seq


def test_the_plain_model_looks_the_far_key_up(tmp_path):
    write_lookup_model(str(tmp_path), "float32")
    plain = PlainGPT2.from_folder(str(tmp_path))
    for far in (0, 100, 268):
        a = plain.logits(sequence(270, far))[-1]
        b = plain.logits(sequence(270, far, planted=False))[-1]
        assert (a - b).abs().max() > 3.0, "the last row does not depend on the far key"
    # and where the far key is, is nearly the same to the last row (the position table's part is small)
    a, b = plain.logits(sequence(270, 3))[-1], plain.logits(sequence(270, 200))[-1]
    assert (a - b).abs().max() < 3.0


CONTEXTS = {270: (0, 15, 16, 255, 256, 268), 1030: (0, 16, 255, 256, 511, 512, 767, 1023, 1024, 1028)}


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
@pytest.mark.parametrize("n", sorted(CONTEXTS))
def test_a_far_key_is_found_by_every_kernel_of_the_engine(tmp_path, dtype, n):
    from denno_beta_amd.config import EngineOptions
    from denno_beta_amd.engine import ModelRunner, StepEntry
    folder = str(tmp_path)
    write_lookup_model(folder, dtype)
    plain = PlainGPT2.from_folder(folder)
    mk = lambda graphs: ModelRunner.from_folder(folder, EngineOptions(   # noqa: E731
        dtype=dtype, page_size=16, cache_tokens=3 * 1104, max_live=4, use_graphs=graphs))
    eager, graphs = mk(False), mk(True)
    other = sequence(200, 7)
    rid = 0
    for far in CONTEXTS[n]:
        seq = sequence(n, far)
        want = plain.logits(seq)[-1]
        effect = (want - plain.logits(sequence(n, far, planted=False))[-1]).abs().max().item()
        assert effect > 3.0
        got = {}
        # the whole prompt in one step
        eager.start_request(rid)
        got["whole"] = eager.step([StepEntry(rid, seq, [n - 1])])[0].cpu()
        eager.end_request(rid)
        # portions of 100 and the rest
        rid += 1
        eager.start_request(rid)
        for at in range(0, n, 100):
            part = seq[at:at + 100]
            out = eager.step([StepEntry(rid, part, [len(part) - 1] if at + 100 >= n else [])])
        got["portions"] = out[0].cpu()
        eager.end_request(rid)
        # all but the last token, then the last token as a decode step: kernel by kernel, and from a graph
        for name, r in (("decode", eager), ("graph", graphs)):
            rid += 1
            r.start_request(rid)
            r.step([StepEntry(rid, seq[:-1], [])])
            got[name] = r.step([StepEntry(rid, seq[-1:], [0])])[0].cpu()
            r.end_request(rid)
        # the last token beside a portion of another request
        rid += 2
        eager.start_request(rid), eager.start_request(rid + 1)
        eager.step([StepEntry(rid, seq[:-1], [])])
        got["mixed"] = eager.step([StepEntry(rid + 1, other[:77], []), StepEntry(rid, seq[-1:], [0])])[0].cpu()
        eager.end_request(rid), eager.end_request(rid + 1)
        rid += 2
        for name, row in got.items():
            worst = (row - want).abs().max().item()
            assert worst < effect / 20, f"{dtype}, context {n}, far key at {far}, {name}: off by {worst:.3g} " \
                                        f"where losing the key costs {effect:.3g}"
            if dtype == "float32":
                assert worst < 2e-4, (far, name, worst)
        eager.cache.manager.check(), graphs.cache.manager.check()
