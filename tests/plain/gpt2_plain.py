"""A plain, slow GPT-2: whole sequences, no cache, one function per part.

It is written from the formulas of ahinore/denno-beta's GPT-2 forward pass and shares
no code with the engine.  Citations are `file:line` under
`crates/denno-engine/src/` of the reference.  Options that the reference fixes
in code (eps, MLP width, activation, attention scale) are parameters here; the
values the reference uses are the defaults.

Every function takes and returns torch tensors on the CPU; `dtype` decides the
precision of the whole computation (float32 as the reference, or float64 to see
how much of a difference is rounding).
"""
from __future__ import annotations

import json
import math
import os

import torch


# ----------------------------------------------------------------------------
# parts
# ----------------------------------------------------------------------------

def embed(tokens, positions, wte, wpe):
    """x[i,:] = wte[token_i,:] + wpe[pos_i,:]                 (model/gpt2.rs:142-150)"""
    return wte[tokens] + wpe[positions]


def layer_norm(x, gamma, beta, eps):
    """Per row: mean, biased variance of (x-mean), (x-mean)/sqrt(var+eps)*gamma+beta
    (tensor.rs:1101-1112)."""
    mean = x.sum(dim=-1, keepdim=True) / x.shape[-1]
    d = x - mean
    var = (d * d).sum(dim=-1, keepdim=True) / x.shape[-1]
    inv = 1.0 / torch.sqrt(var + eps)
    return d * inv * gamma + beta


def linear_in_out(x, w, b):
    """Conv1D: the weight is stored [in, out] and used as it is: x @ W + b
    (model/gpt2.rs:155-156, quant.rs:1049-1051, tensor.rs:1092-1098)."""
    y = x @ w
    if b is not None:
        y = y + b
    return y


def gelu_tanh(t):
    """0.5 t (1 + tanh(0.7978845608028654 (t + 0.044715 t^3)))   (tensor.rs:1156-1161)"""
    return 0.5 * t * (1.0 + torch.tanh(0.7978845608028654 * (t + 0.044715 * t * t * t)))


def gelu_erf(t):
    """0.5 t (1 + erf(t / sqrt 2)): the exact form, which `activation_function: gelu`
    names.  The reference has the tanh form only."""
    return 0.5 * t * (1.0 + torch.erf(t / math.sqrt(2.0)))


ACTIVATIONS = {"gelu_new": gelu_tanh, "gelu_pytorch_tanh": gelu_tanh, "gelu": gelu_erf}


def softmax_rows(s):
    """exp(s - max) / sum, per row                              (tensor.rs:1171-1183)"""
    m = s.max(dim=-1, keepdim=True).values
    e = torch.exp(s - m)
    return e / e.sum(dim=-1, keepdim=True)


def causal_attention(q, k, v, n_head, scale, first_position=0, window=None):
    """q: [n, E] for positions first_position..first_position+n-1; k, v: [m, E] for
    positions 0..m-1 (m >= first_position + n).  Head hd is columns hd*dh..(hd+1)*dh;
    query i sees keys j <= first_position + i (causal by loop bound, no mask tensor);
    scores are (q.k)*scale; heads are written back side by side
    (model/gpt2.rs:170-202).  `window`, if given, keeps only the last `window` keys
    (j > pos - window); the reference's GPT-2 has none."""
    n, e = q.shape
    dh = e // n_head
    out = torch.zeros_like(q)
    for i in range(n):
        pos = first_position + i
        lo = 0 if window is None else max(0, pos - window + 1)
        for hd in range(n_head):
            c = slice(hd * dh, (hd + 1) * dh)
            s = (k[lo:pos + 1, c] @ q[i, c]) * scale
            p = softmax_rows(s[None, :])[0]
            out[i, c] = p @ v[lo:pos + 1, c]
    return out


def causal_attention_by_head(q, k, v, n_head, scale):
    """The same result as causal_attention for a whole sequence from position 0, one head at a time
    as matrices: scores of all pairs, -inf above the diagonal, softmax_rows, times the values.  For
    sequences too long for the loop above; tests/test_plain.py holds the two against each other."""
    n, e = q.shape
    dh = e // n_head
    out = torch.zeros_like(q)
    above = torch.ones(n, n, dtype=torch.bool).triu(1)
    for hd in range(n_head):
        c = slice(hd * dh, (hd + 1) * dh)
        s = (q[:, c] @ k[:, c].t()) * scale
        out[:, c] = softmax_rows(s.masked_fill(above, float("-inf"))) @ v[:, c]
    return out


def attention_scale(head_dim, layer_idx, scale_attn_weights=True, scale_attn_by_inverse_layer_idx=False):
    """1/sqrt(dh) as the reference (model/gpt2.rs:174); config options of the
    architecture switch it off or divide further by (layer_idx + 1)."""
    s = 1.0
    if scale_attn_weights:
        s = s / math.sqrt(head_dim)
    if scale_attn_by_inverse_layer_idx:
        s = s / float(layer_idx + 1)
    return s


def attention_block(h, p, n_head, scale, attention=causal_attention):
    """qkv = h W + b, columns q | k | v; attention; output projection
    (model/gpt2.rs:155-208)."""
    e = h.shape[-1]
    qkv = linear_in_out(h, p["attn.c_attn.weight"], p["attn.c_attn.bias"])
    q, k, v = qkv[:, :e], qkv[:, e:2 * e], qkv[:, 2 * e:]
    a = attention(q, k, v, n_head, scale)
    return linear_in_out(a, p["attn.c_proj.weight"], p["attn.c_proj.bias"])


def mlp_block(h, p, act):
    """f = act(h W_fc + b_fc); f W_proj + b_proj               (model/gpt2.rs:211-219)"""
    f = act(linear_in_out(h, p["mlp.c_fc.weight"], p["mlp.c_fc.bias"]))
    return linear_in_out(f, p["mlp.c_proj.weight"], p["mlp.c_proj.bias"])


def block(x, p, n_head, scale, eps, act, attention=causal_attention):
    """x += attn(LN1(x)); x += mlp(LN2(x))                      (model/gpt2.rs:152-220)"""
    x = x + attention_block(layer_norm(x, p["ln_1.weight"], p["ln_1.bias"], eps), p, n_head, scale, attention)
    x = x + mlp_block(layer_norm(x, p["ln_2.weight"], p["ln_2.bias"], eps), p, act)
    return x


def head(x, gamma, beta, eps, wte):
    """logits = LN_f(x) @ wte^T, tied head, no bias             (model/gpt2.rs:224-229).
    The reference computes the last row only; here every row."""
    return layer_norm(x, gamma, beta, eps) @ wte.t()


# ----------------------------------------------------------------------------
# the whole model
# ----------------------------------------------------------------------------

class PlainGPT2:
    """Weights by name (with or without the `transformer.` prefix) and the config
    dictionary of config.json."""

    def __init__(self, config: dict, tensors: dict, dtype=torch.float32):
        self.cfg = config
        self.dtype = dtype
        t = {}
        for name, w in tensors.items():
            if name.startswith("transformer."):
                name = name[len("transformer."):]
            t[name] = w.to(dtype)
        self.t = t
        self.n_layer = config["n_layer"]
        self.n_head = config["n_head"]
        self.n_embd = config["n_embd"]
        self.eps = config.get("layer_norm_epsilon", 1e-5)
        self.act = ACTIVATIONS[config.get("activation_function", "gelu_new")]
        self.scale_w = config.get("scale_attn_weights", True)
        self.scale_inv = config.get("scale_attn_by_inverse_layer_idx", False)

    @classmethod
    def from_folder(cls, folder, dtype=torch.float32):
        from safetensors.torch import load_file
        with open(os.path.join(folder, "config.json")) as f:
            cfg = json.load(f)
        return cls(cfg, load_file(os.path.join(folder, "model.safetensors")), dtype)

    def layer_params(self, i):
        pre = f"h.{i}."
        return {k[len(pre):]: v for k, v in self.t.items() if k.startswith(pre)}

    def logits(self, tokens, by_head=False, input_table=None) -> torch.Tensor:
        """[len(tokens), vocab] logits of one whole sequence starting at position 0.
        by_head: attention one head at a time as matrices (long sequences of deep models).
        input_table: the token rows come from this table (the head stays the model's own token table)."""
        tok = torch.as_tensor(tokens, dtype=torch.long)
        pos = torch.arange(len(tok))
        x = embed(tok, pos, self.t["wte.weight"] if input_table is None else input_table.to(self.t["wte.weight"].dtype),
                  self.t["wpe.weight"])
        dh = self.n_embd // self.n_head
        for i in range(self.n_layer):
            scale = attention_scale(dh, i, self.scale_w, self.scale_inv)
            x = block(x, self.layer_params(i), self.n_head, scale, self.eps, self.act,
                      causal_attention_by_head if by_head else causal_attention)
        return head(x, self.t["ln_f.weight"], self.t["ln_f.bias"], self.eps, self.t["wte.weight"])

    def greedy(self, prompt, n_new):
        """Greedy continuation, recomputing the whole sequence each time."""
        seq = list(prompt)
        for _ in range(n_new):
            seq.append(int(argmax_first(self.logits(seq)[-1])))
        return seq[len(prompt):]


def argmax_first(row):
    """Index of the first maximum; NaN never wins             (sampler.rs:301-331)."""
    best, best_v = 0, float("-inf")
    for i, v in enumerate(row.tolist()):
        if v > best_v:
            best, best_v = i, v
    return best
