"""Plain PyTorch references of the kernels, one function per entry of
`denno_beta_amd.kernels.ops`, with the same arguments.  Computation is 32-bit (inputs in
bfloat16 are widened first); outputs are rounded to the output tensor's dtype once.

They serve two ends: the GPU tests compare each HIP kernel with its reference here, and the
CPU tests put them in the kernels' place to run the engine's host logic (batching, cache,
scheduling) without a GPU.
"""
from __future__ import annotations

import math

import torch


def embed(tokens, positions, wte, wpe, out, token_scale=1.0):
    x = wte[tokens.long()].float()
    if token_scale != 1.0:
        x = x * torch.tensor(token_scale, dtype=torch.float32)
    if wpe is not None:
        x = x + wpe[positions.long()].float()
    out.copy_(x)
    return out


def embed_sum(parts, out):
    x = None
    for table, index, scale in parts:
        a = table[index.long()].float()
        if scale != 1.0:
            a = a * torch.tensor(scale, dtype=torch.float32)
        x = a if x is None else x + a
    out.copy_(x)
    return out


def logits_post(logits, scale=1.0, softcap=0.0):
    logits.mul_(torch.tensor(scale, dtype=torch.float32))
    if softcap > 0:
        logits.copy_(softcap * torch.tanh(logits / softcap))
    return logits


def layernorm(x, gamma, beta, eps, out, rows=None):
    src = x if rows is None else x[rows.long()]
    mean = src.mean(dim=-1, keepdim=True)
    d = src - mean
    var = (d * d).mean(dim=-1, keepdim=True)
    y = d / torch.sqrt(var + eps) * gamma
    if beta is not None:
        y = y + beta
    out.copy_(y)
    return out


def kv_write(src, k_col, v_col, slot_map, k_pool, v_pool):
    n_pages, hkv, ps, dh = k_pool.shape
    w = hkv * dh
    for t in range(src.shape[0]):
        slot = int(slot_map[t])
        if slot < 0:
            continue
        page, off = divmod(slot, ps)
        k_pool[page, :, off, :] = src[t, k_col:k_col + w].view(hkv, dh)
        v_pool[page, :, :, off] = src[t, v_col:v_col + w].view(hkv, dh)


def cast(x, out):
    out.copy_(x)
    return out


def linear(a, w, bias=None, out=None, epilogue="none", residual=None):
    wide = torch.float64 if a.dtype == torch.float64 else torch.float32
    y = a.to(wide) @ w.to(wide).t()
    if bias is not None:
        y = y + bias
    if residual is not None:
        residual += y
        return residual
    if epilogue == "gelu_tanh":
        y = torch.nn.functional.gelu(y, approximate="tanh")
    elif epilogue == "gelu_erf":
        y = torch.nn.functional.gelu(y)
    elif epilogue != "none":
        raise ValueError(epilogue)
    out.copy_(y)
    return out


def norm_folded(w_rows, bias, gamma, beta):
    w = w_rows.float()
    c1 = w @ gamma.float()
    c2 = torch.zeros_like(c1) if beta is None else w @ beta.float()
    return c1, (c2 if bias is None else c2 + bias.float())


def linear_norm_out(a, w, bias, residual, gamma, copy, stats):
    linear(a, w, bias, residual=residual)
    copy.copy_(residual * gamma)
    blocks = residual.view(residual.shape[0], -1, 16)
    mean = blocks.mean(dim=-1)
    stats[:, :, 0] = mean
    stats[:, :, 1] = ((blocks - mean[:, :, None]) ** 2).sum(dim=-1)
    return residual


def linear_norm_in(copy, stats, c1, c2, eps, w, out, epilogue="none", kv=None, no_mean=False):
    """The kernel's own formula: the product of the rows that are not normalised, then the row's mean
    and 1 / sqrt(var + eps), joined from the blocks' pairs, on the sums.  no_mean: the mean counts as 0."""
    mean = stats[:, :, 0].mean(dim=1, keepdim=True)
    if no_mean:
        mean = torch.zeros_like(mean)
    var = (stats[:, :, 1] + 16.0 * (stats[:, :, 0] - mean) ** 2).sum(dim=1, keepdim=True) / copy.shape[1]
    y = (copy.float() @ w.float().t() - mean * c1) / torch.sqrt(var + eps) + c2
    if epilogue == "gelu_tanh":
        y = torch.nn.functional.gelu(y, approximate="tanh")
    elif epilogue == "gelu_erf":
        y = torch.nn.functional.gelu(y)
    if kv is None:
        out.copy_(y)
        return out
    slot_map, k_pool, v_pool, q_width = kv
    hkv, dh = k_pool.shape[1], k_pool.shape[3]
    full = y.to(out.dtype)
    kv_write(full, q_width, q_width + hkv * dh, slot_map, k_pool, v_pool)
    out.copy_(full[:, :out.shape[1]])
    return out[:, :q_width]


def attention(q, out, k_pool, v_pool, block_tables, tiles, n_heads, scale, window=0, tiles_wide=None,
              single_rows=False, max_context=0, decode_waves=None):
    n_pages, hkv, ps, dh = k_pool.shape
    group = n_heads // hkv
    tl = tiles.cpu().tolist()
    bt = block_tables.cpu()
    kf, vf = k_pool.float(), v_pool.float()
    for seq, row0, nrows, pos0 in zip(*tl):
        if seq < 0:
            continue
        for i in range(nrows):
            pos = pos0 + i
            lo = max(0, pos - window + 1) if window > 0 else 0
            keys = torch.arange(lo, pos + 1)
            pages = bt[seq][keys // ps].long()
            offs = keys % ps
            assert (pages >= 0).all(), "attention reads a page that was given back"
            for h in range(n_heads):
                k = kf[pages, h // group, offs, :]                  # [n, dh]
                v = vf[pages, h // group, :, offs]
                qv = q[row0 + i, h * dh:(h + 1) * dh].float()
                p = torch.softmax((k @ qv) * scale, dim=0)
                out[row0 + i, h * dh:(h + 1) * dh] = (p @ v).to(out.dtype)
    return out


def sample(logits, temperature, uniform, out):
    for r in range(logits.shape[0]):
        row = logits[r]
        t = float(temperature[r])
        if not t > 0:
            best, best_v = 0, float("-inf")
            for i, v in enumerate(row.tolist()):
                if v > best_v:
                    best, best_v = i, v
            out[r] = best
            continue
        z = row / t
        e = torch.exp(z - z.max())
        c = torch.cumsum(e.double(), 0)
        target = float(uniform[r]) * float(c[-1])
        idx = int(torch.searchsorted(c, torch.tensor(target, dtype=torch.float64)))
        out[r] = min(idx, row.shape[0] - 1)
    return out


def penalties(logits, ctx, begin, length, repetition, frequency, presence, ngram, bounds=None):
    from plain import sampler_plain as sp
    for r in range(logits.shape[0]):
        c = ctx[int(begin[r]):int(begin[r]) + int(length[r])].tolist()
        row = logits[r].tolist()
        row = sp.repetition_penalty(row, c, float(repetition[r]))
        row = sp.frequency_presence(row, c, float(frequency[r]), float(presence[r]))
        row = sp.no_repeat_ngram(row, c, int(ngram[r]))
        logits[r] = torch.tensor(row, dtype=torch.float32)
    return logits


def history_append(history, begin, length, rows, tokens, bounds=None):
    for b, n, r in zip(begin.tolist(), length.tolist(), rows.tolist()):
        history[b + n] = tokens[r]
    return history


def sample_top(logits, rows, temperature, uniform, top_k, top_p, out, undecided):
    from plain import sampler_plain as sp
    for j, r in enumerate(rows.tolist()):
        k, p = int(top_k[j]), float(top_p[j])
        if k > 0:
            out[r] = sp.top_k_top_p(logits[r].tolist(), float(temperature[r]), min(k, 2048),
                                    None if p >= 1.0 else p, float(uniform[r]))
            undecided[j] = 0
        else:
            tok, whole = sp.top_p_alone(logits[r].tolist(), float(temperature[r]), p, float(uniform[r]))
            out[r], undecided[j] = tok, int(whole)
    return out


def sample_full(logits, rows, temperature, uniform, top_p, out, only=None):
    from plain import sampler_plain as sp
    for j, r in enumerate(rows.tolist()):
        if only is not None and int(only[j]) == 0:
            continue
        p = float(top_p[j])
        out[r] = sp.top_k_top_p(logits[r].tolist(), float(temperature[r]), None, None if p >= 1.0 else p,
                                float(uniform[r]))
    return out


def linear_qkv(a, w, bias, out, slot_map, k_pool, v_pool, q_width):
    linear(a, w, bias, out=out)
    kvw = k_pool.shape[1] * k_pool.shape[3]
    kv_write(out, q_width, q_width + kvw, slot_map, k_pool, v_pool)
    return out[:, :q_width]
