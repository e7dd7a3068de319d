"""Plain samplers and logit processors, written from the reference's sampler
(`crates/denno-engine/src/sampler.rs`).  Python lists and floats, no torch; the
uniform number `u` in [0,1) is an argument, since the reference's generator
(`rand::StdRng`) is not reproduced.
"""
from __future__ import annotations

import math

import numpy as np


def f32(x):
    return float(np.float32(x))


def greedy(logits):
    """First maximum, NaN ignored (sampler.rs:350-367, 301-331)."""
    best, best_v = 0, float("-inf")
    for i, v in enumerate(logits):
        if v > best_v:
            best, best_v = i, v
    return best


def temperature_walk(logits, t, u):
    """z = logit/T; e_i = exp(z_i - max z); u*sum(e); walk ascending, subtracting,
    until <= 0; the last index otherwise (sampler.rs:440-463).  32-bit like the
    reference."""
    z = np.asarray(logits, dtype=np.float32) / np.float32(t)
    m = np.float32(-np.inf)
    for v in z:
        if v > m:
            m = v
    e = np.exp(z - m).astype(np.float32)
    total = np.float32(0.0)
    for v in e:
        total = np.float32(total + v)
    r = np.float32(np.float32(u) * total)
    for i, v in enumerate(e):
        r = np.float32(r - v)
        if r <= 0.0:
            return i
    return len(e) - 1


def top_k_top_p(logits, t, top_k, top_p, u):
    """Keep the k largest of logit/T (ties: lower index first), softmax over them,
    cut after the cumulative probability reaches p, renormalise, walk
    (sampler.rs:372-385, 487-514).  top_k None = all."""
    z = [(f32(x) / f32(t), i) for i, x in enumerate(logits)]
    z.sort(key=lambda a: (-a[0], a[1]))
    if top_k is not None:
        z = z[:max(1, min(top_k, len(z)))]
    mx = z[0][0]
    probs = [math.exp(a[0] - mx) for a in z]
    if top_p is not None:
        total = sum(probs)
        cum, cutoff = 0.0, len(probs)
        for i, p in enumerate(probs):
            cum += p / total
            if cum >= top_p:
                cutoff = i + 1
                break
        probs = probs[:cutoff]
    total = sum(probs)
    r = u * total
    for i, p in enumerate(probs):
        r -= p
        if r <= 0.0:
            return z[i][1]
    return z[len(probs) - 1][1]


TOP_P_SUBSET = 2048      # sampler.rs:23


def top_p_alone(logits, t, top_p, u):
    """top-p without top-k (sampler.rs:387-435): over a vocabulary larger than 2,048 the cut is
    looked for among the 2,048 largest, with probabilities relative to their sum; if it falls
    before the last of them the token is drawn from that head of the list, else everything is
    done over again on the whole sorted vocabulary (sample_legacy_full, :466-476).
    -> (token, whether the whole vocabulary was needed)."""
    n = len(logits)
    if n > TOP_P_SUBSET:
        z = [(f32(x) / f32(t), i) for i, x in enumerate(logits)]
        z.sort(key=lambda a: (-a[0], a[1]))
        sub = z[:TOP_P_SUBSET]
        mx = sub[0][0]
        probs = [math.exp(a[0] - mx) for a in sub]
        total = sum(probs)
        cum, cutoff = 0.0, TOP_P_SUBSET
        for i, p in enumerate(probs):
            cum += p / total
            if cum >= top_p:
                cutoff = i + 1
                break
        if cutoff < TOP_P_SUBSET:
            pr = probs[:cutoff]
            r = u * sum(pr)
            for i, p in enumerate(pr):
                r -= p
                if r <= 0.0:
                    return sub[i][1], False
            return sub[cutoff - 1][1], False
    return top_k_top_p(logits, t, None, top_p, u), n > TOP_P_SUBSET


def repetition_penalty(logits, context, penalty):
    """Each distinct context token once: l > 0 -> l / p, else l * p (sampler.rs:42-58)."""
    out = list(logits)
    if penalty == 1.0:
        return out
    for t in set(context):
        if 0 <= t < len(out):
            out[t] = out[t] / penalty if out[t] > 0 else out[t] * penalty
    return out


def frequency_presence(logits, context, frequency, presence):
    """l[t] -= f * count(t) + p * (count(t) > 0)               (sampler.rs:99-118)."""
    out = list(logits)
    counts = {}
    for t in context:
        if 0 <= t < len(out):
            counts[t] = counts.get(t, 0) + 1
    for t, c in counts.items():
        out[t] -= frequency * c + presence
    return out


def no_repeat_ngram(logits, context, n):
    """Tokens that would complete an n-gram already in the context get -inf
    (sampler.rs:150-172)."""
    out = list(logits)
    if n <= 1 or len(context) < n:
        return out
    prefix = list(context[len(context) - (n - 1):])
    for i in range(0, len(context) - n + 1):
        if list(context[i:i + n - 1]) == prefix:
            f = context[i + n - 1]
            if 0 <= f < len(out):
                out[f] = float("-inf")
    return out
