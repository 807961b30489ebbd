"""A plain, slow implementation of the Lurirax decoder in float64 numpy: one function per mechanism, whole
sequences only (no cache, no state passing, no batching).  It shares no code with the engine; the tests hold the
engine's kernels, cache, state slots and scheduler to it.

Notation: ``x`` [T, width] is the stream and a sublayer's input, ``w`` the dict of a folder's tensors as float64
arrays, ``pre`` a tensor-name prefix such as ``l3.mix.``, ``m`` the layer's ``mixer`` or ``mlp`` object from the
configuration, ``eps`` the model's ``norm.eps``.
"""
import json
import math
import os

import numpy as np


def load_folder(folder):
    """(configuration dict, tensors as float64) of a model folder."""
    import torch

    from vipera_rs_amd.weights import Checkpoint

    with open(os.path.join(folder, "config.json")) as handle:
        cfg = json.load(handle)
    checkpoint = Checkpoint(folder)
    try:
        w = {name: checkpoint.read(name).to(torch.float64).numpy() for name in checkpoint.names()}
    finally:
        checkpoint.close()
    return cfg, w


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def over_rms(x, eps):
    """x divided by its root mean square over the last axis, eps inside the root."""
    return x / np.sqrt(np.mean(np.square(x), axis=-1, keepdims=True) + eps)


def frequencies(rot):
    """One frequency per rotated pair: base^(-2i/dims), and where ``rot.scaling`` is given the long waves slowed down."""
    dims = int(rot["dims"])
    f = float(rot["base"]) ** (-2.0 * np.arange(dims // 2) / dims)
    s = rot.get("scaling")
    if not s:
        return f
    factor, low, high, original = float(s["factor"]), float(s["low"]), float(s["high"]), float(s["original"])
    out = np.empty_like(f)
    for i, fi in enumerate(f):
        wave = 2.0 * math.pi / fi
        if wave < original / high:
            out[i] = fi
        elif wave > original / low:
            out[i] = fi / factor
        else:
            share = (original / wave - low) / (high - low)
            out[i] = (1.0 - share) * fi / factor + share * fi
    return out


def rotate(x, positions, rot):
    """x [T, heads, dim]: pairs (i, i + dims/2) of the first ``dims`` numbers of a head turn by position * f_i."""
    dims = int((rot or {}).get("dims") or 0)
    if not dims:
        return x
    half = dims // 2
    angle = np.asarray(positions, dtype=np.float64)[:, None] * frequencies(rot)[None, :]
    c, s = np.cos(angle)[:, None, :], np.sin(angle)[:, None, :]
    out = x.copy()
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


def distance_bucket(n, rows, far):
    """Row of the distance table for a distance n >= 0: one row per distance below rows/2, then logarithmic steps up
    to the distance ``far``, at and beyond which it is the last row."""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


def visible(kind, size, keep_first, T):
    """[T, T] booleans: which earlier positions j a position i sees."""
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    causal = j <= i
    if kind == "window":
        return causal & ((i - j < size) | (j < keep_first))
    if kind == "chunk":
        return causal & (i // size == j // size)
    return causal


def softmax_attention(q, k, v, scale, mask, sink=None, bias=None):
    """q [T, H, d], k [T, G, d], v [T, G, dv] -> [T, H, dv]; ``sink`` [H] joins the denominator only; ``bias``
    [T, T, H] is added to the scaled scores."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        if bias is not None:
            s = s + bias[:, :, h]
        s = np.where(mask, s, -np.inf)
        top = s.max(axis=1, keepdims=True)
        if sink is not None:
            top = np.maximum(top, sink[h])
        e = np.exp(s - top)
        den = e.sum(axis=1, keepdims=True)
        if sink is not None:
            den = den + np.exp(sink[h] - top)
        out[:, h] = (e / den) @ v[:, g]
    return out


def windowed_attention(x, w, pre, m, eps):
    """Mixer ``attention``: rotation, then q and k over their root mean square, a sliding window, a sink."""
    T = x.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    pos = np.arange(T)
    q = rotate((x @ w[pre + "q"].T).reshape(T, H, d), pos, m.get("rot"))
    k = rotate((x @ w[pre + "k"].T).reshape(T, G, d), pos, m.get("rot"))
    v = (x @ w[pre + "v"].T).reshape(T, G, dv)
    q, k = over_rms(q, eps), over_rms(k, eps)
    mask = visible("window", int(m["mask"]["size"]), 0, T)
    o = softmax_attention(q, k, v, float(m["scale"]), mask, sink=w[pre + "sink"])
    return o.reshape(T, H * dv) @ w[pre + "o"].T


def biased_chunk_attention(x, w, pre, m, eps):
    """Left half of ``parallel``: biases, a norm per head with a weight, a learned bias by distance, chunks, a sink,
    a gate per head."""
    T = x.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = (x @ w[pre + "q"].T + w[pre + "q.b"]).reshape(T, H, d)
    k = (x @ w[pre + "k"].T + w[pre + "k.b"]).reshape(T, G, d)
    v = (x @ w[pre + "v"].T + w[pre + "v.b"]).reshape(T, G, dv)
    q, k = over_rms(q, eps) * w[pre + "q.norm"], over_rms(k, eps) * w[pre + "k.norm"]
    table = w[pre + "rel"]
    rows = table.shape[0]
    bias = np.zeros((T, T, H))
    for i in range(T):
        for j in range(i + 1):
            bias[i, j] = table[distance_bucket(i - j, rows, float(m["bias_max"]))]
    mask = visible("chunk", int(m["mask"]["size"]), 0, T)
    o = softmax_attention(q, k, v, float(m["scale"]), mask, sink=w[pre + "sink"], bias=bias)
    o = o * sigmoid(x @ w[pre + "g"].T)[:, :, None]
    return o.reshape(T, H * dv) @ w[pre + "o"].T


def retention(x, w, pre, m, eps):
    """Right half of ``parallel``: S <- decay_h S + k v^T, o = S^T q, token by token."""
    T = x.shape[0]
    H, d, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    pos = np.arange(T)
    q = rotate((x @ w[pre + "q"].T).reshape(T, H, d), pos, m.get("rot"))
    k = rotate((x @ w[pre + "k"].T).reshape(T, H, d), pos, m.get("rot")) * d ** -0.5
    v = (x @ w[pre + "v"].T).reshape(T, H, dv)
    o = np.zeros((T, H, dv))
    for h in range(H):
        S = np.zeros((d, dv))
        for t in range(T):
            S = float(m["decay"][h]) * S + np.outer(k[t, h], v[t, h])
            o[t, h] = S.T @ q[t, h]
    o = over_rms(o, eps).reshape(T, H * dv) * silu(x @ w[pre + "g"].T)
    return o @ w[pre + "o"].T


def parallel_mixer(x, w, pre, m, eps):
    return (float(m["left_scale"]) * biased_chunk_attention(x, w, pre + "left.", m["left"], eps)
            + float(m["right_scale"]) * retention(x, w, pre + "right.", m["right"], eps))


def differential_attention(x, w, pre, m, eps):
    """Mixer ``attention_2``: two attention maps per head over the same values, the second subtracted."""
    T = x.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    diff = float(m["diff"])
    q = over_rms((x @ w[pre + "q"].T).reshape(T, H, 2, d), eps) * w[pre + "q.norm"]
    k = over_rms((x @ w[pre + "k"].T).reshape(T, G, 2, d), eps) * w[pre + "k.norm"]
    v = (x @ w[pre + "v"].T).reshape(T, G, dv)
    mask = visible("window", int(m["mask"]["size"]), int(m["mask"].get("keep_first") or 0), T)
    a1 = softmax_attention(q[:, :, 0], k[:, :, 0], v, float(m["scale"]), mask)
    a2 = softmax_attention(q[:, :, 1], k[:, :, 1], v, float(m["scale"]), mask)
    lam = (math.exp(float(np.sum(w[pre + "lq1"] * w[pre + "lk1"])))
           - math.exp(float(np.sum(w[pre + "lq2"] * w[pre + "lk2"]))) + diff)
    o = over_rms(a1 - lam * a2, eps) * (1.0 - diff)
    return o.reshape(T, H * dv) @ w[pre + "o"].T


def gated_feed_forward(x, w, pre, act):
    return (act(x @ w[pre + "gate"].T) * (x @ w[pre + "up"].T)) @ w[pre + "down"].T


def choose(choice_scores, top):
    """Indices of the ``top`` largest scores, the lower index among equals."""
    return sorted(range(len(choice_scores)), key=lambda e: (-choice_scores[e], e))[:top]


def mixture_of_experts(x, w, pre, m, gaps=None):
    """``gaps``: a list that receives, per token, how far the last chosen expert's choice score lies above the best one
    left out (a small gap is a close call that 16-bit rounding may decide the other way)."""
    router = m["router"]
    experts, top, weight = int(router["experts"]), int(router["top"]), float(router.get("scale", 1.0))
    s = sigmoid(x @ w[pre + "router"].T)
    pick = s + w[pre + "correction"] if pre + "correction" in w else s
    out = np.zeros_like(x)
    for t in range(x.shape[0]):
        chosen = choose(list(pick[t]), top)
        if gaps is not None and top < experts:
            rest = [pick[t, e] for e in range(experts) if e not in chosen]
            gaps.append(min(pick[t, e] for e in chosen) - max(rest))
        for e in chosen:
            out[t] += weight * s[t, e] * gated_feed_forward(x[t:t + 1], w, f"{pre}e{e}.", silu)[0]
    if m.get("shared"):
        out += gated_feed_forward(x, w, pre + "shared.", silu) * sigmoid(x @ w[pre + "shared.sg"].T)
    return out


def feed_forward(x, w, pre, m, gaps=None):
    if m is None:
        return None
    if m["kind"] == "dense":
        return gated_feed_forward(x, w, pre, gelu_tanh)
    return mixture_of_experts(x, w, pre, m, gaps)


MIXERS = {"attention": windowed_attention, "parallel": parallel_mixer, "attention_2": differential_attention}


def forward(cfg, w, tokens, layers_out=None, gaps=None):
    """Logits [T, vocab] of a whole sequence.  ``layers_out``: a list that receives the stream after every layer."""
    eps = float(cfg["norm"]["eps"])
    x = w["embed"][np.asarray(tokens)] * float((cfg.get("embedding") or {}).get("scale", 1.0))
    for index, layer in enumerate(cfg["layers"]):
        pre = f"l{index}."
        y = MIXERS[layer["type"]](x, w, pre + "mix.", layer["mixer"], eps)
        x = x + over_rms(y, eps) * w[pre + "norm1"]
        y = feed_forward(x, w, pre + "mlp.", layer.get("mlp"), gaps)
        if y is not None:
            x = x + over_rms(y, eps) * w[pre + "norm2"]
        if layers_out is not None:
            layers_out.append(x.copy())
    return (over_rms(x, eps) * w["final.norm"]) @ w["head"].T


def greedy_generate(cfg, w, prompt, new_tokens):
    tokens = list(prompt)
    for _ in range(new_tokens):
        tokens.append(int(np.argmax(forward(cfg, w, tokens)[-1])))
    return tokens[len(prompt):]
