"""A plain, slow implementation of the Muzasun decoder in float64 numpy: one function per mechanism, whole
sequences only (no cache, no state passing, no batching).  It shares no code with the engine; the tests hold the
engine's kernels, cache, state slots and scheduler to it.

Notation: ``h`` [T, width] is a sublayer's input, ``w`` the dict of a folder's tensors as float64 arrays, ``pre`` a
tensor-name prefix such as ``l3.mix.``, ``m`` the layer's ``mixer`` or ``mlp`` object from the configuration.
"""
import json
import math
import os

import numpy as np

UNIT_EPS = 1e-6      # unit vectors of the delta rule: x / sqrt(sum(x^2) + UNIT_EPS)
READ_EPS = 1e-6      # added to the matrix memory's denominator


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


def log_sigmoid(z):
    return -np.logaddexp(0.0, -z)


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def dynamic_tanh(x, w, name):
    """tanh(alpha x) * weight + bias, elementwise."""
    return np.tanh(float(w[name + ".alpha"]) * x) * w[name] + w[name + ".b"]


def over_rms(x, eps):
    """x divided by its root mean square over the last axis, eps inside the root."""
    return x / np.sqrt(np.mean(np.square(x), axis=-1, keepdims=True) + eps)


def rotate_half(x, positions, dims, base):
    """x [T, heads, dim]: the first ``dims`` numbers of each head turn, number i together with number i + dims/2, by the
    angle position * base^(-2i/dims); the others pass."""
    out = x.copy()
    half = dims // 2
    if half == 0:
        return out
    freq = base ** (-2.0 * np.arange(half) / dims)
    angle = positions[:, None].astype(np.float64) * freq[None, :]
    c, s = np.cos(angle)[:, None, :], np.sin(angle)[:, None, :]
    lo, hi = x[:, :, :half], x[:, :, half:dims]
    out[:, :, :half] = lo * c - hi * s
    out[:, :, half:dims] = hi * c + lo * s
    return out


def attention_mixer(h, w, pre, m, eps, v_first=None):
    """Softmax attention over all earlier positions with grouped heads, biases, a norm per head on q and k, a partial
    rotation and, from the second layer that mixes values on, values blended with the first such layer's.  Returns
    ``(output, the values that this layer attends over)``."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[pre + "q"].T + w[pre + "q.b"]).reshape(T, H, D)
    k = (h @ w[pre + "k"].T + w[pre + "k.b"]).reshape(T, G, D)
    v = (h @ w[pre + "v"].T + w[pre + "v.b"]).reshape(T, G, V)
    q = over_rms(q, eps) * w[pre + "q.norm"]
    k = over_rms(k, eps) * w[pre + "k.norm"]
    positions = np.arange(T)
    rot = m.get("rot")
    if rot:
        q = rotate_half(q, positions, rot["dims"], rot["base"])
        k = rotate_half(k, positions, rot["dims"], rot["base"])
    if m.get("v_mix") and v_first is not None:
        lam = float(w[pre + "vmix"])
        v = (1.0 - lam) * v + lam * v_first
    out = np.zeros((T, H, V))
    visible = np.tril(np.ones((T, T), dtype=bool))
    for head in range(H):
        g = head // (H // G)
        score = (q[:, head] @ k[:, g].T) * m["scale"]
        score = np.where(visible, score, -np.inf)
        p = np.exp(score - score.max(axis=1, keepdims=True))
        p /= p.sum(axis=1, keepdims=True)
        out[:, head] = p @ v[:, g]
    return out.reshape(T, H * V) @ w[pre + "o"].T + w[pre + "o.b"], v


def matrix_memory_mixer(h, w, pre, m, eps):
    """mLSTM: a matrix S [dim, vdim] and a vector n [dim] per head, with gates kept in logarithms under a running
    maximum that starts at 0."""
    T = h.shape[0]
    H, D, V, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = (h @ w[pre + "q"].T).reshape(T, H, D) / math.sqrt(D)
    k = (h @ w[pre + "k"].T).reshape(T, H, D)
    v = (h @ w[pre + "v"].T).reshape(T, H, V)
    log_i = cap * np.tanh((h @ w[pre + "i"].T + w[pre + "i.b"]) / cap)
    log_f = log_sigmoid(cap * np.tanh((h @ w[pre + "f"].T + w[pre + "f.b"]) / cap))
    out = np.zeros((T, H, V))
    for head in range(H):
        S, n, top = np.zeros((D, V)), np.zeros(D), 0.0
        for t in range(T):
            new_top = max(log_f[t, head] + top, log_i[t, head])
            keep, take = math.exp(log_f[t, head] + top - new_top), math.exp(log_i[t, head] - new_top)
            S = keep * S + take * np.outer(k[t, head], v[t, head])
            n = keep * n + take * k[t, head]
            top = new_top
            out[t, head] = (S.T @ q[t, head]) / (max(abs(n @ q[t, head]), math.exp(-top)) + READ_EPS)
    out = over_rms(out, eps).reshape(T, H * V) * w[pre + "norm"]
    return (out * sigmoid(h @ w[pre + "g"].T)) @ w[pre + "o"].T


def short_convolution(x, taps):
    """Causal, per channel: y[t] = sum_j taps[:, j] x[t - (J - 1 - j)], zeros before the start; then silu."""
    count = taps.shape[1]
    y = np.zeros_like(x)
    for t in range(x.shape[0]):
        for j in range(count):
            back = count - 1 - j
            if t - back >= 0:
                y[t] += taps[:, j] * x[t - back]
    return silu(y)


def channel_delta_mixer(h, w, pre, m, eps):
    """The gated delta rule with one decay per head and key channel."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = short_convolution(h @ w[pre + "q"].T, w[pre + "q.conv"]).reshape(T, G, D)
    k = short_convolution(h @ w[pre + "k"].T, w[pre + "k.conv"]).reshape(T, G, D)
    v = short_convolution(h @ w[pre + "v"].T, w[pre + "v.conv"]).reshape(T, H, V)
    q = q / np.sqrt(np.sum(q * q, axis=-1, keepdims=True) + UNIT_EPS) / math.sqrt(D)
    k = k / np.sqrt(np.sum(k * k, axis=-1, keepdims=True) + UNIT_EPS)
    beta = sigmoid(h @ w[pre + "b"].T)
    step = softplus((h @ w[pre + "a1"].T) @ w[pre + "a2"].T + w[pre + "dt_bias"]).reshape(T, H, D)
    decay = np.exp(-np.exp(w[pre + "A_log"])[None, :, None] * step)
    out = np.zeros((T, H, V))
    for head in range(H):
        g = head // (H // G)
        S = np.zeros((D, V))
        for t in range(T):
            S = decay[t, head][:, None] * S
            u = beta[t, head] * (v[t, head] - S.T @ k[t, g])
            S = S + np.outer(k[t, g], u)
            out[t, head] = S.T @ q[t, g]
    out = over_rms(out, eps) * w[pre + "norm"]
    gate = sigmoid((h @ w[pre + "g1"].T) @ w[pre + "g2"].T)
    return (out.reshape(T, H * V) * gate) @ w[pre + "o"].T


def gated_feed_forward(h, w, pre):
    return (silu(h @ w[pre + "gate"].T) * (h @ w[pre + "up"].T)) @ w[pre + "down"].T


def route(scores, top):
    """The ``top`` experts with the largest scores, the lower id among equals."""
    return sorted(range(len(scores)), key=lambda e: (-scores[e], e))[:top]


def mixture_of_experts(h, w, pre, m, gaps=None):
    """Sigmoid scores; the best ``top`` experts, each fed the token times its score; a shared expert for every token.
    ``gaps`` (a list) receives, per token, how far the router's logit of the last chosen expert lies above the best one
    left out (infinite where every expert is chosen)."""
    experts, top = m["router"]["experts"], m["router"]["top"]
    logits = h @ w[pre + "router"].T
    scores = sigmoid(logits)
    out = np.zeros((h.shape[0], w[pre + "e0.down"].shape[0]))
    if gaps is not None:
        ranked = -np.sort(-logits, axis=1)
        gaps.append(ranked[:, top - 1] - ranked[:, top] if top < experts else np.full(h.shape[0], np.inf))
    for t in range(h.shape[0]):
        chosen = route(scores[t], top)
        for e in chosen:
            out[t] += gated_feed_forward(scores[t, e] * h[t][None, :], w, f"{pre}e{e}.")[0]
    if m.get("shared"):
        out += gated_feed_forward(h, w, pre + "shared.")
    return out


def feed_forward(h, w, pre, m, gaps=None):
    if m is None:
        return 0.0
    if m["kind"] == "dense":
        return gated_feed_forward(h, w, pre)
    return mixture_of_experts(h, w, pre, m, gaps)


def forward(cfg, w, tokens, layers_out=None, gaps=None):
    """Logits [T, vocab] of one sequence; ``layers_out`` (a list) receives the stream after every layer, ``gaps`` every
    mixture's routing margins (see :func:`mixture_of_experts`)."""
    eps, mult = cfg["norm"]["eps"], cfg.get("residual_mult", 1.0)
    x = w["embed"][np.asarray(tokens)]
    v_first = None
    for index, layer in enumerate(cfg["layers"]):
        pre = f"l{index}."
        h = dynamic_tanh(x, w, pre + "norm1")
        kind, m = layer["type"], layer["mixer"]
        if kind == "attention":
            mixed, values = attention_mixer(h, w, pre + "mix.", m, eps, v_first)
            if m.get("v_mix") and v_first is None:
                v_first = values
        elif kind == "mlstm":
            mixed = matrix_memory_mixer(h, w, pre + "mix.", m, eps)
        elif kind == "channel_delta":
            mixed = channel_delta_mixer(h, w, pre + "mix.", m, eps)
        else:
            raise ValueError(f"layer {index}: unknown type {kind!r}")
        fed = feed_forward(dynamic_tanh(x, w, pre + "norm2"), w, pre + "mlp.", layer.get("mlp"), gaps) \
            if layer.get("mlp") is not None else 0.0
        x = x + mult * (mixed + fed)
        if layers_out is not None:
            layers_out.append(x.copy())
    return (dynamic_tanh(x, w, "final.norm") @ w["head"].T) * cfg.get("logit_scale", 1.0)
