"""Configurations and weights of the tests' own for the Lurirax decoder.

Weights are drawn at magnitudes that keep every mechanism alive (sinks that take a visible share of a softmax, a table
of biases by distance with clear steps, decays spread below one, routers with clear preferences, corrections that change
some choices) and are bfloat16-exact, so that a 32-bit run, a bfloat16 run and the plain implementation read the same
numbers.
"""
from __future__ import annotations

import json
import os
from typing import Dict, List, Optional

import numpy as np
import torch


# --- layers -----------------------------------------------------------------------------------------------------------
def windowed(heads, kv_heads, dim, vdim, size, rot_dims=None, base=10000.0, scaling=None, scale=None):
    """Mixer ``attention``: a sliding window, a sink, q and k over their root mean square behind the rotation."""
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": size},
         "scale": float(scale if scale is not None else dim ** -0.5)}
    dims = dim if rot_dims is None else rot_dims
    if dims:
        m["rot"] = {"dims": dims, "base": float(base)}
        if scaling:
            m["rot"]["scaling"] = dict(scaling)
    return {"type": "attention", "mixer": m}


def differential(heads, kv_heads, dim, vdim, size, keep_first=0, diff=0.4, scale=None):
    """Mixer ``attention_2``: two maps per head, a window that keeps the first positions."""
    return {"type": "attention_2", "mixer": {
        "heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "diff": float(diff),
        "mask": {"size": size, "keep_first": keep_first}, "scale": float(scale if scale is not None else dim ** -0.5)}}


def chunked(heads, kv_heads, dim, vdim, size, bias_rows=8, bias_max=40, scale=None):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": size},
            "bias_max": bias_max, "bias_rows": bias_rows, "scale": float(scale if scale is not None else dim ** -0.5)}


def retention(heads, dim, vdim, decay=None, rot_dims=None, base=10000.0):
    decay = decay if decay is not None else [1.0 - 2.0 ** -(3 + h) for h in range(heads)]
    m = {"heads": heads, "dim": dim, "vdim": vdim, "decay": [float(d) for d in decay]}
    dims = dim if rot_dims is None else rot_dims
    if dims:
        m["rot"] = {"dims": dims, "base": float(base)}
    return m


def parallel(left, right, left_scale=0.7, right_scale=0.4):
    return {"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": left_scale, "right_scale": right_scale}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, scale=1.5, shared=None):
    mlp = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "scale": float(scale)}}
    if shared:
        mlp["shared"] = {"ff": shared}
    return mlp


def config(vocab, width, layers, mlps, eps=1e-5, embedding_scale=1.5):
    assert len(layers) == len(mlps)
    return {"architecture": "Lurirax", "embedding": {"scale": embedding_scale}, "norm": {"eps": eps}, "vocab": vocab,
            "width": width, "layers": [dict(layer, mlp=mlp) for layer, mlp in zip(layers, mlps)]}


def single(layer, mlp=None, vocab=97, width=64, **kw):
    return config(vocab, width, [layer], [mlp], **kw)


def stored(cfg: dict) -> dict:
    """The configuration as a folder holds it: the rows of the table of biases by distance are given by the tensor."""
    out = json.loads(json.dumps(cfg))
    for layer in out["layers"]:
        if layer["type"] == "parallel":
            layer["mixer"]["left"].pop("bias_rows", None)
    return out


# Two models that have every kind of layer; the second at other sizes: one key head, heads that are no power of two,
# values wider than keys, a partial rotation, all experts chosen in one layer, no shared expert in another, a layer
# without a feed-forward, windows and chunks that are no multiples of a page.
L1 = config(83, 48, [
    differential(4, 2, 8, 16, 11, keep_first=3),
    windowed(4, 2, 16, 16, 9, rot_dims=8, base=500.0, scaling={"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64}),
    parallel(chunked(4, 2, 16, 16, 13, bias_rows=8, bias_max=12), retention(2, 16, 8, rot_dims=16, base=100.0)),
    windowed(2, 2, 16, 8, 21, rot_dims=16),
], [dense(40), moe(6, 2, 24, shared=16), moe(4, 2, 24, scale=0.8, shared=24), dense(32)])

L2 = config(61, 40, [
    parallel(chunked(3, 1, 8, 24, 7, bias_rows=6, bias_max=9.5, scale=0.5), retention(3, 24, 8, rot_dims=8), 0.5, 1.0),
    differential(3, 3, 16, 8, 6, keep_first=5, diff=0.7, scale=0.3),
    windowed(6, 3, 8, 24, 17, rot_dims=4, base=50.0, scale=0.6),
    differential(2, 1, 24, 24, 30, keep_first=0, diff=0.2),
], [moe(3, 3, 16, scale=1.0, shared=8), None, moe(5, 1, 24, scale=2.0), dense(56)], eps=1e-6, embedding_scale=0.75)


def random_config(seed: int) -> dict:
    """A configuration drawn at random: one to five layers of any kind in any order, head counts, widths, windows,
    chunks, kept positions, rotations, tables, decays, experts and constants from lists that hold ones, equal values,
    odd values and values beyond a page or a tile."""
    rng = np.random.default_rng(seed)
    pick = lambda xs: xs[int(rng.integers(0, len(xs)))]
    layers, mlps = [], []
    for _ in range(int(rng.integers(1, 6))):
        kind = pick(["window", "two", "pair"])
        kv = pick([1, 2, 3])
        heads = kv * pick([1, 2, 4])
        dim, vdim = pick([4, 8, 10, 16, 24, 32, 64]), pick([4, 8, 12, 16, 32, 40, 64])
        size = pick([1, 2, 3, 7, 16, 17, 31, 64, 65, 100, 500])
        scale = float(pick([dim ** -0.5, 0.3, 1.0 / dim]))
        if kind == "window":
            rot = pick([0, 2, dim // 2 // 2 * 2, dim // 2 * 2])
            scaling = pick([None, {"factor": float(pick([2.0, 8.0])), "low": 1.0, "high": float(pick([2.0, 4.0])),
                                   "original": pick([16, 64, 1024])}])
            layers.append(windowed(heads, kv, dim, vdim, size, rot_dims=rot, base=float(pick([50.0, 1e4, 1e6])),
                                   scaling=scaling if rot else None, scale=scale))
        elif kind == "two":
            layers.append(differential(heads, kv, dim, vdim, size, keep_first=pick([0, 1, 4, 9, 70]),
                                       diff=float(pick([0.1, 0.5, 0.8])), scale=scale))
        else:
            rows = pick([2, 4, 6, 16, 32])
            far = float(pick([rows // 2 + 1, rows, 4 * rows, 150]))
            rh, rd, rv = pick([1, 2, 3, 5]), pick([4, 8, 16, 24, 40, 64]), pick([4, 8, 16, 20, 32])
            decay = [float(pick([0.5, 0.9, 0.96875, 0.999, 1.0])) for _ in range(rh)]
            layers.append(parallel(chunked(heads, kv, dim, vdim, size, bias_rows=rows, bias_max=far, scale=scale),
                                   retention(rh, rd, rv, decay=decay, rot_dims=pick([0, 2, rd // 2 * 2]),
                                             base=float(pick([100.0, 1e6]))),
                                   float(pick([0.5, 1.0])), float(pick([0.3, 1.0]))))
        mlp = pick(["none", "dense", "moe", "moe"])
        if mlp == "none":
            mlps.append(None)
        elif mlp == "dense":
            mlps.append(dense(pick([16, 24, 40, 64, 100])))
        else:
            experts = pick([1, 2, 3, 8, 9])
            mlps.append(moe(experts, int(rng.integers(1, experts + 1)), pick([8, 16, 24, 40]), scale=float(pick([1.0, 2.0])),
                            shared=pick([None, 8, 24])))
    return config(pick([31, 61, 97, 128]), pick([24, 40, 56, 64, 72, 96]), layers, mlps, eps=float(pick([1e-6, 1e-5])),
                  embedding_scale=float(pick([0.5, 1.0, 3.0])))


# --- weights -----------------------------------------------------------------------------------------------------------
def _bf16(a) -> torch.Tensor:
    return torch.from_numpy(np.asarray(a, dtype=np.float32)).to(torch.bfloat16)


def make_weights(cfg: dict, seed: int, sharp: float = 1.0) -> Dict[str, torch.Tensor]:
    """``sharp`` scales what makes attention weights peaked: the weights of the query norms (layers that have them)."""
    rng = np.random.default_rng(seed)
    W = cfg["width"]
    out: Dict[str, torch.Tensor] = {}

    def mat(rows, cols, gain=1.0):
        return _bf16(rng.standard_normal((rows, cols)) * gain / np.sqrt(cols))

    def gated(prefix, ff):
        out[prefix + "gate"], out[prefix + "up"], out[prefix + "down"] = mat(ff, W, 1.5), mat(ff, W, 1.5), mat(W, ff)

    def softmax_part(p, m, maps=1, biases=False):
        H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        out[p + "q"], out[p + "k"], out[p + "v"] = mat(H * maps * D, W), mat(G * maps * D, W), mat(G * V, W, 1.5)
        out[p + "o"] = mat(W, H * V)
        if biases:
            for n, rows in (("q", H * D), ("k", G * D), ("v", G * V)):
                out[f"{p}{n}.b"] = _bf16(0.3 * rng.standard_normal(rows))

    out["embed"] = _bf16(rng.standard_normal((cfg["vocab"], W)))
    for i, layer in enumerate(cfg["layers"]):
        m, p = layer["mixer"], f"l{i}.mix."
        out[f"l{i}.norm1"] = _bf16(1.0 + 0.1 * rng.standard_normal(W))
        out[f"l{i}.norm2"] = _bf16(1.0 + 0.1 * rng.standard_normal(W))
        if layer["type"] == "attention":
            softmax_part(p, m)
            out[p + "sink"] = _bf16(rng.uniform(-1.0, 2.0, m["heads"]))
        elif layer["type"] == "attention_2":
            softmax_part(p, m, maps=2)
            out[p + "q.norm"] = _bf16(sharp * (1.0 + 0.1 * rng.standard_normal(m["dim"])))
            out[p + "k.norm"] = _bf16(1.0 + 0.1 * rng.standard_normal(m["dim"]))
            for n in ("lq1", "lk1", "lq2", "lk2"):
                out[p + n] = _bf16(0.3 * rng.standard_normal(m["dim"]))
        else:
            left, right = m["left"], m["right"]
            q = p + "left."
            softmax_part(q, left, biases=True)
            out[q + "q.norm"] = _bf16(sharp * (1.0 + 0.1 * rng.standard_normal(left["dim"])))
            out[q + "k.norm"] = _bf16(1.0 + 0.1 * rng.standard_normal(left["dim"]))
            out[q + "rel"] = _bf16(rng.standard_normal((left["bias_rows"], left["heads"])))
            out[q + "sink"] = _bf16(rng.uniform(-1.0, 2.0, left["heads"]))
            out[q + "g"] = mat(left["heads"], W, 2.0)
            r = p + "right."
            H, D, V = right["heads"], right["dim"], right["vdim"]
            out[r + "q"], out[r + "k"] = mat(H * D, W, 1.5), mat(H * D, W, 1.5)
            out[r + "v"], out[r + "g"], out[r + "o"] = mat(H * V, W, 1.5), mat(H * V, W, 2.0), mat(W, H * V)
        mlp = layer.get("mlp")
        if mlp is not None:
            q = f"l{i}.mlp."
            if mlp["kind"] == "dense":
                gated(q, mlp["ff"])
            else:
                experts = mlp["router"]["experts"]
                for e in range(experts):
                    gated(f"{q}e{e}.", mlp["expert"]["ff"])
                out[q + "router"] = mat(experts, W, 2.0)
                out[q + "correction"] = _bf16(0.25 * rng.standard_normal(experts))
                if mlp.get("shared"):
                    gated(q + "shared.", mlp["shared"]["ff"])
                    out[q + "shared.sg"] = mat(1, W, 2.0)
    out["final.norm"] = _bf16(1.0 + 0.1 * rng.standard_normal(W))
    out["head"] = mat(cfg["vocab"], W)
    return out


def make_folder(path, cfg: dict, seed: int, dtype=torch.float32, sharp: float = 1.0, edit=None) -> str:
    """Write ``config.json`` and ``model.safetensors``; ``edit(tensors)`` may change the weights before."""
    from vipera_rs_amd.weights import write_safetensors

    path = str(path)
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as handle:
        json.dump(stored(cfg), handle)
    tensors = make_weights(cfg, seed, sharp)
    if edit is not None:
        edit(tensors)
    write_safetensors(os.path.join(path, "model.safetensors"), [(name, t.to(dtype)) for name, t in tensors.items()])
    return path


def load_folder(folder):
    """(configuration dict, tensors as float64 numpy arrays) of a model folder, for the plain implementation."""
    from safetensors.torch import load_file

    with open(os.path.join(folder, "config.json")) as handle:
        cfg = json.load(handle)
    w = {name: t.to(torch.float64).numpy() for name, t in load_file(os.path.join(folder, "model.safetensors")).items()}
    return cfg, w


def tokens_of(vocab: int, count: int, seed: int) -> List[int]:
    return [int(t) for t in np.random.default_rng(seed).integers(0, vocab, count)]


def clear_tokens(cfg: dict, w: dict, count: int, seed: int, gap: float = 0.02) -> List[int]:
    """Random tokens whose routing is no close call: wherever the plain implementation finds the choice score of a
    token's last chosen expert within ``gap`` of the best one left out (scores are sigmoids: they lie in (0, 1) plus a
    small correction), the token is drawn again (what comes before it does not change, so the sequence settles from the
    left).  A bfloat16 run then chooses as float64 does.  A model without a mixture gets plain random tokens."""
    from plain import lurirax_plain as P

    tokens = tokens_of(cfg["vocab"], count, seed)
    routed = [layer for layer in cfg["layers"] if (layer.get("mlp") or {}).get("kind") == "moe"
              and layer["mlp"]["router"]["top"] < layer["mlp"]["router"]["experts"]]
    if not routed:
        return tokens
    rng = np.random.default_rng(seed + 1000)
    for _ in range(400):
        gaps: list = []
        P.forward(cfg, w, tokens, gaps=gaps)
        per_layer = np.asarray(gaps).reshape(len(routed), len(tokens))
        close = np.nonzero(np.min(per_layer, axis=0) < gap)[0]
        if close.size == 0:
            return tokens
        tokens[int(close[0])] = int(rng.integers(0, cfg["vocab"]))
    raise AssertionError("no sequence with clear routing found")
