"""Small Muzasun configurations and model folders with the tests' own random weights.

The weights are drawn here with numpy (not by the engine's random-weights mode) at magnitudes that keep every
mechanism alive: gates that neither freeze nor wipe the state, decays spread over (0, 1), routers with clear
preferences, norm weights around one.  Every value is rounded to bfloat16 before it is stored, so a 32-bit run, a
bfloat16 run and the plain implementation read the same numbers.
"""
from __future__ import annotations

import copy
import json
import os
from typing import Dict, List

import numpy as np
import torch


def attention(heads, kv_heads, dim, vdim, rot_dims=None, base=10000.0, scale=None, v_mix=False):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
         "scale": float(scale if scale is not None else dim ** -0.5), "v_mix": bool(v_mix)}
    if rot_dims is None:
        rot_dims = dim
    if rot_dims:
        m["rot"] = {"base": base, "dims": rot_dims}
    return {"type": "attention", "mixer": m}


def memory(heads, dim, vdim, cap=15.0):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}}


def delta(heads, kv_heads, dim, vdim, conv, ranks=(6, 5)):
    """``ranks``: rows of the first step of the decay's and of the gate's projection; no key of the configuration,
    only the tensors' shapes give them."""
    return {"type": "channel_delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv},
            "ranks": tuple(ranks)}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, shared=None):
    out = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        out["shared"] = {"ff": shared}
    return out


def config(vocab, width, layers, mlps, eps=1e-5, mult=1.0, logit_scale=1.0):
    out = {"architecture": "Muzasun", "vocab": vocab, "width": width, "norm": {"eps": eps}, "residual_mult": mult,
           "logit_scale": logit_scale, "layers": []}
    for layer, mlp in zip(layers, mlps):
        out["layers"].append(dict(copy.deepcopy(layer), mlp=copy.deepcopy(mlp)))
    return out


def ranks_of(cfg: dict) -> Dict[int, tuple]:
    return {i: tuple(layer.get("ranks", (6, 5))) for i, layer in enumerate(cfg["layers"]) if layer["type"] == "channel_delta"}


def stored(cfg: dict) -> dict:
    """The configuration as a folder holds it: without the helpers' own notes."""
    out = copy.deepcopy(cfg)
    for layer in out["layers"]:
        layer.pop("ranks", None)
    return out


# Five layers of all three kinds, the first of them no attention.  Values wider than keys in one attention and as wide
# in another; a partial rotation beside none beside a full one; four heads over two key heads, as many key heads as
# heads, three over one; two attention layers that blend values (the second with the first's) and one that does not; a
# mixture with a shared expert and one without in which every expert is chosen; a layer without a feed-forward; a
# multiplier on the sublayers' sum and a scale on the logits.
M1 = config(131, 48,
            [memory(3, 24, 8, cap=8.0),
             attention(4, 2, 16, 24, rot_dims=8, base=1000.0, scale=0.3, v_mix=True),
             delta(4, 2, 16, 8, 3),
             attention(2, 2, 24, 24, rot_dims=0, v_mix=True),
             attention(3, 1, 8, 16, scale=0.5)],
            [moe(6, 2, 24, shared=16), dense(40), None, moe(4, 4, 16), dense(24)], mult=0.7, logit_scale=2.0)
# Another order and widths that fit no fast path: nothing is a multiple of 8, the model's width not even of 4; a
# convolution of one tap; one key head under two heads of the delta rule; one wide head of the matrix memory; a single
# layer that says it blends values (it only keeps them); no multiplier and no scale; top 1.
M2 = config(83, 50,
            [delta(2, 1, 10, 14, 1, ranks=(3, 7)), attention(2, 2, 10, 6, rot_dims=4, base=50.0, scale=0.4),
             memory(1, 40, 20, cap=30.0), attention(3, 1, 6, 10, v_mix=True)],
            [moe(5, 1, 18), dense(22), moe(3, 2, 10, shared=30), None], eps=1e-6)


def single(layer, mlp=None, vocab=97, width=64, **kw):
    """A model of one layer: a mechanism alone."""
    return config(vocab, width, [layer], [mlp], **kw)


def _bf16(a) -> torch.Tensor:
    return torch.from_numpy(np.asarray(a, dtype=np.float32)).to(torch.bfloat16)


def make_weights(cfg: dict, seed: int, sharp: float = 1.0) -> Dict[str, torch.Tensor]:
    """``sharp`` scales the weights of the query and key norms of attention layers (peaked attention weights)."""
    rng = np.random.default_rng(seed)
    W = cfg["width"]
    out: Dict[str, torch.Tensor] = {}

    def mat(rows, cols, gain=1.0):
        return _bf16(rng.standard_normal((rows, cols)) * gain / np.sqrt(cols))

    def norm(name):
        out[name] = _bf16(1.0 + 0.1 * rng.standard_normal(W))
        out[name + ".b"] = _bf16(0.1 * rng.standard_normal(W))
        out[name + ".alpha"] = _bf16(rng.uniform(0.6, 1.4))

    def gated(prefix, ff):
        out[prefix + "gate"], out[prefix + "up"], out[prefix + "down"] = mat(ff, W, 1.5), mat(ff, W, 1.5), mat(W, ff)

    out["embed"] = _bf16(rng.standard_normal((cfg["vocab"], W)))
    ranks = ranks_of(cfg)
    for i, layer in enumerate(cfg["layers"]):
        m, p = layer["mixer"], f"l{i}.mix."
        norm(f"l{i}.norm1")
        norm(f"l{i}.norm2")
        H, D, V = m["heads"], m["dim"], m["vdim"]
        if layer["type"] == "attention":
            G = m["kv_heads"]
            out[p + "q"], out[p + "k"], out[p + "v"] = mat(H * D, W), mat(G * D, W), mat(G * V, W, 1.5)
            out[p + "q.b"], out[p + "k.b"] = _bf16(0.2 * rng.standard_normal(H * D)), _bf16(0.2 * rng.standard_normal(G * D))
            out[p + "v.b"] = _bf16(0.2 * rng.standard_normal(G * V))
            out[p + "q.norm"] = _bf16(sharp * (1.0 + 0.1 * rng.standard_normal(D)))
            out[p + "k.norm"] = _bf16(sharp * (1.0 + 0.1 * rng.standard_normal(D)))
            if m.get("v_mix"):
                out[p + "vmix"] = _bf16(rng.uniform(0.3, 0.7))
            out[p + "o"], out[p + "o.b"] = mat(W, H * V), _bf16(0.1 * rng.standard_normal(W))
        elif layer["type"] == "mlstm":
            out[p + "q"], out[p + "k"] = mat(H * D, W, 1.5), mat(H * D, W, 1.5)
            out[p + "v"], out[p + "g"] = mat(H * V, W, 1.5), mat(H * V, W, 2.0)
            out[p + "o"] = mat(W, H * V)
            out[p + "norm"] = _bf16(1.0 + 0.1 * rng.standard_normal(H * V))
            out[p + "i"], out[p + "f"] = mat(H, W, 2.0), mat(H, W, 2.0)
            out[p + "i.b"] = _bf16(rng.uniform(-1.0, 1.0, H))
            out[p + "f.b"] = _bf16(rng.uniform(1.0, 4.0, H))
        else:
            G, J = m["kv_heads"], m["conv"]
            ra, rg = ranks[i]
            out[p + "q"], out[p + "k"], out[p + "v"] = mat(G * D, W, 1.5), mat(G * D, W, 1.5), mat(H * V, W, 1.5)
            for n, rows in (("q", G * D), ("k", G * D), ("v", H * V)):
                out[f"{p}{n}.conv"] = _bf16(rng.standard_normal((rows, J)) * 0.6)
            out[p + "b"] = mat(H, W, 2.0)
            out[p + "A_log"] = _bf16(rng.uniform(-1.5, 1.0, H))
            out[p + "norm"] = _bf16(1.0 + 0.1 * rng.standard_normal(V))
            out[p + "a1"], out[p + "a2"] = mat(ra, W, 1.5), mat(H * D, ra, 1.5)
            out[p + "dt_bias"] = _bf16(rng.uniform(-2.5, 0.0, H * D))
            out[p + "g1"], out[p + "g2"] = mat(rg, W, 1.5), mat(H * V, rg, 2.0)
            out[p + "o"] = mat(W, H * V)
        mlp = layer.get("mlp")
        if mlp is not None:
            q = f"l{i}.mlp."
            if mlp["kind"] == "dense":
                gated(q, mlp["ff"])
            else:
                for e in range(mlp["router"]["experts"]):
                    gated(f"{q}e{e}.", mlp["expert"]["ff"])
                out[q + "router"] = mat(mlp["router"]["experts"], W, 2.0)
                if mlp.get("shared"):
                    gated(q + "shared.", mlp["shared"]["ff"])
    norm("final.norm")
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


def clear_tokens(cfg: dict, w: dict, count: int, seed: int, gap: float = 0.15) -> List[int]:
    """Random tokens whose routing is no close call: wherever the plain implementation finds the router's logit of a
    token's last chosen expert within ``gap`` of the best one left out, the token is drawn again (what comes before it
    does not change, so the sequence settles from the left).  A bfloat16 run then chooses as float64 does, and a
    difference between the two is a difference of the mechanisms.  A model without a mixture gets plain random tokens."""
    from plain import muzasun_plain as P

    tokens = tokens_of(cfg["vocab"], count, seed)
    if not any((layer.get("mlp") or {}).get("kind") == "moe" for layer in cfg["layers"]):
        return tokens
    rng = np.random.default_rng(seed + 1000)
    for _ in range(300):
        gaps: list = []
        P.forward(cfg, w, tokens, gaps=gaps)
        close = np.nonzero(np.min(np.stack(gaps), axis=0) < gap)[0]
        if close.size == 0:
            return tokens
        tokens[int(close[0])] = int(rng.integers(0, cfg["vocab"]))
    raise AssertionError("no sequence with clear routing found")
