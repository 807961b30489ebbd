"""Configuration of the Muzasun decoder, read from its own ``config.json``.

The file lists the layers one by one: ``layers[i]`` has ``type`` (which mixer: ``attention``, ``mlstm`` or
``channel_delta``), ``mixer`` (its sizes and constants) and ``mlp`` (``kind`` ``dense`` or ``moe``, or null for none).
The inner sizes of the delta rule's two-step projections are those of the folder's tensors; ``decay_rank`` and
``gate_rank`` in its ``mixer`` may state them.
Beside the list stand ``vocab``, ``width``, ``norm.eps``, ``residual_mult`` and ``logit_scale``.  Every layer is a
parallel block with a Dynamic Tanh norm of its own in front of each sublayer, both of the same stream:
``x += residual_mult * (mixer(norm1(x)) + mlp(norm2(x)))``; the last layer is followed by such a norm too.  Among the
attention layers that say ``v_mix`` the first keeps its values of a step's tokens and the later ones blend theirs with
them.  Tensor names: ``embed``, ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``, ``head``.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple

from ..errors import InvalidArgumentError, UnsupportedError
from .base import KeyReader, LayerSpec, ModelConfig, PartSpec

MIXER_TYPES = ("attention", "mlstm", "channel_delta")
MLP_KINDS = ("dense", "moe")


def _sub(data: Dict[str, Any], key: str, where: str) -> Dict[str, Any]:
    value = data.get(key)
    if not isinstance(value, dict):
        raise InvalidArgumentError(f"{where}: key \"{key}\" is {value!r}, expected an object")
    return value


@dataclass
class MuzasunConfig(ModelConfig):
    vocab: int
    width: int
    eps: float
    logit_scale: float
    residual_mult: float
    layers: List[Dict[str, Any]] = field(default_factory=list)
    max_positions: int = 1 << 20       # no learned or tabled positions bound the context; a file may give "max_positions"
    eos_token_ids: Tuple[int, ...] = ()

    architecture = "Muzasun"

    # --- reading ----------------------------------------------------------------------
    @classmethod
    def from_dict(cls, data: Dict[str, Any]) -> "MuzasunConfig":
        r = KeyReader(data)
        layers = data.get("layers")
        if not isinstance(layers, list) or not all(isinstance(layer, dict) for layer in layers):
            raise InvalidArgumentError("config.json: key \"layers\" must be a list of objects, one per layer")
        eos = data.get("eos_token_id")
        eos_ids = () if eos is None else (eos,) if isinstance(eos, int) else tuple(eos)
        config = cls(vocab=r.integer("vocab", minimum=1), width=r.integer("width", minimum=1),
                     eps=KeyReader(_sub(data, "norm", "config.json"), "config.json: norm").number("eps"),
                     logit_scale=r.number("logit_scale", default=1.0), residual_mult=r.number("residual_mult", default=1.0),
                     layers=copy.deepcopy(layers), max_positions=r.integer("max_positions", default=1 << 20, minimum=1),
                     eos_token_ids=eos_ids)
        config.validate()
        return config

    def validate(self) -> None:
        if not self.eps >= 0.0:
            raise InvalidArgumentError(f"config.json: norm: key \"eps\" is {self.eps!r}, expected a number at or above 0")
        mixed_values: Optional[Tuple[int, int]] = None
        for index, layer in enumerate(self.layers):
            where = f"config.json: layers[{index}]"
            kind = layer.get("type")
            if kind not in MIXER_TYPES:
                raise UnsupportedError(f"{where}: type {kind!r} is not implemented; known: {', '.join(MIXER_TYPES)}")
            mixer = KeyReader(_sub(layer, "mixer", where), where + ".mixer")
            heads = mixer.integer("heads", minimum=1)
            mixer.integer("dim", minimum=1)
            vdim = mixer.integer("vdim", minimum=1)
            if kind in ("attention", "channel_delta"):
                kv_heads = mixer.integer("kv_heads", minimum=1)
                if heads % kv_heads:
                    raise InvalidArgumentError(f"{where}.mixer: \"heads\" {heads} is not a multiple of \"kv_heads\" {kv_heads}")
            if kind == "attention":
                mixer.number("scale")
                if mixer.has("rot"):
                    rotation = KeyReader(_sub(mixer.data, "rot", where + ".mixer"), where + ".mixer.rot")
                    dims = rotation.integer("dims", minimum=0)
                    if dims % 2 or dims > mixer.integer("dim"):
                        raise InvalidArgumentError(f"{where}.mixer.rot: \"dims\" is {dims}; it must be even and at most "
                                                   f"\"dim\" {mixer.integer('dim')}")
                    if not rotation.number("base") > 0:
                        raise InvalidArgumentError(f"{where}.mixer.rot: \"base\" must be above 0")
                if mixer.boolean("v_mix", False):
                    shape = (kv_heads, vdim)
                    if mixed_values is not None and mixed_values != shape:
                        raise InvalidArgumentError(f"{where}.mixer: \"v_mix\" blends {kv_heads} x {vdim} values with the "
                                                   f"{mixed_values[0]} x {mixed_values[1]} of the first layer that has it")
                    mixed_values = mixed_values or shape
            elif kind == "mlstm":
                if not mixer.number("gate_cap") > 0:
                    raise InvalidArgumentError(f"{where}.mixer: \"gate_cap\" must be above 0")
            else:
                mixer.integer("conv", minimum=1)
            mlp = layer.get("mlp")
            if mlp is None:
                continue
            if not isinstance(mlp, dict) or mlp.get("kind") not in MLP_KINDS:
                raise UnsupportedError(f"{where}: mlp {mlp!r} is not implemented; \"kind\" {' or '.join(MLP_KINDS)}, or null")
            if mlp["kind"] == "dense":
                KeyReader(mlp, where + ".mlp").integer("ff", minimum=1)
                continue
            KeyReader(_sub(mlp, "expert", where + ".mlp"), where + ".mlp.expert").integer("ff", minimum=1)
            router = KeyReader(_sub(mlp, "router", where + ".mlp"), where + ".mlp.router")
            experts, top = router.integer("experts", minimum=1), router.integer("top", minimum=1)
            if top > experts:
                raise InvalidArgumentError(f"{where}.mlp.router: \"top\" {top} is above \"experts\" {experts}")
            if mlp.get("shared") is not None:
                KeyReader(_sub(mlp, "shared", where + ".mlp"), where + ".mlp.shared").integer("ff", minimum=1)

    def to_dict(self) -> Dict[str, Any]:
        data: Dict[str, Any] = {"architecture": self.architecture, "layers": copy.deepcopy(self.layers),
                                "logit_scale": self.logit_scale, "norm": {"eps": self.eps},
                                "residual_mult": self.residual_mult, "vocab": self.vocab, "width": self.width}
        if self.max_positions != 1 << 20:
            data["max_positions"] = self.max_positions
        if self.eos_token_ids:
            data["eos_token_id"] = list(self.eos_token_ids)
        return data

    @property
    def context_limit(self) -> int:
        return int(self.max_positions)

    # --- for callers that ask a configuration for its sizes by the common names ---------------------
    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    # --- the description the generic decoder consumes ---------------------------------------
    def _norm(self, name: str) -> PartSpec:
        return PartSpec("dyt", {"width": self.width, "eps": self.eps, "name": name})

    def _ffn(self, mlp: Optional[Dict[str, Any]]) -> PartSpec:
        if mlp is None:
            return PartSpec("none", {})
        if mlp["kind"] == "dense":
            return PartSpec("gated_mlp", {"hidden": self.width, "intermediate": int(mlp["ff"]), "name": "mlp",
                                          "tensors": {"gate": "gate", "up": "up", "down": "down"}})
        shared = mlp.get("shared")
        return PartSpec("moe", {"hidden": self.width, "intermediate": int(mlp["expert"]["ff"]),
                                "experts": int(mlp["router"]["experts"]), "top": int(mlp["router"]["top"]),
                                "limit": None, "alpha": 1.0, "scores": "sigmoid", "weigh": "input",
                                "shared": int(shared["ff"]) if shared is not None else None, "name": "mlp"})

    def layer_specs(self) -> List[LayerSpec]:
        specs = []
        mixes_values = False      # whether an earlier layer keeps its values for the later ones
        for index, layer in enumerate(self.layers):
            kind, m = layer["type"], layer["mixer"]
            position = PartSpec("none", {})
            if kind == "attention":
                value_mix = None
                if m.get("v_mix"):
                    value_mix = "blend" if mixes_values else "source"
                    mixes_values = True
                mixer = PartSpec("attention", {
                    "hidden": self.width, "heads": int(m["heads"]), "kv_heads": int(m["kv_heads"]),
                    "head_dim": int(m["dim"]), "value_dim": int(m["vdim"]), "scale": float(m["scale"]),
                    "qkv_bias": True, "out_bias": True, "qk_norm": "head", "eps": self.eps, "value_mix": value_mix,
                    "name": "mix",
                    "tensors": {"q": "q", "k": "k", "v": "v", "o": "o", "q_bias": "q.b", "k_bias": "k.b", "v_bias": "v.b",
                                "o_bias": "o.b", "q_norm": "q.norm", "k_norm": "k.norm", "value_mix": "vmix"}})
                rot = m.get("rot")
                if rot and int(rot["dims"]):
                    position = PartSpec("rotary_neox", {"head_dim": int(m["dim"]), "rotary_dim": int(rot["dims"]),
                                                        "base": float(rot["base"])})
            elif kind == "mlstm":
                mixer = PartSpec("matrix_memory", {
                    "hidden": self.width, "heads": int(m["heads"]), "dim": int(m["dim"]), "vdim": int(m["vdim"]),
                    "gate_cap": float(m["gate_cap"]), "eps": self.eps, "name": "mix"})
            else:
                mixer = PartSpec("gated_delta", {
                    "hidden": self.width, "heads": int(m["heads"]), "kv_heads": int(m["kv_heads"]), "dim": int(m["dim"]),
                    "vdim": int(m["vdim"]), "conv": int(m["conv"]), "eps": self.eps, "decay": "channel",
                    # the two-step projections' inner sizes are the folder's tensors' unless the file gives them
                    # (a model of random weights has no folder to ask)
                    "decay_rank": int(m.get("decay_rank") or -1), "gate_rank": int(m.get("gate_rank") or -1),
                    "gate": "sigmoid", "name": "mix"})
            specs.append(LayerSpec("parallel", mixer, self._ffn(layer.get("mlp")), self._norm("norm1"), self._norm("norm2"),
                                   position, f"l{index}.", params={"residual_mult": self.residual_mult}))
        return specs

    def embedding_spec(self) -> PartSpec:
        return PartSpec("embedding", {"vocab": self.vocab, "width": self.width, "name": "embed", "tensor": "embed"})

    def final_norm_spec(self) -> PartSpec:
        return self._norm("final.norm")

    def head_spec(self) -> PartSpec:
        return PartSpec("lm_head", {"vocab": self.vocab, "width": self.width, "name": "head", "tensor": "head",
                                    "tied_to": None, "scale": self.logit_scale})
