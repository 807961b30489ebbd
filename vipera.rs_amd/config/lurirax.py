"""Configuration of the Lurirax decoder, read from its own ``config.json``.

The file lists the layers one by one: ``layers[i]`` has ``type`` (``attention``: softmax attention in a sliding window
with a sink; ``attention_2``: differential attention in a window that keeps a sequence's first positions;
``parallel``: softmax attention within chunks, biased by distance, beside retention), ``mixer`` (its sizes and
constants) and ``mlp`` (``{"kind": "dense", "ff"}``, ``{"kind": "moe", "expert": {"ff"}, "router": {"experts", "top",
"scale"}, "shared": {"ff"}}``, or null).  Beside the list stand ``vocab``, ``width``, ``norm.eps`` and
``embedding.scale``.  A layer norms what its sublayers return, not what they read:
``x += norm1(mixer(x)); x += norm2(mlp(x))``.  Tensor names: ``embed``, ``l<i>.norm1 | norm2``, ``l<i>.mix.*``,
``l<i>.mlp.*``, ``final.norm``, ``head``.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple

from ..errors import InvalidArgumentError, UnsupportedError
from .base import KeyReader, LayerSpec, ModelConfig, PartSpec

MIXER_TYPES = ("attention", "attention_2", "parallel")
MLP_KINDS = ("dense", "moe")


def _sub(data: Dict[str, Any], key: str, where: str) -> Dict[str, Any]:
    value = data.get(key)
    if not isinstance(value, dict):
        raise InvalidArgumentError(f"{where}: key \"{key}\" is {value!r}, expected an object")
    return value


def _optional(data: Dict[str, Any], key: str, where: str) -> Optional[Dict[str, Any]]:
    return _sub(data, key, where) if data.get(key) is not None else None


@dataclass
class LuriraxConfig(ModelConfig):
    vocab: int
    width: int
    eps: float
    embedding_scale: float
    layers: List[Dict[str, Any]] = field(default_factory=list)
    max_positions: int = 1 << 20       # nothing learned or tabled bounds the context; a file may give "max_positions"
    eos_token_ids: Tuple[int, ...] = ()

    architecture = "Lurirax"

    # --- reading ----------------------------------------------------------------------
    @classmethod
    def from_dict(cls, data: Dict[str, Any]) -> "LuriraxConfig":
        r = KeyReader(data)
        layers = data.get("layers")
        if not isinstance(layers, list) or not all(isinstance(layer, dict) for layer in layers):
            raise InvalidArgumentError("config.json: key \"layers\" must be a list of objects, one per layer")
        eos = data.get("eos_token_id")
        eos_ids = () if eos is None else (eos,) if isinstance(eos, int) else tuple(eos)
        embedding = _optional(data, "embedding", "config.json")
        config = cls(
            vocab=r.integer("vocab", minimum=1), width=r.integer("width", minimum=1),
            eps=KeyReader(_sub(data, "norm", "config.json"), "config.json: norm").number("eps"),
            embedding_scale=KeyReader(embedding, "config.json: embedding").number("scale", default=1.0) if embedding else 1.0,
            layers=copy.deepcopy(layers), max_positions=r.integer("max_positions", default=1 << 20, minimum=1),
            eos_token_ids=eos_ids)
        config.validate()
        return config

    def validate(self) -> None:
        if not self.eps >= 0.0:
            raise InvalidArgumentError(f"config.json: norm: key \"eps\" is {self.eps!r}, expected a number at or above 0")
        for index, layer in enumerate(self.layers):
            where = f"config.json: layers[{index}]"
            kind = layer.get("type")
            if kind not in MIXER_TYPES:
                raise UnsupportedError(f"{where}: type {kind!r} is not implemented; known: {', '.join(MIXER_TYPES)}")
            mixer = _sub(layer, "mixer", where)
            if kind == "parallel":
                left = _sub(mixer, "left", where + ".mixer")
                self._check_softmax(left, where + ".mixer.left", window=False)
                lr = KeyReader(left, where + ".mixer.left")
                if lr.has("bias_max") and not lr.number("bias_max") > 0:
                    raise InvalidArgumentError(f"{where}.mixer.left: \"bias_max\" must be above 0")
                self._check_retention(_sub(mixer, "right", where + ".mixer"), where + ".mixer.right")
                scales = KeyReader(mixer, where + ".mixer")
                scales.number("left_scale", default=1.0)
                scales.number("right_scale", default=1.0)
            else:
                self._check_softmax(mixer, where + ".mixer", window=True)
                if kind == "attention_2":
                    KeyReader(mixer, where + ".mixer").number("diff")
            self._check_mlp(layer.get("mlp"), where)

    @staticmethod
    def _check_rot(m: Dict[str, Any], dim: int, where: str) -> None:
        rot = _optional(m, "rot", where)
        if rot is None:
            return
        rr = KeyReader(rot, where + ".rot")
        dims = rr.integer("dims", minimum=0)
        if dims % 2 or dims > dim:
            raise InvalidArgumentError(f"{where}.rot: \"dims\" is {dims}; it must be even and at most \"dim\" {dim}")
        if dims and not rr.number("base") > 0:
            raise InvalidArgumentError(f"{where}.rot: \"base\" must be above 0")
        scaling = _optional(rot, "scaling", where + ".rot")
        if scaling is not None:
            sr = KeyReader(scaling, where + ".rot.scaling")
            factor, low, high = sr.number("factor"), sr.number("low"), sr.number("high")
            if not (factor > 0 and high > low and sr.number("original") > 0):
                raise InvalidArgumentError(f"{where}.rot.scaling: {scaling!r}; \"factor\" and \"original\" must be above 0 "
                                           "and \"high\" above \"low\"")

    @classmethod
    def _check_softmax(cls, m: Dict[str, Any], where: str, window: bool) -> None:
        r = KeyReader(m, where)
        heads, kv_heads = r.integer("heads", minimum=1), r.integer("kv_heads", minimum=1)
        if heads % kv_heads:
            raise InvalidArgumentError(f"{where}: \"heads\" {heads} is not a multiple of \"kv_heads\" {kv_heads}")
        dim = r.integer("dim", minimum=1)
        r.integer("vdim", minimum=1)
        r.number("scale")
        mask = KeyReader(_sub(m, "mask", where), where + ".mask")
        mask.integer("size", minimum=1)
        if window:
            mask.integer("keep_first", default=0, minimum=0)
        cls._check_rot(m, dim, where)

    @classmethod
    def _check_retention(cls, m: Dict[str, Any], where: str) -> None:
        r = KeyReader(m, where)
        heads = r.integer("heads", minimum=1)
        dim = r.integer("dim", minimum=1)
        r.integer("vdim", minimum=1)
        decay = m.get("decay")
        if not isinstance(decay, list) or len(decay) != heads or not all(
                isinstance(d, (int, float)) and not isinstance(d, bool) for d in decay):
            raise InvalidArgumentError(f"{where}: key \"decay\" is {decay!r}, expected one number per head ({heads})")
        cls._check_rot(m, dim, where)

    @staticmethod
    def _check_mlp(mlp: Any, where: str) -> None:
        if mlp is None:
            return
        if not isinstance(mlp, dict) or mlp.get("kind") not in MLP_KINDS:
            raise UnsupportedError(f"{where}: mlp {mlp!r} is not implemented; \"kind\" {' or '.join(MLP_KINDS)}, or null")
        if mlp["kind"] == "dense":
            KeyReader(mlp, where + ".mlp").integer("ff", minimum=1)
            return
        KeyReader(_sub(mlp, "expert", where + ".mlp"), where + ".mlp.expert").integer("ff", minimum=1)
        router = KeyReader(_sub(mlp, "router", where + ".mlp"), where + ".mlp.router")
        experts, top = router.integer("experts", minimum=1), router.integer("top", minimum=1)
        router.number("scale", default=1.0)
        if top > experts:
            raise InvalidArgumentError(f"{where}.mlp.router: \"top\" {top} is above \"experts\" {experts}")
        shared = _optional(mlp, "shared", where + ".mlp")
        if shared is not None:
            KeyReader(shared, where + ".mlp.shared").integer("ff", minimum=1)

    def to_dict(self) -> Dict[str, Any]:
        data: Dict[str, Any] = {"architecture": self.architecture, "embedding": {"scale": self.embedding_scale},
                                "layers": copy.deepcopy(self.layers), "norm": {"eps": self.eps}, "vocab": self.vocab,
                                "width": self.width}
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
        return PartSpec("rmsnorm", {"width": self.width, "eps": self.eps, "name": name, "tensor": name})

    @staticmethod
    def _rotation(m: Dict[str, Any]) -> PartSpec:
        rot = m.get("rot") or {}
        dims = int(rot.get("dims") or 0)
        if not dims:
            return PartSpec("none", {})
        params = {"head_dim": int(m["dim"]), "rotary_dim": dims, "base": float(rot["base"])}
        if rot.get("scaling"):
            params["long_waves"] = {key: float(rot["scaling"][key]) for key in ("factor", "low", "high", "original")}
        return PartSpec("rotary_neox", params)

    def _softmax(self, m: Dict[str, Any], name: str, **options) -> PartSpec:
        params = {"hidden": self.width, "heads": int(m["heads"]), "kv_heads": int(m["kv_heads"]),
                  "head_dim": int(m["dim"]), "value_dim": int(m["vdim"]), "scale": float(m["scale"]), "eps": self.eps,
                  "tensors": {"q": "q", "k": "k", "v": "v", "o": "o", "g": "g", "q_norm": "q.norm", "k_norm": "k.norm",
                              "q_bias": "q.b", "k_bias": "k.b", "v_bias": "v.b"},
                  "name": name}
        params.update(options)
        return PartSpec("attention", params)

    def _windowed(self, m: Dict[str, Any]) -> PartSpec:
        return self._softmax(m, "mix", window=int(m["mask"]["size"]), keep_first=int(m["mask"].get("keep_first") or 0),
                             qk_norm="unit", sink=True)

    def _differential(self, m: Dict[str, Any]) -> PartSpec:
        return self._softmax(m, "mix", window=int(m["mask"]["size"]), keep_first=int(m["mask"].get("keep_first") or 0),
                             qk_norm="head", maps=2, diff=float(m["diff"]))

    def _chunked(self, m: Dict[str, Any], name: str, rows: int) -> PartSpec:
        options = dict(chunk=int(m["mask"]["size"]), qk_norm="head", qkv_bias=True, sink=True, gate="head_sigmoid")
        if m.get("bias_max") is not None:
            options["rel_bias"] = {"rows": rows, "far": float(m["bias_max"])}
        return self._softmax(m, name, **options)

    def _retention(self, m: Dict[str, Any], name: str) -> PartSpec:
        rot = m.get("rot") or {}
        return PartSpec("decay_attention", {
            "hidden": self.width, "heads": int(m["heads"]), "dim": int(m["dim"]), "vdim": int(m["vdim"]),
            "decay": [float(d) for d in m["decay"]], "eps": self.eps, "activation": "none", "gate": "silu",
            "norm": "head", "k_scale": float(m["dim"]) ** -0.5,
            "rotary": {"dims": int(rot.get("dims") or 0), "base": float(rot.get("base") or 10000.0)}, "name": name})

    def _ffn(self, mlp: Optional[Dict[str, Any]]) -> PartSpec:
        if mlp is None:
            return PartSpec("none", {})
        names = {"gate": "gate", "up": "up", "down": "down"}
        if mlp["kind"] == "dense":
            return PartSpec("gated_mlp", {"hidden": self.width, "intermediate": int(mlp["ff"]), "activation": "gelu_tanh",
                                          "tensors": names, "name": "mlp"})
        router = mlp["router"]
        shared = mlp.get("shared") or {}
        return PartSpec("moe", {"hidden": self.width, "intermediate": int(mlp["expert"]["ff"]),
                                "experts": int(router["experts"]), "top": int(router["top"]), "limit": None, "alpha": 1.0,
                                "scores": "steered", "weight_scale": float(router.get("scale", 1.0)),
                                "shared": int(shared["ff"]) if shared else None,
                                "shared_gate": "sigmoid" if shared else None, "name": "mlp"})

    def layer_specs(self) -> List[LayerSpec]:
        specs = []
        for index, layer in enumerate(self.layers):
            m = layer["mixer"]
            position = PartSpec("none", {})
            if layer["type"] == "attention":
                mixer, position = self._windowed(m), self._rotation(m)
            elif layer["type"] == "attention_2":
                mixer, position = self._differential(m), self._rotation(m)
            else:
                # the rows of the table of biases by distance are the stored tensor's (-1); "bias_rows" may give them
                # where weights are made, not read
                left = self._chunked(m["left"], "mix.left", int(m["left"].get("bias_rows") or -1))
                position = self._rotation(m["left"])
                mixer = PartSpec("mixer_pair", {"left": left, "right": self._retention(m["right"], "mix.right"),
                                                "left_scale": float(m.get("left_scale", 1.0)),
                                                "right_scale": float(m.get("right_scale", 1.0))})
            specs.append(LayerSpec("postnorm", mixer, self._ffn(layer.get("mlp")), self._norm("norm1"),
                                   self._norm("norm2"), position, f"l{index}."))
        return specs

    def embedding_spec(self) -> PartSpec:
        return PartSpec("embedding", {"vocab": self.vocab, "width": self.width, "name": "embed", "tensor": "embed",
                                      "scale": self.embedding_scale})

    def final_norm_spec(self) -> PartSpec:
        return self._norm("final.norm")

    def head_spec(self) -> PartSpec:
        return PartSpec("lm_head", {"vocab": self.vocab, "width": self.width, "name": "head", "tensor": "head",
                                    "tied_to": None})
