"""Typed configuration of Koketar, read from its config.json keys.

Koketar is a decoder whose every layer mixes two branches that read the same input: windowed
softmax attention with rotary positions ("left") and a gated delta rule ("right"), followed by a
feed-forward with clamped halves. The norm of a sublayer stands on its output, and what joins the
residual stream is scaled by one factor. ``layers`` lists the layers with all their sizes; a
checkpoint names its tensors ``l<i>.<part>`` without a ".weight" suffix. Two sizes stand in no key:
the inner widths of the right branch's two low-rank maps, which the shapes of its tensors give.
"""

from __future__ import annotations

import json
import math
import os
from dataclasses import dataclass, field
from typing import Any, Dict, List, Mapping, Optional, Tuple

from .spec import ConfigError, LayerSpec, ModelSpec, PartSpec, default_schedule

# The design has no limit on a sequence's length (positions enter through rotation angles and a
# recurrence); the engine sizes what it must by the run's own limit.
UNBOUNDED_POSITIONS = 1 << 30
LAYER_TYPES = ("parallel",)
FF_KINDS = ("dense",)
GLU_ALPHA = 1.702           # the design fixes the activation: g * sigmoid(1.702 g) * (u + 1)
GLU_SHIFT = 1.0


def _get(data: Mapping[str, Any], key: str, where: str):
    if not isinstance(data, Mapping) or key not in data or data[key] is None:
        raise ConfigError(f"config.json: {where} is missing '{key}'")
    return data[key]


def _int(data, key, where, least=1) -> int:
    value = _get(data, key, where)
    if isinstance(value, float) and value.is_integer():
        value = int(value)
    if isinstance(value, bool) or not isinstance(value, int) or value < least:
        raise ConfigError(f"config.json: {where}.{key} must be an integer of at least {least}, found {value!r}")
    return value


def _number(data, key, where, positive=False) -> float:
    value = _get(data, key, where)
    if isinstance(value, bool) or not isinstance(value, (int, float)) or not math.isfinite(value) or (positive and not value > 0):
        raise ConfigError(f"config.json: {where}.{key} must be a {'positive ' if positive else ''}number, found {value!r}")
    return float(value)


@dataclass(frozen=True)
class WindowAttentionSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int
    rot_dims: int
    rot_base: float
    rot_factor: float

    @classmethod
    def from_dict(cls, data, where) -> "WindowAttentionSizes":
        rot = _get(data, "rot", where)
        scaling = rot.get("scaling") if isinstance(rot, Mapping) else None
        sizes = cls(heads=_int(data, "heads", where), kv_heads=_int(data, "kv_heads", where), dim=_int(data, "dim", where),
                    vdim=_int(data, "vdim", where), scale=_number(data, "scale", where),
                    window=_int(_get(data, "mask", where), "size", where + ".mask"),
                    rot_dims=_int(rot, "dims", where + ".rot", least=0), rot_base=_number(rot, "base", where + ".rot", positive=True),
                    rot_factor=_number(scaling, "factor", where + ".rot.scaling", positive=True) if scaling is not None else 1.0)
        if sizes.heads % sizes.kv_heads:
            raise ConfigError(f"config.json: {where}: {sizes.heads} heads are not a multiple of {sizes.kv_heads} kv_heads")
        if sizes.rot_dims % 2 or sizes.rot_dims > sizes.dim:
            raise ConfigError(f"config.json: {where}.rot.dims {sizes.rot_dims} must be even and at most dim {sizes.dim}")
        return sizes

    def to_dict(self) -> Dict[str, Any]:
        rot: Dict[str, Any] = {"base": self.rot_base, "dims": self.rot_dims}
        if self.rot_factor != 1.0:
            rot["scaling"] = {"factor": self.rot_factor}
        return {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "mask": {"size": self.window}, "rot": rot,
                "scale": self.scale, "vdim": self.vdim}


@dataclass(frozen=True)
class DeltaRuleSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    decay_rank: Optional[int] = None        # from the checkpoint's shapes (or given, for random weights)
    gate_rank: Optional[int] = None

    @classmethod
    def from_dict(cls, data, where) -> "DeltaRuleSizes":
        sizes = cls(heads=_int(data, "heads", where), kv_heads=_int(data, "kv_heads", where), dim=_int(data, "dim", where),
                    vdim=_int(data, "vdim", where), conv=_int(data, "conv", where),
                    decay_rank=_int(data, "decay_rank", where) if data.get("decay_rank") is not None else None,
                    gate_rank=_int(data, "gate_rank", where) if data.get("gate_rank") is not None else None)
        if sizes.heads % sizes.kv_heads:
            raise ConfigError(f"config.json: {where}: {sizes.heads} heads are not a multiple of {sizes.kv_heads} kv_heads")
        return sizes

    def to_dict(self) -> Dict[str, Any]:
        out = {"conv": self.conv, "dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "vdim": self.vdim}
        if self.decay_rank is not None:
            out["decay_rank"] = self.decay_rank
        if self.gate_rank is not None:
            out["gate_rank"] = self.gate_rank
        return out


@dataclass(frozen=True)
class KoketarLayer:
    left: WindowAttentionSizes
    right: DeltaRuleSizes
    left_scale: float
    right_scale: float
    ff: Optional[int]               # None: the layer has no feed-forward
    limit: Optional[float]


@dataclass(frozen=True)
class KoketarConfig:
    vocab: int
    width: int
    norm_eps: float
    residual_mult: float
    logit_softcap: float
    layers: Tuple[KoketarLayer, ...]

    architecture = "Koketar"

    @classmethod
    def from_dict(cls, data: Mapping[str, Any]) -> "KoketarConfig":
        if not isinstance(data, Mapping):
            raise ConfigError("config.json must hold a JSON object")
        listed = _get(data, "layers", "the model")
        if not isinstance(listed, list) or not listed:
            raise ConfigError("config.json: 'layers' must be a list of at least one layer")
        layers: List[KoketarLayer] = []
        for index, entry in enumerate(listed):
            where = f"layers[{index}]"
            kind = _get(entry, "type", where)
            if kind not in LAYER_TYPES:
                raise ConfigError(f"config.json: {where}.type is {kind!r}; known: {', '.join(LAYER_TYPES)}")
            mixer = _get(entry, "mixer", where)
            mlp = entry.get("mlp")
            if mlp is not None and _get(mlp, "kind", where + ".mlp") not in FF_KINDS:
                raise ConfigError(f"config.json: {where}.mlp.kind is {mlp['kind']!r}; known: {', '.join(FF_KINDS)}")
            layers.append(KoketarLayer(
                left=WindowAttentionSizes.from_dict(_get(mixer, "left", where + ".mixer"), where + ".mixer.left"),
                right=DeltaRuleSizes.from_dict(_get(mixer, "right", where + ".mixer"), where + ".mixer.right"),
                left_scale=_number(mixer, "left_scale", where + ".mixer"), right_scale=_number(mixer, "right_scale", where + ".mixer"),
                ff=_int(mlp, "ff", where + ".mlp") if mlp is not None else None,
                limit=_number(mlp, "limit", where + ".mlp", positive=True) if mlp is not None else None))
        cap = data.get("logit_softcap")
        return cls(vocab=_int(data, "vocab", "the model"), width=_int(data, "width", "the model"),
                   norm_eps=_number(_get(data, "norm", "the model"), "eps", "norm", positive=True),
                   residual_mult=_number(data, "residual_mult", "the model"),
                   logit_softcap=_number(data, "logit_softcap", "the model", positive=True) if cap else 0.0,
                   layers=tuple(layers))

    @classmethod
    def from_model_dir(cls, model_dir: str, data: Mapping[str, Any]) -> "KoketarConfig":
        """``from_dict``, with the sizes that only the checkpoint's tensors show read from their shapes."""
        from ..weights.safetensors_io import SafetensorsFile, checkpoint_files
        config = cls.from_dict(data)
        shapes: Dict[str, Tuple[int, ...]] = {}
        for path in checkpoint_files(model_dir):
            handle = SafetensorsFile(path)
            try:
                shapes.update({name: tuple(entry.shape) for name, entry in handle.entries.items()})
            finally:
                handle.close()
        layers = []
        for index, layer in enumerate(config.layers):
            ranks = {}
            for key, tensor in (("decay_rank", f"l{index}.mix.right.a1"), ("gate_rank", f"l{index}.mix.right.g1")):
                shape = shapes.get(tensor)
                if getattr(layer.right, key) is None:
                    if shape is None or len(shape) != 2:
                        raise ConfigError(f"{model_dir}: tensor '{tensor}' is missing or no matrix; its rows give layers[{index}].mixer.right's {key}")
                    ranks[key] = int(shape[0])
            layers.append(KoketarLayer(left=layer.left, right=DeltaRuleSizes(**{**layer.right.__dict__, **ranks}),
                                       left_scale=layer.left_scale, right_scale=layer.right_scale, ff=layer.ff, limit=layer.limit))
        return cls(vocab=config.vocab, width=config.width, norm_eps=config.norm_eps, residual_mult=config.residual_mult,
                   logit_softcap=config.logit_softcap, layers=tuple(layers))

    def to_dict(self) -> Dict[str, Any]:
        layers = []
        for layer in self.layers:
            layers.append({
                "mixer": {"left": layer.left.to_dict(), "left_scale": layer.left_scale, "right": layer.right.to_dict(),
                          "right_scale": layer.right_scale},
                "mlp": None if layer.ff is None else {"ff": layer.ff, "kind": "dense", "limit": layer.limit},
                "type": "parallel"})
        data: Dict[str, Any] = {"architecture": self.architecture, "layers": layers, "norm": {"eps": self.norm_eps},
                                "residual_mult": self.residual_mult, "vocab": self.vocab, "width": self.width}
        if self.logit_softcap:
            data["logit_softcap"] = self.logit_softcap
        return data

    def save(self, folder: str) -> None:
        os.makedirs(folder, exist_ok=True)
        with open(os.path.join(folder, "config.json"), "w", encoding="utf-8") as handle:
            json.dump(self.to_dict(), handle, indent=1)

    # sizes the engine's command line and scheduler ask any configuration for
    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def max_position_embeddings(self) -> int:
        return UNBOUNDED_POSITIONS

    def model_spec(self) -> ModelSpec:
        D = self.width
        layers: List[LayerSpec] = []
        for index, layer in enumerate(self.layers):
            base = f"l{index}."
            a, b = layer.left, layer.right
            if b.decay_rank is None or b.gate_rank is None:
                raise ConfigError(f"layers[{index}].mixer.right: the inner widths of its low-rank maps are not known "
                                  "(they come from a checkpoint's tensor shapes, or 'decay_rank' / 'gate_rank')")
            left = PartSpec("gqa_attention", {
                "hidden_size": D, "num_heads": a.heads, "num_kv_heads": a.kv_heads, "head_dim": a.dim, "v_head_dim": a.vdim,
                "qk_norm": True, "qk_norm_eps": self.norm_eps, "window": a.window, "softmax_scale": a.scale,
                "position": PartSpec("rotary_neox", {"theta": a.rot_base, "rotary_dim": a.rot_dims, "head_dim": a.dim,
                                                     "scaling_factor": a.rot_factor}),
                "names": {"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm"},
                "weight_suffix": "",
            }, prefix=base + "mix.left.")
            right = PartSpec("gated_delta_rule", {
                "hidden_size": D, "num_heads": b.heads, "num_kv_heads": b.kv_heads, "head_dim": b.dim, "v_head_dim": b.vdim,
                "conv_taps": b.conv, "decay_rank": b.decay_rank, "gate_rank": b.gate_rank, "norm_eps": self.norm_eps,
            }, prefix=base + "mix.right.")
            norm = {"eps": self.norm_eps, "size": D, "one_centered": True}
            layers.append(LayerSpec(
                arrangement="output_norm_residual",
                mixer_norm=PartSpec("rmsnorm", {**norm, "tensor": base + "norm1"}),
                mixer=PartSpec("parallel_branches", {"branches": (("left", left, layer.left_scale), ("right", right, layer.right_scale))},
                               prefix=base + "mix."),
                ffn_norm=None if layer.ff is None else PartSpec("rmsnorm", {**norm, "tensor": base + "norm2"}),
                ffn=None if layer.ff is None else PartSpec("clamped_glu", {
                    "hidden_size": D, "intermediate_size": layer.ff, "limit": layer.limit, "alpha": GLU_ALPHA, "shift": GLU_SHIFT,
                    "weight_suffix": ""}, prefix=base + "mlp."),
                params={"residual_mult": self.residual_mult},
            ))
        spec = ModelSpec(
            architecture=self.architecture, hidden_size=D, vocab_size=self.vocab, max_positions=UNBOUNDED_POSITIONS,
            layers=tuple(layers), schedule=default_schedule(len(layers)),
            final_norm=PartSpec("rmsnorm", {"eps": self.norm_eps, "size": D, "one_centered": True, "tensor": "final.norm"}),
            embedding_name="embed", lm_head_name=None, logit_softcap=self.logit_softcap)
        spec.validate()
        return spec
