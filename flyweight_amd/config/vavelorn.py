"""Typed configuration of Vavelorn, read from its config.json keys.

Vavelorn is a decoder whose layers each have one of three mixers, named by ``type``: ``attention``
(grouped-query softmax attention with interleaved rotary positions on the first channels of a head, a
soft cap on the scores, and a chunked mask: a row sees the earlier keys of its own chunk of positions
only), ``latent_attention`` (keys and values of every head unfolded from one normed latent per token,
queries through a normed latent of their own, a sigmoid gate on the heads' outputs, no positions) and
``delta`` (a gated delta rule with short convolutions, one decay per head and a silu gate). A norm
stands before and behind each sublayer (layer norms with a weight and no bias), the feed-forward is a
SwiGLU or absent, and after it every layer adds an input of the tokens' own from its slice of a second
embedding table (``token_side.dim`` columns a layer). ``layers`` lists the layers with all their sizes;
a checkpoint names its tensors ``l<i>.<part>`` without a ".weight" suffix; the head is a matrix of its own.
"""

from __future__ import annotations

import json
import math
import os
from dataclasses import dataclass
from typing import Any, Dict, List, Mapping, Optional, Tuple

from .spec import ConfigError, LayerSpec, ModelSpec, PartSpec, default_schedule

UNBOUNDED_POSITIONS = 1 << 30       # positions enter through rotation angles and a recurrence only
LAYER_TYPES = ("attention", "latent_attention", "delta")
FF_KINDS = ("dense",)
NORM_KINDS = {"layer": "layernorm", "layernorm": "layernorm", "rms": "rmsnorm", "rmsnorm": "rmsnorm"}


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


def _or(data, key, where, default, least=1) -> int:
    """A size that may be left out: kv_heads (then every head has keys of its own), vdim (then the keys' size)."""
    return _int(data, key, where, least) if isinstance(data, Mapping) and data.get(key) is not None else default


def _scale(data, where, dim: int) -> float:
    """The factor on the scores; left out, dim^-1/2."""
    return _number(data, "scale", where, positive=True) if data.get("scale") is not None else dim ** -0.5


def _groups(heads: int, kv_heads: int, where: str) -> None:
    if heads % kv_heads:
        raise ConfigError(f"config.json: {where}: {heads} heads are not a multiple of {kv_heads} kv_heads")


@dataclass(frozen=True)
class ChunkedAttentionSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    chunk: Optional[int]            # None: every earlier key
    softcap: Optional[float]        # None: the scores as they are
    rot_dims: int
    rot_base: float

    kind = "attention"

    @classmethod
    def from_dict(cls, data, where) -> "ChunkedAttentionSizes":
        rot, mask, cap = data.get("rot"), data.get("mask"), data.get("softcap")
        heads, dim = _int(data, "heads", where), _int(data, "dim", where)
        sizes = cls(heads=heads, kv_heads=_or(data, "kv_heads", where, heads), dim=dim,
                    vdim=_or(data, "vdim", where, dim), scale=_scale(data, where, dim),
                    chunk=_int(mask, "size", where + ".mask") if mask is not None else None,
                    softcap=_number(data, "softcap", where, positive=True) if cap else None,
                    rot_dims=_int(rot, "dims", where + ".rot", least=0) if rot is not None else 0,
                    rot_base=_number(rot, "base", where + ".rot", positive=True) if rot is not None else 1.0)
        _groups(sizes.heads, sizes.kv_heads, where)
        if sizes.rot_dims % 2 or sizes.rot_dims > sizes.dim:
            raise ConfigError(f"config.json: {where}.rot.dims {sizes.rot_dims} must be even and at most dim {sizes.dim}")
        return sizes

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads,
                               "rot": {"base": self.rot_base, "dims": self.rot_dims}, "scale": self.scale, "vdim": self.vdim}
        if self.chunk is not None:
            out["mask"] = {"size": self.chunk}
        if self.softcap is not None:
            out["softcap"] = self.softcap
        return out


@dataclass(frozen=True)
class LatentAttentionSizes:
    heads: int
    dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float

    kind = "latent_attention"

    @classmethod
    def from_dict(cls, data, where) -> "LatentAttentionSizes":
        dim = _int(data, "dim", where)
        return cls(heads=_int(data, "heads", where), dim=dim, vdim=_or(data, "vdim", where, dim),
                   q_rank=_int(data, "q_rank", where), kv_rank=_int(data, "kv_rank", where), scale=_scale(data, where, dim))

    def to_dict(self) -> Dict[str, Any]:
        return {"dim": self.dim, "heads": self.heads, "kv_rank": self.kv_rank, "q_rank": self.q_rank, "scale": self.scale,
                "vdim": self.vdim}


@dataclass(frozen=True)
class DeltaSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int

    kind = "delta"

    @classmethod
    def from_dict(cls, data, where) -> "DeltaSizes":
        heads, dim = _int(data, "heads", where), _int(data, "dim", where)
        sizes = cls(heads=heads, kv_heads=_or(data, "kv_heads", where, heads), dim=dim, vdim=_or(data, "vdim", where, dim),
                    conv=_int(data, "conv", where))
        _groups(sizes.heads, sizes.kv_heads, where)
        return sizes

    def to_dict(self) -> Dict[str, Any]:
        return {"conv": self.conv, "dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "vdim": self.vdim}


_MIXERS = {cls.kind: cls for cls in (ChunkedAttentionSizes, LatentAttentionSizes, DeltaSizes)}


@dataclass(frozen=True)
class VavelornLayer:
    mixer: Any                      # one of the three sizes classes; its ``kind`` is the layer's type
    ff: Optional[int]               # None: the layer has no feed-forward


@dataclass(frozen=True)
class VavelornConfig:
    vocab: int
    width: int
    norm_eps: float
    side_dim: Optional[int]         # columns of the second token table that a layer reads; None: no such input
    layers: Tuple[VavelornLayer, ...]
    norm_kind: str = "layer"

    architecture = "Vavelorn"

    @classmethod
    def from_dict(cls, data: Mapping[str, Any]) -> "VavelornConfig":
        if not isinstance(data, Mapping):
            raise ConfigError("config.json must hold a JSON object")
        listed = _get(data, "layers", "the model")
        if not isinstance(listed, list) or not listed:
            raise ConfigError("config.json: 'layers' must be a list of at least one layer")
        layers: List[VavelornLayer] = []
        for index, entry in enumerate(listed):
            where = f"layers[{index}]"
            kind = _get(entry, "type", where)
            if kind not in _MIXERS:
                raise ConfigError(f"config.json: {where}.type is {kind!r}; known: {', '.join(LAYER_TYPES)}")
            mlp = entry.get("mlp")
            if mlp is not None and _get(mlp, "kind", where + ".mlp") not in FF_KINDS:
                raise ConfigError(f"config.json: {where}.mlp.kind is {mlp['kind']!r}; known: {', '.join(FF_KINDS)}")
            layers.append(VavelornLayer(mixer=_MIXERS[kind].from_dict(_get(entry, "mixer", where), where + ".mixer"),
                                        ff=_int(mlp, "ff", where + ".mlp") if mlp is not None else None))
        norm = _get(data, "norm", "the model")
        norm_kind = str(norm.get("kind", "layer"))
        if norm_kind not in NORM_KINDS:
            raise ConfigError(f"config.json: norm.kind is {norm_kind!r}; known: layer, rms")
        side = data.get("token_side")
        return cls(vocab=_int(data, "vocab", "the model"), width=_int(data, "width", "the model"),
                   norm_eps=_number(norm, "eps", "norm", positive=True),
                   side_dim=_int(side, "dim", "token_side") if side is not None else None, layers=tuple(layers), norm_kind=norm_kind)

    def to_dict(self) -> Dict[str, Any]:
        layers = [{"mixer": layer.mixer.to_dict(), "mlp": None if layer.ff is None else {"ff": layer.ff, "kind": "dense"},
                   "type": layer.mixer.kind} for layer in self.layers]
        norm: Dict[str, Any] = {"eps": self.norm_eps}
        if self.norm_kind != "layer":
            norm["kind"] = self.norm_kind
        data: Dict[str, Any] = {"architecture": self.architecture, "layers": layers, "norm": norm, "vocab": self.vocab,
                                "width": self.width}
        if self.side_dim is not None:
            data["token_side"] = {"dim": self.side_dim}
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

    def _mixer_spec(self, sizes, prefix: str) -> PartSpec:
        D = self.width
        if sizes.kind == "attention":
            return PartSpec("gqa_attention", {
                "hidden_size": D, "num_heads": sizes.heads, "num_kv_heads": sizes.kv_heads, "head_dim": sizes.dim,
                "v_head_dim": sizes.vdim, "softmax_scale": sizes.scale, "chunk": sizes.chunk, "score_softcap": sizes.softcap,
                "position": PartSpec("rotary_interleaved", {"theta": sizes.rot_base, "rotary_dim": sizes.rot_dims, "head_dim": sizes.dim}),
                "names": {"q": "q", "k": "k", "v": "v", "o": "o"}, "weight_suffix": "",
            }, prefix=prefix)
        if sizes.kind == "latent_attention":
            return PartSpec("latent_attention", {
                "hidden_size": D, "num_heads": sizes.heads, "head_dim": sizes.dim, "v_head_dim": sizes.vdim, "q_rank": sizes.q_rank,
                "kv_rank": sizes.kv_rank, "softmax_scale": sizes.scale, "norm_eps": self.norm_eps, "output_gate": True,
            }, prefix=prefix)
        return PartSpec("gated_delta_rule", {
            "hidden_size": D, "num_heads": sizes.heads, "num_kv_heads": sizes.kv_heads, "head_dim": sizes.dim, "v_head_dim": sizes.vdim,
            "conv_taps": sizes.conv, "norm_eps": self.norm_eps, "decay": "head", "gate": "silu",
        }, prefix=prefix)

    def model_spec(self) -> ModelSpec:
        D = self.width
        norm_part = NORM_KINDS[self.norm_kind]

        def norm(tensor: str) -> PartSpec:
            return PartSpec(norm_part, {"eps": self.norm_eps, "size": D, "tensor": tensor})

        layers: List[LayerSpec] = []
        for index, layer in enumerate(self.layers):
            base = f"l{index}."
            params: Dict[str, Any] = {"mixer_post_norm": norm(base + "norm1b")}
            if layer.ff is not None:
                params["ffn_post_norm"] = norm(base + "norm2b")
            if self.side_dim is not None:
                params["token_input"] = PartSpec("token_input", {
                    "hidden_size": D, "dim": self.side_dim, "first_column": index * self.side_dim,
                    "table_columns": self.side_dim * len(self.layers), "vocab_size": self.vocab, "norm_eps": self.norm_eps,
                    "table": "side.embed"}, prefix=base + "side.")
            layers.append(LayerSpec(
                arrangement="sandwich_norm_residual",
                mixer_norm=norm(base + "norm1"),
                mixer=self._mixer_spec(layer.mixer, base + "mix."),
                ffn_norm=None if layer.ff is None else norm(base + "norm2"),
                ffn=None if layer.ff is None else PartSpec("swiglu", {
                    "hidden_size": D, "intermediate_size": layer.ff, "names": {"gate": "gate", "up": "up", "down": "down"},
                    "weight_suffix": ""}, prefix=base + "mlp."),
                params=params))
        spec = ModelSpec(
            architecture=self.architecture, hidden_size=D, vocab_size=self.vocab, max_positions=UNBOUNDED_POSITIONS,
            layers=tuple(layers), schedule=default_schedule(len(layers)), final_norm=norm("final.norm"),
            embedding_name="embed", lm_head_name="head")
        spec.validate()
        return spec
