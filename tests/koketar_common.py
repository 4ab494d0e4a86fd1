"""Shared by the Koketar tests: small configurations that differ from each other in every size and
option, model folders with random weights that make every part count, and the comparison's limits."""

from __future__ import annotations

import copy
import json
import os
from typing import Dict, List, Optional, Sequence

import numpy as np

import plain_koketar as plain


def _left(heads, kv_heads, dim, vdim, window, rot_dims, base, factor, scale):
    rot = {"base": base, "dims": rot_dims}
    if factor is not None:
        rot["scaling"] = {"factor": factor}
    return {"dim": dim, "heads": heads, "kv_heads": kv_heads, "mask": {"size": window}, "rot": rot, "scale": scale, "vdim": vdim}


def _right(heads, kv_heads, dim, vdim, conv, rank_a, rank_g):
    # rank_a / rank_g are the tests' own keys (plain_koketar.tensor_shapes reads them); a checkpoint shows them by its shapes
    return {"conv": conv, "dim": dim, "heads": heads, "kv_heads": kv_heads, "vdim": vdim, "rank_a": rank_a, "rank_g": rank_g}


def _layer(left, right, left_scale, right_scale, ff, limit):
    return {"mixer": {"left": left, "left_scale": left_scale, "right": right, "right_scale": right_scale},
            "mlp": None if ff is None else {"ff": ff, "kind": "dense", "limit": limit}, "type": "parallel"}


# X: three layers, each of other sizes. Layer 0: grouped heads, values wider than keys, a window that
# crosses page borders, partial rotation with scaling, low-rank widths that are no multiple of 8.
# Layer 1: keys and values of one size (the matrix-core attention in bfloat16), full rotation
# without scaling, value heads wider than one block of the recurrence, two taps, no feed-forward.
# Layer 2: three query heads on one key head, a window of five tokens, a recurrence of one head.
CONFIG_X = {
    "architecture": "Koketar", "vocab": 300, "width": 96, "norm": {"eps": 1e-6}, "residual_mult": 0.6, "logit_softcap": 8.0,
    "layers": [
        _layer(_left(4, 2, 32, 48, 40, 16, 10000.0, 4.0, 0.2), _right(4, 2, 24, 40, 3, 10, 12), 1.3, 0.7, 160, 0.8),
        _layer(_left(2, 2, 64, 64, 70, 64, 500000.0, None, 0.125), _right(2, 1, 64, 80, 2, 16, 8), 0.5, 1.0, None, None),
        _layer(_left(3, 1, 16, 16, 5, 8, 100.0, 2.0, 0.3), _right(1, 1, 16, 16, 4, 8, 24), 1.0, 1.0, 72, 2.5),
    ],
}

# Y: one wide layer with a sharp softmax (a single key decides a row's output, so a window that is one
# token off shows in bfloat16 too) and a recurrence that forgets slowly (see ``make_folder``), values
# narrower than keys, six taps, no soft cap.
CONFIG_Y = {
    "architecture": "Koketar", "vocab": 200, "width": 64, "norm": {"eps": 1e-5}, "residual_mult": 1.0,
    "layers": [
        _layer(_left(2, 1, 48, 32, 33, 24, 1000.0, 1.5, 1.5), _right(3, 3, 40, 24, 6, 8, 8), 1.0, 1.0, 128, 1.0),
        _layer(_left(2, 2, 32, 96, 64, 32, 1000.0, None, 1.0), _right(2, 2, 8, 136, 3, 8, 16), 0.9, 1.1, 96, 0.5),
    ],
}

# Z: the corners. A window of one token (a row sees itself alone) and one wider than any prompt here; no
# rotation at all and rotation of every channel; one tap (no convolution memory); heads of 4 and 8
# channels; values narrower and wider than keys; one head on one key head and six on three; a
# feed-forward width that is no multiple of eight (the products then take the plain kernel); a layer
# without feed-forward; no soft cap; a factor of one on what joins the residual stream.
CONFIG_Z = {
    "architecture": "Koketar", "vocab": 97, "width": 40, "norm": {"eps": 1e-5}, "residual_mult": 1.0,
    "layers": [
        _layer(_left(1, 1, 8, 24, 1, 0, 10000.0, None, 1.0), _right(2, 2, 4, 4, 1, 3, 5), 0.7, 1.2, None, None),
        _layer(_left(6, 3, 24, 8, 200, 24, 10000.0, 1.0, 0.25), _right(4, 1, 12, 20, 2, 8, 8), 1.0, 0.6, 50, 3.0),
    ],
}

# W: wide enough that a prompt of some hundred tokens goes through the tiled prompt products and the
# matrix-core attention (keys of 64 and values of 128 channels in one layer, the reverse in the other), with widths of
# the joined operands that are no multiple of their tiles.
CONFIG_W = {
    "architecture": "Koketar", "vocab": 1000, "width": 512, "norm": {"eps": 1e-5}, "residual_mult": 0.4, "logit_softcap": 20.0,
    "layers": [
        _layer(_left(8, 2, 64, 128, 150, 48, 100000.0, 4.0, 0.11), _right(6, 3, 48, 80, 4, 24, 40), 0.9, 0.6, 1344, 1.5),
        _layer(_left(4, 4, 128, 64, 90, 128, 100000.0, None, 0.09), _right(4, 4, 128, 128, 3, 16, 16), 1.0, 1.0, 1024, 2.0),
    ],
}

CONFIGS = {"X": CONFIG_X, "Y": CONFIG_Y, "Z": CONFIG_Z, "W": CONFIG_W}

# Largest difference from the plain float64 model, as a fraction of the largest logit compared, and
# the same for the root mean square. float32 shows the logic right; the bfloat16 limits have to tell
# rounding (2e-3 at every stored activation) from a fault, and the configurations make faults large.
MAX_TOL = {"float32": 3e-5, "bfloat16": 8e-2}
RMS_TOL = {"float32": 6e-6, "bfloat16": 2e-2}


def only_branch(config: dict, which: str) -> dict:
    """The same model with one branch of every mixer switched off and no feed-forward: the other
    mechanism alone."""
    out = copy.deepcopy(config)
    for layer in out["layers"]:
        layer["mixer"]["left_scale" if which == "right" else "right_scale"] = 0.0
        layer["mlp"] = None
    return out


def file_config(config: dict) -> dict:
    """What stands in config.json: the tests' own keys taken out."""
    out = copy.deepcopy(config)
    for layer in out["layers"]:
        for key in ("rank_a", "rank_g"):
            layer["mixer"]["right"].pop(key, None)
    return out


def make_folder(folder: str, config: dict, seed: int = 0, slow_decay: bool = False):
    """Writes config.json and model.safetensors (bfloat16 matrices) and returns the weights as the
    plain model reads them: the stored values, in float64."""
    import torch
    from safetensors.torch import save_file
    weights = plain.random_weights(config, seed)
    if slow_decay:      # the first head of every recurrence barely forgets: what it wrote long ago still counts
        for name in weights:
            if name.endswith(".A_log"):
                weights[name][0] = -7.0
    stored = {name: torch.from_numpy(value).to(torch.bfloat16) for name, value in weights.items()}
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as handle:
        json.dump(file_config(config), handle)
    save_file({name: value.contiguous() for name, value in stored.items()}, os.path.join(folder, "model.safetensors"))
    return {name: value.to(torch.float64).numpy() for name, value in stored.items()}


def random_tokens(vocab: int, count: int, seed: int) -> List[int]:
    return np.random.default_rng(seed).integers(0, vocab, size=count).tolist()


def assert_close(found: np.ndarray, expected: np.ndarray, dtype: str, what: str = "") -> None:
    assert found.shape == expected.shape, f"{what}: shape {found.shape} vs {expected.shape}"
    assert np.isfinite(found).all(), f"{what}: non-finite logits"
    scale = max(1.0, float(np.abs(expected).max()))
    error = np.abs(found.astype(np.float64) - expected)
    worst, rms = float(error.max()), float(np.sqrt(np.mean(error ** 2)))
    first = int(np.argmax(error.max(axis=-1) > MAX_TOL[dtype] * scale))
    assert worst <= MAX_TOL[dtype] * scale, f"{what}: largest difference {worst:.3e} exceeds {MAX_TOL[dtype] * scale:.3e} (first row over: {first})"
    assert rms <= RMS_TOL[dtype] * scale, f"{what}: rms difference {rms:.3e} exceeds {RMS_TOL[dtype] * scale:.3e}"
