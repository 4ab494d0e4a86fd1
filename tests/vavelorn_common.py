"""Shared by the Vavelorn tests: small configurations that differ from each other in every size and
option, model folders with random weights that make every part count, and the comparison's limits."""

from __future__ import annotations

import copy
import json
import os
from typing import Dict, List, Optional

import numpy as np

import plain_vavelorn as plain


def attention(heads, kv_heads, dim, vdim, chunk, rot_dims, base, scale, softcap):
    out = {"dim": dim, "heads": heads, "kv_heads": kv_heads, "rot": {"base": base, "dims": rot_dims}, "scale": scale, "vdim": vdim}
    if chunk is not None:
        out["mask"] = {"size": chunk}
    if softcap is not None:
        out["softcap"] = softcap
    return {"type": "attention", "mixer": out}


def latent(heads, dim, vdim, q_rank, kv_rank, scale):
    return {"type": "latent_attention", "mixer": {"dim": dim, "heads": heads, "kv_rank": kv_rank, "q_rank": q_rank, "scale": scale, "vdim": vdim}}


def delta(heads, kv_heads, dim, vdim, conv):
    return {"type": "delta", "mixer": {"conv": conv, "dim": dim, "heads": heads, "kv_heads": kv_heads, "vdim": vdim}}


def layer(mixer, ff):
    return {**mixer, "mlp": None if ff is None else {"ff": ff, "kind": "dense"}}


# X: one layer of every mixer and a second attention, each of other sizes. Grouped heads with values wider
# than keys, a chunk that crosses page borders, partial rotation, a low soft cap; a latent that is no
# multiple of sixteen (bfloat16 takes the plain attention kernel); a recurrence with grouped heads and four
# taps; an attention layer without chunks and without a cap, every channel rotated, no feed-forward.
CONFIG_X = {
    "architecture": "Vavelorn", "vocab": 300, "width": 96, "norm": {"eps": 1e-6}, "token_side": {"dim": 12},
    "layers": [
        layer(attention(4, 2, 32, 48, 40, 16, 10000.0, 0.2, 3.0), 160),
        layer(latent(3, 24, 40, 20, 40, 0.25), 136),
        layer(delta(4, 2, 24, 40, 4), 160),
        layer(attention(2, 2, 64, 64, None, 64, 500000.0, 0.125, None), None),
    ],
}

# Y: pointed softmaxes (score spreads of about three, so that a few keys share a row's weight and a chunk
# that is one token off shows in bfloat16 too; sharper ones would make rounding itself visible: the
# kernel tests have those, with keys made for it), chunks of 33 and of 64 tokens, a latent on the matrix-core kernels, a recurrence whose
# first head barely forgets (see ``make_folder``), two taps, values narrower than keys.
CONFIG_Y = {
    "architecture": "Vavelorn", "vocab": 200, "width": 64, "norm": {"eps": 1e-5}, "token_side": {"dim": 8},
    "layers": [
        layer(attention(2, 1, 48, 32, 33, 24, 1000.0, 0.45, 30.0), 128),
        layer(delta(3, 3, 40, 24, 2), 96),
        layer(latent(2, 16, 24, 32, 64, 0.6), 128),
        layer(attention(4, 4, 16, 16, 64, 8, 100.0, 0.7, None), 96),
    ],
}

# Z: the corners. A chunk of one token (a row sees itself alone) and one longer than any prompt here; no
# rotation at all; one tap (no convolution memory) and six; heads of 4 and 8 channels; one head on one key
# head and six on three; a latent of 8 channels with a query rank of 4, and one of 320 channels; a feed-forward width that is no
# multiple of eight; layers without feed-forward; no token input at all.
CONFIG_Z = {
    "architecture": "Vavelorn", "vocab": 97, "width": 40, "norm": {"eps": 1e-5},
    "layers": [
        layer(attention(1, 1, 8, 24, 1, 0, 10000.0, 1.0, 2.0), None),
        layer(delta(2, 2, 4, 4, 1), 50),
        layer(latent(1, 8, 4, 4, 8, 0.5), None),
        layer(attention(6, 3, 24, 8, 500, 24, 10000.0, 0.25, 50.0), 50),
        layer(delta(4, 1, 12, 20, 6), None),
        layer(latent(2, 16, 8, 12, 320, 0.25), None),       # a latent wider than the matrix-core kernels take
    ],
}

# W: wide enough that a prompt of some hundred tokens goes through the tiled prompt products and the
# matrix-core attention (keys of 64 and values of 128 channels, a latent of 128 channels shared by eight
# heads), with widths of the joined operands that are no multiple of their tiles.
CONFIG_W = {
    "architecture": "Vavelorn", "vocab": 1000, "width": 512, "norm": {"eps": 1e-5}, "token_side": {"dim": 40},
    "layers": [
        layer(attention(8, 2, 64, 128, 150, 48, 100000.0, 0.11, 20.0), 1344),
        layer(latent(8, 48, 80, 96, 128, 0.14), 1024),
        layer(delta(6, 3, 48, 80, 4), 1024),
    ],
}

CONFIGS = {"X": CONFIG_X, "Y": CONFIG_Y, "Z": CONFIG_Z, "W": CONFIG_W}

# Largest difference from the plain float64 model, as a fraction of the largest logit compared, and
# the same for the root mean square. float32 shows the logic right; the bfloat16 limits have to tell
# rounding (2e-3 at every stored activation) from a fault, and the configurations make faults large.
# The design divides by the size of small vectors (a head's four read-outs, a sublayer's whole output),
# which now and then is nearly nothing: in bfloat16 one row in fifty may pass the largest difference,
# the root mean square over all rows still has to hold.
MAX_TOL = {"float32": 3e-5, "bfloat16": 8e-2}
RMS_TOL = {"float32": 6e-6, "bfloat16": 2e-2}
ROWS_OVER = {"float32": 0.0, "bfloat16": 0.02}


def only_mixer(config: dict, kind: str) -> dict:
    """The same model with the layers of one mixer alone, no feed-forward and no token input: one
    mechanism between its norms."""
    out = copy.deepcopy(config)
    out["layers"] = [dict(entry, mlp=None) for entry in out["layers"] if entry["type"] == kind]
    out.pop("token_side", None)
    return out


def make_folder(folder: str, config: dict, seed: int = 0, slow_decay: bool = False):
    """Writes config.json and model.safetensors (bfloat16 matrices) and returns the weights as the
    plain model reads them: the stored values, in float64."""
    import torch
    from safetensors.torch import save_file
    weights = plain.random_weights(config, seed)
    # A recurrence's read-out is a sum of values weighted by k . q and is divided by its own size: were
    # its keys and queries independent, k . q would lie around zero and now and then so close to it that
    # the rounding of the layer's input decides the whole output. Keys that lean towards their queries
    # keep the read-outs away from nothing, so that a difference means a fault.
    for index, entry in enumerate(config["layers"]):
        if entry["type"] == "delta":
            base = f"l{index}.mix."
            weights[base + "k"] = 0.8 * weights[base + "q"] + 0.6 * weights[base + "k"]
            weights[base + "k.conv"] = weights[base + "q.conv"].copy()
    if slow_decay:      # the first head of every recurrence barely forgets: what it wrote long ago still counts
        for name in weights:
            if name.endswith(".A_log"):
                weights[name][0] = -7.0
    stored = {name: torch.from_numpy(value).to(torch.bfloat16) for name, value in weights.items()}
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as handle:
        json.dump(config, handle)
    save_file({name: value.contiguous() for name, value in stored.items()}, os.path.join(folder, "model.safetensors"))
    return {name: value.to(torch.float64).numpy() for name, value in stored.items()}


def random_tokens(vocab: int, count: int, seed: int) -> List[int]:
    return np.random.default_rng(seed).integers(0, vocab, size=count).tolist()


def assert_close(found: np.ndarray, expected: np.ndarray, dtype: str, what: str = "", scale: Optional[float] = None) -> None:
    assert found.shape == expected.shape, f"{what}: shape {found.shape} vs {expected.shape}"
    assert np.isfinite(found).all(), f"{what}: non-finite values"
    scale = max(1.0, float(np.abs(expected).max())) if scale is None else scale
    error = np.abs(found.astype(np.float64) - expected)
    worst, rms = float(error.max()), float(np.sqrt(np.mean(error ** 2)))
    over = error.reshape(error.shape[0], -1).max(axis=-1) > MAX_TOL[dtype] * scale
    allowed = int(ROWS_OVER[dtype] * error.shape[0])
    assert int(over.sum()) <= allowed, (f"{what}: largest difference {worst:.3e} exceeds {MAX_TOL[dtype] * scale:.3e} in {int(over.sum())} rows "
                                        f"({allowed} allowed; first row over: {int(np.argmax(over))})")
    assert rms <= RMS_TOL[dtype] * scale, f"{what}: rms difference {rms:.3e} exceeds {RMS_TOL[dtype] * scale:.3e}"
