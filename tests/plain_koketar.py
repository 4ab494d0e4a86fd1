"""A plain, slow Koketar in float64 numpy, one function per mechanism, written from the
design's equations. It shares no code with the package: the tests hold the engine against it.

Notation: T tokens, D model width; a weight W is stored [out, in] and applied as x @ W.T.
Every function takes whole sequences (position 0 first) except ``delta_rule_step``, which takes
one token and the state before it, and ``delta_inputs`` / ``causal_conv``, which may be told what
came before.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional

import numpy as np


# ----- small pieces -------------------------------------------------------------------------
def rms(x: np.ndarray, eps: float) -> np.ndarray:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def sigmoid(x: np.ndarray) -> np.ndarray:
    return 1.0 / (1.0 + np.exp(-x))


def softplus(x: np.ndarray) -> np.ndarray:
    return np.logaddexp(0.0, x)


def silu(x: np.ndarray) -> np.ndarray:
    return x * sigmoid(x)


def output_norm(y: np.ndarray, weight: np.ndarray, eps: float) -> np.ndarray:
    """The norm a sublayer's output passes: weights are stored around zero."""
    return rms(y, eps) * (1.0 + weight)


def rotate(x: np.ndarray, positions: np.ndarray, dims: int, base: float, factor: float) -> np.ndarray:
    """x [T, heads, dim]: channel i < dims/2 of a head turns with channel i + dims/2 by the
    angle position * base^(-2i/dims) / factor; channels from ``dims`` on stay."""
    half = dims // 2
    out = x.copy()
    if half == 0:
        return out
    freq = base ** (-2.0 * np.arange(half) / dims) / factor
    angle = positions[:, None].astype(np.float64) * freq[None, :]          # [T, half]
    c, s = np.cos(angle)[:, None, :], np.sin(angle)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


# ----- the windowed softmax attention ("left") ------------------------------------------------
def window_attention(h: np.ndarray, w: Dict[str, np.ndarray], p: dict, eps: float,
                     positions: Optional[np.ndarray] = None) -> np.ndarray:
    T = h.shape[0]
    H, G, d, dv = p["heads"], p["kv_heads"], p["dim"], p["vdim"]
    positions = np.arange(T) if positions is None else positions
    q = (h @ w["q"].T).reshape(T, H, d)
    k = (h @ w["k"].T).reshape(T, G, d)
    v = (h @ w["v"].T).reshape(T, G, dv)
    q = rms(q, eps) * w["q.norm"]
    k = rms(k, eps) * w["k.norm"]
    rot = p["rot"]
    factor = float((rot.get("scaling") or {}).get("factor", 1.0))
    q = rotate(q, positions, rot["dims"], rot["base"], factor)
    k = rotate(k, positions, rot["dims"], rot["base"], factor)
    size = p["mask"]["size"]
    out = np.zeros((T, H, dv))
    for head in range(H):
        g = head // (H // G)
        for i in range(T):
            lo = max(0, i - size + 1)
            score = (k[lo:i + 1, g] @ q[i, head]) * p["scale"]
            weight = np.exp(score - score.max())
            weight /= weight.sum()
            out[i, head] = weight @ v[lo:i + 1, g]
    return out.reshape(T, H * dv) @ w["o"].T


# ----- the gated delta rule ("right") -----------------------------------------------------------
def causal_conv(x: np.ndarray, taps: np.ndarray, before: Optional[np.ndarray] = None) -> np.ndarray:
    """x [T, C], taps [C, L] (last column: the current token). ``before`` [L-1, C]: the inputs
    that came ahead of x (zeros at the start of a sequence)."""
    L = taps.shape[1]
    before = np.zeros((L - 1, x.shape[1])) if before is None else before
    padded = np.concatenate([before, x], axis=0)
    out = np.zeros_like(x)
    for j in range(L):
        out += padded[j:j + x.shape[0]] * taps[:, j][None, :]
    return out


def unit(x: np.ndarray) -> np.ndarray:
    return x / np.sqrt(np.sum(x * x, axis=-1, keepdims=True) + 1e-6)


def delta_rule_step(S: np.ndarray, q: np.ndarray, k: np.ndarray, v: np.ndarray, beta: float, g: np.ndarray):
    """One token of one head. S [dim, vdim]; g [dim] decays the rows of S. Returns (S, o)."""
    S = g[:, None] * S
    u = beta * (v - S.T @ k)
    S = S + np.outer(k, u)
    return S, S.T @ q


def delta_inputs(h: np.ndarray, w: Dict[str, np.ndarray], p: dict, conv_before: Optional[Dict[str, np.ndarray]] = None):
    """Everything the recurrence reads, for whole sequences: q, k [T, kv_heads, dim] (unit
    vectors, q scaled), v [T, heads, vdim], beta [T, heads], g [T, heads, dim]; and the raw
    projections (the convolution's inputs) for whoever carries them on."""
    T = h.shape[0]
    H, G, d, dv = p["heads"], p["kv_heads"], p["dim"], p["vdim"]
    raw = {n: h @ w[n].T for n in "qkv"}
    conv = {n: silu(causal_conv(raw[n], w[n + ".conv"], None if conv_before is None else conv_before[n])) for n in "qkv"}
    q = unit(conv["q"].reshape(T, G, d)) * d ** -0.5
    k = unit(conv["k"].reshape(T, G, d))
    v = conv["v"].reshape(T, H, dv)
    beta = sigmoid(h @ w["b"].T)
    a = (h @ w["a1"].T) @ w["a2"].T + w["dt_bias"]
    g = np.exp(-np.exp(w["A_log"])[None, :, None] * softplus(a.reshape(T, H, d)))
    return q, k, v, beta, g, raw


def delta_output(o: np.ndarray, h: np.ndarray, w: Dict[str, np.ndarray], p: dict, eps: float) -> np.ndarray:
    """o [T, heads, vdim] -> the mixer's output [T, D]."""
    T = o.shape[0]
    gate = sigmoid((h @ w["g1"].T) @ w["g2"].T).reshape(T, p["heads"], p["vdim"])
    y = rms(o, eps) * w["norm"] * gate
    return y.reshape(T, -1) @ w["o"].T


def gated_delta_rule(h: np.ndarray, w: Dict[str, np.ndarray], p: dict, eps: float) -> np.ndarray:
    T = h.shape[0]
    H, G, d, dv = p["heads"], p["kv_heads"], p["dim"], p["vdim"]
    q, k, v, beta, g, _ = delta_inputs(h, w, p)
    o = np.zeros((T, H, dv))
    for head in range(H):
        kv = head // (H // G)
        S = np.zeros((d, dv))
        for t in range(T):
            S, o[t, head] = delta_rule_step(S, q[t, kv], k[t, kv], v[t, head], beta[t, head], g[t, head])
    return delta_output(o, h, w, p, eps)


# ----- feed-forward, layers, the model ----------------------------------------------------------
def clamped_glu(h: np.ndarray, w: Dict[str, np.ndarray], limit: float) -> np.ndarray:
    gate = np.minimum(h @ w["gate"].T, limit)
    up = np.clip(h @ w["up"].T, -limit, limit)
    return (gate * sigmoid(1.702 * gate) * (up + 1.0)) @ w["down"].T


def _sub(weights: Dict[str, np.ndarray], prefix: str) -> Dict[str, np.ndarray]:
    return {name[len(prefix):]: value for name, value in weights.items() if name.startswith(prefix)}


def parallel_mixer(h, weights, layer: int, mixer: dict, eps: float):
    left = window_attention(h, _sub(weights, f"l{layer}.mix.left."), mixer["left"], eps)
    right = gated_delta_rule(h, _sub(weights, f"l{layer}.mix.right."), mixer["right"], eps)
    return mixer["left_scale"] * left + mixer["right_scale"] * right


def forward(config: dict, weights: Dict[str, np.ndarray], tokens, return_layers: bool = False):
    """Logits [T, vocab] of one whole sequence (and the residual stream after every layer)."""
    eps = config["norm"]["eps"]
    m = config["residual_mult"]
    x = weights["embed"][np.asarray(tokens)]
    after: List[np.ndarray] = []
    for index, layer in enumerate(config["layers"]):
        if layer["type"] != "parallel":
            raise ValueError(f"unknown layer type {layer['type']!r}")
        x = x + m * output_norm(parallel_mixer(x, weights, index, layer["mixer"], eps), weights[f"l{index}.norm1"], eps)
        if layer.get("mlp") is not None:
            y = clamped_glu(x, _sub(weights, f"l{index}.mlp."), layer["mlp"]["limit"])
            x = x + m * output_norm(y, weights[f"l{index}.norm2"], eps)
        after.append(x.copy())
    logits = output_norm(x, weights["final.norm"], eps) @ weights["embed"].T
    cap = config.get("logit_softcap")
    if cap:
        logits = cap * np.tanh(logits / cap)
    return (logits, np.stack(after)) if return_layers else logits


def greedy(config: dict, weights: Dict[str, np.ndarray], prompt, new_tokens: int) -> List[int]:
    tokens = list(prompt)
    for _ in range(new_tokens):
        tokens.append(int(np.argmax(forward(config, weights, tokens)[-1])))
    return tokens[len(prompt):]


# ----- random models for the tests ----------------------------------------------------------------
def tensor_shapes(config: dict) -> Dict[str, tuple]:
    D = config["width"]
    shapes = {"embed": (config["vocab"], D), "final.norm": (D,)}
    for i, layer in enumerate(config["layers"]):
        a, b = layer["mixer"]["left"], layer["mixer"]["right"]
        base = f"l{i}."
        shapes[base + "norm1"] = (D,)
        shapes.update({
            base + "mix.left.q": (a["heads"] * a["dim"], D), base + "mix.left.k": (a["kv_heads"] * a["dim"], D),
            base + "mix.left.v": (a["kv_heads"] * a["vdim"], D), base + "mix.left.q.norm": (a["dim"],),
            base + "mix.left.k.norm": (a["dim"],), base + "mix.left.o": (D, a["heads"] * a["vdim"]),
            base + "mix.right.q": (b["kv_heads"] * b["dim"], D), base + "mix.right.q.conv": (b["kv_heads"] * b["dim"], b["conv"]),
            base + "mix.right.k": (b["kv_heads"] * b["dim"], D), base + "mix.right.k.conv": (b["kv_heads"] * b["dim"], b["conv"]),
            base + "mix.right.v": (b["heads"] * b["vdim"], D), base + "mix.right.v.conv": (b["heads"] * b["vdim"], b["conv"]),
            base + "mix.right.b": (b["heads"], D), base + "mix.right.A_log": (b["heads"],), base + "mix.right.norm": (b["vdim"],),
            base + "mix.right.a1": (b["rank_a"], D), base + "mix.right.a2": (b["heads"] * b["dim"], b["rank_a"]),
            base + "mix.right.dt_bias": (b["heads"] * b["dim"],),
            base + "mix.right.g1": (b["rank_g"], D), base + "mix.right.g2": (b["heads"] * b["vdim"], b["rank_g"]),
            base + "mix.right.o": (D, b["heads"] * b["vdim"]),
        })
        if layer.get("mlp") is not None:
            ff = layer["mlp"]["ff"]
            shapes.update({base + "norm2": (D,), base + "mlp.gate": (ff, D), base + "mlp.up": (ff, D), base + "mlp.down": (D, ff)})
    return shapes


def random_weights(config: dict, seed: int) -> Dict[str, np.ndarray]:
    """Weights that make every part count: matrices 1/sqrt(columns) wide, norm weights around
    zero, taps and decays of visible size. ``rank_a`` / ``rank_g`` in a right mixer's sizes are
    the inner widths of its two low-rank maps (the tests' own key: a checkpoint shows them by
    its tensors' shapes)."""
    rng = np.random.default_rng(seed)
    out = {}
    for name, shape in tensor_shapes(config).items():
        leaf = name.split(".")[-1]
        if leaf in ("norm1", "norm2") or name == "final.norm":
            value = rng.uniform(-0.3, 0.3, shape)
        elif leaf == "norm":
            value = rng.uniform(0.7, 1.3, shape)
        elif leaf == "conv":
            value = rng.normal(0.0, 0.5, shape)
        elif leaf == "A_log":
            value = rng.uniform(-2.0, 0.5, shape)
        elif leaf == "dt_bias":
            value = rng.uniform(-3.0, 0.0, shape)
        elif name == "embed":
            # small beside what the layers add: a token's own embedding must not decide the logits of the
            # tied head (greedy generation would repeat the last token whatever the mixers do), and the
            # logits stay below a soft cap's flat part
            value = rng.normal(0.0, 0.2, shape)
        else:
            value = rng.normal(0.0, 1.0 / math.sqrt(shape[-1]), shape)
        out[name] = value
    return out
