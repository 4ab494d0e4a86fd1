"""A plain, slow Vavelorn in float64 numpy, one function per mechanism, written from the design's
equations. It shares no code with the package: the tests hold the engine against it.

Notation: T tokens, D model width; a weight W is stored [out, in] and applied as x @ W.T. Every
mixer takes a whole sequence (position 0 first); ``delta_step`` takes one token and the state before
it, so that a sequence can also be walked token by token.

The design: x = embed[token]; per layer x += N1b(mixer(N1(x))), x += N2b(ff(N2(x))) (N: layer norm with
a weight and no bias), then a per-layer token input x += rms(P (gelu(G x) * e)) * w, where e is the
layer's slice of a second embedding row; mixers are chunked softmax attention with interleaved rotary
positions and a soft cap on the scores, latent attention (keys and values unfolded from one normed
latent per token, an output gate), and a gated delta rule with one decay per head.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional

import numpy as np


# ----- small pieces -------------------------------------------------------------------------
def rms(x: np.ndarray, eps: float) -> np.ndarray:
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def layer_norm(x: np.ndarray, weight: np.ndarray, eps: float) -> np.ndarray:
    centred = x - np.mean(x, axis=-1, keepdims=True)
    return centred / np.sqrt(np.mean(centred * centred, axis=-1, keepdims=True) + eps) * weight


def sigmoid(x: np.ndarray) -> np.ndarray:
    return 1.0 / (1.0 + np.exp(-x))


def softplus(x: np.ndarray) -> np.ndarray:
    return np.logaddexp(0.0, x)


def silu(x: np.ndarray) -> np.ndarray:
    return x * sigmoid(x)


def gelu_tanh(z: np.ndarray) -> np.ndarray:
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def softmax_rows(score: np.ndarray) -> np.ndarray:
    weight = np.exp(score - score.max())
    return weight / weight.sum()


def rotate_pairs(x: np.ndarray, positions: np.ndarray, dims: int, base: float) -> np.ndarray:
    """x [T, heads, dim]: channels 2i and 2i + 1 (i < dims / 2) of a head turn together by the angle
    position * base^(-2i / dims); channels from ``dims`` on stay."""
    out = x.copy()
    half = dims // 2
    if half == 0:
        return out
    freq = base ** (-2.0 * np.arange(half) / dims)
    angle = positions[:, None].astype(np.float64) * freq[None, :]
    c, s = np.cos(angle)[:, None, :], np.sin(angle)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


# ----- mixer: chunked attention ---------------------------------------------------------------
def chunked_heads(q: np.ndarray, k: np.ndarray, v: np.ndarray, scale: float, size: Optional[int], cap: Optional[float]) -> np.ndarray:
    """q [T, H, d], k [T, G, d], v [T, G, dv] of one sequence from position 0 -> [T, H, dv]: row i sees
    the keys j <= i of its own chunk (i // size == j // size; no size: all), scores capped softly."""
    T, H = q.shape[:2]
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    for head in range(H):
        g = head // (H // G)
        for i in range(T):
            lo = 0 if not size else (i // size) * size
            score = (k[lo:i + 1, g] @ q[i, head]) * scale
            if cap:
                score = cap * np.tanh(score / cap)
            out[i, head] = softmax_rows(score) @ v[lo:i + 1, g]
    return out


def chunked_attention(h: np.ndarray, w: Dict[str, np.ndarray], p: dict) -> np.ndarray:
    T = h.shape[0]
    H, G, d, dv = p["heads"], p["kv_heads"], p["dim"], p["vdim"]
    positions = np.arange(T)
    q = (h @ w["q"].T).reshape(T, H, d)
    k = (h @ w["k"].T).reshape(T, G, d)
    v = (h @ w["v"].T).reshape(T, G, dv)
    rot = p.get("rot") or {"dims": 0, "base": 1.0}
    q = rotate_pairs(q, positions, rot["dims"], rot["base"])
    k = rotate_pairs(k, positions, rot["dims"], rot["base"])
    out = chunked_heads(q, k, v, p["scale"], (p.get("mask") or {}).get("size"), p.get("softcap"))
    return out.reshape(T, H * dv) @ w["o"].T


# ----- mixer: latent attention ----------------------------------------------------------------
def latent_attention(h: np.ndarray, w: Dict[str, np.ndarray], p: dict, eps: float) -> np.ndarray:
    T = h.shape[0]
    H, d, dv = p["heads"], p["dim"], p["vdim"]
    cq = rms(h @ w["dq"].T, eps) * w["dq.norm"]
    q = (cq @ w["uq"].T).reshape(T, H, d)
    c = rms(h @ w["dkv"].T, eps) * w["dkv.norm"]
    k = (c @ w["uk"].T).reshape(T, H, d)
    v = (c @ w["uv"].T).reshape(T, H, dv)
    out = np.zeros((T, H, dv))
    for head in range(H):
        for i in range(T):
            score = (k[:i + 1, head] @ q[i, head]) * p["scale"]
            out[i, head] = softmax_rows(score) @ v[:i + 1, head]
    gated = out.reshape(T, H * dv) * sigmoid(h @ w["g"].T)
    return gated @ w["o"].T


# ----- mixer: gated delta rule ----------------------------------------------------------------
def causal_conv(x: np.ndarray, taps: np.ndarray, before: Optional[np.ndarray] = None) -> np.ndarray:
    """x [T, C], taps [C, L] (last column on the current token), ``before`` [L - 1, C] the inputs
    ahead of x (zeros at a sequence's start)."""
    T, C = x.shape
    L = taps.shape[1]
    before = np.zeros((L - 1, C)) if before is None else before
    padded = np.concatenate([before, x], axis=0)
    out = np.zeros((T, C))
    for t in range(T):
        out[t] = np.sum(padded[t:t + L] * taps.T, axis=0)
    return out


def delta_inputs(h: np.ndarray, w: Dict[str, np.ndarray], p: dict, before: Optional[Dict[str, np.ndarray]] = None):
    """What the recurrence reads: q, k [T, G, d] (unit vectors, q times d^-1/2), v [T, H, dv], beta
    [T, H], decay [T, H]; and the convolutions' inputs (for a caller that goes on later)."""
    T = h.shape[0]
    H, G, d, dv = p["heads"], p["kv_heads"], p["dim"], p["vdim"]
    raw = {name: h @ w[name].T for name in ("q", "k", "v")}
    conv = {name: silu(causal_conv(raw[name], w[name + ".conv"], None if before is None else before[name])) for name in raw}
    q = conv["q"].reshape(T, G, d)
    k = conv["k"].reshape(T, G, d)
    q = q / np.sqrt(np.sum(q * q, axis=-1, keepdims=True) + 1e-6) * d ** -0.5
    k = k / np.sqrt(np.sum(k * k, axis=-1, keepdims=True) + 1e-6)
    beta = sigmoid(h @ w["b"].T)
    decay = np.exp(-np.exp(w["A_log"]) * softplus(h @ w["a"].T + w["dt_bias"]))
    return q, k, conv["v"].reshape(T, H, dv), beta, decay, raw


def delta_step(S: np.ndarray, q: np.ndarray, k: np.ndarray, v: np.ndarray, beta: float, decay: float):
    """One token of one head: S [d, dv] -> (new S, read-out [dv])."""
    S = decay * S
    u = beta * (v - S.T @ k)
    S = S + np.outer(k, u)
    return S, S.T @ q


def gated_delta(h: np.ndarray, w: Dict[str, np.ndarray], p: dict, eps: float) -> np.ndarray:
    T = h.shape[0]
    H, G, d, dv = p["heads"], p["kv_heads"], p["dim"], p["vdim"]
    q, k, v, beta, decay, _ = delta_inputs(h, w, p)
    out = np.zeros((T, H, dv))
    for head in range(H):
        g = head // (H // G)
        S = np.zeros((d, dv))
        for t in range(T):
            S, out[t, head] = delta_step(S, q[t, g], k[t, g], v[t, head], beta[t, head], decay[t, head])
    normed = rms(out, eps) * w["norm"]
    gated = normed.reshape(T, H * dv) * silu(h @ w["g"].T)
    return gated @ w["o"].T


# ----- feed-forward, token input ----------------------------------------------------------------
def dense_ff(h: np.ndarray, w: Dict[str, np.ndarray]) -> np.ndarray:
    return (silu(h @ w["gate"].T) * (h @ w["up"].T)) @ w["down"].T


def token_input(x: np.ndarray, e: np.ndarray, w: Dict[str, np.ndarray], eps: float) -> np.ndarray:
    """What a layer adds from the tokens' own rows e [T, dim] of the second table."""
    y = (gelu_tanh(x @ w["gate"].T) * e) @ w["proj"].T
    return rms(y, eps) * w["norm"]


# ----- the model ----------------------------------------------------------------------------------
def sub(weights: Dict[str, np.ndarray], prefix: str) -> Dict[str, np.ndarray]:
    return {name[len(prefix):]: value for name, value in weights.items() if name.startswith(prefix)}


def mixer(kind: str, h: np.ndarray, w: Dict[str, np.ndarray], p: dict, eps: float) -> np.ndarray:
    if kind == "attention":
        return chunked_attention(h, w, p)
    if kind == "latent_attention":
        return latent_attention(h, w, p, eps)
    if kind == "delta":
        return gated_delta(h, w, p, eps)
    raise ValueError(kind)


def forward(config: dict, weights: Dict[str, np.ndarray], tokens, layers_out: Optional[List[np.ndarray]] = None) -> np.ndarray:
    """Logits [T, vocab] of a whole sequence; ``layers_out`` collects the residual stream after every layer."""
    weights = {name: np.asarray(value, dtype=np.float64) if value.dtype.kind == "f" else value for name, value in weights.items()}
    tokens = np.asarray(tokens, dtype=np.int64)
    eps = config["norm"]["eps"]
    x = weights["embed"][tokens]
    side = config.get("token_side")
    for index, layer in enumerate(config["layers"]):
        base = f"l{index}."
        h = layer_norm(x, weights[base + "norm1"], eps)
        x = x + layer_norm(mixer(layer["type"], h, sub(weights, base + "mix."), layer["mixer"], eps), weights[base + "norm1b"], eps)
        if layer.get("mlp") is not None:
            h = layer_norm(x, weights[base + "norm2"], eps)
            x = x + layer_norm(dense_ff(h, sub(weights, base + "mlp.")), weights[base + "norm2b"], eps)
        if side:
            dim = side["dim"]
            e = weights["side.embed"][tokens][:, index * dim:(index + 1) * dim]
            x = x + token_input(x, e, sub(weights, base + "side."), eps)
        if layers_out is not None:
            layers_out.append(x.copy())
    return layer_norm(x, weights["final.norm"], eps) @ weights["head"].T


def tensor_shapes(config: dict) -> Dict[str, tuple]:
    """Every tensor of a model of this configuration, by name."""
    D, V = config["width"], config["vocab"]
    side = config.get("token_side")
    shapes: Dict[str, tuple] = {"embed": (V, D), "final.norm": (D,), "head": (V, D)}
    if side:
        shapes["side.embed"] = (V, side["dim"] * len(config["layers"]))
    for index, layer in enumerate(config["layers"]):
        base, p = f"l{index}.", layer["mixer"]
        for name in ("norm1", "norm1b"):
            shapes[base + name] = (D,)
        m = base + "mix."
        if layer["type"] == "attention":
            H, G, d, dv = p["heads"], p["kv_heads"], p["dim"], p["vdim"]
            shapes.update({m + "q": (H * d, D), m + "k": (G * d, D), m + "v": (G * dv, D), m + "o": (D, H * dv)})
        elif layer["type"] == "latent_attention":
            H, d, dv, rq, rk = p["heads"], p["dim"], p["vdim"], p["q_rank"], p["kv_rank"]
            shapes.update({m + "dq": (rq, D), m + "dq.norm": (rq,), m + "uq": (H * d, rq), m + "dkv": (rk, D), m + "dkv.norm": (rk,),
                           m + "uk": (H * d, rk), m + "uv": (H * dv, rk), m + "g": (H * dv, D), m + "o": (D, H * dv)})
        else:
            H, G, d, dv, L = p["heads"], p["kv_heads"], p["dim"], p["vdim"], p["conv"]
            shapes.update({m + "q": (G * d, D), m + "q.conv": (G * d, L), m + "k": (G * d, D), m + "k.conv": (G * d, L),
                           m + "v": (H * dv, D), m + "v.conv": (H * dv, L), m + "b": (H, D), m + "A_log": (H,), m + "norm": (dv,),
                           m + "a": (H, D), m + "dt_bias": (H,), m + "g": (H * dv, D), m + "o": (D, H * dv)})
        if layer.get("mlp") is not None:
            ff = layer["mlp"]["ff"]
            shapes.update({base + "norm2": (D,), base + "norm2b": (D,), base + "mlp.gate": (ff, D), base + "mlp.up": (ff, D),
                           base + "mlp.down": (D, ff)})
        if side:
            shapes.update({base + "side.gate": (side["dim"], D), base + "side.proj": (D, side["dim"]), base + "side.norm": (D,)})
    return shapes


def greedy(config: dict, weights: Dict[str, np.ndarray], prompt, new: int) -> List[int]:
    """The most likely token, ``new`` times (ties to the lowest id); the whole sequence is run again for each."""
    tokens, out = list(prompt), []
    for _ in range(new):
        token = int(np.argmax(forward(config, weights, tokens)[-1]))
        out.append(token)
        tokens.append(token)
    return out


def random_weights(config: dict, seed: int) -> Dict[str, np.ndarray]:
    """Weights that make every part count: matrices 1 / sqrt(columns) wide, norm weights of visible
    spread, taps, decays and write strengths of visible size."""
    rng = np.random.default_rng(seed)
    out = {}
    for name, shape in tensor_shapes(config).items():
        leaf = name.split(".")[-1]
        if leaf in ("norm1", "norm2", "norm1b", "norm2b", "norm") or name == "final.norm":
            value = rng.uniform(0.6, 1.4, shape)
        elif leaf == "conv":
            value = rng.normal(0.0, 0.5, shape)
        elif leaf == "A_log":
            value = rng.uniform(-3.0, 0.5, shape)
        elif leaf == "dt_bias":
            value = rng.uniform(-3.0, 0.0, shape)
        elif name == "side.embed":
            value = rng.normal(0.0, 1.0, shape)
        else:
            value = rng.normal(0.0, 1.0 / math.sqrt(shape[-1]), shape)
        out[name] = value
    return out
