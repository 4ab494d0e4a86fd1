"""Gated delta rule: a linear recurrence over a matrix state per head.

q = W_q h, k = W_k h (kv_heads heads of ``dim`` channels), v = W_v h (heads of ``vdim`` channels);
each passes a short causal convolution per channel over the sequence (``taps`` wide, the last tap on
the current token, zeros before the start) and silu; q and k are then made unit vectors per head
(sum of squares + 1e-6 under the root) and q is scaled by dim^-1/2. Per head, with beta =
sigmoid(W_b h) and a decay per key channel g = exp(-exp(A_log) * softplus(W_a2 W_a1 h + dt_bias)):

    S <- diag(g) S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q

(head i reads q/k head i // (heads / kv_heads)). o is divided by its root mean square per head, times
a weight of vdim shared by the heads, times sigmoid(W_g2 W_g1 h); out = W_o of the heads side by
side. The state S and everything that enters the recurrence besides the projections is float32.
A request keeps S (zero at the start) and the convolutions' last taps - 1 inputs.

Two parameters choose between forms of the decay and of the output gate. ``decay`` "channel_low_rank" (the
default) is the above; "head" is one decay for all key channels of a head, g = exp(-exp(A_log) *
softplus(W_a h + dt_bias)) with W_a [heads, hidden] and dt_bias [heads]. ``gate`` "low_rank_sigmoid" (the
default) is the above; "silu" multiplies by silu(W_g h) with W_g [heads vdim, hidden].
"""

from __future__ import annotations

from typing import Dict

import torch

from ..cache.needs import FixedState
from ..config.spec import ConfigError
from ..kernels import ops
from ..weights.loader import TensorDecl
from .base import Mixer, register_mixer
from .linear import Linear

_DEFAULT_NAMES = {"q": "q", "k": "k", "v": "v", "b": "b", "a": "a", "a1": "a1", "a2": "a2", "g": "g", "g1": "g1", "g2": "g2", "o": "o",
                  "q_conv": "q.conv", "k_conv": "k.conv", "v_conv": "v.conv", "A_log": "A_log", "dt_bias": "dt_bias",
                  "norm": "norm"}


@register_mixer("gated_delta_rule")
class GatedDeltaRule(Mixer):
    graph_safe = True

    def __init__(self, spec):
        super().__init__(spec)
        self.hidden = int(spec["hidden_size"])
        self.heads = int(spec["num_heads"])
        self.kv_heads = int(spec["num_kv_heads"])
        self.dim = int(spec["head_dim"])
        self.vdim = int(spec["v_head_dim"])
        self.taps_count = int(spec["conv_taps"])
        self.decay = str(spec.get("decay", "channel_low_rank"))
        self.gate = str(spec.get("gate", "low_rank_sigmoid"))
        if self.decay not in ("channel_low_rank", "head") or self.gate not in ("low_rank_sigmoid", "silu"):
            raise ConfigError(f"gated delta rule: unknown form of the decay '{self.decay}' or of the gate '{self.gate}'")
        self.rank_a = int(spec["decay_rank"]) if self.decay == "channel_low_rank" else 0
        self.rank_g = int(spec["gate_rank"]) if self.gate == "low_rank_sigmoid" else 0
        self.eps = float(spec["norm_eps"])
        self.names = {**_DEFAULT_NAMES, **dict(spec.get("names", {}))}
        if self.heads % self.kv_heads:
            raise ConfigError(f"{self.heads} heads are not a multiple of {self.kv_heads} q/k heads")
        if not 1 <= self.dim <= 256 or not 1 <= self.vdim <= 256:
            raise ConfigError(f"the recurrence's head sizes ({self.dim}, {self.vdim}) must lie in 1..256")
        if not 1 <= self.taps_count <= 17:
            raise ConfigError(f"a short convolution of {self.taps_count} taps (1..17)")
        self.channels = 2 * self.kv_heads * self.dim + self.heads * self.vdim

    def cache_need(self):
        need = {"state": FixedState((self.heads, self.vdim, self.dim), torch.float32)}
        if self.taps_count > 1:
            need["conv"] = FixedState((self.channels, self.taps_count - 1), torch.float32)
        return need

    def _name(self, which: str) -> str:
        return self.prefix + self.names[which]

    def mixing_flops(self, rows: int, keys_before: int = 0) -> int:
        """Flops of the recurrence itself: per token and head three passes over the state (decay and
        read with the key, write, read with the query), a multiply and an add each."""
        return 6 * self.heads * self.dim * self.vdim * rows

    def tensors(self) -> Dict[str, TensorDecl]:
        D, H, G, d, dv, L = self.hidden, self.heads, self.kv_heads, self.dim, self.vdim, self.taps_count
        declared = {
            self._name("q"): TensorDecl((G * d, D)), self._name("k"): TensorDecl((G * d, D)), self._name("v"): TensorDecl((H * dv, D)),
            self._name("q_conv"): TensorDecl((G * d, L), "vector", "conv"), self._name("k_conv"): TensorDecl((G * d, L), "vector", "conv"),
            self._name("v_conv"): TensorDecl((H * dv, L), "vector", "conv"),
            self._name("b"): TensorDecl((H, D)), self._name("A_log"): TensorDecl((H,), "vector", "bias"),
            self._name("norm"): TensorDecl((dv,), "vector", "norm"),
            self._name("o"): TensorDecl((D, H * dv)),
        }
        if self.decay == "head":
            declared[self._name("a")] = TensorDecl((H, D))
            declared[self._name("dt_bias")] = TensorDecl((H,), "vector", "bias")
        else:
            declared[self._name("a1")] = TensorDecl((self.rank_a, D))
            declared[self._name("a2")] = TensorDecl((H * d, self.rank_a))
            declared[self._name("dt_bias")] = TensorDecl((H * d,), "vector", "bias")
        if self.gate == "silu":
            declared[self._name("g")] = TensorDecl((H * dv, D))
        else:
            declared[self._name("g1")] = TensorDecl((self.rank_g, D))
            declared[self._name("g2")] = TensorDecl((H * dv, self.rank_g))
        return declared

    def bind(self, tensors, dtype, device) -> None:
        super().bind(tensors, dtype, device)
        t = {which: tensors[self._name(which)] for which in self.names if self._name(which) in self.tensors()}
        # One operand for what the recurrence reads of h in float32: q | k | v (the convolutions' inputs)
        # and the write strengths. The two low-rank maps share their two products: the inner halves
        # side by side (their activations leave in the activation dtype, as any product's input), and
        # the outer halves as one block-diagonal operand whose zeros add nothing, so that one product
        # gives the decays' arguments and the gates side by side.
        self.beta_col = self.channels
        # Maps that read h directly (a decay per head, a full-rank gate) join that operand: the decays'
        # arguments behind the write strengths, the gates behind them, all float32 sums of one product.
        direct = [t["q"], t["k"], t["v"], t["b"]]
        self.a_col = self.gate_col = None
        if self.decay == "head":
            self.a_col = sum(m.shape[0] for m in direct)
            direct.append(t["a"])
        if self.gate == "silu":
            self.gate_col = sum(m.shape[0] for m in direct)
            direct.append(t["g"])
        self.in_proj = Linear(torch.cat(direct, dim=0))
        inner = ([t["a1"]] if self.decay != "head" else []) + ([t["g1"]] if self.gate != "silu" else [])
        self.low = self.outer = None
        if inner:
            self.low = Linear(torch.cat(inner, dim=0))
            blocks = ([t["a2"]] if self.decay != "head" else []) + ([t["g2"]] if self.gate != "silu" else [])
            outer = torch.zeros((sum(b.shape[0] for b in blocks), sum(b.shape[1] for b in blocks)), dtype=blocks[0].dtype,
                                device=blocks[0].device)
            row = col = 0
            for b in blocks:
                outer[row:row + b.shape[0], col:col + b.shape[1]] = b
                row, col = row + b.shape[0], col + b.shape[1]
            self.outer = Linear(outer)
        self.out = Linear(t["o"])
        self.taps = torch.cat([t["q_conv"], t["k_conv"], t["v_conv"]], dim=0).contiguous()
        self.A_log, self.dt_bias, self.norm_weight = t["A_log"], t["dt_bias"], t["norm"]
        self._no_conv_state = None

    def _conv_state(self, cache):
        if "conv" in cache:
            return cache["conv"].state
        if self._no_conv_state is None or self._no_conv_state.shape[0] != cache["state"].state.shape[0]:
            self._no_conv_state = torch.zeros((cache["state"].state.shape[0], self.channels, 0), dtype=torch.float32, device=self.device)
        return self._no_conv_state

    def heads_output(self, h, ctx, cache) -> torch.Tensor:
        """The heads' normed and gated read-outs [rows, heads * vdim] in the activation dtype; the
        request's state moves on by the step's rows."""
        proj = self.in_proj.forward(h, out_dtype=torch.float32)
        both = self.outer.forward(self.low.forward(h), out_dtype=torch.float32) if self.outer is not None else None
        per_head = self.decay == "head"
        if per_head:
            a = proj[:, self.a_col:self.a_col + self.heads]
        else:
            a = both[:, :self.heads * self.dim]
        if self.gate == "silu":
            gate = proj[:, self.gate_col:self.gate_col + self.heads * self.vdim]
        else:
            gate = both[:, both.shape[1] - self.heads * self.vdim:]
        records = ops.delta_prepare(proj, self.beta_col, a, self.taps, self._conv_state(cache), self.A_log, self.dt_bias,
                                    ctx.row_seg, ctx.seg_row0, ctx.seg_slot, ctx.num_segments, self.heads, self.kv_heads,
                                    self.dim, self.vdim, decay_per_head=per_head)
        o = ops.gated_delta_rule(records, cache["state"].state, ctx.seg_row0, ctx.seg_slot, ctx.num_segments,
                                 self.heads, self.dim, self.vdim)
        return ops.gated_head_norm(o, gate, self.norm_weight, self.heads, self.vdim, self.eps, self.dtype,
                                   gate_silu=self.gate == "silu")

    def output(self, h, ctx, cache) -> torch.Tensor:
        return self.out.forward(self.heads_output(h, ctx, cache), out_dtype=torch.float32)

    def forward(self, h, residual, ctx, cache):
        return self.out.accumulate(self.heads_output(h, ctx, cache), residual, then=getattr(ctx, "upcoming_norm", None))
