"""Dense gated feed-forward (reference models/qwen3.py:42-51)."""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import FeedForward, ParamSpec, PendingNorm, register_part
from .linear import Linear


class TokenGated:
    """A feed-forward's output that is still to be multiplied, token by token, by the sigmoid of one number per token:
    (rows [T, hidden], gate rows: a view [T, 1]). A feed-forward returns one only to a caller that asked for it
    (`defer_gate`), which multiplies where it adds the output to others (`ops.weighted_sum`)."""

    def __init__(self, rows, gate):
        self.rows, self.gate = rows, gate

    def value(self):
        return ops.weighted_sum([(self.rows, 1.0, None, self.gate)])


@register_part("feed_forward", "swiglu")
class SwiGLU(FeedForward):
    """down(silu(gate(x)) * up(x)); gate and up are one packed product with gate's rows first
    (reference layers/linear.py:29-45, layers/activation.py:5-7)."""

    takes_pending_norm = True      # x goes to the packed product and nowhere else

    def __init__(self, hidden_size: int, intermediate_size: int):
        super().__init__()
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.add_child("gate_up", Linear(hidden_size, 2 * intermediate_size,
                                         parts={"gate": intermediate_size, "up": intermediate_size}))
        self.add_child("down", Linear(intermediate_size, hidden_size))

    def forward(self, x):
        rows = x.x.shape[-2] if isinstance(x, PendingNorm) else x.shape[0]
        if ops.gated_linear_rows(rows, self.gate_up.weight):
            # few rows (or a few hundred over a small weight): the gating in the gate/up product's epilogue (every gate formed
            # once), a plain down product
            return self.down.forward(self.gate_up.forward(x, gated=True), allow_partials=True)
        gu = self.gate_up.forward(x)
        return ops.silu_mul_linear(gu, self.down.weight, allow_partials=True)


@register_part("feed_forward", "dense")
class ActivatedMLP(FeedForward):
    """down(act(up(x))) without a gate; `activation`: "relu2" (the square of relu), "silu", "tanh" or "gelu_tanh" (the
    tanh form of gelu). `token_gate`: the output is multiplied by sigmoid(w_gate . x), one number per token; the gate's
    row rides behind the up rows in one product (`token_gate_weight` [1, hidden], packed when the weights are bound)."""

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "relu2", token_gate: bool = False):
        super().__init__()
        if activation not in ops.ACTIVATIONS:
            raise ValueError(f"activation {activation!r} is not one of {sorted(ops.ACTIVATIONS)}")
        self.hidden_size, self.intermediate_size, self.activation = hidden_size, intermediate_size, activation
        self.token_gate = bool(token_gate)
        self.add_child("up", Linear(hidden_size, intermediate_size))
        self.add_child("down", Linear(intermediate_size, hidden_size))
        self._packed = None
        if self.token_gate:
            self.add_param("token_gate_weight", ParamSpec((1, hidden_size), init="matrix", dtype="compute"))

    def set_param(self, local, tensor):
        super().set_param(local, tensor)
        self._packed = None

    def finalize(self, device, dtype, max_positions):
        if self.token_gate:
            # the up rows, the gate's row, and zero rows up to a whole step of 8
            w, g = self.up.weight, self.token_gate_weight.to(self.up.weight.dtype)
            self._packed = torch.cat((w, g, w.new_zeros(-(w.shape[0] + 1) % 8, w.shape[1])), 0).contiguous()

    def forward(self, x, defer_gate: bool = False):
        if not self.token_gate:
            return self.down.forward(ops.activation(self.up.forward(x), self.activation), allow_partials=True)
        F = self.intermediate_size
        rows = ops.linear(x, self._packed)
        out = TokenGated(self.down.forward(ops.activation(rows[:, :F], self.activation), allow_partials=True), rows[:, F:F + 1])
        return out if defer_gate else out.value()


@register_part("feed_forward", "clamped_glu")
class ClampedGLU(FeedForward):
    """g = min(gate(x), limit), u = clamp(up(x), -limit, limit); down(g * sigmoid(alpha * g) * (u + 1)). Gate and up are
    one packed product with gate's rows first."""

    def __init__(self, hidden_size: int, intermediate_size: int, limit: float, alpha: float = 1.702):
        super().__init__()
        if not limit > 0:
            raise ValueError("the limit must be positive")
        self.hidden_size, self.intermediate_size = hidden_size, intermediate_size
        self.limit, self.alpha = float(limit), float(alpha)
        self.add_child("gate_up", Linear(hidden_size, 2 * intermediate_size,
                                         parts={"gate": intermediate_size, "up": intermediate_size}))
        self.add_child("down", Linear(intermediate_size, hidden_size))

    def forward(self, x):
        return self.down.forward(ops.glu_clamped(self.gate_up.forward(x), self.limit, self.alpha), allow_partials=True)
