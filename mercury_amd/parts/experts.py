"""A feed-forward of routed experts."""

from __future__ import annotations

import torch

from ..hostcore import core
from .base import FeedForward, TensorSpec
from .feedforward import ACTIVATION_CODES
from .lowering import OneOp

DEFAULT_NAMES = {"router": "router", "expert": "e{}.", "gate": "gate", "up": "up", "down": "down"}


class RoutedExperts(FeedForward):
    """`experts` small gated feed-forwards without biases, of which each token uses `top`.

        s = softmax(W_router x)                 (float32, over all experts)
        E = the `top` experts of largest s      (ties: the lower index)
        w_e = scale * s_e  (s_e / sum_{E} s first, when `renormalize`)
        y = sum_{e in E} w_e * W_down[e] act(W_gate[e] x, W_up[e] x)

    `activation` and its constants are those of :class:`GatedMLP`.  A token's sum runs over
    its experts in the order they were chosen, whatever else is in the batch.
    """

    graph_safe = True
    lowerable = True

    def __init__(self, hidden: int, experts: int, top: int, intermediate: int,
                 scale: float = 1.0, renormalize: bool = False, activation: str = "silu",
                 limit: float = 0.0, alpha: float = 1.0, beta: float = 0.0,
                 names: dict | None = None):
        if activation not in ACTIVATION_CODES:
            raise ValueError(f"activation {activation!r} is not implemented; known: {sorted(ACTIVATION_CODES)}")
        self.hidden, self.experts, self.top = int(hidden), int(experts), int(top)
        self.intermediate = int(intermediate)
        if not 0 < self.top <= self.experts:
            raise ValueError(f"top {self.top} of {self.experts} experts")
        self.scale, self.renormalize = float(scale), bool(renormalize)
        self.activation = activation
        self.limit, self.alpha, self.beta = float(limit), float(alpha), float(beta)
        self.names = {**DEFAULT_NAMES, **(names or {})}
        self.w_router = self.w_gate_up = self.w_down = None
        self._alone = None

    def _expert(self, e: int, leaf: str) -> str:
        return f"{self.names['expert'].format(e)}{self.names[leaf]}.weight"

    def param_specs(self) -> dict:
        i, h = self.intermediate, self.hidden
        specs = {f"{self.names['router']}.weight": TensorSpec((self.experts, h))}
        for e in range(self.experts):
            specs[self._expert(e, "gate")] = TensorSpec((i, h))
            specs[self._expert(e, "up")] = TensorSpec((i, h))
            specs[self._expert(e, "down")] = TensorSpec((h, i))
        return specs

    def bind(self, params, dtype, device) -> None:
        self.w_router = params[f"{self.names['router']}.weight"]
        # [experts, gate rows | up rows, hidden] and [experts, hidden, intermediate]
        self.w_gate_up = torch.stack([
            torch.cat([params[self._expert(e, "gate")], params[self._expert(e, "up")]], dim=0)
            for e in range(self.experts)]).contiguous()
        self.w_down = torch.stack([params[self._expert(e, "down")]
                                   for e in range(self.experts)]).contiguous()
        self._alone = None

    def weight_bytes(self) -> int:
        """Bytes a step of one token reads: the router and `top` experts."""
        per_expert = 3 * self.intermediate * self.hidden * self.w_down.element_size()
        return self.w_router.numel() * self.w_router.element_size() + self.top * per_expert

    def lower(self, program) -> None:
        program.append("routed_experts", core.routed_experts_params(
            w_router=self.w_router.data_ptr(), w_gate_up=self.w_gate_up.data_ptr(),
            w_down=self.w_down.data_ptr(), experts=self.experts, top=self.top,
            ff=self.intermediate, scale=self.scale, renormalize=self.renormalize,
            act=ACTIVATION_CODES[self.activation], limit=self.limit, alpha=self.alpha,
            beta=self.beta))

    def forward(self, x, step, accum):
        if self._alone is None:
            self._alone = OneOp(x.dtype, self.hidden, 0, self.lower)
        _logits, _x, pending = self._alone.run(step, accum, x=x)
        return pending
