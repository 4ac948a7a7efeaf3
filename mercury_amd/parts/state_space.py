"""A state-space mixer with per-request recurrent state."""

from __future__ import annotations

import torch

from ..hostcore import core
from ..kernels import ops
from .base import Mixer, StateSpec, TensorSpec
from .lowering import OneOp

DEFAULT_NAMES = {"in": "in_proj", "conv": "conv1d", "dt_bias": "dt_bias", "a_log": "A_log",
                 "d": "D", "norm": "norm", "out": "out_proj"}


class StateSpaceMixer(Mixer):
    """The Mamba-2 make of a state-space mixer.

    One projection of the input gives [z | x | B | C | dt] (inner = heads * vdim columns of z
    and of x, groups * state of B and of C, one dt per head).  x, B and C together pass a
    causal convolution per channel over `taps` tokens (weights [channels, taps], the last
    column meeting the current token, zeros before the sequence, a bias) and SiLU.  Per head h,
    which reads group h // (heads / groups):

        dt_t = softplus(dt_t + dt_bias_h)
        S_t  = exp(-exp(A_log_h) dt_t) S_(t-1) + dt_t B_t x_t^T        (S is state x vdim)
        y_t  = S_t^T C_t + D_h x_t

    y times silu(z) is RMS-normed in `norm_groups` equal parts (plain weight) and projected
    back.  Everything between the in-projection and the out-projection is float32.  The state
    a request carries from step to step is the recurrence's S per head and the convolution's
    last taps - 1 inputs, one float32 row per request slot (zeroed when a request takes it).
    """

    graph_safe = True
    lowerable = True
    lowers_state = True

    def __init__(self, hidden: int, heads: int, vdim: int, state: int, groups: int, conv: int,
                 norm_groups: int = 1, eps: float = 1e-6, names: dict | None = None):
        self.hidden, self.heads, self.vdim = int(hidden), int(heads), int(vdim)
        self.state_size, self.groups, self.taps = int(state), int(groups), int(conv)
        self.norm_groups, self.eps = int(norm_groups), float(eps)
        if min(self.hidden, self.heads, self.vdim, self.state_size, self.groups, self.taps,
               self.norm_groups) <= 0:
            raise ValueError("a state-space mixer's sizes are positive")
        if self.heads % self.groups:
            raise ValueError(f"{self.heads} heads are not a multiple of {self.groups} groups")
        if self.inner % self.norm_groups:
            raise ValueError(f"{self.inner} inner columns do not split into {self.norm_groups} parts")
        self.names = {**DEFAULT_NAMES, **(names or {})}
        self.w_in = self.w_out = self.vectors = None
        self._offsets: dict = {}
        self._alone: dict = {}

    @property
    def inner(self) -> int:
        return self.heads * self.vdim

    @property
    def channels(self) -> int:
        return self.inner + 2 * self.groups * self.state_size

    @property
    def in_width(self) -> int:
        return 2 * self.inner + 2 * self.groups * self.state_size + self.heads

    def carried_floats(self) -> int:
        return (self.taps - 1) * self.channels

    def recurrent_floats(self) -> int:
        """Floats of recurrent state per request, as the recurrence kernel lays it out (what
        ``core.ssm_state_floats`` answers once the kernel library is loaded): per head, blocks of
        8 columns in whole groups of four, a lane of 64 holding ceil(state / 8) entries rounded
        up to a power of two, at least 4."""
        if self.state_size > 256:
            raise ValueError("the recurrence kernel holds states of up to 256 rows")
        entries = 4
        while entries < -(-self.state_size // 8):
            entries *= 2
        return self.heads * (-(-self.vdim // 32) * 4) * entries * 64

    def state_spec(self) -> StateSpec:
        return StateSpec((self.carried_floats() + self.recurrent_floats(),), torch.float32)

    def param_specs(self) -> dict:
        n = self.names
        return {
            f"{n['in']}.weight": TensorSpec((self.in_width, self.hidden)),
            f"{n['conv']}.weight": TensorSpec((self.channels, self.taps), role="vector"),
            f"{n['conv']}.bias": TensorSpec((self.channels,), role="vector"),
            f"{n['dt_bias']}": TensorSpec((self.heads,), role="vector"),
            f"{n['a_log']}": TensorSpec((self.heads,), role="vector"),
            f"{n['d']}": TensorSpec((self.heads,), role="vector", init="one_plus_normal"),
            f"{n['norm']}.weight": TensorSpec((self.inner,), role="vector", init="one_plus_normal"),
            f"{n['out']}.weight": TensorSpec((self.hidden, self.inner)),
        }

    def bind(self, params, dtype, device) -> None:
        n = self.names
        self.w_in = params[f"{n['in']}.weight"]
        self.w_out = params[f"{n['out']}.weight"]
        # the small tensors in one float32 buffer: one dtype code for all of them
        order = [("conv_w", f"{n['conv']}.weight"), ("conv_b", f"{n['conv']}.bias"),
                 ("dt_bias", n["dt_bias"]), ("a_log", n["a_log"]), ("d_skip", n["d"]),
                 ("norm", f"{n['norm']}.weight")]
        flat, self._offsets, at = [], {}, 0
        for key, name in order:
            t = params[name].float().reshape(-1)
            self._offsets[key] = at
            flat.append(t)
            at += (t.numel() + 3) // 4 * 4       # every tensor starts 16-byte aligned
            if at > sum(x.numel() for x in flat):
                flat.append(torch.zeros(at - sum(x.numel() for x in flat), device=t.device))
        self.vectors = torch.cat(flat).contiguous()
        self._alone.clear()

    def weight_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in (self.w_in, self.w_out, self.vectors))

    def lower(self, program, cache=None, state=None) -> None:
        if state is None:
            raise ValueError("a state-space mixer runs over a state tensor")
        if state.dtype != torch.float32 or state.dim() != 2:
            raise ValueError("the state is float32 [slots, floats]")
        at = lambda key: self.vectors.data_ptr() + 4 * self._offsets[key]
        program.append("state_space", core.state_space_params(
            w_in=self.w_in.data_ptr(), conv_w=at("conv_w"), conv_b=at("conv_b"),
            dt_bias=at("dt_bias"), a_log=at("a_log"), d_skip=at("d_skip"), norm=at("norm"),
            vector_dtype=ops.F32, w_out=self.w_out.data_ptr(), heads=self.heads, vdim=self.vdim,
            state_size=self.state_size, groups=self.groups, taps=self.taps,
            norm_groups=self.norm_groups, eps=self.eps, state=state.data_ptr(),
            slot_floats=state.shape[1]))

    def forward(self, x, step, cache, state, accum):
        alone = self._alone.get(state.data_ptr())
        if alone is None:
            alone = self._alone[state.data_ptr()] = OneOp(
                x.dtype, self.hidden, 0, lambda program: self.lower(program, None, state))
        _logits, _x, pending = alone.run(step, accum, x=x)
        return pending
