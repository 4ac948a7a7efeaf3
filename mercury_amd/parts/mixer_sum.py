"""Mixers side by side."""

from __future__ import annotations

from ..hostcore import core
from ..kernels import ops
from .base import Mixer, TensorSpec
from .block import _Recorder
from .lowering import OneOp


class NormedMixerSum(Mixer):
    """Two mixers read the same input; each one's output is RMS-normed over the model width
    with a plain weight of its own (``<name>.weight``, eps inside the root), and the mixer's
    output is `mult` times their sum:  mult * (norm_a(a(x)) + norm_b(b(x))).

    At most one of the two keeps a paged cache and at most one a per-request state: they
    become this mixer's.  `names` gives the stored sub-prefix of each mixer and the names of
    the two norms: ``{"a": "left.", "b": "right.", "norm_a": "left.out", "norm_b": "right.out"}``.
    """

    lowers_state = True

    def __init__(self, hidden: int, a: Mixer, b: Mixer, names: dict, eps: float = 1e-6,
                 mult: float = 0.5):
        self.hidden = int(hidden)
        self.a, self.b = a, b
        self.eps, self.mult = float(eps), float(mult)
        self.names = dict(names)
        if sum(m.cache_spec() is not None for m in (a, b)) > 1:
            raise ValueError("at most one of two mixers side by side keeps a paged cache")
        if sum(m.state_spec() is not None for m in (a, b)) > 1:
            raise ValueError("at most one of two mixers side by side keeps per-request state")
        self.w_a = self.w_b = None
        self._alone: dict = {}

    def _children(self):
        return [("a", self.a), ("b", self.b)]

    @property
    def graph_safe(self) -> bool:
        return all(m.graph_safe for _, m in self._children())

    @property
    def lowerable(self) -> bool:
        return all(m.can_lower() for _, m in self._children()) and all(
            m.state_spec() is None or getattr(m, "lowers_state", False) for _, m in self._children())

    def cache_spec(self):
        return self.a.cache_spec() or self.b.cache_spec()

    def state_spec(self):
        return self.a.state_spec() or self.b.state_spec()

    def prepare(self, max_positions: int, device) -> None:
        self.a.prepare(max_positions, device)
        self.b.prepare(max_positions, device)

    def param_specs(self) -> dict:
        specs = {}
        for key, part in self._children():
            for name, spec in part.param_specs().items():
                specs[self.names[key] + name] = spec
            specs[self.names["norm_" + key] + ".weight"] = TensorSpec(
                (self.hidden,), role="vector", init="one_plus_normal")
        return specs

    def bind(self, params, dtype, device) -> None:
        for key, part in self._children():
            prefix = self.names[key]
            norm_name = self.names["norm_" + key] + ".weight"
            part.bind({n[len(prefix):]: t for n, t in params.items()
                       if n.startswith(prefix) and n != norm_name}, dtype, device)
        self.w_a = params[self.names["norm_a"] + ".weight"].float().contiguous()
        self.w_b = params[self.names["norm_b"] + ".weight"].float().contiguous()
        self._alone.clear()

    def weight_bytes(self) -> int:
        return (self.a.weight_bytes() + self.b.weight_bytes()
                + sum(t.numel() * t.element_size() for t in (self.w_a, self.w_b)))

    def lower(self, program, cache=None, state=None) -> None:
        subs = []
        for (key, mixer), weight in zip(self._children(), (self.w_a, self.w_b)):
            sub = _Recorder()
            mine_cache = cache if mixer.cache_spec() is not None else None
            if mixer.state_spec() is not None:
                mixer.lower(sub, mine_cache, state)
            else:
                mixer.lower(sub, mine_cache)
            if len(sub.ops) != 1:
                raise ValueError("a mixer beside another lowers itself to one operation")
            subs.append((sub.ops[0][0], sub.ops[0][1], weight.data_ptr()))
        program.append("normed_sum", core.normed_sum_params(self.mult, self.eps, ops.F32, subs))

    def forward(self, x, step, cache, state, accum):
        if not self.lowerable:
            raise NotImplementedError("mixers side by side run as operations of the host core")
        key = (None if cache is None else cache.k.data_ptr(),
               None if state is None else state.data_ptr())
        alone = self._alone.get(key)
        if alone is None:
            alone = self._alone[key] = OneOp(x.dtype, self.hidden, 0,
                                             lambda program: self.lower(program, cache, state))
        _logits, _x, pending = alone.run(step, accum, x=x)
        return pending
