"""The residual stream re-entered through a projection."""

from __future__ import annotations

from ..hostcore import core
from .base import Part, TensorSpec


class StreamMix(Part):
    """h <- W [h ; h0], W [hidden, 2 hidden] applied to the stream beside the stream as the
    embedding left it (h first).  The model keeps h0 for the step when it holds this part; an
    execution-list entry with `mix` set runs it right before its layer.  The tensor is stored
    as ``<prefix>weight``."""

    graph_safe = True
    lowerable = True

    def __init__(self, hidden: int):
        self.hidden = int(hidden)
        self.weight = None

    def param_specs(self) -> dict:
        return {"weight": TensorSpec((self.hidden, 2 * self.hidden))}

    def bind(self, params, dtype, device) -> None:
        self.weight = params["weight"]

    def weight_bytes(self) -> int:
        return self.weight.numel() * self.weight.element_size()

    def lower_keep(self, program) -> None:
        program.append("keep_stream", b"")

    def lower(self, program) -> None:
        program.append("stream_mix", core.stream_mix_params(self.weight.data_ptr()))
