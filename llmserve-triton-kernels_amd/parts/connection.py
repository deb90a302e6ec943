"""Connections between a sublayer and a residual stream.

"residual"  one stream: the sublayer reads it and its result is added to it.
"hyper"     `streams` parallel copies x_1 .. x_S (all equal to the embedding at the start).  The sublayer reads
            u = sum_s in[s] x_s, and its result y is written to all copies at once from the old ones:
            x_t <- sum_s mix[s, t] x_s + out[t] y.  Tensors: in [S], out [S], mix [S, S] indexed [from, to]
            (local names from `names`; defaults ".in", ".out", ".mix").
"none"      for a sublayer that a layer does not have.
The arithmetic belongs to the norm that reads the streams next (ops.streams_norm), in 32-bit.
"""

from __future__ import annotations

import torch

from .registry import Connection, register_connection
from .spec import ParamInfo


def _fill_read(shape, generator, device, options):
    """Coefficients of a mean of the streams, a little off."""
    return 1.0 / shape[0] + 0.1 * torch.randn(shape, generator=generator, dtype=torch.float32, device=device)


def _fill_write(shape, generator, device, options):
    return 1.0 + 0.2 * torch.randn(shape, generator=generator, dtype=torch.float32, device=device)


def _fill_mix(shape, generator, device, options):
    """Near the identity, so that the streams neither die out nor blow up over many layers."""
    return torch.eye(shape[0], dtype=torch.float32, device=device) + 0.15 * torch.randn(
        shape, generator=generator, dtype=torch.float32, device=device)


@register_connection("residual")
class ResidualConnection(Connection):
    graph_safe = True


@register_connection("none")
class NoConnection(Connection):
    graph_safe = True


@register_connection("hyper")
class HyperConnection(Connection):
    graph_safe = True

    def __init__(self, spec, ctx):
        super().__init__(spec, ctx)
        self.streams = int(spec["streams"])
        if not 1 <= self.streams <= 8:
            raise ValueError(f"1 to 8 streams, got {self.streams}")
        names = spec.get("names") or {}
        self.names = {k: names.get(k, "." + k) for k in ("in", "out", "mix")}

    def param_infos(self):
        s = self.streams
        return {self.names["in"]: ParamInfo((s,), _fill_read), self.names["out"]: ParamInfo((s,), _fill_write),
                self.names["mix"]: ParamInfo((s, s), _fill_mix)}

    def libraries(self, dtype_name):
        return ("stream32",)

    def load(self, tensors):
        self.read = tensors[self.names["in"]].float().contiguous()
        self.write = tensors[self.names["out"]].float().contiguous()
        self.mix = tensors[self.names["mix"]].float().contiguous()
