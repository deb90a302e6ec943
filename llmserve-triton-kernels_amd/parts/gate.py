"""Gates of a branch's result: g = sigmoid(W h + b), element by element, h being the branch's input.
Parameters: hidden, names (local names of "weight" and "bias"; defaults "weight" and "bias").
The product is formed in the model's dtype with 32-bit sums and left unrounded; the bias, the sigmoid and the
multiplication belong to the kernel that sums the residual stream (ops.gated_add)."""

from __future__ import annotations

import torch

from .linear import linear
from .registry import Gate, register_gate
from .spec import ParamInfo


@register_gate("none")
class NoGate(Gate):
    """The branch joins the stream as it is."""

    graph_safe = True


@register_gate("sigmoid_linear")
class SigmoidLinearGate(Gate):
    graph_safe = True

    def __init__(self, spec, ctx):
        super().__init__(spec, ctx)
        self.hidden = int(spec["hidden"])
        names = spec.get("names") or {}
        self.names = {k: names.get(k, k) for k in ("weight", "bias")}

    def param_infos(self):
        return {self.names["weight"]: ParamInfo((self.hidden, self.hidden)),
                self.names["bias"]: ParamInfo((self.hidden,), "around_zero")}

    def load(self, tensors):
        self.weight = tensors[self.names["weight"]].contiguous()
        self.bias = tensors[self.names["bias"]].float().contiguous()

    def products(self, h):
        return linear(h, self.weight, out_dtype=torch.float32)
