"""RMSNorm: weight * cast(x * rsqrt(mean(x^2) + eps)), statistics in 32-bit
(src/llmserve/model/llama.py:18-28).  Parameters: hidden, eps."""

from __future__ import annotations

import torch

from ..ops import library as ops
from .registry import GatedSum, PartialSums, Norm, register_norm
from .spec import ParamInfo


@register_norm("rmsnorm")
class RMSNorm(Norm):
    graph_safe = True

    def __init__(self, spec, ctx):
        super().__init__(spec, ctx)
        self.hidden = int(spec["hidden"])
        self.eps = float(spec["eps"])
        self.weight: torch.Tensor | None = None

    def param_infos(self):
        return {"weight": ParamInfo((self.hidden,), "norm")}

    def load(self, tensors):
        self.weight = tensors["weight"].contiguous()

    def rms_params(self):
        """(weight, eps): what a kernel that norms its rows on the way in needs."""
        return self.weight, self.eps

    def forward(self, x):
        return ops.rmsnorm(torch.empty_like(x), x, self.weight, self.eps)

    def add_norm(self, residual, delta):
        if delta is None:
            return self.forward(residual)
        if isinstance(delta, PartialSums):  # the kernel adds the partial sums up itself
            delta = delta.parts
        return ops.rmsnorm(torch.empty_like(residual), residual, self.weight, self.eps, delta=delta,
                           resid_out=residual)

    def norm_rows(self, x, delta, rows):
        out = torch.empty((rows.numel(), self.hidden), dtype=x.dtype, device=x.device)
        if isinstance(delta, PartialSums):
            delta = delta.parts
        return ops.rmsnorm(out, x, self.weight, self.eps, delta=delta, rows=rows)


@register_norm("rmsnorm32")
class RMSNorm32(Norm):
    """RMSNorm of a residual stream that is kept in 32-bit: x / sqrt(mean(x^2) + eps) * (offset + w), everything in
    32-bit, rounded once to the model's dtype.  Parameters: hidden, eps, weight_offset (1.0 for a weight that is
    stored as its deviation from one; default 0.0), tensor (the weight's local name; default "weight").  It offers
    no `rms_params`: the products that norm their rows on the way in round where this norm does not."""

    graph_safe = True
    closes_gated_sums = True  # `add_norm` and `norm_rows` take a `GatedSum` in the place of delta

    def __init__(self, spec, ctx):
        super().__init__(spec, ctx)
        self.hidden = int(spec["hidden"])
        self.eps = float(spec["eps"])
        self.offset = float(spec.get("weight_offset", 0.0))
        self.tensor = spec.get("tensor", "weight")
        self.weight: torch.Tensor | None = None

    def param_infos(self):
        return {self.tensor: ParamInfo((self.hidden,), "around_zero" if self.offset else "norm")}

    def libraries(self, dtype_name):
        return ("stream32",)

    def load(self, tensors):
        self.weight = tensors[self.tensor].float().contiguous()

    def forward(self, x):
        out = torch.empty(x.shape, dtype=self.ctx.dtype, device=x.device)
        return ops.rmsnorm32(out, self._stream(x), self.weight, self.eps, self.offset)

    def add_norm(self, residual, delta):
        """`delta`: None, or the open gated sum of the layer before (closed here, in the norm's own kernel)."""
        if delta is None:
            return self.forward(residual)
        if not isinstance(delta, GatedSum) or residual.dtype != torch.float32:
            raise ValueError("a 32-bit residual stream takes an open gated sum or nothing")
        out = torch.empty(residual.shape, dtype=self.ctx.dtype, device=residual.device)
        return ops.gated_add_norm(out, residual, delta.branches, delta.gate_products, self.weight, self.eps, self.offset)

    def norm_rows(self, x, delta, rows):
        if delta is not None:  # (few rows are wanted, but every row's sum is closed: the stream is the caller's)
            if not isinstance(delta, GatedSum) or x.dtype != torch.float32:
                raise ValueError("a 32-bit residual stream takes an open gated sum or nothing")
            ops.gated_add(x, delta.branches, delta.gate_products)
        out = torch.empty((rows.numel(), self.hidden), dtype=self.ctx.dtype, device=x.device)
        return ops.rmsnorm32(out, self._stream(x), self.weight, self.eps, self.offset, rows=rows)

    @staticmethod
    def _stream(x):
        return x if x.dtype == torch.float32 else x.float()
