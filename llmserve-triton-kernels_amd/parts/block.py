"""Arrangements of a layer's parts.

"parallel" has one norm that both branches read: with h = norm(x),
    x = x + g_mixer * mixer(h) + g_feed_forward * feed_forward(h)
where each g is the branch's gate (a part of the family "gate"; kind "none": no gate) and the residual
stream x is 32-bit whatever the model's dtype: the branches' results arrive unrounded and one kernel
applies the gates and sums.

"prenorm" is the reference's decoder layer (src/llmserve/model/llama.py:131-135):
    x = x + mixer(norm1(x));  x = x + feed_forward(norm2(x))
The hidden state travels as (x, delta) with the last sum still open, so each residual
sum is done, in 32-bit, by the norm kernel that needs its result.
"""

from __future__ import annotations

import torch

from ..ops import library as ops
from .linear import linear
from .registry import ADDED_IN_PLACE, Block, DeferredNorm, GatedSum, register_block


@register_block("prenorm")
class PreNormBlock(Block):
    def forward(self, x, delta, batch, cache):
        # x + delta, normed: by the norm's kernel or by the mixer's; what the mixer returns is added to the
        # residual rows by the next norm's kernel, or by the mixer's last kernel (ADDED_IN_PLACE)
        h = DeferredNorm(self.mixer_norm, x, delta, may_add_in_place=True)
        a = self.mixer.forward(h if self.mixer.accepts_deferred_norm else h.materialize(), batch, cache)
        if not h.resolved:
            raise RuntimeError(f"{type(self.mixer).__name__} took a deferred input and left it unresolved")
        h2 = DeferredNorm(self.feed_forward_norm, h.residual, None if a is ADDED_IN_PLACE else a, may_add_in_place=True)
        f = self.feed_forward.forward(h2 if self.feed_forward.accepts_deferred_norm else h2.materialize())
        if not h2.resolved:
            raise RuntimeError(f"{type(self.feed_forward).__name__} took a deferred input and left it unresolved")
        return h2.residual, None if f is ADDED_IN_PLACE else f


@register_block("parallel")
class ParallelBlock(Block):
    """One norm, two branches beside each other, each with a gate of its own; a 32-bit residual stream, summed in
    place.  The feed-forward may be of kind "none" (the layer has a mixer only)."""

    ROLES = {"mixer": "mixer", "feed_forward": "feed_forward", "norm": "norm", "mixer_gate": "gate",
             "feed_forward_gate": "gate"}

    def __init__(self, parts):
        super().__init__(parts)
        self._stacked = None  # the gates' weights (and the mixer's input projection) as one matrix, made at the first step
        self._mixer_columns = None

    def _stack(self):
        """One matrix for every product of h whose result stays 32-bit: the two gates, and the mixer's input
        projection where the mixer offers it (`input_weight`, taken back as `projected`).  The parts' own
        weights become views of it, so nothing is held twice."""
        gm, gf = self.mixer_gate, self.feed_forward_gate
        wm, wf = gm.weight, gf.weight
        if wm is None or wf is None:
            return False
        if self._stacked is None:
            pieces = [wm, wf]
            mixer_w = getattr(self.mixer, "input_weight", None)
            if mixer_w is not None and mixer_w.dtype == wm.dtype and mixer_w.shape[1] == wm.shape[1]:
                pieces.append(mixer_w)
            self._stacked = torch.cat(pieces, dim=0).contiguous()
            a, b = wm.shape[0], wm.shape[0] + wf.shape[0]
            gm.weight, gf.weight = self._stacked[:a], self._stacked[a:b]
            if len(pieces) == 3:
                self.mixer.input_weight = self._stacked[b:]
                self._mixer_columns = (b, self._stacked.shape[0])
        return True

    def _gate_products(self, h):
        """(products [N, columns] or None, column of the mixer's gate or None, column of the feed-forward's,
        the mixer's projected input or None)."""
        gm, gf = self.mixer_gate, self.feed_forward_gate
        if self._stack():  # one product for all
            out = linear(h, self._stacked, out_dtype=torch.float32)
            projected = None
            if self._mixer_columns is not None:
                projected = out[:, self._mixer_columns[0]: self._mixer_columns[1]]
            return out, 0, gm.weight.shape[0], projected
        zm, zf = gm.products(h), gf.products(h)
        if zm is not None and zf is not None:
            return torch.cat([zm, zf], dim=1), 0, zm.shape[1], None
        one = zm if zm is not None else zf
        return one, (0 if zm is not None else None), (0 if zf is not None else None), None

    def forward(self, x, delta, batch, cache):
        if x.dtype != torch.float32:
            raise ValueError("the parallel arrangement keeps a 32-bit residual stream")
        # (the layer before may have left its gated sum open: this layer's norm closes it in its own kernel)
        h = self.norm.add_norm(x, delta)
        z, col_m, col_f, projected = self._gate_products(h)
        a = self.mixer.forward(h, batch, cache) if projected is None else self.mixer.forward(h, batch, cache, projected=projected)
        f = self.feed_forward.forward(h)
        branches = []
        for y, col, gate in ((a, col_m, self.mixer_gate), (f, col_f, self.feed_forward_gate)):
            if y is not None:
                branches.append((y if y.dtype == torch.float32 else y.float(), col, gate.bias))
        if not branches:
            return x, None
        if getattr(self.norm, "closes_gated_sums", False):  # left open for the next norm (the next layer's, or the last)
            return x, GatedSum(branches, z)
        ops.gated_add(x, branches, z)
        return x, None
