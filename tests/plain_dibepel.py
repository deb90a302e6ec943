"""The Dibepel decoder, plainly: one function per mechanism, whole sequences, no cache, no kernels.

Everything is computed on the CPU in the dtype the caller names (float64 to have an oracle
whose own rounding does not matter).  `forward` takes a config.json dictionary and the
checkpoint's tensors by name and returns the logits of every position, and on request the
residual stream after every layer run.

Notation: t, i, j are positions (from 0), H query heads, G key/value heads, dk the size of a
query or key, dv of a value.  Linear weights are [out, in].
"""

from __future__ import annotations

import math

import torch


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x divided by its root mean square over the last axis, eps inside the root."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def norm_zero_centred(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """RMS norm whose stored weight is the deviation from one."""
    return rms_unit(x, eps) * (1.0 + w)


def kv_head_of(h: int, heads: int, kv_heads: int) -> int:
    return h // (heads // kv_heads)


def visible_window(t: int, size: int | None, keep_first: int) -> torch.Tensor:
    """[t, t] bool: j <= i and (i - j < size or j < keep_first); size None: every earlier key."""
    i = torch.arange(t)[:, None]
    j = torch.arange(t)[None, :]
    near = (i - j < size) if size is not None else torch.ones(t, t, dtype=torch.bool)
    return (j <= i) & (near | (j < keep_first))


def visible_chunk(t: int, size: int | None) -> torch.Tensor:
    """[t, t] bool: j <= i and both in the same chunk of `size` positions counted from 0."""
    i = torch.arange(t)[:, None]
    j = torch.arange(t)[None, :]
    same = (i // size == j // size) if size is not None else torch.ones(t, t, dtype=torch.bool)
    return (j <= i) & same


def masked_softmax(scores: torch.Tensor, visible: torch.Tensor) -> torch.Tensor:
    return torch.softmax(scores.masked_fill(~visible, float("-inf")), dim=-1)


def short_conv(u: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """u [t, C], w [C, taps]: y_t = sum_j w[:, j] * u_(t - taps + 1 + j), zeros before position 0."""
    t, taps = u.shape[0], w.shape[1]
    y = torch.zeros_like(u)
    for j in range(taps):
        back = taps - 1 - j
        if back < t:
            y[back:] += w[:, j] * u[: t - back]
    return y


def distance_slopes(heads: int) -> torch.Tensor:
    """slope_h = 2^(-8 (h + 1) / H)."""
    return torch.tensor([2.0 ** (-8.0 * (h + 1) / heads) for h in range(heads)], dtype=torch.float64)


def differential_heads(q, k, v, visible, scale: float, lam: float, diff: float, eps: float) -> torch.Tensor:
    """q [t, H, 2, dk], k [t, G, 2, dk], v [t, G, dv] -> [t, H, dv]: per head a_1 - lam a_2 over the same values,
    divided by its root mean square, times (1 - diff)."""
    t, H = q.shape[0], q.shape[1]
    G = k.shape[1]
    out = torch.zeros(t, H, v.shape[-1], dtype=q.dtype)
    for head in range(H):
        g = kv_head_of(head, H, G)
        a = [masked_softmax((q[:, head, which] @ k[:, g, which].T) * scale, visible) @ v[:, g] for which in range(2)]
        out[:, head] = rms_unit(a[0] - lam * a[1], eps) * (1.0 - diff)
    return out


def differential_attention(h: torch.Tensor, w: dict, p: str, m: dict, eps: float) -> torch.Tensor:
    """Two score maps per head over the same values; o = a1 - lambda a2, divided by its root mean square
    per head, times (1 - diff); then the output projection."""
    t = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    mask = m.get("mask") or {}
    q = (h @ w[p + "q"].T).view(t, H, 2, dk)
    k = (h @ w[p + "k"].T).view(t, G, 2, dk)
    v = (h @ w[p + "v"].T).view(t, G, dv)
    visible = visible_window(t, mask.get("size"), int(mask.get("keep_first") or 0))
    lam = (torch.exp((w[p + "lq1"] * w[p + "lk1"]).sum()) - torch.exp((w[p + "lq2"] * w[p + "lk2"]).sum())
           + m["diff"])
    out = differential_heads(q, k, v, visible, m["scale"], lam, m["diff"], eps)
    return out.reshape(t, H * dv) @ w[p + "o"].T


def talking_heads(q, k, v, visible, scale: float, slopes, talk) -> torch.Tensor:
    """q [t, H, dk], k [t, G, dk], v [t, G, dv] -> [t, H, dv]: slope_h * (i - j) taken off the scores (slopes None:
    nothing), softmax, the heads' weights mixed by `talk` (None: not mixed), each head on its own value head."""
    t, H = q.shape[0], q.shape[1]
    G = k.shape[1]
    distance = (torch.arange(t)[:, None] - torch.arange(t)[None, :]).to(q.dtype)
    weights = torch.zeros(H, t, t, dtype=q.dtype)
    for head in range(H):
        s = (q[:, head] @ k[:, kv_head_of(head, H, G)].T) * scale
        if slopes is not None:
            s = s - slopes[head] * distance
        weights[head] = masked_softmax(s, visible)
    if talk is not None:
        weights = torch.einsum("hg,gij->hij", talk, weights)
    out = torch.zeros(t, H, v.shape[-1], dtype=q.dtype)
    for head in range(H):
        out[:, head] = weights[head] @ v[:, kv_head_of(head, H, G)]
    return out


def talking_chunk_attention(h: torch.Tensor, w: dict, p: str, m: dict) -> torch.Tensor:
    """Short convolutions behind the projections, a bias slope_h * (i - j) taken off the scores, keys of
    the query's own chunk only, and the heads' softmax weights mixed by `talk` before they meet the values."""
    t = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    mask = m.get("mask") or {}

    def projected(name):
        u = h @ w[p + name].T
        return short_conv(u, w[p + name + ".conv"]) if (p + name + ".conv") in w else u

    q = projected("q").view(t, H, dk)
    k = projected("k").view(t, G, dk)
    v = projected("v").view(t, G, dv)
    out = talking_heads(q, k, v, visible_chunk(t, mask.get("size")), m["scale"], distance_slopes(H).to(h.dtype),
                        w[p + "talk"])
    return out.reshape(t, H * dv) @ w[p + "o"].T


def dense_feed_forward(h: torch.Tensor, w: dict, p: str) -> torch.Tensor:
    gate = h @ w[p + "gate"].T
    return ((gate * torch.sigmoid(gate)) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def branch_gate(h: torch.Tensor, w: dict, name: str) -> torch.Tensor:
    return torch.sigmoid(h @ w[name].T + w[name + ".b"])


MIXERS = {"attention": lambda h, w, p, m, eps: differential_attention(h, w, p, m, eps),
          "attention_2": lambda h, w, p, m, eps: talking_chunk_attention(h, w, p, m)}


def layer(x: torch.Tensor, w: dict, p: str, entry: dict, eps: float) -> torch.Tensor:
    """One norm; mixer and feed-forward both read it; each result goes through its gate into the sum."""
    h = norm_zero_centred(x, w[p + "norm1"], eps)
    total = branch_gate(h, w, p + "rg1") * MIXERS[entry["type"]](h, w, p + "mix.", entry["mixer"], eps)
    if entry.get("mlp"):
        total = total + branch_gate(h, w, p + "rg2") * dense_feed_forward(h, w, p + "mlp.")
    return x + total


def forward(config: dict, tensors: dict, ids: list[int], dtype=torch.float64, with_layers: bool = False):
    w = {k: v.to(dtype) for k, v in tensors.items()}
    eps = config["norm"]["eps"]
    x = w["embed"][torch.tensor(ids)] * config["embedding"]["scale"]
    after = []
    for i, entry in enumerate(config["layers"]):
        owner = i
        while config["layers"][owner].get("weights_of") is not None:
            owner = config["layers"][owner]["weights_of"]
        x = layer(x, w, f"l{owner}.", entry, eps)
        after.append(x)
    logits = norm_zero_centred(x, w["final.norm"], eps) @ w["head"].T
    return (logits, torch.stack(after)) if with_layers else logits


def lambda_of(w: dict, p: str, diff: float) -> float:
    return float(math.exp(float((w[p + "lq1"].double() * w[p + "lk1"].double()).sum()))
                 - math.exp(float((w[p + "lq2"].double() * w[p + "lk2"].double()).sum())) + diff)


def greedy(config: dict, tensors: dict, prompt: list[int], n: int, dtype=torch.float64) -> list[int]:
    """`n` tokens after `prompt`, each the argmax (lowest index wins) of a whole forward pass."""
    ids, out = list(prompt), []
    for _ in range(n):
        tok = int(forward(config, tensors, ids, dtype)[-1].argmax())
        out.append(tok)
        ids.append(tok)
    return out
