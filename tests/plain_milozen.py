"""The Milozen decoder, plainly: one function per mechanism, whole sequences, no cache, no kernels.

Everything runs on the CPU in the dtype the caller names (float64 for an oracle whose own rounding does not
matter).  `forward` takes a config.json dictionary and the checkpoint's tensors by name and returns the logits
of every position and, on request, the summed streams after every layer.

Notation: T tokens, i and j positions (from 0), H heads, dn the unrotated and dr the rotated size of a query or
key, dv of a value, r the latent's size.  Linear weights are [out, in].
"""

from __future__ import annotations

import math

import torch


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def layer_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """(x - mean) / sqrt(var + eps) * w with the variance as the mean squared deviation; no bias."""
    mu = x.mean(dim=-1, keepdim=True)
    var = ((x - mu) ** 2).mean(dim=-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w


def rotate_interleaved(x: torch.Tensor, positions: torch.Tensor, base: float, dims: int) -> torch.Tensor:
    """x [T, ..., D]: the first `dims` of the last axis are turned, (2i, 2i+1) being a pair with the angle
    p * base^(-2i/dims); the rest passes."""
    out = x.clone()
    for i in range(dims // 2):
        angle = positions.to(x.dtype) * (base ** (-2.0 * i / dims))
        shape = (-1,) + (1,) * (x.dim() - 2)
        c, s = torch.cos(angle).reshape(shape), torch.sin(angle).reshape(shape)
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * c - v * s
        out[..., 2 * i + 1] = v * c + u * s
    return out


def window_visible(t: int, size: int | None) -> torch.Tensor:
    """[T, T] bool: 0 <= i - j < size (size None: every j <= i)."""
    i = torch.arange(t)[:, None]
    j = torch.arange(t)[None, :]
    ok = j <= i
    if size is not None:
        ok = ok & (i - j < size)
    return ok


def latent_kv(h: torch.Tensor, w_dkv: torch.Tensor, w_norm: torch.Tensor, eps: float, r: int, base: float, dims: int):
    """h [T, W] -> (latent [T, r] normed, shared rotated key part [T, dr] after rotation)."""
    z = h @ w_dkv.T
    c = rms_unit(z[:, :r], eps) * w_norm
    positions = torch.arange(h.shape[0])
    return c, rotate_interleaved(z[:, r:], positions, base, dims)


def latent_attention(h: torch.Tensor, m: dict, w: dict, eps: float, shared=None):
    """The mixer on its input h [T, W].  `m`: the layer's mixer sizes; `w`: its tensors by local name; `shared`:
    (latent, rotated key part) of the layer named by kv_from, or None.  Returns (result [T, W], (latent, key part))."""
    t = h.shape[0]
    heads, dn, dr, dv, r = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
    rot = m.get("rot") or {}
    base, dims = float(rot.get("base", 10000.0)), int(rot.get("dims", dr))
    size = (m.get("mask") or {}).get("size")
    positions = torch.arange(t)
    cq = rms_unit(h @ w["dq"].T, eps) * w["dq.norm"]
    q = (cq @ w["uq"].T).reshape(t, heads, dn + dr)
    q_plain, q_rot = q[..., :dn], rotate_interleaved(q[..., dn:], positions, base, dims)
    if shared is None:
        shared = latent_kv(h, w["dkv"], w["dkv.norm"], eps, r, base, dims)
    c, k_rot = shared
    k_plain = (c @ w["uk"].T).reshape(t, heads, dn)
    v = (c @ w["uv"].T).reshape(t, heads, dv)
    visible = window_visible(t, None if size is None else int(size))
    out = torch.zeros(t, heads, dv, dtype=h.dtype)
    for a in range(heads):
        scores = (q_plain[:, a] @ k_plain[:, a].T + q_rot[:, a] @ k_rot.T) * float(m["scale"])
        p = torch.softmax(scores.masked_fill(~visible, float("-inf")), dim=-1)
        out[:, a] = p @ v[:, a]
    gated = out.reshape(t, heads * dv) * torch.sigmoid(h @ w["g"].T)
    return gated @ w["o"].T, shared


def dense_ff(h: torch.Tensor, w: dict) -> torch.Tensor:
    g = h @ w["gate"].T
    return (g * torch.sigmoid(g) * (h @ w["up"].T)) @ w["down"].T


def expert(x: torch.Tensor, w_gate, w_up, w_down, limit: float) -> torch.Tensor:
    g = torch.clamp(x @ w_gate.T, max=limit)
    u = torch.clamp(x @ w_up.T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w_down.T


def route(h: torch.Tensor, w_router: torch.Tensor, top: int):
    """(chosen experts [T, top], their weights [T, top]): sigmoid scores, the largest `top`, not renormalised."""
    s = torch.sigmoid(h @ w_router.T)
    weight, chosen = torch.topk(s, top, dim=-1)
    return chosen, weight


def moe_ff(h: torch.Tensor, mlp: dict, w: dict) -> torch.Tensor:
    top, limit = int(mlp["router"]["top"]), float(mlp["expert"]["limit"])
    chosen, weight = route(h, w["router"], top)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for k in range(top):
            e = int(chosen[t, k])
            out[t] += expert(weight[t, k] * h[t], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"], limit)
    return out


def feed_forward(h: torch.Tensor, mlp: dict, w: dict) -> torch.Tensor:
    return dense_ff(h, w) if mlp.get("kind", "dense") == "dense" else moe_ff(h, mlp, w)


def streams_read(xs: torch.Tensor, w_in: torch.Tensor) -> torch.Tensor:
    """xs [S, T, W] -> sum_s in[s] xs[s]."""
    return torch.einsum("s,stw->tw", w_in, xs)


def streams_write(xs: torch.Tensor, y: torch.Tensor, w_mix: torch.Tensor, w_out: torch.Tensor) -> torch.Tensor:
    """new[t] = sum_s mix[s, t] xs[s] + out[t] y, all streams at once from the old ones."""
    return torch.einsum("sk,stw->ktw", w_mix, xs) + w_out[:, None, None] * y[None]


def local(tensors: dict, prefix: str) -> dict:
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def forward(config: dict, tensors: dict, tokens, dtype=torch.float64, layers_out: list | None = None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence."""
    ts = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in tensors.items()}
    eps = float(config["norm"]["eps"])
    ids = torch.as_tensor(tokens, dtype=torch.long)
    x0 = ts["embed"][ids] * float((config.get("embedding") or {}).get("scale", 1.0))
    streams = config.get("streams")
    xs = x0[None].repeat(int(streams), 1, 1) if streams is not None else x0[None].clone()
    kept = {}
    for i, entry in enumerate(config["layers"]):
        p = f"l{i}."
        for q, name in ((1, "mixer"), (2, "mlp")):
            if q == 2 and entry.get("mlp") is None:
                continue
            if streams is not None:
                u = streams_read(xs, ts[f"{p}hc{q}.in"])
            else:
                u = xs[0]
            hn = layer_norm(u, ts[f"{p}norm{q}"], eps)
            if q == 1:
                src = entry["mixer"].get("kv_from")
                y, kept[i] = latent_attention(hn, entry["mixer"], local(ts, p + "mix."), eps,
                                              None if src is None else kept[int(src)])
            else:
                y = feed_forward(hn, entry["mlp"], local(ts, p + "mlp."))
            if streams is not None:
                xs = streams_write(xs, y, ts[f"{p}hc{q}.mix"], ts[f"{p}hc{q}.out"])
            else:
                xs = xs + y[None]
        if layers_out is not None:
            layers_out.append(xs.sum(dim=0).clone())
    x = xs.sum(dim=0)
    return layer_norm(x, ts["final.norm"], eps) @ ts["embed"].T


def greedy(config: dict, tensors: dict, prompt, n_new: int, dtype=torch.float64) -> list[int]:
    ids = list(prompt)
    for _ in range(n_new):
        ids.append(int(forward(config, tensors, ids, dtype)[-1].argmax()))
    return ids[len(prompt):]
