"""The Dibepel decoder as a `ModelSpec`.

config.json: "architecture": "Dibepel", "vocab", "width", "embedding": {"scale"}, "norm": {"eps"} and "layers", a
list whose entries give "type" (the mixer: "attention" or "attention_2"), "mixer" (its sizes and constants), "mlp"
({"kind": "dense", "ff"} or null) and optionally "weights_of": j, the layer whose tensors this one uses (with a cache
and state of its own).  Tensors: embed, l<i>.norm1, l<i>.mix.*, l<i>.mlp.{gate,up,down}, l<i>.rg1, l<i>.rg1.b,
l<i>.rg2, l<i>.rg2.b, final.norm, head.

Every layer is the parallel arrangement over a 32-bit residual stream: one RMS norm whose weight is stored as its
deviation from one, mixer and feed-forward both reading it, each result gated by sigmoid(W h + b).
  "attention"    two score maps per head (differential), no rotation, a sliding window that keeps the first tokens,
                 per-head RMS norm of the difference times (1 - diff)
  "attention_2"  short causal convolutions behind the q, k, v projections, a distance bias with slopes
                 2^(-8 (h + 1) / H), keys of the query's own chunk only, the heads' softmax weights mixed ("talk")
A layer with "weights_of" is a second run of that layer in the schedule: same parts, a cache of its own.
"""

from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path

from ..config.model_config import ConfigError
from ..config.registry import register_architecture
from ..parts.spec import LayerSpec, ModelSpec, PartSpec

MIXER_TYPES = ("attention", "attention_2")
DISTANCE_SLOPE_BASE = 8.0  # slope_h = 2^(-8 (h + 1) / H)
MAX_POSITIONS = 1 << 17  # no part of the design limits positions; what the engine sizes its block tables for


@dataclass(frozen=True)
class DibepelConfig:
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    layers: tuple  # of dictionaries as config.json holds them
    max_positions: int = MAX_POSITIONS

    @classmethod
    def from_dict(cls, d: dict) -> "DibepelConfig":
        missing = [k for k in ("vocab", "width", "layers") if k not in d]
        if missing:
            raise ConfigError(f"config.json lacks required keys {missing}")
        cfg = cls(vocab=int(d["vocab"]), width=int(d["width"]),
                  embedding_scale=float((d.get("embedding") or {}).get("scale", 1.0)),
                  norm_eps=float((d.get("norm") or {}).get("eps", 1e-5)),
                  layers=tuple(json.loads(json.dumps(entry)) for entry in d["layers"]),
                  max_positions=int(d.get("max_positions", MAX_POSITIONS)))
        cfg.validate()
        return cfg

    @classmethod
    def from_json(cls, path: str | Path) -> "DibepelConfig":
        path = Path(path)
        if path.is_dir():
            path = path / "config.json"
        return cls.from_dict(json.loads(path.read_text()))

    def owner(self, i: int) -> int:
        """The layer whose tensors layer `i` uses (itself, unless it names another with "weights_of")."""
        seen = set()
        while self.layers[i].get("weights_of") is not None:
            if i in seen:
                raise ConfigError(f"layer {i}: weights_of runs in a circle")
            seen.add(i)
            i = int(self.layers[i]["weights_of"])
        return i

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0 or not self.layers:
            raise ConfigError("vocab and width must be positive and there must be a layer")
        if self.norm_eps <= 0:
            raise ConfigError("norm.eps must be positive")
        for i, entry in enumerate(self.layers):
            if entry.get("type") not in MIXER_TYPES:
                raise ConfigError(f"layer {i}: type {entry.get('type')!r} is not one of {MIXER_TYPES}")
            src = entry.get("weights_of")
            if src is not None and not 0 <= int(src) < len(self.layers):
                raise ConfigError(f"layer {i}: weights_of={src} names no layer")
            m = entry.get("mixer") or {}
            for key in ("heads", "kv_heads", "dim", "vdim"):
                if int(m.get(key, 0)) <= 0:
                    raise ConfigError(f"layer {i}: mixer.{key} must be positive")
            if int(m["heads"]) % int(m["kv_heads"]):
                raise ConfigError(f"layer {i}: heads is not a multiple of kv_heads")
            mlp = entry.get("mlp")
            if mlp is not None and (mlp.get("kind", "dense") != "dense" or int(mlp.get("ff", 0)) <= 0):
                raise ConfigError(f"layer {i}: mlp must be null or {{'kind': 'dense', 'ff': > 0}}")
            self.owner(i)

    def to_dict(self) -> dict:
        return {"architecture": "Dibepel", "vocab": self.vocab, "width": self.width,
                "embedding": {"scale": self.embedding_scale}, "norm": {"eps": self.norm_eps},
                "layers": [dict(entry) for entry in self.layers]}


def _mixer_spec(kind: str, m: dict, width: int, eps: float) -> PartSpec:
    mask = m.get("mask") or {}
    size = mask.get("size")
    common = {"hidden": width, "num_heads": int(m["heads"]), "num_kv_heads": int(m["kv_heads"]),
              "head_dim": int(m["dim"]), "value_dim": int(m["vdim"]), "scale": m.get("scale"), "result": "float32"}
    if kind == "attention":
        diff = float(m.get("diff", 0.0))
        return PartSpec("composed_attention", dict(
            common, differential=True, diff=diff, window=None if size is None else int(size),
            keep_first=int(mask.get("keep_first") or 0), head_norm_eps=eps, head_norm_scale=1.0 - diff))
    return PartSpec("composed_attention", dict(
        common, conv_taps=int(m.get("conv") or 0), distance_slope_base=DISTANCE_SLOPE_BASE, talking_heads=True,
        chunk=None if size is None else int(size)))


def dibepel_spec(cfg: DibepelConfig) -> ModelSpec:
    w = cfg.width
    own = [i for i in range(len(cfg.layers)) if cfg.owner(i) == i]  # layers that hold tensors
    index = {layer: k for k, layer in enumerate(own)}
    layers, unused = [], []
    for i in own:
        entry, p = cfg.layers[i], f"l{i}."
        mlp = entry.get("mlp")
        gate = PartSpec("sigmoid_linear", {"hidden": w, "names": {"weight": "", "bias": ".b"}})
        parts = {
            "norm": PartSpec("rmsnorm32", {"hidden": w, "eps": cfg.norm_eps, "weight_offset": 1.0, "tensor": ""}),
            "mixer": _mixer_spec(entry["type"], entry["mixer"], w, cfg.norm_eps),
            "mixer_gate": gate,
            "feed_forward": PartSpec("none", {}) if mlp is None else PartSpec("swiglu", {
                "hidden": w, "intermediate": int(mlp["ff"]), "result": "float32",
                "names": {"gate": "gate", "up": "up", "down": "down"}}),
            "feed_forward_gate": PartSpec("none", {}) if mlp is None else gate}
        if mlp is None:  # (a gate without a branch has nothing to gate; its tensors may be there all the same)
            unused += [p + "rg2", p + "rg2.b"]
        layers.append(LayerSpec(block="parallel", parts=parts, weights={
            "norm": p + "norm1", "mixer": p + "mix.", "mixer_gate": p + "rg1", "feed_forward": p + "mlp.",
            "feed_forward_gate": p + "rg2"}))
    return ModelSpec(
        hidden_size=w, vocab_size=cfg.vocab, max_positions=cfg.max_positions,
        embedding=PartSpec("embedding", {"vocab": cfg.vocab, "hidden": w, "scale": cfg.embedding_scale,
                                         "stream": "float32", "tensor": ""}),
        layers=tuple(layers), schedule=tuple(index[cfg.owner(i)] for i in range(len(cfg.layers))),
        final_norm=PartSpec("rmsnorm32", {"hidden": w, "eps": cfg.norm_eps, "weight_offset": 1.0, "tensor": ""}),
        head=PartSpec("lm_head", {"vocab": cfg.vocab, "hidden": w, "tied": False, "tensor": ""}),
        weights={"embedding": "embed", "final_norm": "final.norm", "head": "head"},
        unused_tensors=tuple(unused))


DIBEPEL_PRESETS: dict[str, dict] = {}


def _preset(width: int, ff: int, heads: int, kv_heads: int, dim: int, layers: int, vocab: int, window: int,
            keep_first: int, chunk: int, conv: int = 4) -> dict:
    """A named size: every third layer is the windowed differential attention, the others the chunked one; the
    second half of the layers runs on the tensors of the first."""
    entries = []
    half = max(1, layers // 2)
    for i in range(layers):
        if i % 3 == 2:
            entry = {"type": "attention", "mixer": {
                "heads": heads // 2, "kv_heads": max(1, kv_heads // 2), "dim": dim, "vdim": 2 * dim, "diff": 0.5,
                "scale": dim ** -0.5, "mask": {"size": window, "keep_first": keep_first}}}
        else:
            entry = {"type": "attention_2", "mixer": {
                "heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "conv": conv, "scale": dim ** -0.5,
                "mask": {"size": chunk}}}
        entry["mlp"] = {"kind": "dense", "ff": ff}
        if i >= half and i - half < half and entries[i - half]["type"] == entry["type"]:
            entry["weights_of"] = i - half
        entries.append(entry)
    return {"architecture": "Dibepel", "vocab": vocab, "width": width, "embedding": {"scale": 2.0},
            "norm": {"eps": 1e-5}, "layers": entries}


DIBEPEL_PRESETS["dibepel-tiny"] = _preset(width=96, ff=160, heads=4, kv_heads=2, dim=16, layers=6, vocab=211,
                                          window=24, keep_first=5, chunk=32, conv=3)
# layer sizes of the 1.1B Llama shape (width 2048, 32 heads of 64, 4 key/value heads, feed-forward 5632)
DIBEPEL_PRESETS["dibepel-1b"] = _preset(width=2048, ff=5632, heads=32, kv_heads=4, dim=64, layers=22, vocab=32000,
                                        window=1024, keep_first=64, chunk=1024)

register_architecture("Dibepel", DibepelConfig, dibepel_spec, model_type="dibepel", presets=DIBEPEL_PRESETS)
