"""The Milozen decoder as a `ModelSpec`.

config.json: "architecture": "Milozen", "vocab", "width", "embedding": {"scale"}, "norm": {"eps"}, optionally
"streams" (the number of parallel copies of the residual stream), and "layers", a list whose entries give "type"
(the mixer: "latent_attention"), "mixer" (its sizes and constants: heads, dim, rot_dim, vdim, q_rank, kv_rank, scale,
mask {size}, rot {base, dims}, and optionally kv_from: j, the layer whose cache rows this one reads) and "mlp"
({"kind": "dense", "ff"}, {"kind": "moe", "expert": {ff, limit}, "router": {experts, top}} or null).
Tensors: embed, l<i>.norm1, l<i>.norm2, l<i>.mix.*, l<i>.mlp.*, l<i>.hc1.{in,out,mix}, l<i>.hc2.{in,out,mix},
final.norm.  The output head is the embedding table.

Every layer is the pre-norm arrangement over a 32-bit residual stream (layer norm with a weight and no bias); with
"streams" the sublayers read and write the copies through hyper-connections, without it the stream is one and the
sums are plain.  A layer with kv_from keeps no cache of its own: the cache of the layer it names is kept for the
widest window among its readers.
"""

from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path

from ..config.model_config import ConfigError
from ..config.registry import register_architecture
from ..parts.spec import LayerSpec, ModelSpec, PartSpec

MIXER_TYPES = ("latent_attention",)
MLP_KINDS = ("dense", "moe")
MAX_POSITIONS = 1 << 17  # no part of the design limits positions; what the engine sizes its block tables for


@dataclass(frozen=True)
class MilozenConfig:
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    streams: int | None
    layers: tuple  # of dictionaries as config.json holds them
    max_positions: int = MAX_POSITIONS

    @classmethod
    def from_dict(cls, d: dict) -> "MilozenConfig":
        missing = [k for k in ("vocab", "width", "layers") if k not in d]
        if missing:
            raise ConfigError(f"config.json lacks required keys {missing}")
        cfg = cls(vocab=int(d["vocab"]), width=int(d["width"]),
                  embedding_scale=float((d.get("embedding") or {}).get("scale", 1.0)),
                  norm_eps=float((d.get("norm") or {}).get("eps", 1e-5)),
                  streams=None if d.get("streams") is None else int(d["streams"]),
                  layers=tuple(json.loads(json.dumps(entry)) for entry in d["layers"]),
                  max_positions=int(d.get("max_positions", MAX_POSITIONS)))
        cfg.validate()
        return cfg

    @classmethod
    def from_json(cls, path: str | Path) -> "MilozenConfig":
        path = Path(path)
        if path.is_dir():
            path = path / "config.json"
        return cls.from_dict(json.loads(path.read_text()))

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0 or not self.layers:
            raise ConfigError("vocab and width must be positive and there must be a layer")
        if self.norm_eps <= 0:
            raise ConfigError("norm.eps must be positive")
        if self.streams is not None and not 1 <= self.streams <= 8:
            raise ConfigError("streams must be 1 to 8")
        for i, entry in enumerate(self.layers):
            if entry.get("type") not in MIXER_TYPES:
                raise ConfigError(f"layer {i}: type {entry.get('type')!r} is not one of {MIXER_TYPES}")
            m = entry.get("mixer") or {}
            for key in ("heads", "dim", "vdim", "q_rank", "kv_rank"):
                if int(m.get(key, 0)) <= 0:
                    raise ConfigError(f"layer {i}: mixer.{key} must be positive")
            if int(m.get("rot_dim", 0)) < 0 or "scale" not in m:
                raise ConfigError(f"layer {i}: mixer.rot_dim must not be negative and mixer.scale must be given")
            size = (m.get("mask") or {}).get("size")
            if size is not None and int(size) < 1:
                raise ConfigError(f"layer {i}: mask.size must be positive")
            src = m.get("kv_from")
            if src is not None:
                if not 0 <= int(src) < i:
                    raise ConfigError(f"layer {i}: kv_from={src} names no earlier layer")
                other = self.layers[int(src)]["mixer"]
                if other.get("kv_from") is not None:
                    raise ConfigError(f"layer {i}: kv_from={src} names a layer that keeps no cache of its own")
                for key in ("kv_rank", "rot_dim", "rot"):
                    if other.get(key) != m.get(key):
                        raise ConfigError(f"layer {i}: {key} differs from layer {src}, whose cache it reads")
            mlp = entry.get("mlp")
            if mlp is None:
                continue
            kind = mlp.get("kind", "dense")
            if kind not in MLP_KINDS:
                raise ConfigError(f"layer {i}: mlp.kind {kind!r} is not one of {MLP_KINDS}")
            if kind == "dense" and int(mlp.get("ff", 0)) <= 0:
                raise ConfigError(f"layer {i}: mlp.ff must be positive")
            if kind == "moe":
                expert, router = mlp.get("expert") or {}, mlp.get("router") or {}
                if int(expert.get("ff", 0)) <= 0 or "limit" not in expert:
                    raise ConfigError(f"layer {i}: mlp.expert needs ff > 0 and limit")
                if not 1 <= int(router.get("top", 0)) <= int(router.get("experts", 0)):
                    raise ConfigError(f"layer {i}: mlp.router needs 1 <= top <= experts")

    def to_dict(self) -> dict:
        d = {"architecture": "Milozen", "vocab": self.vocab, "width": self.width,
             "embedding": {"scale": self.embedding_scale}, "norm": {"eps": self.norm_eps},
             "layers": [dict(entry) for entry in self.layers]}
        if self.streams is not None:
            d["streams"] = self.streams
        return d

    def cache_window(self, i: int) -> int | None:
        """What the cache of layer `i` has to keep: the widest window among it and the layers that read its rows."""
        sizes = [(self.layers[j]["mixer"].get("mask") or {}).get("size") for j in range(len(self.layers))
                 if j == i or self.layers[j]["mixer"].get("kv_from") == i]
        return None if any(s is None for s in sizes) else max(int(s) for s in sizes)


def _mixer_spec(cfg: MilozenConfig, i: int) -> PartSpec:
    m = cfg.layers[i]["mixer"]
    rot = m.get("rot") or {}
    size = (m.get("mask") or {}).get("size")
    rot_dim = int(m.get("rot_dim", 0))
    src = m.get("kv_from")
    return PartSpec("latent_attention", {
        "hidden": cfg.width, "num_heads": int(m["heads"]), "head_dim_plain": int(m["dim"]), "head_dim_rotated": rot_dim,
        "value_dim": int(m["vdim"]), "q_rank": int(m["q_rank"]), "kv_rank": int(m["kv_rank"]), "scale": float(m["scale"]),
        "window": None if size is None else int(size),
        "cache_window": cfg.cache_window(i if src is None else int(src)),
        "rotary_base": float(rot.get("base", 10000.0)), "rotary_dims": int(rot.get("dims", rot_dim)),
        "eps": cfg.norm_eps, "own_latent": src is None, "output_gate": True,
        "num_kv_heads": 1, "head_dim": int(m["kv_rank"]) + rot_dim})


def _mlp_spec(cfg: MilozenConfig, mlp: dict | None) -> PartSpec:
    if mlp is None:
        return PartSpec("none", {})
    if mlp.get("kind", "dense") == "dense":
        return PartSpec("swiglu", {"hidden": cfg.width, "intermediate": int(mlp["ff"]), "result": "float32",
                                   "names": {"gate": "gate", "up": "up", "down": "down"}})
    return PartSpec("experts", {"hidden": cfg.width, "intermediate": int(mlp["expert"]["ff"]),
                                "experts": int(mlp["router"]["experts"]), "top": int(mlp["router"]["top"]),
                                "limit": float(mlp["expert"]["limit"])})


def milozen_spec(cfg: MilozenConfig) -> ModelSpec:
    w = cfg.width
    norm = PartSpec("layernorm32", {"hidden": w, "eps": cfg.norm_eps, "tensor": ""})
    connection = PartSpec("residual", {}) if cfg.streams is None else PartSpec("hyper", {"streams": cfg.streams})
    layers, unused = [], []
    for i, entry in enumerate(cfg.layers):
        p = f"l{i}."
        mlp = entry.get("mlp")
        absent = mlp is None
        parts = {"mixer": _mixer_spec(cfg, i), "mixer_norm": norm, "mixer_connection": connection,
                 "feed_forward": _mlp_spec(cfg, mlp), "feed_forward_norm": PartSpec("none", {}) if absent else norm,
                 "feed_forward_connection": PartSpec("none", {}) if absent else connection}
        if absent:  # (a checkpoint may hold the second sublayer's norm and connection all the same)
            unused += [p + "norm2"] + [p + "hc2" + t for t in (".in", ".out", ".mix")]
        if cfg.streams is None:
            unused += [p + hc + t for hc in ("hc1", "hc2") for t in (".in", ".out", ".mix")]
        src = entry["mixer"].get("kv_from")
        layers.append(LayerSpec(block="streams", parts=parts, cache_from=None if src is None else int(src), weights={
            "mixer": p + "mix.", "mixer_norm": p + "norm1", "mixer_connection": p + "hc1",
            "feed_forward": p + "mlp.", "feed_forward_norm": p + "norm2", "feed_forward_connection": p + "hc2"}))
    return ModelSpec(
        hidden_size=w, vocab_size=cfg.vocab, max_positions=cfg.max_positions,
        embedding=PartSpec("embedding", {"vocab": cfg.vocab, "hidden": w, "scale": cfg.embedding_scale,
                                         "stream": "float32", "tensor": ""}),
        layers=tuple(layers), schedule=tuple(range(len(layers))), final_norm=norm,
        head=PartSpec("lm_head", {"vocab": cfg.vocab, "hidden": w, "tied": True}),
        weights={"embedding": "embed", "final_norm": "final.norm", "head": "head."},
        unused_tensors=tuple(unused))


def _preset(width: int, layers: int, heads: int, dim: int, rot_dim: int, vdim: int, q_rank: int, kv_rank: int,
            window: int, ff: int, experts: int, top: int, expert_ff: int, vocab: int, streams: int | None) -> dict:
    """A named size: the first layer has a dense feed-forward, the others experts; every third layer from the
    fourth on reads the cache rows of the layer before it."""
    entries = []
    for i in range(layers):
        mixer = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
                 "scale": (dim + rot_dim) ** -0.5, "mask": {"size": window}, "rot": {"base": 10000.0, "dims": rot_dim}}
        if i >= 3 and i % 3 == 0:
            mixer["kv_from"] = i - 1
        mlp = {"kind": "dense", "ff": ff} if i == 0 else {
            "kind": "moe", "expert": {"ff": expert_ff, "limit": 7.0}, "router": {"experts": experts, "top": top}}
        entries.append({"type": "latent_attention", "mixer": mixer, "mlp": mlp})
    d = {"architecture": "Milozen", "vocab": vocab, "width": width, "embedding": {"scale": 1.0}, "norm": {"eps": 1e-5},
         "layers": entries}
    if streams is not None:
        d["streams"] = streams
    return d


MILOZEN_PRESETS = {
    "milozen-tiny": _preset(width=96, layers=4, heads=3, dim=16, rot_dim=8, vdim=24, q_rank=40, kv_rank=48, window=20,
                            ff=160, experts=4, top=2, expert_ff=32, vocab=211, streams=3),
    # layer sizes near the 1.1B Llama shape: width 2048, 16 heads of 128 + 64, latent 512, 16 experts of 1408 (2 used)
    "milozen-1b": _preset(width=2048, layers=22, heads=16, dim=128, rot_dim=64, vdim=128, q_rank=768, kv_rank=512,
                          window=4096, ff=5632, experts=16, top=2, expert_ff=1408, vocab=32000, streams=2),
}

register_architecture("Milozen", MilozenConfig, milozen_spec, model_type="milozen", presets=MILOZEN_PRESETS)
