"""Small Dibepel configurations for the tests: every size differs from layer kind to layer kind, and the values
that a configuration may happen to make equal or 1 (key and value sizes, query and key/value heads, one tap, no
kept tokens, no mask at all, an embedding scale of 1) appear both ways."""

from __future__ import annotations

import copy

DEFAULT_MIXERS = {
    "attention_2": {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 24, "conv": 3, "scale": 0.3, "mask": {"size": 12}},
    "attention": {"heads": 2, "kv_heads": 1, "dim": 24, "vdim": 16, "diff": 0.3, "scale": 0.25,
                  "mask": {"size": 9, "keep_first": 4}},
}


def config_of(width=72, vocab=151, scale=1.7, eps=1e-5, ff=88, layers=None) -> dict:
    """config.json of a model whose layers are (type, changes): `changes` may replace "mixer" keys ("mixer": {...} is
    merged into the type's default), set "mlp" (None: no feed-forward) or "weights_of"."""
    layers = layers if layers is not None else [("attention_2", {}), ("attention", {})]
    entries = []
    for kind, changes in layers:
        changes = dict(changes)
        src = changes.get("weights_of")
        if src is not None:
            entry = copy.deepcopy(entries[src])
            entry["weights_of"] = src
        else:
            mixer = dict(copy.deepcopy(DEFAULT_MIXERS[kind]), **changes.pop("mixer", {}))
            entry = {"type": kind, "mixer": mixer, "mlp": changes.pop("mlp", {"kind": "dense", "ff": ff})}
            entry.update(changes)
        entries.append(entry)
    return {"architecture": "Dibepel", "vocab": vocab, "width": width, "embedding": {"scale": scale},
            "norm": {"eps": eps}, "layers": entries}


SMALL = config_of(layers=[
    ("attention_2", {}),
    ("attention", {}),
    ("attention_2", {}),
    ("attention_2", {"mixer": {"heads": 3, "kv_heads": 3, "dim": 8, "vdim": 8, "conv": 1, "mask": {"size": 7}}, "mlp": None}),
    ("attention", {"weights_of": 1}),
    ("attention_2", {"weights_of": 2}),
])

SMALL_B = config_of(width=64, vocab=97, scale=1.0, eps=1e-6, ff=40, layers=[
    ("attention", {"mixer": {"heads": 4, "kv_heads": 4, "dim": 8, "vdim": 8, "diff": 0.0, "scale": 0.4,
                             "mask": {"size": 5, "keep_first": 0}}}),
    ("attention_2", {"mixer": {"heads": 2, "kv_heads": 1, "dim": 16, "vdim": 8, "conv": 2, "scale": 0.2,
                               "mask": {"size": 16}}}),
    ("attention", {"mixer": {"heads": 3, "kv_heads": 1, "dim": 8, "vdim": 24, "diff": 0.6, "scale": 0.3,
                             "mask": {"size": 6, "keep_first": 11}}}),  # more kept tokens than the window is wide
    ("attention", {"mixer": {"mask": {}}}),  # no window: every earlier key
    ("attention_2", {"weights_of": 1}),
    ("attention_2", {"mixer": {"heads": 5, "kv_heads": 5, "dim": 12, "vdim": 20, "conv": 4, "mask": {"size": 3}}}),
])

# sizes the matrix-core attention takes (keys and values in multiples of 16), with 1, 2 and 8 query heads per
# key/value head
SMALL_C = config_of(width=64, vocab=131, scale=0.8, ff=48, layers=[
    ("attention_2", {"mixer": {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 32, "conv": 3, "mask": {"size": 20}}}),
    ("attention", {"mixer": {"heads": 2, "kv_heads": 1, "dim": 32, "vdim": 16, "mask": {"size": 11, "keep_first": 6}}}),
    ("attention_2", {"mixer": {"heads": 8, "kv_heads": 1, "dim": 16, "vdim": 16, "conv": 2, "mask": {"size": 64}}}),
    ("attention", {"weights_of": 1}),
    ("attention_2", {"mixer": {"heads": 3, "kv_heads": 3, "dim": 16, "vdim": 16, "conv": 1, "mask": {"size": 9}}}),
    ("attention", {"mixer": {"heads": 4, "kv_heads": 4, "dim": 16, "vdim": 48, "diff": 0.1, "mask": {"size": 40, "keep_first": 20}}}),
])
