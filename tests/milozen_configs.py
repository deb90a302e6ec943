"""Small Milozen configurations for the tests: sizes differ from layer to layer, and what a configuration may happen
to make equal or 1 (plain and rotated sizes, key and value sizes, one head, one expert chosen, one stream, no streams
at all, a rotation over part of the rotated dimensions, no mask) appears both ways."""

from __future__ import annotations

import copy

DEFAULT_MIXER = {"heads": 3, "dim": 16, "rot_dim": 8, "vdim": 24, "q_rank": 40, "kv_rank": 32, "scale": 0.21,
                 "mask": {"size": 11}, "rot": {"base": 10000.0, "dims": 8}}
DENSE = {"kind": "dense", "ff": 56}


def moe(experts=5, top=2, ff=24, limit=1.25):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}


def config_of(width=72, vocab=151, scale=1.7, eps=1e-5, streams=2, layers=None) -> dict:
    """config.json of a model whose layers are dictionaries of changes: "mixer" is merged into the default mixer (or,
    with "kv_from", into the mixer of the layer named), "mlp" replaces the dense default."""
    entries = []
    for changes in (layers if layers is not None else [{}, {"mlp": moe()}]):
        changes = dict(changes)
        mixer_changes = dict(changes.pop("mixer", {}))
        src = mixer_changes.get("kv_from")
        base = entries[src]["mixer"] if src is not None else DEFAULT_MIXER
        mixer = dict(copy.deepcopy(base), **mixer_changes)
        entries.append({"type": "latent_attention", "mixer": mixer, "mlp": changes.pop("mlp", dict(DENSE))})
    d = {"architecture": "Milozen", "vocab": vocab, "width": width, "embedding": {"scale": scale}, "norm": {"eps": eps},
         "layers": entries}
    if streams is not None:
        d["streams"] = streams
    return d


SMALL = config_of(layers=[
    {},
    {"mlp": moe(experts=5, top=2)},
    {"mixer": {"heads": 2, "dim": 8, "rot_dim": 16, "vdim": 8, "q_rank": 24, "kv_rank": 48, "mask": {"size": 7},
               "rot": {"base": 500.0, "dims": 16}}, "mlp": moe(experts=3, top=1, ff=40, limit=0.8)},
    {"mixer": {"kv_from": 2, "heads": 4, "dim": 12, "vdim": 20, "q_rank": 16, "mask": {"size": 19}}, "mlp": None},
    {"mixer": {"kv_from": 0, "mask": {"size": 5}}, "mlp": moe(experts=4, top=4, ff=16, limit=2.0)},
])

# one stream through hyper-connections, a rotation over part of the rotated dimensions, one head, no mask
SMALL_B = config_of(width=64, vocab=97, scale=1.0, eps=1e-6, streams=1, layers=[
    {"mixer": {"heads": 1, "dim": 24, "rot_dim": 12, "vdim": 16, "q_rank": 20, "kv_rank": 20, "mask": {"size": 1},
               "rot": {"base": 100.0, "dims": 4}}, "mlp": moe(experts=2, top=1, ff=8)},
    {"mixer": {"heads": 5, "dim": 8, "rot_dim": 8, "vdim": 8, "q_rank": 64, "kv_rank": 16, "mask": {},
               "rot": {"base": 10000.0, "dims": 8}}},
    {"mixer": {"kv_from": 1, "heads": 2, "mask": {"size": 16}}, "mlp": moe(experts=7, top=3, ff=12, limit=0.5)},
    {"mixer": {"kv_from": 1, "mask": {"size": 33}}},
    {"mixer": {"rot_dim": 2, "rot": {"base": 10.0, "dims": 2}, "mask": {"size": 64}}, "mlp": None},
])

# no "streams" at all: the plain residual sum; four copies in the other
SMALL_C = config_of(width=40, vocab=131, scale=0.8, streams=None, layers=[
    {"mlp": moe(experts=6, top=2, ff=20)},
    {"mixer": {"heads": 6, "dim": 4, "rot_dim": 4, "vdim": 12, "q_rank": 8, "kv_rank": 72, "mask": {"size": 40},
               "rot": {"base": 3.0, "dims": 4}}},
    {"mixer": {"kv_from": 1, "mask": {"size": 9}}, "mlp": moe(experts=8, top=1, ff=4, limit=3.0)},
])
SMALL_D = config_of(width=48, vocab=77, scale=3.0, streams=4, layers=[
    {"mixer": {"mask": {"size": 17}}, "mlp": moe(experts=3, top=2, ff=24)},
    {"mixer": {"mask": {"size": 8}}},
])
