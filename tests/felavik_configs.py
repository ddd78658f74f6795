"""Small Felavik configurations for the tests: sizes differ from layer to layer, and what a configuration may happen
to make equal or 1 (key and value sizes, one head, as many key/value heads as query heads, a rotation over all or part
of a head, one group of experts, every group kept, one expert chosen, no soft cap, no feed-forward) appears both ways."""

from __future__ import annotations

import copy

LIGHTNING = {"heads": 3, "dim": 12, "vdim": 20, "decay": [0.5, 0.9, 0.99]}
LEFT = {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 24, "scale": 0.3, "bias_max": 40, "bias_rows": 10,
        "q_temp": {"coef": 0.4, "every": 9}}
RIGHT = {"heads": 2, "dim": 16, "vdim": 8, "decay": [0.8, 0.97], "rot": {"base": 100.0, "dims": 8}}


def moe(experts=6, top=2, ff=24, groups=3, keep=2):
    router = {"experts": experts, "top": top}
    if groups is not None:
        router["groups"] = {"count": groups, "keep": keep}
    return {"kind": "moe", "expert": {"ff": ff}, "router": router}


def lightning(mlp="default", **changes):
    return {"type": "lightning", "mixer": dict(copy.deepcopy(LIGHTNING), **changes), "mlp": moe() if mlp == "default" else mlp}


def parallel(left=None, right=None, left_scale=0.7, right_scale=1.3, mlp="default"):
    mixer = {"left": dict(copy.deepcopy(LEFT), **(left or {})), "right": dict(copy.deepcopy(RIGHT), **(right or {})),
             "left_scale": left_scale, "right_scale": right_scale}
    return {"type": "parallel", "mixer": mixer, "mlp": moe() if mlp == "default" else mlp}


def again(layers: list, j: int) -> dict:
    """A layer that runs on the tensors of layer j."""
    return dict(copy.deepcopy(layers[j]), weights_of=j)


def config_of(layers, width=72, vocab=151, scale=1.7, eps=1e-5, softcap=20.0) -> dict:
    d = {"architecture": "Felavik", "vocab": vocab, "width": width, "embedding": {"scale": scale}, "norm": {"eps": eps},
         "layers": layers}
    if softcap is not None:
        d["logit_softcap"] = softcap
    return d


def _small():
    layers = [lightning(), parallel(), lightning(heads=2, dim=40, vdim=72, decay=[0.6, 0.995], mlp=moe(5, 1, 16, None))]
    layers.append(again(layers, 1))
    layers.append(lightning(mlp=None))
    return config_of(layers)


def _small_b():
    # one head each; as many key/value heads as query heads; a rotation over all of a head; every group kept; no cap
    layers = [parallel(left={"heads": 3, "kv_heads": 3, "dim": 8, "vdim": 8, "bias_max": 17, "bias_rows": 4,
                             "q_temp": {"coef": 1.5, "every": 2}},
                       right={"heads": 1, "dim": 8, "vdim": 80, "decay": [0.9], "rot": {"base": 10000.0, "dims": 8}},
                       left_scale=1.0, right_scale=0.25, mlp=moe(4, 4, 12, 2, 2)),
              lightning(heads=1, dim=72, vdim=8, decay=[0.75], mlp=moe(3, 2, 8, 1, 1))]
    layers.append(again(layers, 1))
    layers.append(again(layers, 2))
    return config_of(layers, width=64, vocab=97, scale=1.0, eps=1e-6, softcap=None)


def _small_c():
    # one key/value head for all; keys wider than 64; values of another size; two layers side by side in a row
    layers = [parallel(left={"heads": 5, "kv_heads": 1, "dim": 24, "vdim": 12, "bias_max": 200, "bias_rows": 32,
                             "q_temp": {"coef": 0.2, "every": 50}},
                       right={"heads": 3, "dim": 24, "vdim": 24, "decay": [0.9, 0.95, 0.999], "rot": {"base": 50.0, "dims": 2}},
                       mlp=None),
              parallel(mlp=moe(8, 2, 20, 4, 1)), lightning(heads=4, dim=8, vdim=8, decay=[0.3, 0.6, 0.9, 1.0])]
    return config_of(layers, width=40, vocab=131, scale=0.8)


def _small_d():
    # sizes that the matrix cores take (multiples of 16), pages of 16 keys, a table that most keys lie beyond
    layers = [lightning(heads=2, dim=16, vdim=48, decay=[0.7, 0.99]),
              parallel(left={"heads": 4, "kv_heads": 2, "dim": 32, "vdim": 16, "bias_max": 24, "bias_rows": 12,
                             "q_temp": {"coef": 0.4, "every": 16}},
                       right={"heads": 2, "dim": 32, "vdim": 16, "decay": [0.9, 0.999], "rot": {"base": 1000.0, "dims": 16}}),
              lightning(heads=1, dim=64, vdim=32, decay=[0.98], mlp=moe(4, 2, 32, 2, 1))]
    layers.append(again(layers, 1))
    # keys and values of one size: portions of prompts take the plain attention's kernel with a table
    layers.append(parallel(left={"heads": 2, "kv_heads": 1, "dim": 32, "vdim": 32, "bias_max": 20, "bias_rows": 6,
                                 "q_temp": {"coef": 0.3, "every": 7}}, mlp=None))
    return config_of(layers, width=64, vocab=173, scale=1.2)


SMALL, SMALL_B, SMALL_C, SMALL_D = _small(), _small_b(), _small_c(), _small_d()
