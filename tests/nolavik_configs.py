"""Small Nolavik configurations for the tests: sizes differ from layer to layer, and what a configuration may happen
to make equal or 1 (key and value sizes, one head, as many key/value heads as query heads, a rotation over all or part
of a head, stretched frequencies or plain ones, one expert chosen, every expert chosen, no shared expert, no
feed-forward, no loop, a loop of one layer, a loop from the first layer or to the last) appears both ways."""

from __future__ import annotations

import copy

LATENT = {"heads": 3, "dim": 12, "rot_dim": 8, "vdim": 20, "q_rank": 24, "kv_rank": 40, "scale": 0.21,
          "rot": {"base": 100.0, "dims": 8}}
DELTA = {"heads": 4, "kv_heads": 2, "dim": 12, "vdim": 20, "conv": 3}
LEFT = {"heads": 4, "kv_heads": 2, "dim": 24, "vdim": 12, "scale": 0.9,
        "rot": {"base": 50.0, "dims": 16, "scaling": {"factor": 3.0, "low": 1.0, "high": 5.0, "original": 64}}}
RIGHT = {"inner": 56, "state": 5, "dt_rank": 6, "conv": 4}


def moe(experts=6, top=2, ff=24, shared=40):
    d = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        d["shared"] = {"ff": shared}
    return d


def _mlp(mlp):
    return moe() if mlp == "default" else mlp


def latent(mlp="default", **changes):
    return {"type": "latent_attention", "mixer": dict(copy.deepcopy(LATENT), **changes), "mlp": _mlp(mlp)}


def delta(mlp="default", **changes):
    return {"type": "delta", "mixer": dict(copy.deepcopy(DELTA), **changes), "mlp": _mlp(mlp)}


def parallel(left=None, right=None, left_scale=0.7, right_scale=1.3, mlp="default"):
    mixer = {"left": dict(copy.deepcopy(LEFT), **(left or {})), "right": dict(copy.deepcopy(RIGHT), **(right or {})),
             "left_scale": left_scale, "right_scale": right_scale}
    return {"type": "parallel", "mixer": mixer, "mlp": _mlp(mlp)}


def config_of(layers, width=72, vocab=151, eps=1e-5, loop=None) -> dict:
    d = {"architecture": "Nolavik", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if loop is not None:
        d["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return d


def _small():
    # the middle two layers three times
    layers = [latent(), delta(), parallel(), delta(heads=2, kv_heads=2, dim=40, vdim=8, conv=2, mlp=moe(5, 1, 16, None))]
    return config_of(layers, loop=(1, 3, 3))


def _small_b():
    # one head each; as many key/value heads as query heads; rotations over all of a head, plain frequencies; every
    # expert chosen; one tap; no loop
    layers = [parallel(left={"heads": 3, "kv_heads": 3, "dim": 8, "vdim": 8, "scale": 1.5, "rot": {"base": 10000.0, "dims": 8}},
                       right={"inner": 9, "state": 24, "dt_rank": 1, "conv": 1}, left_scale=1.0, right_scale=0.25,
                       mlp=moe(4, 4, 12, 8)),
              latent(heads=1, dim=8, rot_dim=8, vdim=80, q_rank=8, kv_rank=16, rot={"base": 10.0, "dims": 8}, mlp=None),
              delta(heads=1, kv_heads=1, dim=72, vdim=8, conv=1, mlp=moe(3, 2, 8, None))]
    return config_of(layers, width=64, vocab=97, eps=1e-6)


def _small_c():
    # the whole model twice; one key/value head for all; no rotation at all on the left; a part of the rotated part
    # turned; states beyond 16 a channel; two layers side by side in a row
    layers = [parallel(left={"heads": 5, "kv_heads": 1, "dim": 24, "vdim": 12, "scale": 0.5, "rot": {"base": 50.0, "dims": 0}},
                       right={"inner": 40, "state": 37, "dt_rank": 3, "conv": 2}, mlp=None),
              parallel(mlp=moe(8, 3, 20, 12)),
              latent(heads=4, dim=8, rot_dim=12, vdim=8, q_rank=20, kv_rank=12, rot={"base": 1e6, "dims": 4})]
    return config_of(layers, width=40, vocab=131, loop=(0, 3, 2))


def _small_d():
    # sizes that the matrix cores take (multiples of 16), pages of 16 keys; the last layer looped alone
    layers = [latent(heads=4, dim=32, rot_dim=16, vdim=32, q_rank=32, kv_rank=48, scale=0.15, rot={"base": 1e4, "dims": 16}),
              parallel(left={"heads": 4, "kv_heads": 2, "dim": 32, "vdim": 16, "scale": 0.6,
                             "rot": {"base": 1000.0, "dims": 16, "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 32}}},
                       right={"inner": 64, "state": 16, "dt_rank": 8, "conv": 4}),
              delta(heads=2, kv_heads=1, dim=64, vdim=32, conv=4, mlp=moe(4, 2, 32, 32)),
              parallel(left={"heads": 2, "kv_heads": 1, "dim": 64, "vdim": 64, "scale": 0.4, "rot": {"base": 1e5, "dims": 64}},
                       right={"inner": 128, "state": 8, "dt_rank": 16, "conv": 3}, mlp=None)]
    return config_of(layers, width=64, vocab=173, loop=(3, 4, 2))


SMALL, SMALL_B, SMALL_C, SMALL_D = _small(), _small_b(), _small_c(), _small_d()
