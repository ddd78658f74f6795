"""The Nolavik decoder as a `ModelSpec`.

config.json: "architecture": "Nolavik", "vocab", "width", "norm": {"eps"}, "layers" and optionally "loop": {"start",
"stop", "times"}.  An entry of "layers" gives "type" (its mixer), "mixer" (the mixer's sizes and constants) and "mlp"
({"kind": "moe", "expert": {ff}, "router": {experts, top}, "shared": {ff}} or null):
  "latent_attention": heads, dim (unrotated), rot_dim (rotated), vdim, q_rank, kv_rank, scale, rot {base, dims[, scaling]}
  "delta":            heads, kv_heads, dim, vdim, conv
  "parallel":         left {heads, kv_heads, dim, vdim, scale, rot {base, dims[, scaling {factor, low, high, original}]}},
                      right {inner, state, dt_rank, conv}, left_scale, right_scale
Tensors: embed, loop.step [times, width], l<i>.norm1, norm1b, norm2, norm2b, l<i>.mix.*, l<i>.mlp.{router, router.b,
e<k>.gate, e<k>.up, e<k>.down, shared.gate, shared.up, shared.down, shared.sg}, final.norm, head.

Layers start .. stop-1 of the loop run `times` times in a row on the same tensors, every pass with a cache and state of
its own; before the first layer of pass t, row t of loop.step is added to the hidden state.  A layer is the sandwich
arrangement over one 32-bit stream: x += norm1b(mixer(norm1(x))), x += norm2b(mlp(norm2(x))), RMS norms with weights.
"latent_attention" keeps one latent row and one rotated key part per token for all heads; "delta" is the gated delta rule
behind short convolutions; "parallel" is softmax attention with a sink (rotated, then unit-RMS queries and keys) beside a
selective state-space recurrence, added with a factor each.  The feed-forward is a set of SiLU-gated experts chosen by
the largest router logits (with a bias), weighted by the softmax over the chosen logits, and a shared expert that every
token uses, times the sigmoid of one number per token.
"""

from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path

from ..config.model_config import ConfigError
from ..config.registry import register_architecture
from ..parts.attention_composed import scaled_frequencies
from ..parts.spec import LayerSpec, ModelSpec, PartSpec

MIXER_TYPES = ("latent_attention", "delta", "parallel")
MAX_POSITIONS = 1 << 17  # no part of the design limits positions; what the engine sizes its block tables for
UNIT_EPS = 1e-6  # under the root that makes the delta rule's queries and keys unit vectors


def _positive(where: str, m: dict, keys) -> None:
    for key in keys:
        if int(m.get(key, 0)) <= 0:
            raise ConfigError(f"{where}.{key} must be positive")


def _check_rot(where: str, rot: dict, within: int) -> None:
    dims = int(rot.get("dims", 0))
    if dims % 2 or not 0 <= dims <= within:
        raise ConfigError(f"{where}.rot.dims must be even and at most {within}")
    scaling = rot.get("scaling")
    if scaling:
        missing = [k for k in ("factor", "low", "high", "original") if k not in scaling]
        if missing or float(scaling["high"]) == float(scaling["low"]) or float(scaling["factor"]) <= 0:
            raise ConfigError(f"{where}.rot.scaling needs a positive factor, low, high (different from low) and original")


@dataclass(frozen=True)
class NolavikConfig:
    vocab: int
    width: int
    norm_eps: float
    layers: tuple  # of dictionaries as config.json holds them
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    max_positions: int = MAX_POSITIONS

    @classmethod
    def from_dict(cls, d: dict) -> "NolavikConfig":
        missing = [k for k in ("vocab", "width", "layers") if k not in d]
        if missing:
            raise ConfigError(f"config.json lacks required keys {missing}")
        loop = d.get("loop") or {}
        cfg = cls(vocab=int(d["vocab"]), width=int(d["width"]), norm_eps=float((d.get("norm") or {}).get("eps", 1e-6)),
                  layers=tuple(json.loads(json.dumps(entry)) for entry in d["layers"]),
                  loop_start=int(loop.get("start", 0)), loop_stop=int(loop.get("stop", 0)), loop_times=int(loop.get("times", 1)),
                  max_positions=int(d.get("max_positions", MAX_POSITIONS)))
        cfg.validate()
        return cfg

    @classmethod
    def from_json(cls, path: str | Path) -> "NolavikConfig":
        path = Path(path)
        if path.is_dir():
            path = path / "config.json"
        return cls.from_dict(json.loads(path.read_text()))

    @property
    def looped(self) -> bool:
        return self.loop_stop > self.loop_start

    def runs(self) -> list[tuple[int, int | None]]:
        """(layer, pass) in running order; `pass` is the number of the loop's pass at that pass's first layer, else None."""
        n = len(self.layers)
        if not self.looped:
            return [(i, None) for i in range(n)]
        out = [(i, None) for i in range(self.loop_start)]
        for t in range(self.loop_times):
            out += [(i, t if i == self.loop_start else None) for i in range(self.loop_start, self.loop_stop)]
        return out + [(i, None) for i in range(self.loop_stop, n)]

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0 or not self.layers:
            raise ConfigError("vocab and width must be positive and there must be a layer")
        if self.norm_eps <= 0:
            raise ConfigError("norm.eps must be positive")
        if self.looped and not (0 <= self.loop_start < self.loop_stop <= len(self.layers) and self.loop_times >= 1):
            raise ConfigError(f"loop {self.loop_start}..{self.loop_stop} x {self.loop_times} does not fit {len(self.layers)} layers")
        for i, entry in enumerate(self.layers):
            kind, m, where = entry.get("type"), entry.get("mixer") or {}, f"layer {i}: mixer"
            if kind not in MIXER_TYPES:
                raise ConfigError(f"layer {i}: type {kind!r} is not one of {MIXER_TYPES}")
            if kind == "latent_attention":
                _positive(where, m, ("heads", "dim", "vdim", "q_rank", "kv_rank"))
                if int(m.get("rot_dim", 0)) < 0 or "scale" not in m:
                    raise ConfigError(f"{where} needs rot_dim >= 0 and scale")
                _check_rot(where, m.get("rot") or {}, int(m.get("rot_dim", 0)))
            elif kind == "delta":
                _positive(where, m, ("heads", "kv_heads", "dim", "vdim", "conv"))
                if int(m["heads"]) % int(m["kv_heads"]):
                    raise ConfigError(f"{where}.heads is not a multiple of kv_heads")
            else:
                left, right = m.get("left") or {}, m.get("right") or {}
                _positive(where + ".left", left, ("heads", "kv_heads", "dim", "vdim"))
                if int(left["heads"]) % int(left["kv_heads"]) or "scale" not in left:
                    raise ConfigError(f"{where}.left needs heads as a multiple of kv_heads, and scale")
                _check_rot(where + ".left", left.get("rot") or {}, int(left["dim"]))
                _positive(where + ".right", right, ("inner", "state", "dt_rank", "conv"))
            mlp = entry.get("mlp")
            if mlp is None:
                continue
            if mlp.get("kind", "moe") != "moe":
                raise ConfigError(f"layer {i}: mlp.kind {mlp.get('kind')!r} is not 'moe'")
            expert, router = mlp.get("expert") or {}, mlp.get("router") or {}
            experts, top = int(router.get("experts", 0)), int(router.get("top", 0))
            if int(expert.get("ff", 0)) <= 0 or not 1 <= top <= experts:
                raise ConfigError(f"layer {i}: mlp needs expert.ff > 0 and 1 <= router.top <= router.experts")
            if mlp.get("shared") and int(mlp["shared"].get("ff", 0)) <= 0:
                raise ConfigError(f"layer {i}: mlp.shared.ff must be positive")

    def to_dict(self) -> dict:
        d = {"architecture": "Nolavik", "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
             "layers": [dict(entry) for entry in self.layers]}
        if self.looped:
            d["loop"] = {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times}
        return d


def _frequencies(rot: dict):
    """The frequencies as numbers where they are stretched, else None (the part forms base^(-2i / dims) itself)."""
    dims = int(rot.get("dims", 0))
    return tuple(scaled_frequencies(float(rot.get("base", 10000.0)), dims, rot["scaling"])) if dims and rot.get("scaling") else None


def _latent_spec(m: dict, width: int, eps: float) -> PartSpec:
    rot = m.get("rot") or {}
    return PartSpec("latent_attention", {
        "hidden": width, "num_heads": int(m["heads"]), "head_dim_plain": int(m["dim"]), "head_dim_rotated": int(m["rot_dim"]),
        "value_dim": int(m["vdim"]), "q_rank": int(m["q_rank"]), "kv_rank": int(m["kv_rank"]), "scale": float(m["scale"]),
        "window": None, "rotary_base": float(rot.get("base", 10000.0)), "rotary_dims": int(rot.get("dims", m["rot_dim"])),
        "rotary_pairing": "half", "rotary_frequencies": _frequencies(rot), "eps": eps, "output_gate": False})


def _delta_spec(m: dict, width: int, eps: float) -> PartSpec:
    return PartSpec("gated_delta", {
        "hidden": width, "num_heads": int(m["heads"]), "num_kv_heads": int(m["kv_heads"]), "head_dim": int(m["dim"]),
        "value_dim": int(m["vdim"]), "conv_taps": int(m["conv"]), "eps": eps, "unit_eps": UNIT_EPS, "result": "float32"})


def _sink_attention_spec(m: dict, width: int, eps: float) -> PartSpec:
    rot = m.get("rot") or {}
    dims = int(rot.get("dims", 0))
    rotary = {"base": float(rot.get("base", 10000.0)), "dims": dims, "scaling": rot.get("scaling")} if dims else None
    return PartSpec("composed_attention", {
        "hidden": width, "num_heads": int(m["heads"]), "num_kv_heads": int(m["kv_heads"]), "head_dim": int(m["dim"]),
        "value_dim": int(m["vdim"]), "scale": float(m["scale"]), "rotary": rotary, "qk_norm_eps": eps,
        "qk_norm_weight": False, "sink": True, "result": "float32"})


def _scan_spec(m: dict, width: int) -> PartSpec:
    return PartSpec("selective_scan", {"hidden": width, "inner": int(m["inner"]), "states": int(m["state"]),
                                       "dt_rank": int(m["dt_rank"]), "conv_taps": int(m["conv"]), "result": "float32"})


def _mixer_spec(entry: dict, width: int, eps: float) -> PartSpec:
    m = entry["mixer"]
    if entry["type"] == "latent_attention":
        return _latent_spec(m, width, eps)
    if entry["type"] == "delta":
        return _delta_spec(m, width, eps)
    return PartSpec("side_by_side", {"mixers": (
        {"spec": _sink_attention_spec(m["left"], width, eps), "scale": float(m.get("left_scale", 1.0)), "prefix": "left."},
        {"spec": _scan_spec(m["right"], width), "scale": float(m.get("right_scale", 1.0)), "prefix": "right."})})


def _mlp_spec(cfg: NolavikConfig, mlp: dict | None) -> PartSpec:
    if mlp is None:
        return PartSpec("none", {})
    router, shared = mlp["router"], mlp.get("shared")
    # (softmax over all experts, then the chosen scores over their sum: the softmax over the chosen logits)
    return PartSpec("experts", {
        "hidden": cfg.width, "intermediate": int(mlp["expert"]["ff"]), "experts": int(router["experts"]),
        "top": int(router["top"]), "unit": "silu", "scores": "softmax", "renormalize": True, "weight_on": "output",
        "router_bias": True, "shared": {"intermediate": int(shared["ff"]), "gate": True} if shared else None})


def nolavik_spec(cfg: NolavikConfig) -> ModelSpec:
    w = cfg.width
    norm = PartSpec("rmsnorm_streams", {"hidden": w, "eps": cfg.norm_eps, "tensor": ""})
    none = PartSpec("none", {})
    connection = PartSpec("residual", {})
    layers, unused = [], []
    for i, entry in enumerate(cfg.layers):
        p = f"l{i}."
        absent = entry.get("mlp") is None
        parts = {"mixer": _mixer_spec(entry, w, cfg.norm_eps), "mixer_norm": norm, "mixer_post_norm": norm,
                 "mixer_connection": connection, "feed_forward": _mlp_spec(cfg, entry.get("mlp")),
                 "feed_forward_norm": none if absent else norm, "feed_forward_post_norm": none if absent else norm,
                 "feed_forward_connection": none if absent else connection}
        if absent:  # (a checkpoint may hold the second pair of norms all the same)
            unused += [p + "norm2", p + "norm2b"]
        layers.append(LayerSpec(block="sandwich", parts=parts, weights={
            "mixer": p + "mix.", "mixer_norm": p + "norm1", "mixer_post_norm": p + "norm1b", "mixer_connection": p + "c1",
            "feed_forward": p + "mlp.", "feed_forward_norm": p + "norm2", "feed_forward_post_norm": p + "norm2b",
            "feed_forward_connection": p + "c2"}))
    runs = cfg.runs()
    weights = {"embedding": "embed", "final_norm": "final.norm", "head": "head"}
    shifts = tuple((pos, t) for pos, (_layer, t) in enumerate(runs) if t is not None)
    if shifts:
        weights["shifts"] = "loop.step"
    else:  # (a checkpoint of a model without a loop may hold the tensor all the same)
        unused.append("loop.step")
    return ModelSpec(
        hidden_size=w, vocab_size=cfg.vocab, max_positions=cfg.max_positions,
        embedding=PartSpec("embedding", {"vocab": cfg.vocab, "hidden": w, "stream": "float32", "tensor": ""}),
        layers=tuple(layers), schedule=tuple(layer for layer, _t in runs), final_norm=norm,
        head=PartSpec("lm_head", {"vocab": cfg.vocab, "hidden": w, "tied": False, "tensor": ""}),
        weights=weights, unused_tensors=tuple(unused), shifts=shifts)


def _preset(width: int, vocab: int, heads: int, kv_heads: int, dim: int, experts: int, top: int, ff: int, blocks: int,
            times: int) -> dict:
    """A named size: `blocks` times the three kinds of layer in turn (latent attention, delta rule, attention beside a
    scan), the middle of the model run `times` times."""
    mlp = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}, "shared": {"ff": 2 * ff}}
    latent = {"heads": heads, "dim": dim, "rot_dim": dim // 2, "vdim": dim, "q_rank": 3 * width // 8, "kv_rank": width // 4,
              "scale": (dim + dim // 2) ** -0.5, "rot": {"base": 10000.0, "dims": dim // 2}}
    delta = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": 2 * dim, "conv": 4}
    pair = {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": 8.0 / dim,
                     "rot": {"base": 500000.0, "dims": dim // 2,
                             "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}}},
            "right": {"inner": 2 * width, "state": 16, "dt_rank": max(8, width // 16), "conv": 4},
            "left_scale": 1.0, "right_scale": 1.0}
    entries = []
    for _ in range(blocks):
        entries += [{"type": "latent_attention", "mixer": latent, "mlp": mlp}, {"type": "delta", "mixer": delta, "mlp": mlp},
                    {"type": "parallel", "mixer": pair, "mlp": mlp}]
    n = len(entries)
    return {"architecture": "Nolavik", "vocab": vocab, "width": width, "norm": {"eps": 1e-5}, "layers": entries,
            "loop": {"start": n // 3, "stop": n - n // 3, "times": times}}


NOLAVIK_PRESETS = {
    "nolavik-tiny": _preset(width=96, vocab=193, heads=4, kv_heads=2, dim=16, experts=6, top=2, ff=40, blocks=1, times=2),
    # layer sizes near the 1.1B Llama shape
    "nolavik-1b": _preset(width=2048, vocab=32000, heads=32, kv_heads=4, dim=64, experts=16, top=4, ff=1408, blocks=6, times=2),
}

register_architecture("Nolavik", NolavikConfig, nolavik_spec, model_type="nolavik", presets=NOLAVIK_PRESETS)
