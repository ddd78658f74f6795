"""The Felavik decoder as a `ModelSpec`.

config.json: "architecture": "Felavik", "vocab", "width", "embedding": {"scale"}, "norm": {"eps"}, optionally
"logit_softcap", and "layers", a list whose entries give "type" (the mixer: "parallel" or "lightning"), "mixer" (its
sizes and constants, below), "mlp" ({"kind": "moe", "expert": {ff}, "router": {experts, top, groups: {count, keep}}}
or null) and optionally "weights_of": j, the layer whose tensors (mixer, feed-forward and norms) the layer runs on,
with a cache and state of its own.
  "lightning": heads, dim, vdim, decay (a number per head).
  "parallel":  left {heads, kv_heads, dim, vdim, scale, bias_max, q_temp {coef, every}}, right {heads, dim, vdim, decay,
               rot {base, dims}}, left_scale, right_scale.
Tensors: embed, l<i>.norm1, l<i>.norm2, l<i>.mix.*, l<i>.mlp.{router, e<k>.gate, e<k>.up, e<k>.down}, final.norm, head.

Every layer is the pre-norm arrangement over a 32-bit residual stream with RMS norms.  "lightning" is linear
attention with a decay per head (SiLU on q, k, v; one norm with a weight over all heads; a sigmoid gate).  "parallel"
is two mixers on the same input: softmax attention without rotation (biases, normed queries and keys, a query factor
that grows with the position, a learned bias per distance bucket, a sigmoid gate on the heads) and a retention (the
same linear attention with rotated q and k, keys scaled by dim^(-1/2), every head normed by itself, a SiLU gate), added
with a factor each.  The feed-forward is a set of experts chosen by softmax scores within the best groups of
experts.  The logits go through a soft cap.
"""

from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path

from ..config.model_config import ConfigError
from ..config.registry import register_architecture
from ..parts.spec import LayerSpec, ModelSpec, PartSpec

MIXER_TYPES = ("parallel", "lightning")
MAX_POSITIONS = 1 << 17  # no part of the design limits positions; what the engine sizes its block tables for
RENORM_EPS = 1e-20  # added to the sum of the chosen experts' scores before they are divided by it


@dataclass(frozen=True)
class FelavikConfig:
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    logit_softcap: float | None
    layers: tuple  # of dictionaries as config.json holds them
    max_positions: int = MAX_POSITIONS

    @classmethod
    def from_dict(cls, d: dict) -> "FelavikConfig":
        missing = [k for k in ("vocab", "width", "layers") if k not in d]
        if missing:
            raise ConfigError(f"config.json lacks required keys {missing}")
        cap = d.get("logit_softcap")
        cfg = cls(vocab=int(d["vocab"]), width=int(d["width"]),
                  embedding_scale=float((d.get("embedding") or {}).get("scale", 1.0)),
                  norm_eps=float((d.get("norm") or {}).get("eps", 1e-5)),
                  logit_softcap=None if cap is None else float(cap),
                  layers=tuple(json.loads(json.dumps(entry)) for entry in d["layers"]),
                  max_positions=int(d.get("max_positions", MAX_POSITIONS)))
        cfg.validate()
        return cfg

    @classmethod
    def from_json(cls, path: str | Path) -> "FelavikConfig":
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

    @staticmethod
    def _linear(where: str, m: dict) -> None:
        for key in ("heads", "dim", "vdim"):
            if int(m.get(key, 0)) <= 0:
                raise ConfigError(f"{where}.{key} must be positive")
        if len(m.get("decay") or ()) != int(m["heads"]):
            raise ConfigError(f"{where}.decay needs a number per head")

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0 or not self.layers:
            raise ConfigError("vocab and width must be positive and there must be a layer")
        if self.norm_eps <= 0:
            raise ConfigError("norm.eps must be positive")
        if self.logit_softcap is not None and self.logit_softcap <= 0:
            raise ConfigError("logit_softcap must be positive")
        for i, entry in enumerate(self.layers):
            if entry.get("type") not in MIXER_TYPES:
                raise ConfigError(f"layer {i}: type {entry.get('type')!r} is not one of {MIXER_TYPES}")
            src = entry.get("weights_of")
            if src is not None and not 0 <= int(src) < len(self.layers):
                raise ConfigError(f"layer {i}: weights_of={src} names no layer")
            self.owner(i)
            m = entry.get("mixer") or {}
            if entry["type"] == "lightning":
                self._linear(f"layer {i}: mixer", m)
            else:
                left, right = m.get("left") or {}, m.get("right") or {}
                for key in ("heads", "kv_heads", "dim", "vdim"):
                    if int(left.get(key, 0)) <= 0:
                        raise ConfigError(f"layer {i}: mixer.left.{key} must be positive")
                if int(left["heads"]) % int(left["kv_heads"]):
                    raise ConfigError(f"layer {i}: mixer.left.heads is not a multiple of kv_heads")
                if "scale" not in left or "bias_max" not in left:
                    raise ConfigError(f"layer {i}: mixer.left needs scale and bias_max")
                self._linear(f"layer {i}: mixer.right", right)
                rot = right.get("rot") or {}
                if rot and (int(rot.get("dims", 0)) % 2 or not 0 <= int(rot.get("dims", 0)) <= int(right["dim"])):
                    raise ConfigError(f"layer {i}: mixer.right.rot.dims must be even and at most dim")
            mlp = entry.get("mlp")
            if mlp is None:
                continue
            if mlp.get("kind", "moe") != "moe":
                raise ConfigError(f"layer {i}: mlp.kind {mlp.get('kind')!r} is not 'moe'")
            expert, router = mlp.get("expert") or {}, mlp.get("router") or {}
            experts, top = int(router.get("experts", 0)), int(router.get("top", 0))
            if int(expert.get("ff", 0)) <= 0 or not 1 <= top <= experts:
                raise ConfigError(f"layer {i}: mlp needs expert.ff > 0 and 1 <= router.top <= router.experts")
            groups = router.get("groups") or {}
            count = int(groups.get("count", 1))
            keep = int(groups.get("keep", count))
            if count < 1 or experts % count or not 1 <= keep <= count or top > keep * (experts // count):
                raise ConfigError(f"layer {i}: router.groups {groups} do not fit {experts} experts of which {top} are chosen")

    def with_tensor_shapes(self, shapes: dict) -> "FelavikConfig":
        """The configuration with what only the checkpoint's tensor shapes tell: the rows of every distance table
        (kept as mixer.left.bias_rows)."""
        layers = json.loads(json.dumps(self.layers))
        for i, entry in enumerate(layers):
            shape = shapes.get(f"l{self.owner(i)}.mix.left.rel")
            if entry["type"] == "parallel" and shape is not None:
                entry["mixer"]["left"]["bias_rows"] = int(shape[0])
        return FelavikConfig(self.vocab, self.width, self.embedding_scale, self.norm_eps, self.logit_softcap, tuple(layers),
                             self.max_positions)

    def to_dict(self) -> dict:
        d = {"architecture": "Felavik", "vocab": self.vocab, "width": self.width,
             "embedding": {"scale": self.embedding_scale}, "norm": {"eps": self.norm_eps},
             "layers": [dict(entry) for entry in self.layers]}
        if self.logit_softcap is not None:
            d["logit_softcap"] = self.logit_softcap
        return d


def _lightning_spec(m: dict, width: int, eps: float) -> PartSpec:
    return PartSpec("decay_attention", {
        "hidden": width, "num_heads": int(m["heads"]), "head_dim": int(m["dim"]), "value_dim": int(m["vdim"]),
        "decay": tuple(float(d) for d in m["decay"]), "activation": "silu", "output_norm": "joint", "eps": eps,
        "gate": "sigmoid", "result": "float32"})


def _retention_spec(m: dict, width: int, eps: float) -> PartSpec:
    rot = m.get("rot") or {}
    return PartSpec("decay_attention", {
        "hidden": width, "num_heads": int(m["heads"]), "head_dim": int(m["dim"]), "value_dim": int(m["vdim"]),
        "decay": tuple(float(d) for d in m["decay"]), "activation": None,
        "rotary": {"base": float(rot.get("base", 10000.0)), "dims": int(rot.get("dims", 0))} if rot else None,
        "key_scale": int(m["dim"]) ** -0.5, "output_norm": "heads", "eps": eps, "gate": "silu", "result": "float32"})


def _softmax_spec(m: dict, width: int, eps: float, rel_rows: int | None) -> PartSpec:
    temp = m.get("q_temp")
    return PartSpec("composed_attention", {
        "hidden": width, "num_heads": int(m["heads"]), "num_kv_heads": int(m["kv_heads"]), "head_dim": int(m["dim"]),
        "value_dim": int(m["vdim"]), "scale": float(m["scale"]), "bias": True, "qk_norm_eps": eps,
        "query_temperature": None if not temp else {"coef": float(temp["coef"]), "every": int(temp["every"])},
        "distance_table": None if rel_rows is None else {"rows": int(rel_rows), "farthest": int(m["bias_max"])},
        "output_gate": True, "result": "float32"})


def _mixer_spec(entry: dict, width: int, eps: float, rel_rows: int | None) -> PartSpec:
    m = entry["mixer"]
    if entry["type"] == "lightning":
        return _lightning_spec(m, width, eps)
    return PartSpec("side_by_side", {"mixers": (
        {"spec": _softmax_spec(m["left"], width, eps, rel_rows), "scale": float(m.get("left_scale", 1.0)), "prefix": "left."},
        {"spec": _retention_spec(m["right"], width, eps), "scale": float(m.get("right_scale", 1.0)), "prefix": "right."})})


def _mlp_spec(cfg: FelavikConfig, mlp: dict | None) -> PartSpec:
    if mlp is None:
        return PartSpec("none", {})
    router = mlp["router"]
    groups = router.get("groups") or {}
    count = int(groups.get("count", 1))
    return PartSpec("experts", {
        "hidden": cfg.width, "intermediate": int(mlp["expert"]["ff"]), "experts": int(router["experts"]),
        "top": int(router["top"]), "unit": "silu", "scores": "softmax", "groups": count,
        "keep": int(groups.get("keep", count)), "renormalize": True, "renorm_eps": RENORM_EPS, "weight_on": "output"})


DEFAULT_REL_ROWS = 16  # rows of a distance table where no checkpoint says (random weights)


def felavik_spec(cfg: FelavikConfig) -> ModelSpec:
    """(The rows of a distance table are a tensor's shape: `with_tensor_shapes` notes them as mixer.left.bias_rows.)"""
    w = cfg.width
    norm = PartSpec("rmsnorm_streams", {"hidden": w, "eps": cfg.norm_eps, "tensor": ""})
    connection = PartSpec("residual", {})
    own = [i for i in range(len(cfg.layers)) if cfg.owner(i) == i]  # layers that hold tensors
    index = {layer: k for k, layer in enumerate(own)}
    layers, unused = [], []
    for i in own:
        entry, p = cfg.layers[i], f"l{i}."
        mlp = entry.get("mlp")
        absent = mlp is None
        rows = None
        if entry["type"] == "parallel":
            rows = int(entry["mixer"]["left"].get("bias_rows") or DEFAULT_REL_ROWS)
        parts = {"mixer": _mixer_spec(entry, w, cfg.norm_eps, rows), "mixer_norm": norm, "mixer_connection": connection,
                 "feed_forward": _mlp_spec(cfg, mlp), "feed_forward_norm": PartSpec("none", {}) if absent else norm,
                 "feed_forward_connection": PartSpec("none", {}) if absent else connection}
        if absent:  # (a checkpoint may hold the second norm all the same)
            unused.append(p + "norm2")
        layers.append(LayerSpec(block="streams", parts=parts, weights={
            "mixer": p + "mix.", "mixer_norm": p + "norm1", "mixer_connection": p + "hc1",
            "feed_forward": p + "mlp.", "feed_forward_norm": p + "norm2", "feed_forward_connection": p + "hc2"}))
    return ModelSpec(
        hidden_size=w, vocab_size=cfg.vocab, max_positions=cfg.max_positions,
        embedding=PartSpec("embedding", {"vocab": cfg.vocab, "hidden": w, "scale": cfg.embedding_scale,
                                         "stream": "float32", "tensor": ""}),
        layers=tuple(layers), schedule=tuple(index[cfg.owner(i)] for i in range(len(cfg.layers))), final_norm=norm,
        head=PartSpec("lm_head", {"vocab": cfg.vocab, "hidden": w, "tied": False, "tensor": "", "softcap": cfg.logit_softcap}),
        weights={"embedding": "embed", "final_norm": "final.norm", "head": "head"},
        unused_tensors=tuple(unused))


def _preset(width: int, layers: int, heads: int, kv_heads: int, dim: int, linear_heads: int, linear_dim: int, experts: int,
            top: int, groups: int, keep: int, expert_ff: int, vocab: int) -> dict:
    """A named size: every fourth layer (from the second) has the two mixers side by side, the others the linear
    attention alone; the last side-by-side layer runs on the tensors of the first."""
    def decays(n):
        return [1.0 - 2.0 ** (-5.0 - 5.0 * k / max(n - 1, 1)) for k in range(n)]

    entries, first = [], None
    mlp = {"kind": "moe", "expert": {"ff": expert_ff},
           "router": {"experts": experts, "top": top, "groups": {"count": groups, "keep": keep}}}
    for i in range(layers):
        if i % 4 == 1:
            mixer = {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": dim ** -0.5,
                              "bias_max": 1024, "bias_rows": 32, "q_temp": {"coef": 0.1, "every": 1024}},
                     "right": {"heads": linear_heads, "dim": linear_dim, "vdim": linear_dim, "decay": decays(linear_heads),
                               "rot": {"base": 10000.0, "dims": linear_dim}},
                     "left_scale": 1.0, "right_scale": 1.0}
            entry = {"type": "parallel", "mixer": mixer, "mlp": mlp}
            if first is None:
                first = i
            elif i + 4 >= layers:
                entry["weights_of"] = first
        else:
            entry = {"type": "lightning", "mlp": mlp,
                     "mixer": {"heads": linear_heads, "dim": linear_dim, "vdim": linear_dim, "decay": decays(linear_heads)}}
        entries.append(entry)
    return {"architecture": "Felavik", "vocab": vocab, "width": width, "embedding": {"scale": 1.0}, "norm": {"eps": 1e-6},
            "logit_softcap": 30.0, "layers": entries}


FELAVIK_PRESETS = {
    "felavik-tiny": _preset(width=96, layers=6, heads=4, kv_heads=2, dim=16, linear_heads=3, linear_dim=24, experts=6, top=2,
                            groups=3, keep=2, expert_ff=40, vocab=211),
    # layer sizes near the 1.1B Llama shape: width 2048, 32 heads of 64, 16 linear heads of 128, 16 experts of 1408 (4 used)
    "felavik-1b": _preset(width=2048, layers=22, heads=32, kv_heads=4, dim=64, linear_heads=16, linear_dim=128, experts=16,
                          top=4, groups=4, keep=2, expert_ff=1408, vocab=32000),
}

register_architecture("Felavik", FelavikConfig, felavik_spec, model_type="felavik", presets=FELAVIK_PRESETS)
