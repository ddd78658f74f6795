"""Linear attention with a fixed decay per head and no softmax or denominator, over a state of fixed size.

Per head, with S = 0 before position 0:   S_t = decay_h S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t.

Parameters (a `PartSpec` of kind "decay_attention"):
  hidden, num_heads (H), head_dim (dk, of queries and keys), value_dim (dv; default dk)
  decay             a list of H numbers
  activation        "silu" on q, k and v behind their projections, or None
  rotary            {base, dims}: q and k are turned by position on the first `dims` dimensions of every head,
                    dimension i together with dimension i + dims/2 by the angle p * base^(-2i/dims); None: no rotation
  key_scale         k is multiplied by it (after the rotation); default 1
  output_norm       "heads": each head's o is divided by its own root mean square, no weight;
                    "joint": all heads together are RMS-normed with a weight (tensor "norm")
  eps               of that norm (inside the root)
  gate              "sigmoid" or "silu": the normed heads are multiplied by it of W_g h (tensor "g"); None: no gate
  result            "float32": the output projection's result stays unrounded (for a 32-bit residual stream)
  names             local tensor names (defaults: q, k, v, g, o, norm)

A request keeps S, [H, dk, dv] in 32-bit, in its state slot; a portion of a prompt starts from the stored state and
leaves the state behind its last token, so any cut of a prompt gives the same recurrence.  The projections leave
32-bit results; activation, rotation, the recurrence, the norm and the gate are computed in 32-bit and the gated
heads are rounded once.  The kernels of the recurrence apply activation, rotation and the key's factor to q, k and v
on their way in (no pass over the projection of its own), except for long portions with values wider than 64.
"""

from __future__ import annotations

import torch

from ..ops import library as ops
from .linear import linear
from .registry import Mixer, register_mixer
from .spec import ParamInfo, StateCacheSpec

_DEFAULT_NAMES = {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o", "norm": "norm"}


@register_mixer("decay_attention")
class DecayAttention(Mixer):
    graph_safe = True
    SCAN_UP_TO = 16  # new tokens of the longest portion up to which the recurrence runs token by token

    def __init__(self, spec, ctx):
        super().__init__(spec, ctx)
        self.hidden = int(spec["hidden"])
        self.num_heads = int(spec["num_heads"])
        self.head_dim = int(spec["head_dim"])
        self.value_dim = int(spec.get("value_dim") or self.head_dim)
        self.decay_values = [float(d) for d in spec["decay"]]
        self.activation = spec.get("activation")
        rotary = spec.get("rotary") or {}
        self.rot_dims = int(rotary.get("dims", 0))
        self.rot_base = float(rotary.get("base", 10000.0))
        self.key_scale = float(spec.get("key_scale", 1.0))
        self.output_norm = spec.get("output_norm", "heads")
        self.eps = float(spec["eps"])
        self.gate = spec.get("gate")
        self.result_dtype = torch.float32 if spec.get("result", "model") == "float32" else None
        self.names = dict(_DEFAULT_NAMES, **(spec.get("names") or {}))
        if len(self.decay_values) != self.num_heads:
            raise ValueError(f"{len(self.decay_values)} decays for {self.num_heads} heads")
        if self.activation not in (None, "silu") or self.gate not in (None, "sigmoid", "silu") or \
                self.output_norm not in ("heads", "joint"):
            raise ValueError(f"activation={self.activation!r}, gate={self.gate!r}, output_norm={self.output_norm!r}")
        if self.rot_dims % 2 or not 0 <= self.rot_dims <= self.head_dim:
            raise ValueError(f"rotary.dims={self.rot_dims} must be even and at most head_dim={self.head_dim}")
        if self.head_dim > ops.DECAY_MAX_KEY:
            raise ValueError(f"head_dim up to {ops.DECAY_MAX_KEY}, got {self.head_dim}")
        self.cq = self.num_heads * self.head_dim
        self.cv = self.num_heads * self.value_dim
        self.in_weight = self.o_weight = self.norm_weight = self.decay = self.freq = None

    def libraries(self, dtype_name):
        return ("decay_attention",)

    def cache_spec(self):
        return StateCacheSpec((self.num_heads, self.head_dim, self.value_dim), "float32")

    def param_infos(self):
        n, h = self.names, self.hidden
        infos = {n["q"]: ParamInfo((self.cq, h)), n["k"]: ParamInfo((self.cq, h)), n["v"]: ParamInfo((self.cv, h)),
                 n["o"]: ParamInfo((h, self.cv))}
        if self.gate is not None:
            infos[n["g"]] = ParamInfo((self.cv, h))
        if self.output_norm == "joint":
            infos[n["norm"]] = ParamInfo((self.cv,), "norm")
        return infos

    def load(self, tensors):
        n = self.names
        dev = tensors[n["q"]].device
        pieces = [tensors[n[x]] for x in "qkv"] + ([tensors[n["g"]]] if self.gate is not None else [])
        self.in_weight = torch.cat(pieces, dim=0).contiguous()  # q, k, v and the gate in one product
        self.o_weight = tensors[n["o"]].contiguous()
        if self.output_norm == "joint":
            self.norm_weight = tensors[n["norm"]].float().contiguous()
        self.decay = torch.tensor(self.decay_values, dtype=torch.float32, device=dev)
        if self.rot_dims:
            self.freq = torch.tensor([self.rot_base ** (-2.0 * i / self.rot_dims) for i in range(self.rot_dims // 2)],
                                     dtype=torch.float32, device=dev)

    def forward(self, x, batch, cache):
        heads, dk, dv = self.num_heads, self.head_dim, self.value_dim
        proj = linear(x, self.in_weight, out_dtype=torch.float32)
        cols = dict(col_q=0, col_k=self.cq, col_v=2 * self.cq, heads=heads, dk=dk, dv=dv)
        prepare = None
        if self.activation is not None or self.rot_dims or self.key_scale != 1.0:
            prepare = dict(activation=self.activation, freq=self.freq, rot_dims=self.rot_dims, positions=batch.positions,
                           key_scale=self.key_scale)
        o = torch.empty((proj.shape[0], self.cv), dtype=torch.float32, device=x.device)
        self.recur(o, proj, cache.state, batch, cols, prepare)
        out = torch.empty((proj.shape[0], self.cv), dtype=x.dtype, device=x.device)
        ops.decay_finish(out, o, heads=heads, dv=dv, eps=self.eps, weight=self.norm_weight,
                         gate=proj[:, 2 * self.cq + self.cv:] if self.gate is not None else None, gate_activation=self.gate)
        return linear(out, self.o_weight, out_dtype=self.result_dtype)

    def recur(self, o, proj, state, batch, cols, prepare=None):
        """o[n] = S^T q over the step's tokens, and the requests' states brought up to date: token by token where every
        request brings few, in runs of 64 tokens on the matrix cores where one brings many."""
        if batch.max_count > self.SCAN_UP_TO and self.head_dim <= ops.DECAY_CHUNKS_MAX_KEY:
            if prepare is not None and self.value_dim > ops.DECAY_CHUNKS_SLAB:
                # values wider than a workgroup's columns: several workgroups would prepare the same q and k, and a pass
                # over the projection of its own is cheaper (measured at 128: 2,048 tokens 12.5 against 12.1 ms a step)
                ops.decay_prepare(proj, **prepare, **cols)
                prepare = None
            ops.decay_chunks(o, proj, state, batch.state_slots, batch.cu_seqlens, batch.context_lens, self.decay,
                             batch.max_count, prepare=prepare, **cols)
            return
        ops.decay_scan(o, proj, state, batch.state_slots, batch.cu_seqlens, batch.context_lens, self.decay, prepare=prepare,
                       **cols)
