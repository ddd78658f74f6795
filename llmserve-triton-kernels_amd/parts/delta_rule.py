"""The gated delta rule: linear attention over a state per head that every token first decays, then corrects.

Parameters (a `PartSpec` of kind "gated_delta"):
  hidden, num_heads (H, of values), num_kv_heads (G, of queries and keys), head_dim (dk), value_dim (dv), conv_taps
  eps          of the norm over each head's result
  unit_eps     added to the sum of squares under the root that makes q and k unit vectors (default 1e-6)
  result       "float32": the output projection's result stays unrounded (for a 32-bit residual stream)
  names        local tensor names (defaults: q, k, v, q.conv, k.conv, v.conv, b, a, A_log, dt_bias, g, norm, o)

q = W_q h and k = W_k h (G heads of dk), v = W_v h (H heads of dv); each passes a causal convolution per channel (taps
[channels, conv_taps], the last column for the present token, no bias, zeros before the sequence) and SiLU; q and k are
then divided head by head by sqrt(sum of squares + unit_eps) and q is multiplied by dk^(-1/2).  beta = sigmoid(W_b h)
and decay = exp(-exp(A_log) softplus(W_a h + dt_bias)), a number per head each.  Head h (with q and k of head
h / (H / G)), S [dk, dv] zero before position 0:
    S <- decay S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q.
o is divided head by head by its root mean square (eps inside the root), multiplied by a weight of dv numbers that all
heads share and by silu(W_g h); W_o follows.

A request keeps, in one state slot, S of every head (32-bit) and the last conv_taps - 1 rows of [q ; k ; v] before the
convolution (a ring indexed by position).  Everything behind the projections is computed in 32-bit; the gated heads are
rounded once as the operand of W_o.
"""

from __future__ import annotations

import torch

from ..ops import library as ops
from .attention_composed import _fill_taps
from .linear import linear
from .registry import Mixer, register_mixer
from .spec import ParamInfo, StateCacheSpec

_DEFAULT_NAMES = {"q": "q", "k": "k", "v": "v", "q_conv": "q.conv", "k_conv": "k.conv", "v_conv": "v.conv", "b": "b", "a": "a",
                  "A_log": "A_log", "dt_bias": "dt_bias", "g": "g", "norm": "norm", "o": "o"}


def _fill_rate(shape, generator, device, options):
    """log of decay rates between 1/16 and 1."""
    return -2.8 * torch.rand(shape, generator=generator, dtype=torch.float32, device=device)


@register_mixer("gated_delta")
class GatedDelta(Mixer):
    graph_safe = True
    PREPARE_FROM = 4  # new tokens of the longest portion beyond which the gates are formed by a launch of their own

    def __init__(self, spec, ctx):
        super().__init__(spec, ctx)
        self.hidden = int(spec["hidden"])
        self.heads = int(spec["num_heads"])
        self.kv_heads = int(spec.get("num_kv_heads") or self.heads)
        self.dk = int(spec["head_dim"])
        self.dv = int(spec.get("value_dim") or self.dk)
        self.taps = int(spec["conv_taps"])
        self.eps = float(spec["eps"])
        self.unit_eps = float(spec.get("unit_eps", 1e-6))
        self.result_dtype = torch.float32 if spec.get("result", "model") == "float32" else None
        self.names = dict(_DEFAULT_NAMES, **(spec.get("names") or {}))
        if min(self.hidden, self.heads, self.kv_heads, self.dv, self.taps) < 1 or self.heads % self.kv_heads:
            raise ValueError("sizes must be positive and num_heads a multiple of num_kv_heads")
        if not 1 <= self.dk <= ops.DELTA_MAX_KEY:
            raise ValueError(f"head_dim of 1 to {ops.DELTA_MAX_KEY}, got {self.dk}")
        self.cq = self.kv_heads * self.dk
        self.cv = self.heads * self.dv
        self.channels = 2 * self.cq + self.cv
        self.scan_numbers = self.heads * self.dk * self.dv  # S first, then the ring
        self.w_in = self.w_o = self.taps_w = self.a_log = self.dt_bias = self.norm_weight = None

    def libraries(self, dtype_name):
        return ("recurrent",)

    def cache_spec(self):
        return StateCacheSpec((self.scan_numbers + (self.taps - 1) * self.channels,), "float32")

    def param_infos(self):
        n, h = self.names, self.hidden
        infos = {n["q"]: ParamInfo((self.cq, h)), n["k"]: ParamInfo((self.cq, h)), n["v"]: ParamInfo((self.cv, h)),
                 n["b"]: ParamInfo((self.heads, h)), n["a"]: ParamInfo((self.heads, h)), n["g"]: ParamInfo((self.cv, h)),
                 n["o"]: ParamInfo((h, self.cv)), n["A_log"]: ParamInfo((self.heads,), _fill_rate),
                 n["dt_bias"]: ParamInfo((self.heads,), "around_zero"), n["norm"]: ParamInfo((self.dv,), "norm")}
        for key, channels in (("q_conv", self.cq), ("k_conv", self.cq), ("v_conv", self.cv)):
            infos[n[key]] = ParamInfo((channels, self.taps), _fill_taps)
        return infos

    def load(self, tensors):
        n = self.names
        # one product for everything that reads h: [q ; k ; v ; gate ; a ; b], results in 32-bit
        self.w_in = torch.cat([tensors[n[x]] for x in ("q", "k", "v", "g", "a", "b")], dim=0).contiguous()
        self.col_g = self.channels
        self.col_a = self.channels + self.cv
        self.col_b = self.col_a + self.heads
        self.w_o = tensors[n["o"]].contiguous()
        self.taps_w = torch.cat([tensors[n[x + "_conv"]].float() for x in "qkv"], dim=0).contiguous()
        self.a_log = tensors[n["A_log"]].float().contiguous()
        self.dt_bias = tensors[n["dt_bias"]].float().contiguous()
        self.norm_weight = tensors[n["norm"]].float().contiguous()

    def forward(self, x, batch, cache):
        rows, dev = x.shape[0], x.device
        proj = linear(x, self.w_in, out_dtype=torch.float32)
        qkv = torch.empty((rows, self.channels), dtype=torch.float32, device=dev)
        gates = dict(gates=proj, a_col=self.col_a, b_col=self.col_b, a_log=self.a_log, dt_bias=self.dt_bias, heads=self.heads)
        # (steps of many tokens: decay and beta are formed beside the recurrence, not inside its chain from token to token)
        many = batch.max_count > self.PREPARE_FROM
        # the convolution, SiLU, the unit vectors (and the gates) in one launch
        ops.conv_heads(proj, 0, self.channels, self.taps_w, qkv, q_heads=self.kv_heads, k_heads=self.kv_heads, dk=self.dk,
                       eps=self.unit_eps, q_factor=self.dk ** -0.5, state=cache.state, ring_offset=self.scan_numbers, batch=batch,
                       gates=gates if many else None)
        o = torch.empty((rows, self.cv), dtype=torch.float32, device=dev)
        ops.delta_scan(o, qkv, q_col=0, k_col=self.cq, v_col=2 * self.cq, kv_heads=self.kv_heads, dk=self.dk, dv=self.dv,
                       state=cache.state, scan_offset=0, batch=batch, prepared=many, **gates)
        out = torch.empty((rows, self.cv), dtype=x.dtype, device=dev)
        ops.delta_finish(out, o, proj, self.col_g, self.norm_weight, heads=self.heads, dv=self.dv, eps=self.eps)
        return linear(out, self.w_o, out_dtype=self.result_dtype)
