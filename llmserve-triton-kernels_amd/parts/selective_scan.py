"""A selective state-space mixer: a recurrence per channel whose step size, input and read-out depend on the token.

Parameters (a `PartSpec` of kind "selective_scan"):
  hidden, inner (channels), states (N, per channel), dt_rank (R), conv_taps
  result   "float32": the output projection's result stays unrounded (for a 32-bit residual stream)
  names    local tensor names (defaults: in, conv, conv.b, x, dt, dt.b, A_log, D, o)

[x ; z] = W_in h (inner numbers each).  x goes through a causal convolution per channel (taps [inner, conv_taps], the
last column for the present token, a bias, zeros before the sequence) and SiLU.  [d ; B ; C] = W_x x with R, N and N
numbers; dt = softplus(W_dt d + b_dt), one per channel; A = -exp(A_log) [inner, N].  Per channel c and state n
    S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n,        y_c = sum_n S[c, n] C_n + D_c x_c,
and the mixer's result is W_o (y * silu(z)).

A request keeps, in one state slot, S (32-bit, zero before position 0) and the last conv_taps - 1 rows of x before the
convolution (a ring indexed by position); a portion of a prompt starts from them and leaves them behind its last token.
The projections take the model's dtype with 32-bit sums and leave 32-bit results; convolution, SiLU, softplus, the
exponentials, the recurrence and the gate are 32-bit, and y silu(z) is rounded once as the operand of W_o.
"""

from __future__ import annotations

import torch

from ..ops import library as ops
from .attention_composed import _fill_taps
from .linear import linear
from .registry import Mixer, register_mixer
from .spec import ParamInfo, StateCacheSpec

_DEFAULT_NAMES = {"in": "in", "conv": "conv", "conv_bias": "conv.b", "x": "x", "dt": "dt", "dt_bias": "dt.b",
                  "A_log": "A_log", "D": "D", "o": "o"}


def _fill_a_log(shape, generator, device, options):
    """log of 1 .. N along the states, a little off: decays from slow to fast."""
    n = shape[-1]
    base = torch.log(torch.arange(1, n + 1, dtype=torch.float32, device=device)).expand(shape).clone()
    return base + 0.1 * torch.randn(shape, generator=generator, dtype=torch.float32, device=device)


def _fill_dt_bias(shape, generator, device, options):
    """Step sizes around softplus(-2 .. -1)."""
    return -2.0 + torch.rand(shape, generator=generator, dtype=torch.float32, device=device)


def _fill_skip(shape, generator, device, options):
    return 1.0 + 0.1 * torch.randn(shape, generator=generator, dtype=torch.float32, device=device)


@register_mixer("selective_scan")
class SelectiveScan(Mixer):
    graph_safe = True
    PREPARE_FROM = 4  # new tokens of the longest portion beyond which silu(z) is formed beside the recurrence

    def __init__(self, spec, ctx):
        super().__init__(spec, ctx)
        self.hidden = int(spec["hidden"])
        self.inner = int(spec["inner"])
        self.states = int(spec["states"])
        self.dt_rank = int(spec["dt_rank"])
        self.taps = int(spec["conv_taps"])
        self.result_dtype = torch.float32 if spec.get("result", "model") == "float32" else None
        self.names = dict(_DEFAULT_NAMES, **(spec.get("names") or {}))
        if min(self.hidden, self.inner, self.dt_rank, self.taps) < 1 or not 1 <= self.states <= ops.SCAN_MAX_STATES:
            raise ValueError(f"sizes must be positive, with 1 to {ops.SCAN_MAX_STATES} states per channel")
        self.scan_numbers = self.inner * self.states  # S first, then the ring
        self.w_in = self.w_x = self.w_dt_t = self.w_o = self.taps_w = self.conv_bias = self.dt_bias = self.a_neg = self.skip = None

    def libraries(self, dtype_name):
        return ("recurrent",)

    def cache_spec(self):
        return StateCacheSpec((self.scan_numbers + (self.taps - 1) * self.inner,), "float32")

    def param_infos(self):
        n, h, c = self.names, self.hidden, self.inner
        return {n["in"]: ParamInfo((2 * c, h)), n["conv"]: ParamInfo((c, self.taps), _fill_taps),
                n["conv_bias"]: ParamInfo((c,), "around_zero"), n["x"]: ParamInfo((self.dt_rank + 2 * self.states, c)),
                n["dt"]: ParamInfo((c, self.dt_rank)), n["dt_bias"]: ParamInfo((c,), _fill_dt_bias),
                n["A_log"]: ParamInfo((c, self.states), _fill_a_log), n["D"]: ParamInfo((c,), _fill_skip),
                n["o"]: ParamInfo((h, c))}

    def load(self, tensors):
        n = self.names
        self.w_in = tensors[n["in"]].contiguous()
        self.w_x = tensors[n["x"]].contiguous()
        self.w_dt_t = tensors[n["dt"]].float().t().contiguous()  # [dt_rank, inner]
        self.w_o = tensors[n["o"]].contiguous()
        self.taps_w = tensors[n["conv"]].float().contiguous()
        self.conv_bias = tensors[n["conv_bias"]].float().contiguous()
        self.dt_bias = tensors[n["dt_bias"]].float().contiguous()
        self.a_neg = (-torch.exp(tensors[n["A_log"]].float())).contiguous()
        self.skip = tensors[n["D"]].float().contiguous()

    def forward(self, x, batch, cache):
        rows, c, dev = x.shape[0], self.inner, x.device
        xz = linear(x, self.w_in, out_dtype=torch.float32)
        x32 = torch.empty((rows, c), dtype=torch.float32, device=dev)
        x16 = x32 if x.dtype == torch.float32 else torch.empty((rows, c), dtype=x.dtype, device=dev)
        ops.conv_act(xz, 0, c, self.taps_w, bias=self.conv_bias, state=cache.state, ring_offset=self.scan_numbers,
                     batch=batch, out32=x32, out16=None if x16 is x32 else x16)
        low = linear(x16, self.w_x, out_dtype=torch.float32)
        # the step sizes' product is small and stays 32-bit whatever the model's dtype (its input is not rounded): one kernel
        # with the bias and softplus; with many tokens it also forms silu(z), which then stands beside the recurrence's chain
        many = batch.max_count > self.PREPARE_FROM
        dt = ops.step_sizes(torch.empty((rows, c), dtype=torch.float32, device=dev), low, 0, self.w_dt_t, self.dt_bias,
                            z=xz if many else None, z_col=c)
        out = torch.empty((rows, c), dtype=x.dtype, device=dev)
        ops.selective_scan(out, x32, xz, c, low, self.dt_rank, self.dt_rank + self.states, dt, self.a_neg, self.skip, cache.state,
                           0, batch, z_prepared=many)
        return linear(out, self.w_o, out_dtype=self.result_dtype)
