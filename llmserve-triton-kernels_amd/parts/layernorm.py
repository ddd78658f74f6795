"""Layer norm with a weight and no bias over a residual stream that is kept in 32-bit:
(x - mean) / sqrt(var + eps) * w with the variance as the mean squared deviation, all in 32-bit, rounded once to the
model's dtype.  Parameters: hidden, eps, tensor (the weight's local name; default "weight").

The stream may be several parallel copies [N, S, hidden] that sublayers read and write through `Connection`s: the
norm's kernel then closes the write of the sublayer before (`OpenStreams`), forms what the next one reads and norms
it, in one pass over the row.
"""

from __future__ import annotations

import torch

from ..ops import library as ops
from .registry import Norm, NormedSum, OpenStreams, register_norm
from .spec import ParamInfo


@register_norm("layernorm32")
class LayerNorm32(Norm):
    graph_safe = True
    closes_streams = True  # `read_streams`, `add_norm` and `norm_rows` take an `OpenStreams` in the place of delta
    center = True  # the mean is taken off

    def __init__(self, spec, ctx):
        super().__init__(spec, ctx)
        self.hidden = int(spec["hidden"])
        self.eps = float(spec["eps"])
        self.tensor = spec.get("tensor", "weight")
        self.weight: torch.Tensor | None = None

    def param_infos(self):
        return {self.tensor: ParamInfo((self.hidden,), "norm")}

    def libraries(self, dtype_name):
        return ("stream32",)

    def load(self, tensors):
        self.weight = tensors[self.tensor].float().contiguous()

    @staticmethod
    def _streams(x):
        if x.dtype != torch.float32:
            raise ValueError("this norm reads a 32-bit residual stream")
        return x.unsqueeze(1) if x.dim() == 2 else x

    @staticmethod
    def _open(delta):
        if delta is None:
            return {}
        if not isinstance(delta, OpenStreams):
            raise ValueError("a 32-bit residual stream takes an open write of streams or nothing")
        return {"y": delta.y, "mix": delta.connection.mix, "write": delta.connection.write}

    def read_streams(self, x, delta, connection=None, source=None):
        """The normed input of the sublayer behind `connection` from the streams x [N, S, hidden], after the open
        write `delta` (done in place).  `source` [N, hidden]: the streams start as copies of it."""
        x = self._streams(x)
        out = torch.empty((x.shape[0], self.hidden), dtype=self.ctx.dtype, device=x.device)
        read = None if connection is None else connection.read
        return ops.streams_norm(out, x, self.weight, self.eps, source=source, read=read, center=self.center,
                                **self._open(delta))

    def forward(self, x):
        return self.read_streams(x, None)

    def add_norm(self, residual, delta):
        return self.read_streams(residual, delta)

    def norm_rows(self, x, delta, rows):
        x = self._streams(x)
        out = torch.empty((rows.numel(), self.hidden), dtype=self.ctx.dtype, device=x.device)
        return ops.streams_norm(out, x, self.weight, self.eps, rows=rows, center=self.center, **self._open(delta))


@register_norm("rmsnorm_streams")
class RMSNormStreams(LayerNorm32):
    """The same over the same streams without taking the mean off: u / sqrt(mean(u^2) + eps) * w, all in 32-bit,
    rounded once.  Parameters as above."""

    center = False
    closes_normed_sums = True  # `read_streams`, `add_norm` and `norm_rows` also take a `NormedSum` in the place of delta

    def _one_stream(self, x):
        x = self._streams(x)
        if x.shape[1] != 1:
            raise ValueError("a sum through a norm joins a stream of one copy")
        return x.view(x.shape[0], self.hidden)

    def read_streams(self, x, delta, connection=None, source=None):
        if not isinstance(delta, NormedSum):
            return super().read_streams(x, delta, connection, source)
        if source is not None or (connection is not None and connection.read is not None):
            raise ValueError("a sum through a norm joins one plain stream")
        rows = self._one_stream(x)
        out = torch.empty((rows.shape[0], self.hidden), dtype=self.ctx.dtype, device=x.device)
        return ops.normed_add_norm(out, rows, self.weight, self.eps, y=delta.y, y_weight=delta.weight, y_eps=delta.eps)

    def norm_rows(self, x, delta, rows):
        if not isinstance(delta, NormedSum):
            return super().norm_rows(x, delta, rows)
        out = torch.empty((rows.numel(), self.hidden), dtype=self.ctx.dtype, device=x.device)
        return ops.normed_add_norm(out, self._one_stream(x), self.weight, self.eps, y=delta.y, y_weight=delta.weight,
                                   y_eps=delta.eps, rows=rows)


@register_norm("none")
class NoNorm(Norm):
    """For a sublayer that a layer does not have."""

    graph_safe = True

    def forward(self, x):
        return x
