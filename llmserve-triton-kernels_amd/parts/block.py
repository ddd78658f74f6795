"""Arrangements of a layer's parts.

"parallel" has one norm that both branches read: with h = norm(x),
    x = x + g_mixer * mixer(h) + g_feed_forward * feed_forward(h)
where each g is the branch's gate (a part of the family "gate"; kind "none": no gate) and the residual
stream x is 32-bit whatever the model's dtype: the branches' results arrive unrounded and one kernel
applies the gates and sums.

"streams" is the pre-norm layer over a 32-bit residual stream of one or several parallel copies:
    x <- write_1(x, mixer(norm1(read_1(x))));  x <- write_2(x, feed_forward(norm2(read_2(x))))
where read and write are the sublayer's `Connection` (kind "residual": read is x itself and write adds; kind "hyper":
weighted sums over the copies).  Each write is left open and done by the kernel that reads the streams next.

"sandwich" is "streams" with a norm behind every sublayer as well as before it, over one stream:
    x <- x + post_1(mixer(norm1(x)));  x <- x + post_2(feed_forward(norm2(x)))
The sum through the second norm is left open (`NormedSum`) and done by the kernel that norms the stream next.

"prenorm" is the reference's decoder layer (src/llmserve/model/llama.py:131-135):
    x = x + mixer(norm1(x));  x = x + feed_forward(norm2(x))
The hidden state travels as (x, delta) with the last sum still open, so each residual
sum is done, in 32-bit, by the norm kernel that needs its result.
"""

from __future__ import annotations

import torch

from ..ops import library as ops
from .linear import linear
from .registry import ADDED_IN_PLACE, Block, DeferredNorm, GatedSum, NormedSum, OpenStreams, register_block


@register_block("prenorm")
class PreNormBlock(Block):
    def forward(self, x, delta, batch, cache):
        # x + delta, normed: by the norm's kernel or by the mixer's; what the mixer returns is added to the
        # residual rows by the next norm's kernel, or by the mixer's last kernel (ADDED_IN_PLACE)
        h = DeferredNorm(self.mixer_norm, x, delta, may_add_in_place=True)
        a = self.mixer.forward(h if self.mixer.accepts_deferred_norm else h.materialize(), batch, cache)
        if not h.resolved:
            raise RuntimeError(f"{type(self.mixer).__name__} took a deferred input and left it unresolved")
        h2 = DeferredNorm(self.feed_forward_norm, h.residual, None if a is ADDED_IN_PLACE else a, may_add_in_place=True)
        f = self.feed_forward.forward(h2 if self.feed_forward.accepts_deferred_norm else h2.materialize())
        if not h2.resolved:
            raise RuntimeError(f"{type(self.feed_forward).__name__} took a deferred input and left it unresolved")
        return h2.residual, None if f is ADDED_IN_PLACE else f


@register_block("parallel")
class ParallelBlock(Block):
    """One norm, two branches beside each other, each with a gate of its own; a 32-bit residual stream, summed in
    place.  The feed-forward may be of kind "none" (the layer has a mixer only)."""

    ROLES = {"mixer": "mixer", "feed_forward": "feed_forward", "norm": "norm", "mixer_gate": "gate",
             "feed_forward_gate": "gate"}

    def __init__(self, parts):
        super().__init__(parts)
        self._stacked = None  # the gates' weights (and the mixer's input projection) as one matrix, made at the first step
        self._mixer_columns = None

    def _stack(self):
        """One matrix for every product of h whose result stays 32-bit: the two gates, and the mixer's input
        projection where the mixer offers it (`input_weight`, taken back as `projected`).  The parts' own
        weights become views of it, so nothing is held twice."""
        gm, gf = self.mixer_gate, self.feed_forward_gate
        wm, wf = gm.weight, gf.weight
        if wm is None or wf is None:
            return False
        if self._stacked is None:
            pieces = [wm, wf]
            mixer_w = getattr(self.mixer, "input_weight", None)
            if mixer_w is not None and mixer_w.dtype == wm.dtype and mixer_w.shape[1] == wm.shape[1]:
                pieces.append(mixer_w)
            self._stacked = torch.cat(pieces, dim=0).contiguous()
            a, b = wm.shape[0], wm.shape[0] + wf.shape[0]
            gm.weight, gf.weight = self._stacked[:a], self._stacked[a:b]
            if len(pieces) == 3:
                self.mixer.input_weight = self._stacked[b:]
                self._mixer_columns = (b, self._stacked.shape[0])
        return True

    def _gate_products(self, h):
        """(products [N, columns] or None, column of the mixer's gate or None, column of the feed-forward's,
        the mixer's projected input or None)."""
        gm, gf = self.mixer_gate, self.feed_forward_gate
        if self._stack():  # one product for all
            out = linear(h, self._stacked, out_dtype=torch.float32)
            projected = None
            if self._mixer_columns is not None:
                projected = out[:, self._mixer_columns[0]: self._mixer_columns[1]]
            return out, 0, gm.weight.shape[0], projected
        zm, zf = gm.products(h), gf.products(h)
        if zm is not None and zf is not None:
            return torch.cat([zm, zf], dim=1), 0, zm.shape[1], None
        one = zm if zm is not None else zf
        return one, (0 if zm is not None else None), (0 if zf is not None else None), None

    def forward(self, x, delta, batch, cache):
        if x.dtype != torch.float32:
            raise ValueError("the parallel arrangement keeps a 32-bit residual stream")
        # (the layer before may have left its gated sum open: this layer's norm closes it in its own kernel)
        h = self.norm.add_norm(x, delta)
        z, col_m, col_f, projected = self._gate_products(h)
        a = self.mixer.forward(h, batch, cache) if projected is None else self.mixer.forward(h, batch, cache, projected=projected)
        f = self.feed_forward.forward(h)
        branches = []
        for y, col, gate in ((a, col_m, self.mixer_gate), (f, col_f, self.feed_forward_gate)):
            if y is not None:
                branches.append((y if y.dtype == torch.float32 else y.float(), col, gate.bias))
        if not branches:
            return x, None
        if getattr(self.norm, "closes_gated_sums", False):  # left open for the next norm (the next layer's, or the last)
            return x, GatedSum(branches, z)
        ops.gated_add(x, branches, z)
        return x, None


@register_block("streams")
class StreamsBlock(Block):
    """Pre-norm sublayers that meet the residual stream through connections; the stream is float32 [N, S, hidden]
    whatever the model's dtype (the embedding's [N, hidden] becomes S equal copies at the first read).  The
    feed-forward may be of kind "none": the layer then has a mixer only, and its second norm and connection are unused."""

    ROLES = {"mixer": "mixer", "feed_forward": "feed_forward", "mixer_norm": "norm", "feed_forward_norm": "norm",
             "mixer_connection": "connection", "feed_forward_connection": "connection"}

    def _read(self, norm, connection, x, delta):
        if not getattr(norm, "closes_streams", False):
            raise ValueError(f"{type(norm).__name__} cannot read a stream of several copies")
        if x.dim() == 2:  # the embedding's output: every copy starts as it
            if delta is not None:
                raise ValueError("an open write before the streams exist")
            streams = torch.empty((x.shape[0], connection.streams, x.shape[1]), dtype=torch.float32, device=x.device)
            return norm.read_streams(streams, None, connection, source=x), streams
        if x.shape[1] != connection.streams:
            raise ValueError(f"the stream has {x.shape[1]} copies, the connection {connection.streams}")
        return norm.read_streams(x, delta, connection), x

    def forward(self, x, delta, batch, cache):
        h, x = self._read(self.mixer_norm, self.mixer_connection, x, delta)
        delta = OpenStreams(self._result(self.mixer.forward(h, batch, cache)), self.mixer_connection)
        if getattr(self.feed_forward, "absent", False):
            return x, delta
        h, x = self._read(self.feed_forward_norm, self.feed_forward_connection, x, delta)
        return x, OpenStreams(self._result(self.feed_forward.forward(h)), self.feed_forward_connection)

    @staticmethod
    def _result(y):
        return y if y.dtype == torch.float32 else y.float()


@register_block("sandwich")
class SandwichBlock(StreamsBlock):
    """Norms before and behind each sublayer over one 32-bit stream: the roles of "streams" and, of the family "norm",
    `mixer_post_norm` and `feed_forward_post_norm` (RMS norms with a weight: parts that offer `weight` and `eps`).  The
    connections are plain ("residual"); the norms before the sublayers must close a `NormedSum`."""

    ROLES = dict(StreamsBlock.ROLES, mixer_post_norm="norm", feed_forward_post_norm="norm")

    def _read(self, norm, connection, x, delta):
        if not getattr(norm, "closes_normed_sums", False):
            raise ValueError(f"{type(norm).__name__} cannot close a sum through a norm")
        if connection.streams != 1 or connection.read is not None:
            raise ValueError("the sandwich arrangement keeps one plain stream")
        return super()._read(norm, connection, x, delta)

    def _joined(self, y, post):
        return NormedSum(self._result(y), post.weight, post.eps)

    def forward(self, x, delta, batch, cache):
        h, x = self._read(self.mixer_norm, self.mixer_connection, x, delta)
        delta = self._joined(self.mixer.forward(h, batch, cache), self.mixer_post_norm)
        if getattr(self.feed_forward, "absent", False):
            return x, delta
        h, x = self._read(self.feed_forward_norm, self.feed_forward_connection, x, delta)
        return x, self._joined(self.feed_forward.forward(h), self.feed_forward_post_norm)
