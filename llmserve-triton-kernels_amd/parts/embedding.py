"""Token embedding (row gather, no scaling: src/llmserve/model/llama.py:141,171) and the
output head (logits = h W^T in 32-bit, W being the embedding table itself when tied:
src/llmserve/model/llama.py:151-153,185)."""

from __future__ import annotations

import torch

from ..ops import library as ops
from .linear import decode_product, linear
from .registry import EMBEDDINGS, HEADS, DeferredNorm, Part
from .spec import ParamInfo


@EMBEDDINGS.register("embedding")
class TokenEmbedding(Part):
    graph_safe = True

    def __init__(self, spec, ctx):
        super().__init__(spec, ctx)
        self.vocab = int(spec["vocab"])
        self.hidden = int(spec["hidden"])
        # `scale`: the row is multiplied by it; `stream`: "float32" starts a residual stream that is kept in 32-bit
        # whatever the model's dtype (the product is then formed in 32-bit as well); `tensor`: the table's local name
        self.scale = spec.get("scale")
        self.stream = spec.get("stream", "model")
        self.tensor = spec.get("tensor", "weight")
        if self.stream not in ("model", "float32"):
            raise ValueError(f"stream={self.stream!r}; choose 'model' or 'float32'")
        if self.scale is not None and self.stream != "float32":
            raise ValueError("a scaled embedding starts a 32-bit residual stream (stream='float32')")
        self.weight: torch.Tensor | None = None

    def param_infos(self):
        return {self.tensor: ParamInfo((self.vocab, self.hidden))}

    def libraries(self, dtype_name):
        return ("stream32",) if self.stream == "float32" else ()

    def load(self, tensors):
        self.weight = tensors[self.tensor].contiguous()

    def forward(self, token_ids: torch.Tensor) -> torch.Tensor:
        if self.stream == "float32":
            out = torch.empty((token_ids.numel(), self.hidden), dtype=torch.float32, device=self.weight.device)
            return ops.embed_scale(out, self.weight, token_ids, 1.0 if self.scale is None else float(self.scale))
        out = torch.empty((token_ids.numel(), self.hidden), dtype=self.weight.dtype, device=self.weight.device)
        return ops.embed_gather(out, self.weight, token_ids)


@HEADS.register("lm_head")
class LMHead(Part):
    """Parameters: vocab, hidden, tied, tensor, softcap.  A tied head has no tensor of its own: the model
    hands it the embedding table.  `softcap` c: the logits become c tanh(logits / c), in 32-bit."""
    graph_safe = True
    accepts_deferred_norm = True  # (when every row's logits are wanted the model hands over the final norm's input)

    def __init__(self, spec, ctx):
        super().__init__(spec, ctx)
        self.vocab = int(spec["vocab"])
        self.hidden = int(spec["hidden"])
        self.tied = bool(spec.get("tied", False))
        self.tensor = spec.get("tensor", "weight")  # the matrix's local name
        self.softcap = None if spec.get("softcap") is None else float(spec["softcap"])
        self.weight: torch.Tensor | None = None

    def libraries(self, dtype_name):
        return ("stream32",) if self.softcap is not None else ()

    def param_infos(self):
        return {} if self.tied else {self.tensor: ParamInfo((self.vocab, self.hidden))}

    def load(self, tensors):
        self.weight = tensors["weight" if self.tied else self.tensor].contiguous()

    def forward(self, h) -> torch.Tensor:
        logits = self._logits(h)
        return logits if self.softcap is None else ops.softcap(logits, self.softcap)

    def _logits(self, h) -> torch.Tensor:
        if isinstance(h, DeferredNorm):
            rows, norm = h.residual, h.fused()
            if norm is not None and rows.shape[0] <= ops.GEMM_DECODE_NORM_ROWS and decode_product(rows, self.weight):
                h.resolve(None)  # few rows: the product norms them on the way in, and the norm kernel is not launched
                out = torch.empty((rows.shape[0], self.weight.shape[0]), dtype=torch.float32, device=rows.device)
                return ops.gemm_decode(out, rows, self.weight, norm=norm)
            h = h.materialize()
        return linear(h, self.weight, out_dtype=torch.float32)
