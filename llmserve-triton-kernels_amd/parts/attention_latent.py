"""Attention whose keys and values come from one small latent per token, over the paged cache.

Parameters (a `PartSpec` of kind "latent_attention"):
  hidden, num_heads (H), head_dim_plain (dn), head_dim_rotated (dr), value_dim (dv), q_rank, kv_rank (r)
  scale                the scores' factor
  window               a query at i sees j with 0 <= i - j < window (None: every j <= i)
  cache_window         what the cache keeps (the widest window among this layer and the layers that read its cache;
                       None: everything); default: window
  rotary_base, rotary_dims   pairs (2i, 2i+1) of the first rotary_dims numbers of a rotated part are turned by
                       position * base^(-2i / rotary_dims); the rest of the part passes
  rotary_pairing       "neighbours" (default) or "half": dimension i turns together with dimension i + rotary_dims / 2
  rotary_frequencies   the rotary_dims / 2 frequencies themselves, where they are not base^(-2i / rotary_dims)
  eps                  of the two latents' RMS norms (plain weights)
  own_latent           False: the layer has no key/value projection and reads another layer's cache rows
  output_gate          the heads' results are multiplied by sigmoid(W_g h) before the output projection
  num_kv_heads, head_dim   what a cache row looks like to the rest of the engine: 1 and r + dr
  names                local tensor names (defaults: dq, dq.norm, uq, dkv, dkv.norm, uk, uv, g, o)

h -> c_q = rms(W_dq h) w, q = W_uq c_q laid out head by head as [dn plain, dr rotated];
[z_c ; z_r] = W_dkv h, c = rms(z_c) w, k_r = rotated z_r (one for all heads); head a has keys [W_uk,a c ; k_r] and
values W_uv,a c.  A token's cache row is [c ; k_r] and nothing else: the keys' projection is folded into the query,
q'_a = [W_uk,a^T q_a ; q_r,a], so that the score is q'_a . [c ; k_r], and the attention's result over the rows'
c-part is projected by W_uv,a afterwards.  Norms, angles, scores and softmax are 32-bit.
"""

from __future__ import annotations

import torch

from ..ops import library as ops
from .linear import linear
from .registry import Mixer, register_mixer
from .spec import PagedCacheSpec, ParamInfo

_DEFAULT_NAMES = {"dq": "dq", "dq_norm": "dq.norm", "uq": "uq", "dkv": "dkv", "dkv_norm": "dkv.norm", "uk": "uk",
                  "uv": "uv", "g": "g", "o": "o"}


@register_mixer("latent_attention")
class LatentAttention(Mixer):
    graph_safe = True

    def __init__(self, spec, ctx):
        super().__init__(spec, ctx)
        self.hidden = int(spec["hidden"])
        self.heads = int(spec["num_heads"])
        self.dn = int(spec["head_dim_plain"])
        self.dr = int(spec["head_dim_rotated"])
        self.dv = int(spec["value_dim"])
        self.q_rank = int(spec["q_rank"])
        self.r = int(spec["kv_rank"])
        self.scale = float(spec["scale"])
        self.window = None if spec.get("window") is None else int(spec["window"])
        self.cache_window = spec.get("cache_window", self.window)
        self.base = float(spec.get("rotary_base", 10000.0))
        self.dims = int(spec.get("rotary_dims", self.dr))
        self.pairing = spec.get("rotary_pairing", "neighbours")
        self.frequencies = spec.get("rotary_frequencies")
        if self.frequencies is not None and 2 * len(self.frequencies) != self.dims:
            raise ValueError("rotary_frequencies holds a frequency per turned pair")
        self.eps = float(spec["eps"])
        self.own_latent = bool(spec.get("own_latent", True))
        self.output_gate = bool(spec.get("output_gate", True))
        self.names = dict(_DEFAULT_NAMES, **(spec.get("names") or {}))
        if min(self.heads, self.dn, self.dv, self.q_rank, self.r) < 1 or self.dr < 0:
            raise ValueError("sizes must be positive")
        if self.dims % 2 or not 0 <= self.dims <= self.dr:
            raise ValueError(f"rotary_dims={self.dims} must be even and within the rotated part of {self.dr}")
        if self.window is not None and self.window < 1:
            raise ValueError("window must be >= 1")
        if self.r + self.dr > ops.LATENT_ROW_MAX:
            raise ValueError(f"a cache row of {self.r + self.dr} numbers; the kernels take {ops.LATENT_ROW_MAX}")
        if int(spec.get("num_kv_heads", 1)) != 1 or int(spec.get("head_dim", self.r + self.dr)) != self.r + self.dr:
            raise ValueError("a cache row is one head of kv_rank + head_dim_rotated numbers")
        self.w_in = self.w_uq = self.w_absorb = self.w_uv = self.w_o = self.wq_norm = self.wc_norm = self.freq = None

    def libraries(self, dtype_name):
        if dtype_name == "bfloat16" and ops.attend_latent_mfma_supported(torch.bfloat16, self.r, self.dr):
            return ("latent", "grouped_gemm", "latent_mfma")
        return ("latent", "grouped_gemm")

    # ---- what it keeps between steps -------------------------------------------------------------
    def cache_spec(self):
        window = None if self.cache_window is None else int(self.cache_window)
        return PagedCacheSpec(num_kv_heads=1, head_dim=self.r + self.dr, window=window, value_heads=0, value_dim=0)

    # ---- tensors -----------------------------------------------------------------------------------
    def param_infos(self):
        n, w, heads = self.names, self.hidden, self.heads
        infos = {n["dq"]: ParamInfo((self.q_rank, w)), n["dq_norm"]: ParamInfo((self.q_rank,), "norm"),
                 n["uq"]: ParamInfo((heads * (self.dn + self.dr), self.q_rank)),
                 n["uk"]: ParamInfo((heads * self.dn, self.r)), n["uv"]: ParamInfo((heads * self.dv, self.r)),
                 n["o"]: ParamInfo((w, heads * self.dv))}
        if self.own_latent:
            infos[n["dkv"]] = ParamInfo((self.r + self.dr, w))
            infos[n["dkv_norm"]] = ParamInfo((self.r,), "norm")
        if self.output_gate:
            infos[n["g"]] = ParamInfo((heads * self.dv, w))
        return infos

    def load(self, tensors):
        n = self.names
        # every product of h in one: [query latent ; latent and rotated key part ; gate], results in 32-bit
        pieces = [tensors[n["dq"]]] + ([tensors[n["dkv"]]] if self.own_latent else []) + (
            [tensors[n["g"]]] if self.output_gate else [])
        self.w_in = torch.cat(pieces, dim=0).contiguous()
        self.col_c = self.q_rank if self.own_latent else None
        self.col_g = self.q_rank + (self.r + self.dr if self.own_latent else 0)
        self.w_uq = tensors[n["uq"]].contiguous()
        # W_uk [H dn, r] head by head -> [H, r, dn]: the weight of q'_a[:r] = W_uk,a^T q_a
        self.w_absorb = tensors[n["uk"]].reshape(self.heads, self.dn, self.r).transpose(1, 2).contiguous()
        self.w_uv = tensors[n["uv"]].reshape(self.heads, self.dv, self.r).contiguous()
        self.w_o = tensors[n["o"]].contiguous()
        self.wq_norm = tensors[n["dq_norm"]].float().contiguous()
        self.wc_norm = tensors[n["dkv_norm"]].float().contiguous() if self.own_latent else None
        if self.dims and self.frequencies is not None:
            self.freq = torch.tensor([float(f) for f in self.frequencies], dtype=torch.float64).to(torch.float32).to(self.w_o.device)
        elif self.dims:
            exponent = torch.arange(0, self.dims, 2, dtype=torch.float64) / self.dims
            self.freq = (1.0 / (self.base ** exponent)).to(torch.float32).to(self.w_o.device)

    # ---- one step ------------------------------------------------------------------------------------
    def forward(self, x, batch, cache):
        view = batch.groups[cache.group_id]
        heads, dn, dr, dv, r = self.heads, self.dn, self.dr, self.dv, self.r
        rows, dtype, dev = x.shape[0], x.dtype, x.device
        if self.own_latent != bool(cache.store):
            raise ValueError("a layer keeps a latent of its own exactly when it owns its cache")
        z = linear(x, self.w_in, out_dtype=torch.float32)
        cq = torch.empty((rows, self.q_rank), dtype=dtype, device=dev)
        ops.latent_prepare(z, col_q=0, q_rank=self.q_rank, col_c=self.col_c, r=r, dr=dr, wq=self.wq_norm, wc=self.wc_norm,
                           freq=self.freq, positions=batch.positions, eps=self.eps, cq=cq,
                           pool=cache.k_pool if self.own_latent else None, slots=view.slots if self.own_latent else None,
                           pairing=self.pairing)
        q = linear(cq, self.w_uq, out_dtype=torch.float32)
        plain = torch.empty((rows, heads * dn), dtype=dtype, device=dev)
        folded = torch.empty((rows, heads * (r + dr)), dtype=dtype, device=dev)
        ops.latent_query(plain, folded, q, heads=heads, dn=dn, dr=dr, r=r, freq=self.freq, positions=batch.positions,
                         pairing=self.pairing)
        ops.grouped_product(folded.view(rows, heads, r + dr)[:, :, :r], plain.view(rows, heads, dn), self.w_absorb)
        mixed = torch.empty((rows, heads * r), dtype=dtype, device=dev)
        self.attend(mixed, folded, cache, view, batch)
        out = torch.empty((rows, heads * dv), dtype=dtype, device=dev)
        if self.output_gate:
            ops.grouped_product(out.view(rows, heads, dv), mixed.view(rows, heads, r), self.w_uv, epilogue="gated",
                                gate=z, gate_column=self.col_g)
        else:
            ops.grouped_product(out.view(rows, heads, dv), mixed.view(rows, heads, r), self.w_uv)
        return linear(out, self.w_o, out_dtype=torch.float32)

    def attend(self, out, folded, cache, view, batch):
        """out[n, a] = the softmax-weighted sum of the cache rows' latent parts for head a of token n: on the matrix
        cores where the sizes allow (bfloat16), else by the kernel that takes any size and dtype."""
        common = dict(heads=self.heads, r=self.r, dr=self.dr, block_size=cache.block_size, window=int(self.window or 0),
                      scale=self.scale, table_rows=batch.state_slots)
        if not ops.attend_latent_mfma_supported(folded.dtype, self.r, self.dr):
            ops.attend_latent(out, folded, cache.k_pool, view.block_tables, batch.token_seq, batch.positions,
                              batch.context_lens, **common)
            return
        splits = self.key_shares(batch.num_seqs, batch.max_count, batch.max_context, ops.compute_units(folded.device))
        ops.attend_latent_mfma(out, folded, cache.k_pool, view.block_tables, batch.cu_seqlens, batch.context_lens,
                               n_seqs=batch.num_seqs, max_count=batch.max_count, splits=splits, **common)

    def key_shares(self, n_requests: int, max_new: int, max_context: int, cus: int = 256) -> int:
        """Workgroups that share the keys of one block of 64 (token, head) pairs.  While the blocks alone leave
        compute units idle (decoding, short portions), the tiles of 32 keys of each go to several workgroups, two
        tiles a share at least, and a second kernel adds the shares up."""
        blocks = n_requests * -(-max_new * self.heads // ops.LATENT_MFMA_PAIRS)
        reach = max_context if self.window is None else min(max_context, self.window + max_new - 1)
        tiles = -(-reach // ops.LATENT_MFMA_KEYS) + 1
        return max(1, min(16, cus // max(blocks, 1), tiles // 2))
