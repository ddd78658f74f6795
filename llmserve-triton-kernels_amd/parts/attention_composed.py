"""Attention put together from ingredients that its parameters choose, over the paged cache.

Parameters (a `PartSpec` of kind "composed_attention"):
  hidden, num_heads (H), num_kv_heads (G), head_dim (dk, of queries and keys), value_dim (dv; default dk),
  scale                 the scores' factor (default 1 / sqrt(dk))
  window, keep_first    a query at i sees j <= i with i - j < window, and beside them the keys j < keep_first
                        (window None: every earlier key)
  chunk                 a query sees only keys of its own run of `chunk` positions, counted from position 0
  conv_taps             a causal convolution over time on every channel of q, k and v, directly behind the
                        projection: y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros before the sequence (0: none).
                        The last taps - 1 projected rows of a request are its state.
  distance_slope_base   b: slope_h * (i - j) is taken off the scores, slope_h = 2^(-b (h + 1) / H)  (None: no bias)
  talking_heads         the heads' softmax weights are mixed before they meet the values: w_h = sum_g T[h, g] w_g,
                        head h applying its mixed weights to the values of its own key/value head
  differential          two score maps per head over the same values (q and k hold [map 1, map 2] head by head),
                        o = a_1 - lambda a_2 with lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + `diff`
  head_norm_eps         each head's result is divided by its root mean square (eps inside the root), no weight,
                        and multiplied by `head_norm_scale` (None: no such norm)
  bias                  q, k and v have biases (tensors "<name>.b"), added in the projection
  qk_norm_eps           every head of q and of k is RMS-normed over its dk numbers with a weight of size dk that all
                        heads share (tensors "q.norm", "k.norm"; eps inside the root); None: no such norm
  qk_norm_weight        False: that norm has no weight (and no tensors)
  rotary                {base, dims, scaling}: before that norm the first `dims` numbers of every head of q and k are
                        turned by the position, dimension i together with dimension i + dims / 2 by the angle
                        p * f_i, f_i = base^(-2i / dims); `scaling` {factor, low, high, original} stretches long
                        wavelengths (see `scaled_frequencies`); None: no rotation
  sink                  the softmax's denominator holds one more term exp(0): a key of score zero without a value
  query_temperature     {coef, every}: q at position p is multiplied by 1 + coef ln(floor((p + 1) / every) + 1)
  distance_table        {rows: B, farthest: D}: a learned bias per head and distance, tensor "rel" [B, H], added to the
                        scaled score: rel[bucket(i - j), h] with bucket(n) = n for n < B/2 and
                        min(B - 1, B/2 + floor(ln(n / (B/2)) / ln(D / (B/2)) (B - B/2))) beyond
  output_gate           the heads' results are multiplied by sigmoid(W_g h) (tensor "g") before the output projection
  result                "float32": the output projection's result stays unrounded (for a 32-bit residual stream)
  names                 local tensor names (defaults: q, k, v, o, q.conv, k.conv, v.conv, talk, lq1, lk1, lq2, lk2,
                        q.b, k.b, v.b, q.norm, k.norm, rel, g)

Scores, softmax, the mixing of heads, the difference of the maps and the head norm are computed in 32-bit; the
convolution is computed in 32-bit from the unrounded projection and rounded once.  Keys are cached as [pages,
G * maps, block, dk] and values as [pages, G, dv, block]; a windowed or chunked layer gives the pages that no
later query can reach back while the request runs.
"""

from __future__ import annotations

import math

import torch

from ..ops import library as ops
from .linear import linear
from .registry import Mixer, register_mixer
from .spec import PagedCacheSpec, ParamInfo, StateCacheSpec

_DEFAULT_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "q_conv": "q.conv", "k_conv": "k.conv", "v_conv": "v.conv",
                  "talk": "talk", "lq1": "lq1", "lk1": "lk1", "lq2": "lq2", "lk2": "lk2", "q_bias": "q.b", "k_bias": "k.b",
                  "v_bias": "v.b", "q_norm": "q.norm", "k_norm": "k.norm", "rel": "rel", "g": "g"}


def distance_bucket(n: int, rows: int, farthest: int) -> int:
    """Row of a distance table of `rows` rows for the distance n >= 0: a row per distance below rows / 2, then rows
    whose spans grow geometrically up to `farthest`; everything beyond shares the last row."""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(farthest / half) * (rows - half))))


def bias_by_distance(table: torch.Tensor, farthest: int) -> torch.Tensor:
    """table [rows, H] -> float32 [H, R + 1] with the bias of every distance 0 .. R, R being the first distance from
    which the last row holds for good: what the attention kernels index by min(i - j, R)."""
    rows = table.shape[0]
    reach = max(int(farthest), rows // 2)
    while reach > 0 and distance_bucket(reach - 1, rows, farthest) == rows - 1:
        reach -= 1
    index = torch.tensor([distance_bucket(n, rows, farthest) for n in range(reach + 1)], dtype=torch.long,
                         device=table.device)
    return table.float()[index].t().contiguous()


def scaled_frequencies(base: float, dims: int, scaling: dict | None = None) -> list[float]:
    """f_i = base^(-2i / dims) for i < dims / 2.  With `scaling` {factor, low, high, original} a frequency whose
    wavelength 2 pi / f lies below original / high stays, one beyond original / low is divided by factor, and between
    the two it is (1 - s) f / factor + s f with s = (original / wavelength - low) / (high - low)."""
    out = []
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        if scaling:
            factor, low, high, original = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
            wavelength = 2.0 * math.pi / f
            if wavelength > original / low:
                f = f / factor
            elif wavelength >= original / high:
                s = (original / wavelength - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return out


def _fill_rel(shape, generator, device, options):
    """A distance table: moderate biases."""
    return 0.5 * torch.randn(shape, generator=generator, dtype=torch.float32, device=device)


def _fill_taps(shape, generator, device, options):
    """Taps of a short convolution: the newest tap near one, the older ones smaller."""
    w = 0.3 * torch.randn(shape, generator=generator, dtype=torch.float32, device=device)
    w[:, -1] += 1.0
    return w


def _fill_talk(shape, generator, device, options):
    """A mixing matrix of heads: near the identity."""
    w = 0.2 * torch.randn(shape, generator=generator, dtype=torch.float32, device=device)
    return w + torch.eye(shape[0], dtype=torch.float32, device=device)


@register_mixer("composed_attention")
class ComposedAttention(Mixer):
    graph_safe = True

    def __init__(self, spec, ctx):
        super().__init__(spec, ctx)
        self.hidden = int(spec["hidden"])
        self.num_heads = int(spec["num_heads"])
        self.num_kv_heads = int(spec["num_kv_heads"])
        self.head_dim = int(spec["head_dim"])
        self.value_dim = int(spec.get("value_dim") or self.head_dim)
        self.scale = float(spec["scale"]) if spec.get("scale") is not None else 1.0 / math.sqrt(self.head_dim)
        self.window = spec.get("window")
        self.keep_first = int(spec.get("keep_first") or 0) if self.window is not None else 0
        self.chunk = spec.get("chunk")
        self.taps = int(spec.get("conv_taps") or 0)
        self.slope_base = spec.get("distance_slope_base")
        self.talking = bool(spec.get("talking_heads", False))
        self.differential = bool(spec.get("differential", False))
        self.diff = float(spec.get("diff", 0.0))
        self.head_norm_eps = spec.get("head_norm_eps")
        self.head_norm_scale = float(spec.get("head_norm_scale", 1.0))
        self.result_dtype = torch.float32 if spec.get("result", "model") == "float32" else None
        self.names = dict(_DEFAULT_NAMES, **(spec.get("names") or {}))
        self.maps = 2 if self.differential else 1
        self.bias = bool(spec.get("bias", False))
        self.qk_norm_eps = spec.get("qk_norm_eps")
        self.qk_norm_weight = bool(spec.get("qk_norm_weight", True))
        rotary = spec.get("rotary") or None
        self.rot_dims = int(rotary.get("dims", 0)) if rotary else 0
        self.rot_freq = scaled_frequencies(float(rotary.get("base", 10000.0)), self.rot_dims, rotary.get("scaling")) \
            if self.rot_dims else None
        self.sink = bool(spec.get("sink", False))
        self.freq = None
        temp = spec.get("query_temperature") or {}
        self.temp_coef, self.temp_every = float(temp.get("coef", 0.0)), int(temp.get("every", 0))
        table = spec.get("distance_table")
        self.rel_rows = int(table["rows"]) if table else 0
        self.rel_farthest = int(table["farthest"]) if table else 0
        self.output_gate = bool(spec.get("output_gate", False))
        if table and (self.rel_rows < 2 or self.rel_farthest <= self.rel_rows // 2):
            raise ValueError("a distance table has at least 2 rows and reaches beyond the distances that have a row each")
        if (self.qk_norm_eps is not None or self.temp_every or self.rot_dims) and self.taps > 0:
            raise ValueError("normed, turned or position-scaled queries do not go together with a convolution")
        if self.rot_dims % 2 or not 0 <= self.rot_dims <= self.head_dim:
            raise ValueError(f"rotary.dims={self.rot_dims} must be even and at most head_dim={self.head_dim}")
        if self.rot_dims and self.differential:
            raise ValueError("a rotation and two score maps per head do not go together")
        if self.temp_every < 0:
            raise ValueError("query_temperature.every must be positive")
        self.dist_bias = self.q_norm = self.k_norm = self.in_bias = None
        if self.num_heads % self.num_kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        for name in ("window", "chunk"):
            value = getattr(self, name)
            if value is not None and int(value) < 1:
                raise ValueError(f"{name} must be >= 1")
        if self.talking and self.differential:
            raise ValueError("mixing the heads' weights and two score maps per head do not go together")
        lds = ops.attend_composed_lds_bytes(self.num_heads, self.maps, self.head_dim, self.value_dim, self.talking)
        if lds > ops.ATTEND_COMPOSED_LDS:
            raise ValueError(f"{self.num_heads} heads of sizes {self.head_dim} and {self.value_dim} need {lds} bytes "
                             f"of LDS per token; the kernel has {ops.ATTEND_COMPOSED_LDS}")
        self.cq = self.num_heads * self.maps * self.head_dim
        self.ck = self.num_kv_heads * self.maps * self.head_dim
        self.cv = self.num_kv_heads * self.value_dim
        self.qkv_weight = self.o_weight = self.taps_w = self.talk = self.slopes = None
        self.lam = 0.0

    def libraries(self, dtype_name):
        if dtype_name != "bfloat16":
            return ("attention_composed",)
        names = ("attention_composed", "attention_composed_mfma")
        return names + ("attention_biased",) if self.plain_but_for_bias_and_gate else names

    @property
    def plain_but_for_bias_and_gate(self) -> bool:
        """One score map over every earlier key, with nothing between the scores and the values but a distance table,
        and nothing behind them but a gate: what the prompt kernel of the plain attention takes in its variant with a
        table (keys and values of one size of 32, 64, 96 or 128)."""
        return (self.rel_rows > 0 and self.maps == 1 and self.window is None and self.chunk is None and not self.talking
                and self.slope_base is None and self.head_norm_eps is None and self.head_dim == self.value_dim
                and self.head_dim in (32, 64, 96, 128))

    # ---- what it keeps between steps -------------------------------------------------------------
    def cache_spec(self):
        paged = PagedCacheSpec(num_kv_heads=self.num_kv_heads * self.maps, head_dim=self.head_dim,
                               window=None if self.window is None else int(self.window), keep_first=self.keep_first,
                               chunk=None if self.chunk is None else int(self.chunk),
                               value_heads=self.num_kv_heads, value_dim=self.value_dim)
        if self.taps > 1:
            return (paged, StateCacheSpec((self.taps - 1, self.cq + self.ck + self.cv), "float32"))
        return paged

    # ---- tensors -----------------------------------------------------------------------------------
    def param_infos(self):
        n, h = self.names, self.hidden
        infos = {n["q"]: ParamInfo((self.cq, h)), n["k"]: ParamInfo((self.ck, h)), n["v"]: ParamInfo((self.cv, h)),
                 n["o"]: ParamInfo((h, self.num_heads * self.value_dim))}
        if self.taps > 0:
            for key, channels in (("q_conv", self.cq), ("k_conv", self.ck), ("v_conv", self.cv)):
                infos[n[key]] = ParamInfo((channels, self.taps), _fill_taps)
        if self.talking:
            infos[n["talk"]] = ParamInfo((self.num_heads, self.num_heads), _fill_talk)
        if self.differential:
            for key in ("lq1", "lk1", "lq2", "lk2"):
                infos[n[key]] = ParamInfo((self.head_dim,), "around_zero")
        if self.bias:
            for key, channels in (("q_bias", self.cq), ("k_bias", self.ck), ("v_bias", self.cv)):
                infos[n[key]] = ParamInfo((channels,), "around_zero")
        if self.qk_norm_eps is not None and self.qk_norm_weight:
            infos[n["q_norm"]] = ParamInfo((self.head_dim,), "norm")
            infos[n["k_norm"]] = ParamInfo((self.head_dim,), "norm")
        if self.rel_rows:
            infos[n["rel"]] = ParamInfo((self.rel_rows, self.num_heads), _fill_rel)
        if self.output_gate:
            infos[n["g"]] = ParamInfo((self.num_heads * self.value_dim, h))
        return infos

    def load(self, tensors):
        n = self.names
        dev = tensors[n["q"]].device
        pieces = [tensors[n[x]] for x in "qkv"] + ([tensors[n["g"]]] if self.output_gate else [])
        self.qkv_weight = torch.cat(pieces, dim=0).contiguous()  # (the gate's rows lie behind those of q, k and v)
        self.o_weight = tensors[n["o"]].contiguous()
        if self.bias:
            biases = [tensors[n[x + "_bias"]] for x in "qkv"]
            if self.output_gate:
                biases.append(torch.zeros(self.num_heads * self.value_dim, dtype=biases[0].dtype, device=dev))
            self.in_bias = torch.cat(biases).contiguous()
        if self.rot_dims:
            self.freq = torch.tensor(self.rot_freq, dtype=torch.float64).to(torch.float32).to(dev)
        if self.qk_norm_eps is not None and self.qk_norm_weight:
            self.q_norm, self.k_norm = tensors[n["q_norm"]].float().contiguous(), tensors[n["k_norm"]].float().contiguous()
        if self.rel_rows:
            self.dist_bias = bias_by_distance(tensors[n["rel"]], self.rel_farthest)
        if self.taps > 0:
            self.taps_w = torch.cat([tensors[n[x + "_conv"]].float() for x in "qkv"], dim=0).contiguous()
        if self.talking:
            self.talk = tensors[n["talk"]].float().contiguous()
        if self.slope_base is not None:
            heads = self.num_heads
            self.slopes = torch.tensor([2.0 ** (-float(self.slope_base) * (i + 1) / heads) for i in range(heads)],
                                       dtype=torch.float32, device=dev)
        if self.differential:  # one number for the layer, worked out once
            dot = [float((tensors[n[a]].double() * tensors[n[b]].double()).sum()) for a, b in (("lq1", "lk1"), ("lq2", "lk2"))]
            self.lam = math.exp(dot[0]) - math.exp(dot[1]) + self.diff

    # ---- one step ------------------------------------------------------------------------------------
    @property
    def input_weight(self):
        """The stacked q, k, v projection: an arrangement may fold it into a product of its own (32-bit result) and
        hand the result back as `projected`.  (None where the projection has biases, which such a product lacks.)"""
        return None if self.bias else self.qkv_weight

    @input_weight.setter
    def input_weight(self, weight):
        self.qkv_weight = weight

    def forward(self, x, batch, cache, projected=None):
        paged, state = cache if isinstance(cache, tuple) else (cache, None)
        view = batch.groups[paged.group_id]
        heads, kv, dk, dv = self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim
        # q, k and v side by side, unrounded
        proj = projected if projected is not None else linear(x, self.qkv_weight, self.in_bias, out_dtype=torch.float32)
        q = torch.empty((proj.shape[0], self.cq), dtype=x.dtype, device=x.device)
        gate = proj[:, self.cq + self.ck + self.cv:] if self.output_gate else None
        if self.qk_norm_eps is not None or self.temp_every or self.rot_dims:
            ops.norm_store(q, proj, q_heads=heads * self.maps, k_heads=kv * self.maps, dk=dk, v_heads=kv, dv=dv,
                           q_norm=self.q_norm, k_norm=self.k_norm, eps=float(self.qk_norm_eps or 0.0),
                           temp_coef=self.temp_coef, temp_every=self.temp_every, positions=batch.positions,
                           slots=view.slots if paged.store else None, k_pool=paged.k_pool, v_pool=paged.v_pool,
                           block_size=paged.block_size, freq=self.freq,
                           unit_norm=self.qk_norm_eps is not None and not self.qk_norm_weight)
            out = torch.empty((proj.shape[0], heads * dv), dtype=x.dtype, device=x.device)
            self.attend(out, q, paged, view, batch, gate)
            return linear(out, self.o_weight, out_dtype=self.result_dtype)
        if self.output_gate:
            proj = proj[:, : self.cq + self.ck + self.cv]
        conv, taps = self.taps > 1, self.taps > 0  # (one tap is a factor per channel and needs no state)
        single = conv and batch.max_count == 1 and batch.num_seqs == proj.shape[0]  # every request brings one token
        ops.conv_store(q, proj, cq=self.cq, k_heads=kv * self.maps, dk=dk, v_heads=kv, dv=dv,
                       taps_w=self.taps_w if taps else None,
                       state=state.state if conv else None, state_slots=batch.state_slots if conv else None,
                       token_seq=batch.token_seq if taps else None, positions=batch.positions if taps else None,
                       cu_seqlens=batch.cu_seqlens if taps else None, slots=view.slots if paged.store else None,
                       k_pool=paged.k_pool, v_pool=paged.v_pool, block_size=paged.block_size, update_state=single,
                       context_lens=batch.context_lens if single else None)
        if conv and not single:
            ops.conv_state(state.state, proj, batch.state_slots, batch.cu_seqlens, batch.context_lens)
        out = torch.empty((proj.shape[0], heads * dv), dtype=x.dtype, device=x.device)
        self.attend(out, q, paged, view, batch, gate)
        return linear(out, self.o_weight, out_dtype=self.result_dtype)

    def attend(self, out, q, paged, view, batch, gate=None):
        """out[n] = this attention of token n's heads over its request's pages: on the matrix cores where the
        sizes allow (bfloat16; requests that bring one token in one launch, portions of prompts in another), else
        by the kernel that takes any size and dtype."""
        common = dict(heads=self.num_heads, kv_heads=self.num_kv_heads, dk=self.head_dim, dv=self.value_dim,
                      block_size=paged.block_size, scale=self.scale, maps=self.maps, window=int(self.window or 0),
                      keep_first=self.keep_first, chunk=int(self.chunk or 0), slopes=self.slopes, talk=self.talk,
                      lam=self.lam, head_norm=self.head_norm_eps is not None, eps=float(self.head_norm_eps or 0.0),
                      out_scale=self.head_norm_scale, table_rows=batch.state_slots)
        if (self.sink and self.talking) or (gate is not None and (self.talking or gate.data_ptr() % 16 or gate.stride(0) % 4)) or \
                not ops.attend_composed_mfma_supported(
                q.dtype, self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim, paged.block_size, self.talking):
            ops.attend_composed(out, q, paged.k_pool, paged.v_pool, view.block_tables, batch.token_seq, batch.positions,
                                context_lens=batch.context_lens, dist_bias=self.dist_bias, gate=gate, sink=self.sink,
                                **common)
            return
        args = (out, q, paged.k_pool, paged.v_pool, view.block_tables, batch.cu_seqlens, batch.context_lens)
        common.update(dist_bias=self.dist_bias, gate=gate, sink=self.sink)
        n_dec = batch.num_decode
        if n_dec:
            ops.attend_composed_mfma(*args, 0, n_dec, 1, shares=self.decode_shares(n_dec, batch.max_decode_context,
                                                                                  ops.compute_units(q.device)), **common)
        if n_dec < batch.num_seqs and self.plain_but_for_bias_and_gate and \
                ops.attention_prompt_biased_supported(q.dtype, self.head_dim, self.value_dim, paged.block_size) and \
                (gate is None or (gate.data_ptr() % 16 == 0 and gate.stride(0) % 4 == 0)) and q.stride(0) % 8 == 0:
            # portions of prompts: the plain attention's kernel (keys and values shared by a workgroup's waves through LDS)
            ops.attention_prompt_biased(out, q, paged.k_pool, paged.v_pool, view.block_tables, batch.cu_seqlens,
                                        batch.context_lens, n_dec, batch.num_seqs - n_dec, batch.max_count, n_dec,
                                        batch.num_tokens - n_dec, n_heads=self.num_heads, n_kv_heads=self.num_kv_heads,
                                        head_dim=self.head_dim, block_size=paged.block_size, scale=self.scale,
                                        dist_bias=self.dist_bias, gate=gate, table_rows=batch.state_slots)
            return
        if n_dec < batch.num_seqs:
            shares = self.prompt_shares(batch.num_seqs - n_dec, batch.max_count, batch.max_context,
                                        ops.compute_units(q.device))
            ops.attend_composed_mfma(*args, n_dec, batch.num_seqs - n_dec, batch.max_count, shares=shares, **common)

    def prompt_shares(self, n_requests: int, max_new: int, max_context: int, cus: int = 256) -> int:
        """Workgroups that share the keys of one block of prompt tokens when the heads' weights are mixed.  All heads
        of a block are one workgroup; while the blocks alone leave compute units idle, the keys of each go to up to 4
        workgroups of 256 keys at least (measured at 32 heads of 64 in chunks of 1,024: a portion of 512 tokens 210 ->
        97 microseconds with 4 shares; 2,048 tokens are a workgroup for every compute unit and gain nothing)."""
        if not self.talking:
            return 1
        tokens = ops.attend_composed_mfma_tokens(self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim, max_new)
        if tokens <= 0:
            return 1
        blocks = n_requests * -(-max_new // tokens)
        reach = min(x for x in (max_context, self.chunk) if x is not None)
        return max(1, min(4, cus // max(blocks, 1), int(reach) // 256))

    def decode_shares(self, n_requests: int, max_context: int, cus: int = 256) -> int:
        """Workgroups that share the keys of one decoding request when the heads' weights are mixed.  Such a request is
        one workgroup (all its heads must meet for the mixing), which alone keeps one compute unit busy for as long
        as its keys last; while the batch leaves compute units idle its keys go to several, down to one group of 64
        keys a share, at the price of two more launches (measured at batch 8 behind 520 keys, 32 heads of 64: 71
        microseconds in one workgroup of 16 waves, 43 in 4 shares, 26 in 12)."""
        if not self.talking:
            return 1
        reach = min(x for x in (max_context, self.chunk, None if self.window is None else self.window + self.keep_first)
                    if x is not None)
        return max(1, min(16, cus // max(n_requests, 1), -(-int(reach) // 64)))
