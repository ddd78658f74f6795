"""Python face of the HIP kernels: loads the compiled libraries with ctypes and checks,
on the host, every shape and dtype a kernel relies on before launching it.

There is no fallback: a call fails with `KernelLibraryError` when its library cannot be
built or loaded, and with `ValueError` when the arguments are not what the kernel takes.
Kernels run on the current torch stream of the tensors' device.
"""

from __future__ import annotations

import ctypes
import math
import os
import threading

import torch

from . import build as _build

c_void_p, c_int, c_float = ctypes.c_void_p, ctypes.c_int, ctypes.c_float


class KernelLibraryError(RuntimeError):
    pass


_DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 1}
_libs: dict[str, ctypes.CDLL] = {}
_lock = threading.Lock()


def load(name: str) -> ctypes.CDLL:
    """The compiled library of ``csrc/<name>.hip`` (built at the first call if need be)."""
    lib = _libs.get(name)
    if lib is not None:
        return lib
    with _lock:
        if name in _libs:
            return _libs[name]
        try:
            path = _build.build([name])[name]
            lib = ctypes.CDLL(str(path))
        except (OSError, _build.BuildError) as e:
            raise KernelLibraryError(f"HIP kernel library '{name}' is not available: {e}") from e
        _libs[name] = lib
        return lib


def ensure_built(dtype_name: str, verbose: bool = True, extra=None) -> None:
    """Compile (if missing, side by side) and load the libraries a model of this dtype uses: with `extra` (what the
    model's parts name) the products and elementwise kernels and those; without, the Llama decoder's."""
    names = _build.GROUPS[dtype_name] if extra is None else tuple(dict.fromkeys(_build.BASE[dtype_name] + tuple(extra)))
    _build.build(names, verbose=verbose)
    for n in names:
        load(n)


def loaded_libraries() -> dict[str, str]:
    return {k: v._name for k, v in _libs.items()}


# ------------------------------------------------------------------------------ checks


def _code(t: torch.Tensor) -> int:
    try:
        return _DTYPE_CODE[t.dtype]
    except KeyError:
        raise ValueError(f"kernels take float32 or bfloat16 tensors, not {t.dtype}") from None


def _dev(*tensors: torch.Tensor | None) -> torch.device:
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise ValueError("kernels take GPU tensors only (there is no CPU path)")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise ValueError(f"tensors on different devices: {dev} and {t.device}")
    return dev


def _ptr(t: torch.Tensor | None) -> c_void_p:
    return c_void_p(0 if t is None else t.data_ptr())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(dev: torch.device) -> c_void_p:
    """torch's current stream on `dev` (under graph capture: the capturing stream), as a raw handle."""
    if _raw_stream is not None:  # the same handle without building a Stream object (a launch costs less host time)
        return c_void_p(_raw_stream(dev.index if dev.index is not None else torch.cuda.current_device()))
    return c_void_p(torch.cuda.current_stream(dev).cuda_stream)


def _i32(t: torch.Tensor, name: str, numel: int | None = None) -> None:
    if t.dtype != torch.int32 or not t.is_contiguous():
        raise ValueError(f"{name} must be a contiguous int32 tensor")
    if numel is not None and t.numel() != numel:
        raise ValueError(f"{name} has {t.numel()} elements, expected {numel}")


def _f32(t: torch.Tensor, name: str, numel: int | None = None) -> None:
    if t.dtype != torch.float32 or not t.is_contiguous():
        raise ValueError(f"{name} must be a contiguous float32 tensor")
    if numel is not None and t.numel() != numel:
        raise ValueError(f"{name} has {t.numel()} elements, expected {numel}")


def _rows(t: torch.Tensor, name: str, cols: int | None = None) -> None:
    if t.dim() != 2 or t.stride(1) != 1 or not t.is_contiguous():
        raise ValueError(f"{name} must be a contiguous 2-d tensor, got shape {tuple(t.shape)} stride {t.stride()}")
    if cols is not None and t.shape[1] != cols:
        raise ValueError(f"{name} has {t.shape[1]} columns, expected {cols}")


def _check(status: int, what: str) -> None:
    if status != 0:
        raise KernelLibraryError(f"{what}: kernel launcher returned {status} (see stderr)")


# ------------------------------------------------------------------------------ elementwise


def embed_gather(out: torch.Tensor, table: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
    """out[n] = table[ids[n]]; out [N,H], table [V,H], ids int32 [N]."""
    dev = _dev(out, table, ids)
    _rows(out, "out")
    _rows(table, "table", out.shape[1])
    _i32(ids, "ids", out.shape[0])
    if out.dtype != table.dtype:
        raise ValueError("out and table differ in dtype")
    if out.shape[0] == 0:
        return out
    _check(load("elementwise").llms_embed_gather(
        c_int(_code(out)), _ptr(out), _ptr(table), _ptr(ids), c_int(out.shape[0]), c_int(out.shape[1]),
        c_int(table.shape[0]), _stream(dev)), "embed_gather")
    return out


def rmsnorm(out: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, eps: float, *,
            delta: torch.Tensor | None = None, resid_out: torch.Tensor | None = None,
            rows: torch.Tensor | None = None) -> torch.Tensor:
    """out[r] = weight * norm(x[s] + delta[s]), s = rows[r] or r; resid_out[s] = x[s] + delta[s].
    `delta` may be a float32 [S, N, hidden] tensor of partial sums (ops.gemm_stream(k_splits=S)): it then
    stands for their sum in order, rounded to the dtype of x."""
    dev = _dev(out, x, weight, delta, resid_out, rows)
    _rows(x, "x")
    hidden = x.shape[1]
    parts, n_parts, part_stride = None, 0, 0
    if delta is not None and delta.dim() == 3:
        if delta.dtype != torch.float32 or tuple(delta.shape[1:]) != tuple(x.shape) or not delta.is_contiguous():
            raise ValueError("partial sums must be a contiguous float32 [S, rows, hidden] tensor matching x")
        parts, n_parts, part_stride, delta = delta, delta.shape[0], delta.stride(0), None
    _rows(out, "out", hidden)
    n_out = out.shape[0]
    if weight.dim() != 1 or weight.numel() != hidden or not weight.is_contiguous():
        raise ValueError(f"weight must have {hidden} elements")
    for name, t in (("delta", delta), ("resid_out", resid_out)):
        if t is not None:
            _rows(t, name, hidden)
            if t.shape != x.shape or t.dtype != x.dtype:
                raise ValueError(f"{name} must match x in shape and dtype")
    if out.dtype != x.dtype or weight.dtype != x.dtype:
        raise ValueError("out, x and weight must share one dtype")
    if rows is not None:
        _i32(rows, "rows", n_out)
        if resid_out is not None:
            raise ValueError("a row gather cannot also write the residual back")
    elif n_out != x.shape[0]:
        raise ValueError("out and x differ in rows")
    if n_out == 0:
        return out
    _check(load("elementwise").llms_rmsnorm(
        c_int(_code(x)), _ptr(out), _ptr(x), _ptr(delta), _ptr(resid_out), _ptr(weight), _ptr(rows),
        c_float(eps), c_int(n_out), c_int(hidden), _ptr(parts), c_int(n_parts), ctypes.c_size_t(part_stride),
        _stream(dev)), "rmsnorm")
    return out


def rope_store(qkv: torch.Tensor, inv_freq: torch.Tensor | None, positions: torch.Tensor,
               slots: torch.Tensor | None, k_pool: torch.Tensor | None, v_pool: torch.Tensor | None,
               n_heads: int, n_kv_heads: int, head_dim: int, block_size: int) -> None:
    """Rotate q (in place) and k, store k and v of each token at its cache slot.

    qkv [N, (n_heads + 2 n_kv_heads) * head_dim]; k_pool [pages, n_kv_heads, block_size, head_dim];
    v_pool [pages, n_kv_heads, head_dim, block_size]; slots int32 [N] (page * block_size + offset, or -1).
    """
    dev = _dev(qkv, inv_freq, positions, slots, k_pool, v_pool)
    _rows(qkv, "qkv", (n_heads + 2 * n_kv_heads) * head_dim)
    n = qkv.shape[0]
    _i32(positions, "positions", n)
    if inv_freq is not None:
        _f32(inv_freq, "inv_freq", head_dim // 2)
    if slots is not None:
        _i32(slots, "slots", n)
        if k_pool is None or v_pool is None:
            raise ValueError("slots given without pools")
        pages = k_pool.shape[0]
        if tuple(k_pool.shape) != (pages, n_kv_heads, block_size, head_dim) or not k_pool.is_contiguous():
            raise ValueError(f"k_pool shape {tuple(k_pool.shape)} is not [pages,{n_kv_heads},{block_size},{head_dim}]")
        if tuple(v_pool.shape) != (pages, n_kv_heads, head_dim, block_size) or not v_pool.is_contiguous():
            raise ValueError(f"v_pool shape {tuple(v_pool.shape)} is not [pages,{n_kv_heads},{head_dim},{block_size}]")
        if k_pool.dtype != qkv.dtype or v_pool.dtype != qkv.dtype:
            raise ValueError("pools and qkv differ in dtype")
    if n == 0:
        return
    _check(load("elementwise").llms_rope_store(
        c_int(_code(qkv)), _ptr(qkv), _ptr(inv_freq), _ptr(positions), _ptr(slots), _ptr(k_pool), _ptr(v_pool),
        c_int(n), c_int(n_heads), c_int(n_kv_heads), c_int(head_dim), c_int(block_size), _stream(dev)),
        "rope_store")


def rotary_angles(positions: torch.Tensor, inv_freq: torch.Tensor) -> torch.Tensor:
    """float32 [N, half, 2]: (sine, cosine) of positions[n] * inv_freq[i], by the arithmetic of the kernels that
    rotate: a step's angles worked out once, for every layer's product with the rotary epilogue to read."""
    dev = _dev(positions, inv_freq)
    _i32(positions, "positions")
    _f32(inv_freq, "inv_freq")
    n, half = positions.numel(), inv_freq.numel()
    out = torch.empty((n, half, 2), dtype=torch.float32, device=dev)
    if n and half:
        _check(load("elementwise").llms_rotary_angles(_ptr(out), _ptr(positions), _ptr(inv_freq), c_int(n), c_int(half),
                                                      _stream(dev)), "rotary_angles")
    return out


def scatter_i32(dst: torch.Tensor, index: torch.Tensor, value: torch.Tensor) -> None:
    """dst.flatten()[index[i]] = value[i] wherever index[i] >= 0.  The caller has checked the indices."""
    dev = _dev(dst, index, value)
    if dst.dtype != torch.int32 or not dst.is_contiguous():
        raise ValueError("dst must be a contiguous int32 tensor")
    _i32(index, "index")
    _i32(value, "value", index.numel())
    if index.numel() == 0:
        return
    _check(load("elementwise").llms_scatter_i32(_ptr(dst), _ptr(index), _ptr(value), c_int(index.numel()),
                                                _stream(dev)), "scatter_i32")


def silu_mul(out: torch.Tensor, gate_up: torch.Tensor) -> torch.Tensor:
    """out = silu(gate_up[:, :I]) * gate_up[:, I:]."""
    dev = _dev(out, gate_up)
    _rows(out, "out")
    _rows(gate_up, "gate_up", 2 * out.shape[1])
    if out.shape[0] != gate_up.shape[0] or out.dtype != gate_up.dtype:
        raise ValueError("out and gate_up disagree")
    if out.shape[0] == 0:
        return out
    _check(load("elementwise").llms_silu_mul(
        c_int(_code(out)), _ptr(out), _ptr(gate_up), c_int(out.shape[0]), c_int(out.shape[1]), _stream(dev)),
        "silu_mul")
    return out


# ------------------------------------------------------------------------------ matrix products


def gemm_fma(out: torch.Tensor, a: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    """out[M,N] = a[M,K] w[N,K]^T (+ bias): 32-bit multiply-add on the vector units."""
    dev = _dev(out, a, w, bias)
    if a.dim() != 2 or a.stride(1) != 1 or out.dim() != 2 or out.stride(1) != 1:
        raise ValueError("a and out must be 2-d with unit inner stride")
    _rows(w, "w", a.shape[1])
    m, k = a.shape
    n = w.shape[0]
    if tuple(out.shape) != (m, n):
        raise ValueError(f"out shape {tuple(out.shape)} is not {(m, n)}")
    if a.dtype != w.dtype or (bias is not None and (bias.dtype != w.dtype or bias.numel() != n)):
        raise ValueError("a, w and bias must share one dtype; bias has N elements")
    if (a.dtype, out.dtype) not in ((torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16),
                                    (torch.bfloat16, torch.float32)):
        raise ValueError(f"gemm_fma does not take {a.dtype} -> {out.dtype}")
    if m == 0:
        return out
    _check(load("gemm").llms_gemm_fma(
        c_int(_code(a)), c_int(_code(out)), _ptr(out), _ptr(a), _ptr(w), _ptr(bias), c_int(m), c_int(n), c_int(k),
        c_int(a.stride(0)), c_int(out.stride(0)), _stream(dev)), "gemm_fma")
    return out


def gemm_bf16_supported(a: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether the matrix-core kernels take these operands (else `gemm_fma` does)."""
    k = a.shape[1]
    return (a.dtype == torch.bfloat16 and k % 8 == 0 and a.stride(0) % 8 == 0 and a.data_ptr() % 16 == 0
            and w.data_ptr() % 16 == 0)


def gemm_bf16(out: torch.Tensor, a: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None = None,
              kernel: str | None = None) -> torch.Tensor:
    """out[M,N] (bfloat16 or float32) = a[M,K] w[N,K]^T (+ bias) on the matrix cores, 32-bit sums.
    `kernel`: "stream" (M <= 16), "skinny" (M <= 64) or "tile"; default by M."""
    dev = _dev(out, a, w, bias)
    if a.dim() != 2 or a.stride(1) != 1 or out.dim() != 2 or out.stride(1) != 1:
        raise ValueError("a and out must be 2-d with unit inner stride")
    _rows(w, "w", a.shape[1])
    m, k = a.shape
    n = w.shape[0]
    if tuple(out.shape) != (m, n):
        raise ValueError(f"out shape {tuple(out.shape)} is not {(m, n)}")
    if a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise ValueError("gemm_bf16 takes bfloat16 operands")
    if bias is not None and (bias.dtype != torch.bfloat16 or bias.numel() != n or not bias.is_contiguous()):
        raise ValueError("bias must be a contiguous bfloat16 vector of N elements")
    if out.dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("gemm_bf16 stores bfloat16 or float32")
    if not gemm_bf16_supported(a, w):
        raise ValueError(f"gemm_bf16 needs K ({k}) and the row stride of a ({a.stride(0)}) to be multiples of 8 "
                         "and 16-byte aligned operands")
    if m == 0:
        return out
    kernel = kernel or ("stream" if m <= 16 else "skinny" if m <= 64 else "tile")
    if kernel == "stream":
        return gemm_stream(out, a, w, bias)
    if kernel == "skinny" and m > 64:
        raise ValueError("the skinny kernel takes at most 64 rows")
    lib = load("gemm_mfma")
    fn = {"skinny": lib.llms_gemm_bf16_skinny, "tile": lib.llms_gemm_bf16_tile}[kernel]
    _check(fn(c_int(_code(out)), _ptr(out), _ptr(a), _ptr(w), _ptr(bias), c_int(m), c_int(n), c_int(k),
              c_int(a.stride(0)), c_int(out.stride(0)), _stream(dev)), f"gemm_bf16[{kernel}]")
    return out


def gemm_stream(out: torch.Tensor, x: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None = None, *,
                swiglu: bool = False, rope: dict | None = None, k_splits: int = 1) -> torch.Tensor:
    """The product for up to 64 bfloat16 rows (built for up to 16), with what surrounds it fused in.

    plain:   out[M, N] = x w^T (+ bias).
    swiglu:  w = [gate; up] ([2I, K]); out[M, I] = silu(gate) * up.
    rope = dict(n_heads, n_kv_heads, head_dim, inv_freq | None, positions, slots | None, k_pool, v_pool,
             block_size): w = [q; k; v]; out[M, n_heads * head_dim] = rotated q; rotated k and v are stored at
             the tokens' cache slots.
    k_splits > 1 (plain, float32): out is [k_splits, M, N], partial sums over shares of K (a short, wide
             matrix then fills the chip); their sum in order is the product, the bias is in the first."""
    dev = _dev(out, x, w, bias)
    if k_splits != 1:
        if not 1 < k_splits <= 16 or swiglu or rope is not None:
            raise ValueError("k_splits is 1..16 and goes with the plain epilogue only")
        if out.dim() != 3 or out.shape[0] != k_splits or out.dtype != torch.float32 or not out.is_contiguous():
            raise ValueError("with k_splits the output is a contiguous float32 [k_splits, M, N] tensor")
        parts, out = out, out[0]
    if x.dim() != 2 or x.stride(1) != 1 or out.dim() != 2 or out.stride(1) != 1:
        raise ValueError("x and out must be 2-d with unit inner stride")
    _rows(w, "w", x.shape[1])
    m, k = x.shape
    n = w.shape[0]
    if not 0 < m <= 64:
        raise ValueError("gemm_stream takes 1..64 rows")
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or out.dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("gemm_stream takes bfloat16 operands and stores bfloat16 or float32")
    if not gemm_bf16_supported(x, w):
        raise ValueError(f"gemm_stream needs K ({k}) and the row stride of x ({x.stride(0)}) to be multiples of 8 "
                         "and 16-byte aligned operands")
    if bias is not None and (bias.dtype != torch.bfloat16 or bias.numel() != n or not bias.is_contiguous()):
        raise ValueError("bias must be a contiguous bfloat16 vector of N elements")
    if swiglu and rope is not None:
        raise ValueError("one epilogue at a time")
    epilogue, inter, cols = 0, 0, n
    r = dict(n_heads=0, n_kv_heads=0, head_dim=0, block_size=0, inv_freq=None, positions=None, slots=None,
             k_pool=None, v_pool=None, angles=None)
    if swiglu:
        if n % 16 or bias is not None:
            raise ValueError("the gated epilogue needs 2I % 16 == 0 and no bias")
        epilogue, inter, cols = 1, n // 2, n // 2
    elif rope is not None:
        r.update(rope)
        nh, nkv, d = r["n_heads"], r["n_kv_heads"], r["head_dim"]
        if d % 16 or n != (nh + 2 * nkv) * d:
            raise ValueError("the rotary epilogue needs head_dim % 16 == 0 and N = (heads + 2 kv heads) * head_dim")
        _i32(r["positions"], "positions", m)
        if r["inv_freq"] is not None:
            _f32(r["inv_freq"], "inv_freq", d // 2)
        if r["angles"] is not None:
            _f32(r["angles"], "angles", m * d)
        if r["slots"] is not None:
            _i32(r["slots"], "slots", m)
            bs, kp, vp = r["block_size"], r["k_pool"], r["v_pool"]
            pages = kp.shape[0]
            if (tuple(kp.shape) != (pages, nkv, bs, d) or tuple(vp.shape) != (pages, nkv, d, bs)
                    or not kp.is_contiguous() or not vp.is_contiguous() or kp.dtype != x.dtype or vp.dtype != x.dtype):
                raise ValueError("pools do not have the cache layout [pages, kv, block, D] / [pages, kv, D, block]")
        _dev(x, r["inv_freq"], r["angles"], r["positions"], r["slots"], r["k_pool"], r["v_pool"])
        epilogue, cols = 2, nh * d
    if tuple(out.shape) != (m, cols):
        raise ValueError(f"out shape {tuple(out.shape)} is not {(m, cols)}")
    _check(load("gemm_stream").llms_gemm_stream(
        c_int(_code(out)), c_int(epilogue), _ptr(out), c_int(out.stride(0)), _ptr(x), c_int(x.stride(0)), _ptr(w),
        _ptr(bias), c_int(m), c_int(n), c_int(k), c_int(inter), c_int(r["n_heads"]), c_int(r["n_kv_heads"]), c_int(r["head_dim"]), c_int(r["block_size"]),
        _ptr(r["inv_freq"]), _ptr(r["positions"]), _ptr(r["slots"]), _ptr(r["k_pool"]), _ptr(r["v_pool"]),
        c_int(k_splits), _stream(dev)), "gemm_stream")
    return parts if k_splits != 1 else out


_cu_count: dict[int, int] = {}


def compute_units(dev: torch.device) -> int:
    index = dev.index if dev.index is not None else torch.cuda.current_device()
    if index not in _cu_count:
        _cu_count[index] = torch.cuda.get_device_properties(index).multi_processor_count
    return _cu_count[index]


GEMM_DECODE_MAX_ROWS = 64
GEMM_DECODE_NORM_ROWS = 16  # up to here the kernel norms its rows on the way in (with more rows that costs a compute
# unit more vector arithmetic than a norm kernel of its own: measured at 32 rows, 4 microseconds)
GEMM_DECODE_MAX_K = 16 * 3 * 128  # 16 waves with up to three chunks of 128 each


def gemm_decode_fits(m: int, k: int) -> bool:
    """Whether m rows of k elements fit ops.gemm_decode: up to 16 rows stay in LDS or, where K is too long for that, in
    the registers of 16 waves (k up to 6,144 either way); 17 to 64 rows in the registers of 8 waves: four chunks of
    128 each up to 32 rows (k up to 4,096), two beyond (k up to 2,048)."""
    if not (0 < m <= GEMM_DECODE_MAX_ROWS and 0 < k <= GEMM_DECODE_MAX_K):
        return False
    return m <= 16 or k <= 2 * 8 * 128 or (m <= 32 and k <= 4 * 8 * 128)


GEMM_DECODE_ROWS_K = 2 * 8 * 128  # 17 to 64 rows: what 8 waves hold of a row in registers


def gemm_decode_k_parts(m: int, k: int) -> int:
    """Into how many parts ops.gemm_decode best shares K out when it leaves partial sums for 17 to 64 rows (0: it
    cannot take them).  At least what makes a part fit the registers; beyond that about 1,408 columns a part, a compute
    unit then pulls as little of X as of its weights (measured on 2048 x 2048, 2048 x 5632 and 4096 x 4096 at 24 to 64
    rows: 2, 4 and 4 parts), and a count that divides K's chunks of 128 evenly where one is near."""
    if not 16 < m <= GEMM_DECODE_MAX_ROWS or k <= 0:
        return 0
    chunks = -(-k // 128)
    first = max(-(-k // GEMM_DECODE_ROWS_K), -(-k // 1408))
    if first > 8:
        return 0
    for parts in range(first, min(8, first + 2) + 1):
        if chunks % parts == 0:
            return parts
    return first if (first - 1) * (-(-chunks // first) * 128) < k else 0


def gemm_decode_supported(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether ops.gemm_decode takes x [M, K] against w [N, K]."""
    return x.dtype == torch.bfloat16 and gemm_decode_fits(x.shape[0], x.shape[1]) and gemm_bf16_supported(x, w)


def gemm_decode(out: torch.Tensor | None, x: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None = None, *,
                norm: tuple[torch.Tensor, float] | None = None, swiglu: bool = False, rope: dict | None = None,
                residual: torch.Tensor | None = None, k_parts: int = 1) -> torch.Tensor:
    """The product for up to 64 bfloat16 rows with one workgroup per compute unit, and what surrounds it fused in.

    norm = (weight [K], eps): the rows of x are replaced by RMSNorm(x) * weight on the way in (up to 16 rows).
    plain:     out[M, N] = x w^T (+ bias), bfloat16 or float32.
    swiglu:    w = [gate; up] ([2I, K]); out[M, I] = silu(gate) * up.
    rope = dict(n_heads, n_kv_heads, head_dim, inv_freq | None, positions, slots | None, k_pool, v_pool,
               block_size, angles | None): w = [q; k; v]; out[M, n_heads * head_dim] = rotated q; rotated k and v
               are stored at the tokens' cache slots.  `angles` (rotary_angles(positions, inv_freq), float32
               [M, head_dim / 2, 2]) saves the kernel the sines and cosines; the result is the same to the bit.
    residual:  residual[M, N] += x w^T (+ bias) in place (32-bit sum of the rounded product and the row, rounded
               once); `out` is not used and `residual` is returned.
    k_parts > 1 (17 to 64 rows, plain, no bias, no norm): K is shared out to that many sets of workgroups and `out` is
               float32 [k_parts, M, N], the parts' sums, for a norm to add up (gemm_decode_k_parts says how many
               parts a K needs)."""
    dev = _dev(out, x, w, bias, residual, norm[0] if norm else None)
    if x.dim() != 2 or x.stride(1) != 1:
        raise ValueError("x must be 2-d with unit inner stride")
    _rows(w, "w", x.shape[1])
    m, k = x.shape
    n = w.shape[0]
    if not 0 < m <= GEMM_DECODE_MAX_ROWS:
        raise ValueError(f"gemm_decode takes 1..{GEMM_DECODE_MAX_ROWS} rows")
    if k_parts != 1:
        if not 1 < k_parts <= 16 or m <= 16 or bias is not None or norm is not None or swiglu or rope is not None \
                or residual is not None:
            raise ValueError("K is shared out (k_parts 2..16) only for 17 to 64 rows with the plain epilogue, no bias, no norm")
        if (k_parts - 1) * (-(-(-(-k // 128)) // k_parts) * 128) >= k:
            raise ValueError(f"K = {k} has too few chunks of 128 for {k_parts} parts")
        if out is None or out.dtype != torch.float32 or tuple(out.shape) != (k_parts, m, n) or not out.is_contiguous():
            raise ValueError(f"out must be a contiguous float32 [{k_parts}, {m}, {n}] tensor")
    if not gemm_decode_fits(m, -(-(-(-k // 128)) // k_parts) * 128 if k_parts > 1 else k):
        raise ValueError(f"gemm_decode keeps the rows of x in a compute unit: {m} rows of K = {k} do not fit (K up to "
                         f"{GEMM_DECODE_MAX_K} with up to 16 rows, 4,096 with up to 32, 2,048 beyond, per part)")
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise ValueError("gemm_decode takes bfloat16 operands")
    if not gemm_bf16_supported(x, w):
        raise ValueError(f"gemm_decode needs K ({k}) and the row stride of x ({x.stride(0)}) to be multiples of 8 "
                         "and 16-byte aligned operands")
    if bias is not None and (bias.dtype != torch.bfloat16 or bias.numel() != n or not bias.is_contiguous()):
        raise ValueError("bias must be a contiguous bfloat16 vector of N elements")
    if sum((swiglu, rope is not None, residual is not None)) > 1:
        raise ValueError("one epilogue at a time")
    norm_weight, eps = None, 0.0
    if norm is not None:
        norm_weight, eps = norm
        if m > GEMM_DECODE_NORM_ROWS:
            raise ValueError(f"gemm_decode norms up to {GEMM_DECODE_NORM_ROWS} rows on the way in; {m} rows are taken as they are")
        if norm_weight.dtype != torch.bfloat16 or norm_weight.numel() != k or not norm_weight.is_contiguous() \
                or norm_weight.data_ptr() % 16:
            raise ValueError("the norm's weight must be a contiguous, 16-byte aligned bfloat16 vector of K elements")
    epilogue, inter, cols = 0, 0, n
    r = dict(n_heads=0, n_kv_heads=0, head_dim=0, block_size=0, inv_freq=None, positions=None, slots=None,
             k_pool=None, v_pool=None, angles=None)
    if swiglu:
        if n % 2 or bias is not None:
            raise ValueError("the gated epilogue needs an even number of weight rows and no bias")
        epilogue, inter, cols = 1, n // 2, n // 2
    elif rope is not None:
        r.update(rope)
        nh, nkv, d = r["n_heads"], r["n_kv_heads"], r["head_dim"]
        if d % 2 or n != (nh + 2 * nkv) * d:
            raise ValueError("the rotary epilogue needs an even head_dim and N = (heads + 2 kv heads) * head_dim")
        _i32(r["positions"], "positions", m)
        if r["inv_freq"] is not None:
            _f32(r["inv_freq"], "inv_freq", d // 2)
        if r["angles"] is not None:
            _f32(r["angles"], "angles", m * d)
        if r["slots"] is not None:
            _i32(r["slots"], "slots", m)
            bs, kp, vp = r["block_size"], r["k_pool"], r["v_pool"]
            pages = kp.shape[0]
            if (tuple(kp.shape) != (pages, nkv, bs, d) or tuple(vp.shape) != (pages, nkv, d, bs)
                    or not kp.is_contiguous() or not vp.is_contiguous() or kp.dtype != x.dtype or vp.dtype != x.dtype):
                raise ValueError("pools do not have the cache layout [pages, kv, block, D] / [pages, kv, D, block]")
        _dev(x, r["inv_freq"], r["angles"], r["positions"], r["slots"], r["k_pool"], r["v_pool"])
        epilogue, cols = 2, nh * d
    elif residual is not None:
        if (residual.dim() != 2 or residual.stride(1) != 1 or tuple(residual.shape) != (m, n)
                or residual.dtype != torch.bfloat16):
            raise ValueError(f"residual must be a bfloat16 [{m}, {n}] tensor with unit inner stride")
        epilogue = 3
    if epilogue != 3 and k_parts == 1:
        if out is None or out.dim() != 2 or out.stride(1) != 1 or tuple(out.shape) != (m, cols):
            raise ValueError(f"out must be 2-d [{m}, {cols}] with unit inner stride")
        if out.dtype != torch.bfloat16 and not (epilogue == 0 and out.dtype == torch.float32):
            raise ValueError("gemm_decode stores bfloat16 (the plain epilogue also float32)")
    _check(load("gemm_decode").llms_gemm_decode(
        c_int(1 if epilogue == 3 else _code(out)), c_int(epilogue), _ptr(None if epilogue == 3 else out),
        c_int(0 if epilogue == 3 else out.stride(-2)), _ptr(x), c_int(x.stride(0)), _ptr(w), _ptr(bias),
        _ptr(norm_weight), c_float(eps), c_int(m), c_int(n), c_int(k), c_int(inter), c_int(r["n_heads"]),
        c_int(r["n_kv_heads"]), c_int(r["head_dim"]), c_int(r["block_size"]), _ptr(r["inv_freq"]), _ptr(r["angles"]), _ptr(r["positions"]),
        _ptr(r["slots"]), _ptr(r["k_pool"]), _ptr(r["v_pool"]), _ptr(residual),
        c_int(residual.stride(0) if residual is not None else 0), c_int(compute_units(dev)), c_int(k_parts),
        _stream(dev)), "gemm_decode")
    return residual if epilogue == 3 else out


SLICE_K = 512  # what one workgroup of gemm_slices takes of K


def gemm_slices(parts: torch.Tensor, x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """parts[s] = x[:, 512 s : 512 (s+1)] w[:, likewise]^T for the ceil(K / 512) slices of K: float32
    [slices, M, N], whose sum in order is x w^T.  For 17 to 64 bfloat16 rows (fewer are taken too) against a
    short, wide weight: every workgroup keeps its slice of all rows in LDS and reads its weights once."""
    dev = _dev(parts, x, w)
    if x.dim() != 2 or x.stride(1) != 1:
        raise ValueError("x must be 2-d with unit inner stride")
    _rows(w, "w", x.shape[1])
    m, k = x.shape
    n = w.shape[0]
    if not 0 < m <= 64:
        raise ValueError("gemm_slices takes 1..64 rows")
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise ValueError("gemm_slices takes bfloat16 operands")
    if not gemm_bf16_supported(x, w):
        raise ValueError(f"gemm_slices needs K ({k}) and the row stride of x ({x.stride(0)}) to be multiples of 8 "
                         "and 16-byte aligned operands")
    slices = -(-k // SLICE_K)
    if parts.dtype != torch.float32 or tuple(parts.shape) != (slices, m, n) or not parts.is_contiguous():
        raise ValueError(f"parts must be a contiguous float32 tensor of shape {(slices, m, n)}")
    _check(load("gemm_stream").llms_gemm_slices(_ptr(parts), _ptr(x), c_int(x.stride(0)), _ptr(w), c_int(m),
                                                c_int(n), c_int(k), _stream(dev)), "gemm_slices")
    return parts


# ------------------------------------------------------------------------------ attention


_ARRIVAL_COUNTERS: dict = {}
ARRIVAL_COUNTERS = 1 << 16
# LLMSERVE_ATTN_MERGE=kernel: the shares of a split decode attention are always added up by the second kernel
MERGE_BY_KERNEL = os.environ.get("LLMSERVE_ATTN_MERGE", "") == "kernel"


def _arrival_counters(dev) -> torch.Tensor | None:
    """The device's counters for workgroups that add each other's shares up inside a kernel: all zero between
    launches, and every kernel that uses them leaves them so.  Launches that use them must not overlap in time:
    the engine keeps all of a device's steps on one stream (a graph replays where its launches were ordered at
    capture), and whoever runs decode attention with splits on two streams at once passes `merge_kernel=True`
    (or sets LLMSERVE_ATTN_MERGE=kernel).  Made at the first call that is not being captured into a graph (a fill
    inside a graph would run at every replay); until then there are none and the caller takes its other way.  A
    launch that dies half-way may leave a count behind: whoever catches such an error calls
    `reset_arrival_counters` before the next step (the runner does)."""
    key = (dev.type, dev.index)
    if key not in _ARRIVAL_COUNTERS:
        if torch.cuda.is_current_stream_capturing():
            return None
        _ARRIVAL_COUNTERS[key] = torch.zeros(ARRIVAL_COUNTERS, dtype=torch.int32, device=dev)
    return _ARRIVAL_COUNTERS[key]


def reset_arrival_counters(dev=None) -> None:
    """Zero the counters (of one device, or of all): after an error in the middle of a step, and when a runner is
    built.  A small fill kernel, on the current stream."""
    for (kind, index), counters in _ARRIVAL_COUNTERS.items():
        if dev is None or (kind, index) == (dev.type, dev.index):
            counters.zero_()


def arrival_counters_are_zero(dev=None) -> bool:
    """Whether every launch so far has left its counters as it found them (tests ask after their workloads)."""
    return all(int(c.abs().max()) == 0 for (kind, index), c in _ARRIVAL_COUNTERS.items()
               if dev is None or (kind, index) == (dev.type, dev.index))


def _check_paged(q, out, k_pool, v_pool, block_tables, n_heads, n_kv_heads, head_dim, block_size):
    if q.dim() != 2 or q.stride(1) != 1 or q.shape[1] < n_heads * head_dim:
        raise ValueError("q must be [N, >= n_heads*head_dim] with unit inner stride")
    _rows(out, "out", n_heads * head_dim)
    if out.shape[0] != q.shape[0] or out.dtype != q.dtype:
        raise ValueError("out and q disagree")
    pages = k_pool.shape[0]
    if tuple(k_pool.shape) != (pages, n_kv_heads, block_size, head_dim) or not k_pool.is_contiguous():
        raise ValueError(f"k_pool shape {tuple(k_pool.shape)} is not [pages,{n_kv_heads},{block_size},{head_dim}]")
    if tuple(v_pool.shape) != (pages, n_kv_heads, head_dim, block_size) or not v_pool.is_contiguous():
        raise ValueError(f"v_pool shape {tuple(v_pool.shape)} is not [pages,{n_kv_heads},{head_dim},{block_size}]")
    if k_pool.dtype != q.dtype or v_pool.dtype != q.dtype:
        raise ValueError("pools and q differ in dtype")
    if block_tables.dim() != 2 or block_tables.dtype != torch.int32 or not block_tables.is_contiguous():
        raise ValueError("block_tables must be a contiguous int32 [B, M] tensor")
    if n_heads % n_kv_heads:
        raise ValueError("n_heads must be a multiple of n_kv_heads")


def _table_rows(table_rows, block_tables, n_seqs: int | None):
    if table_rows is not None:
        _i32(table_rows, "table_rows", n_seqs)
    return table_rows


def attention_wave(out: torch.Tensor, q: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                   block_tables: torch.Tensor, token_seq: torch.Tensor, positions: torch.Tensor,
                   n_heads: int, n_kv_heads: int, head_dim: int, block_size: int, window: int = 0,
                   scale: float | None = None, table_rows: torch.Tensor | None = None) -> torch.Tensor:
    """Causal attention of N new tokens over the paged cache (one wave per token and head).

    q: rows of width >= n_heads*head_dim (the q part of a qkv buffer is fine); out [N, n_heads*head_dim];
    token_seq[n] = request (0..B-1) of token n; positions[n] = its absolute position; table_rows[b] =
    row of block_tables that request b owns (default: b).
    """
    dev = _dev(out, q, k_pool, v_pool, block_tables, token_seq, positions, table_rows)
    _table_rows(table_rows, block_tables, None)
    _check_paged(q, out, k_pool, v_pool, block_tables, n_heads, n_kv_heads, head_dim, block_size)
    n = q.shape[0]
    _i32(token_seq, "token_seq", n)
    _i32(positions, "positions", n)
    if not 0 < head_dim <= 256:
        raise ValueError(f"head_dim={head_dim} is outside 1..256")
    if n == 0:
        return out
    scale = 1.0 / math.sqrt(head_dim) if scale is None else scale
    _check(load("attention").llms_attention_wave(
        c_int(_code(q)), _ptr(out), c_int(out.stride(0)), _ptr(q), c_int(q.stride(0)), _ptr(k_pool), _ptr(v_pool),
        _ptr(block_tables), _ptr(table_rows), c_int(block_tables.shape[1]), _ptr(token_seq), _ptr(positions), c_int(n),
        c_int(n_heads), c_int(n_kv_heads), c_int(head_dim), c_int(block_size), c_int(window), c_float(scale),
        _stream(dev)), "attention_wave")
    return out


def attention_mfma_supported(dtype: torch.dtype, head_dim: int, block_size: int) -> bool:
    """Whether the matrix-core attention kernel takes this cache (else `attention_wave` does)."""
    return dtype == torch.bfloat16 and head_dim % 16 == 0 and 16 <= head_dim <= 256 and block_size % 8 == 0


def attention_mfma(out: torch.Tensor, q: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                   block_tables: torch.Tensor, cu_seqlens: torch.Tensor, context_lens: torch.Tensor,
                   seq_begin: int, n_seqs: int, max_new: int, token_begin: int, n_tokens: int,
                   n_heads: int, n_kv_heads: int, head_dim: int, block_size: int, window: int = 0,
                   scale: float | None = None, split_waves: bool = False, num_splits: int = 1,
                   table_rows: torch.Tensor | None = None, waves: int = 4, merge_kernel: bool = False) -> torch.Tensor:
    """bfloat16 causal attention on the matrix cores for requests [seq_begin, seq_begin + n_seqs) of a
    step, whose new tokens are rows [token_begin, token_begin + n_tokens) of q and out and bring at most
    `max_new` tokens each.  `split_waves` (with `waves` = 4 or 8 and `num_splits`) spreads each request's keys
    over the waves of a workgroup and over workgroups: the arrangement for single decoded tokens.  Without
    it the 4 waves of a block of tokens take neighbouring tokens and share each tile of keys through LDS (in a
    large launch without a window each has a twin wave that takes every other tile); `num_splits` instead
    shares the keys of such a block of tokens out to several workgroups (short portions, long prefixes).
    The shares of workgroups are added up, in the order of the splits, by a second kernel, or for decoding with up
    to 16 splits by the workgroup of each group that finishes last (`merge_kernel=True` asks for the second kernel
    there too: the same bits).  (For prompt portions the last workgroup was tried as well: no faster.)"""
    dev = _dev(out, q, k_pool, v_pool, block_tables, cu_seqlens, context_lens, table_rows)
    _check_paged(q, out, k_pool, v_pool, block_tables, n_heads, n_kv_heads, head_dim, block_size)
    if not attention_mfma_supported(q.dtype, head_dim, block_size):
        raise ValueError(f"attention_mfma needs bfloat16, head_dim a multiple of 16 up to 256 and block_size a "
                         f"multiple of 8; got {q.dtype}, {head_dim}, {block_size}")
    b = cu_seqlens.numel() - 1
    _i32(cu_seqlens, "cu_seqlens")
    _i32(context_lens, "context_lens", b)
    if table_rows is not None:
        _i32(table_rows, "table_rows", b)
    elif block_tables.shape[0] < b:
        raise ValueError("block_tables has fewer rows than there are requests")
    if not (0 <= seq_begin and n_seqs >= 0 and seq_begin + n_seqs <= b):
        raise ValueError("request range is outside the batch")
    if not (0 <= token_begin and token_begin + n_tokens <= q.shape[0]):
        raise ValueError("token range is outside the batch")
    if q.stride(0) % 8 or q.data_ptr() % 16 or out.data_ptr() % 16:
        raise ValueError("q rows must be 16-byte aligned")
    if num_splits > 1 and not split_waves and window:
        raise ValueError("portions of prompts with a window are not split over workgroups")
    if waves != 4 and not (split_waves and waves == 8):
        raise ValueError("4 waves, or 8 when the waves share the keys")
    if waves == 8 and head_dim > 160:
        raise ValueError("8 waves take head_dim up to 160 (wider heads would not fit the registers)")
    if n_seqs == 0 or n_tokens == 0:
        return out
    ws_o = ws_ml = arrive = None
    if num_splits > 1 and split_waves and not (merge_kernel or MERGE_BY_KERNEL):
        arrive = _arrival_counters(dev)
    if num_splits > 1:
        ws_o = torch.empty((q.shape[0] * n_heads * num_splits * head_dim,), dtype=torch.float32, device=dev)
        ws_ml = torch.empty((q.shape[0] * n_heads * num_splits * 2,), dtype=torch.float32, device=dev)
    scale = 1.0 / math.sqrt(head_dim) if scale is None else scale
    _check(load("attention_mfma").llms_attention_mfma(
        _ptr(out), c_int(out.stride(0)), _ptr(q), c_int(q.stride(0)), _ptr(k_pool), _ptr(v_pool),
        _ptr(block_tables), _ptr(table_rows), c_int(block_tables.shape[1]), _ptr(cu_seqlens), _ptr(context_lens),
        c_int(seq_begin),
        c_int(n_seqs), c_int(max_new), c_int(token_begin), c_int(n_tokens), c_int(n_heads), c_int(n_kv_heads),
        c_int(head_dim), c_int(block_size), c_int(window), c_float(scale),
        c_int(1 if split_waves else 0),
        c_int(num_splits), c_int(waves), _ptr(ws_o), _ptr(ws_ml), _ptr(arrive),
        c_int(arrive.numel() if arrive is not None else 0), _stream(dev)), "attention_mfma")
    return out


def attention_prompt_biased_supported(dtype: torch.dtype, dk: int, dv: int, block_size: int) -> bool:
    """Whether `attention_prompt_biased` takes this cache: bfloat16, keys and values of one size, 32, 64, 96 or 128."""
    return dtype == torch.bfloat16 and dk == dv and dk in (32, 64, 96, 128) and block_size % 8 == 0


def attention_prompt_biased(out: torch.Tensor, q: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                            block_tables: torch.Tensor, cu_seqlens: torch.Tensor, context_lens: torch.Tensor,
                            seq_begin: int, n_seqs: int, max_new: int, token_begin: int, n_tokens: int, *, n_heads: int,
                            n_kv_heads: int, head_dim: int, block_size: int, scale: float, dist_bias: torch.Tensor,
                            gate: torch.Tensor | None = None, table_rows: torch.Tensor | None = None) -> torch.Tensor:
    """The prompt kernel of `attention_mfma` (no window, no splits) with dist_bias[h, min(i - j, R)] added to the scaled
    score of head h between positions i >= j (float32 [heads, R + 1]) and, with `gate` (float32 [N, >= heads * head_dim],
    16-byte aligned rows), the result multiplied by the sigmoid of the gate's products."""
    dev = _dev(out, q, k_pool, v_pool, block_tables, cu_seqlens, context_lens, table_rows, dist_bias, gate)
    _check_paged(q, out, k_pool, v_pool, block_tables, n_heads, n_kv_heads, head_dim, block_size)
    if not attention_prompt_biased_supported(q.dtype, head_dim, head_dim, block_size):
        raise ValueError("attention_prompt_biased needs bfloat16, heads of 32, 64, 96 or 128 and pages of a multiple of 8 keys")
    b = cu_seqlens.numel() - 1
    _i32(cu_seqlens, "cu_seqlens")
    _i32(context_lens, "context_lens", b)
    if table_rows is not None:
        _i32(table_rows, "table_rows", b)
    elif block_tables.shape[0] < b:
        raise ValueError("block_tables has fewer rows than there are requests")
    if not (0 <= seq_begin and n_seqs >= 0 and seq_begin + n_seqs <= b):
        raise ValueError("request range is outside the batch")
    if not (0 <= token_begin and token_begin + n_tokens <= q.shape[0]):
        raise ValueError("token range is outside the batch")
    if q.stride(0) % 8 or q.data_ptr() % 16 or out.data_ptr() % 16:
        raise ValueError("q rows must be 16-byte aligned")
    if dist_bias.dtype != torch.float32 or dist_bias.dim() != 2 or dist_bias.shape[0] != n_heads or dist_bias.shape[1] < 1 \
            or not dist_bias.is_contiguous():
        raise ValueError("dist_bias must be a contiguous float32 [heads, reach + 1] tensor")
    if gate is not None and (gate.dtype != torch.float32 or gate.dim() != 2 or gate.stride(1) != 1 or gate.shape[0] != q.shape[0]
                             or gate.shape[1] < n_heads * head_dim or gate.stride(0) % 4 or gate.data_ptr() % 16):
        raise ValueError("gate must be float32 [N, >= heads*head_dim] with unit inner stride and 16-byte aligned rows")
    if n_seqs == 0 or n_tokens == 0:
        return out
    _check(load("attention_biased").llms_attention_prompt_biased(
        _ptr(out), c_int(out.stride(0)), _ptr(q), c_int(q.stride(0)), _ptr(k_pool), _ptr(v_pool), _ptr(block_tables),
        _ptr(table_rows), c_int(block_tables.shape[1]), _ptr(cu_seqlens), _ptr(context_lens), c_int(seq_begin), c_int(n_seqs),
        c_int(max_new), c_int(token_begin), c_int(n_tokens), c_int(n_heads), c_int(n_kv_heads), c_int(head_dim),
        c_int(block_size), c_float(scale), _ptr(dist_bias), c_int(dist_bias.shape[1] - 1), _ptr(gate),
        c_int(gate.stride(0) if gate is not None else 0), _stream(dev)), "attention_prompt_biased")
    return out


# ------------------------------------------------------------------------------ a residual stream in 32-bit


def embed_scale(out: torch.Tensor, table: torch.Tensor, ids: torch.Tensor, scale: float) -> torch.Tensor:
    """out[n] = table[ids[n]] * scale in 32-bit; out float32 [N, H], table [V, H] float32 or bfloat16."""
    dev = _dev(out, table, ids)
    _rows(out, "out")
    _rows(table, "table", out.shape[1])
    _i32(ids, "ids", out.shape[0])
    if out.dtype != torch.float32:
        raise ValueError("out must be float32")
    if out.shape[0] == 0:
        return out
    _check(load("stream32").llms_embed_scale(
        c_int(_code(table)), _ptr(out), _ptr(table), _ptr(ids), c_int(out.shape[0]), c_int(out.shape[1]),
        c_int(table.shape[0]), c_float(scale), _stream(dev)), "embed_scale")
    return out


def softcap(x: torch.Tensor, cap: float) -> torch.Tensor:
    """x <- cap * tanh(x / cap) in place; x float32, contiguous."""
    dev = _dev(x)
    _f32(x, "x")
    if not cap > 0:
        raise ValueError("the cap must be positive")
    if x.numel():
        _check(load("stream32").llms_softcap(_ptr(x), ctypes.c_size_t(x.numel()), c_float(cap), _stream(dev)), "softcap")
    return x


def rmsnorm32(out: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, eps: float, offset: float = 0.0,
              rows: torch.Tensor | None = None) -> torch.Tensor:
    """out[r] = x[s] / sqrt(mean(x[s]^2) + eps) * (offset + weight), s = rows[r] or r, all in 32-bit and rounded
    once; x and weight float32, out float32 or bfloat16."""
    dev = _dev(out, x, weight, rows)
    _rows(x, "x")
    hidden = x.shape[1]
    _rows(out, "out", hidden)
    _f32(weight, "weight", hidden)
    if x.dtype != torch.float32:
        raise ValueError("x must be float32")
    if rows is not None:
        _i32(rows, "rows", out.shape[0])
    elif out.shape[0] != x.shape[0]:
        raise ValueError("out and x differ in rows")
    if out.shape[0] == 0:
        return out
    _check(load("stream32").llms_rmsnorm32(
        c_int(_code(out)), _ptr(out), _ptr(x), _ptr(weight), _ptr(rows), c_float(eps), c_float(offset),
        c_int(out.shape[0]), c_int(hidden), _stream(dev)), "rmsnorm32")
    return out


def _gated_branches(x: torch.Tensor, branches: list, gate_products: torch.Tensor | None):
    """Checks the operands of a gated sum; returns (device, z stride, [(y, column or -1, bias)] * 2)."""
    ys = [b for b in branches if b is not None]
    if not 1 <= len(ys) <= 2:
        raise ValueError("one or two branches")
    dev = _dev(x, gate_products, *[t for y, _c, bias in ys for t in (y, bias)])
    _rows(x, "x")
    n, hidden = x.shape
    if x.dtype != torch.float32:
        raise ValueError("x must be float32")
    z_stride = 0
    if gate_products is not None:
        if gate_products.dim() != 2 or gate_products.stride(1) != 1 or gate_products.dtype != torch.float32 \
                or gate_products.shape[0] != n:
            raise ValueError("gate_products must be float32 [N, columns] with unit inner stride")
        z_stride = gate_products.stride(0)
    args = []
    for y, column, bias in ys + [(None, None, None)] * (2 - len(ys)):
        if y is not None:
            if y.dim() != 2 or y.stride(1) != 1 or y.dtype != torch.float32 or tuple(y.shape) != (n, hidden):
                raise ValueError("a branch must be float32 [N, hidden] with unit inner stride")
            if column is not None:
                if gate_products is None or not 0 <= column <= gate_products.shape[1] - hidden:
                    raise ValueError("a gate's columns lie outside gate_products")
                if bias is not None:
                    _f32(bias, "bias", hidden)
        args.append((y, -1 if column is None else column, bias if column is not None else None))
    return dev, z_stride, args


def gated_add(x: torch.Tensor, branches: list, gate_products: torch.Tensor | None = None) -> torch.Tensor:
    """x += sum over up to two branches of g * y, in place, all float32.  A branch is (y [N, hidden], column, bias):
    g = sigmoid(gate_products[:, column : column + hidden] + bias) where `column` is not None, else 1."""
    dev, z_stride, args = _gated_branches(x, branches, gate_products)
    n, hidden = x.shape
    if n == 0:
        return x
    (y0, c0, b0), (y1, c1, b1) = args
    _check(load("stream32").llms_gated_add(
        _ptr(x), _ptr(gate_products), c_int(z_stride), c_int(c0), c_int(c1), _ptr(b0), _ptr(b1), _ptr(y0),
        c_int(y0.stride(0) if y0 is not None else 0), _ptr(y1), c_int(y1.stride(0) if y1 is not None else 0),
        c_int(n), c_int(hidden), _stream(dev)), "gated_add")
    return x


# Up to this many rows the sum and the norm are one kernel (a launch less in a step that is a chain of launches);
# measured at 2,048 rows of 2,048: one kernel that walks a row in two turns 4 % of a prompt step slower than two.
GATED_ADD_NORM_ROWS = 256


def gated_add_norm(out: torch.Tensor, x: torch.Tensor, branches: list, gate_products: torch.Tensor | None,
                   weight: torch.Tensor, eps: float, offset: float = 0.0) -> torch.Tensor:
    """`gated_add(x, branches, gate_products)` and `rmsnorm32(out, x, weight, eps, offset)` of the summed rows, in
    one kernel where the sizes allow (rows of a multiple of 4 up to 8,192), else one after the other."""
    dev, z_stride, args = _gated_branches(x, branches, gate_products)
    n, hidden = x.shape
    _rows(out, "out", hidden)
    _f32(weight, "weight", hidden)
    if out.shape[0] != n:
        raise ValueError("out and x differ in rows")
    if n == 0:
        return out
    (y0, c0, b0), (y1, c1, b1) = args
    if n > GATED_ADD_NORM_ROWS:  # many rows fill the chip either way, and two kernels that each read a row at once are faster
        gated_add(x, branches, gate_products)
        return rmsnorm32(out, x, weight, eps, offset)
    status = load("stream32").llms_gated_add_norm(
        c_int(_code(out)), _ptr(out), _ptr(x), _ptr(gate_products), c_int(z_stride), c_int(c0), c_int(c1), _ptr(b0),
        _ptr(b1), _ptr(y0), c_int(y0.stride(0) if y0 is not None else 0), _ptr(y1),
        c_int(y1.stride(0) if y1 is not None else 0), _ptr(weight), c_float(eps), c_float(offset), c_int(n),
        c_int(hidden), _stream(dev))
    if status == 3:  # sizes the fused kernel does not take
        gated_add(x, branches, gate_products)
        return rmsnorm32(out, x, weight, eps, offset)
    _check(status, "gated_add_norm")
    return out


# ------------------------------------------------------------------------------ attention from chosen ingredients


def conv_store(q_out: torch.Tensor, proj: torch.Tensor, *, cq: int, k_heads: int, dk: int, v_heads: int, dv: int,
               taps_w: torch.Tensor | None = None, state: torch.Tensor | None = None,
               state_slots: torch.Tensor | None = None, token_seq: torch.Tensor | None = None,
               positions: torch.Tensor | None = None, cu_seqlens: torch.Tensor | None = None,
               slots: torch.Tensor | None = None, k_pool: torch.Tensor | None = None,
               v_pool: torch.Tensor | None = None, block_size: int = 0, update_state: bool = False,
               context_lens: torch.Tensor | None = None) -> torch.Tensor:
    """proj float32 [N, cq + k_heads*dk + v_heads*dv] (what the stacked q, k, v projection gave), optionally through a
    causal convolution per channel (`taps_w` float32 [channels, taps], `state` float32 [slots, taps-1, channels]: a
    ring of each request's last projected rows, indexed by position), rounded once: queries to q_out [N, cq], keys
    and values to the tokens' cache slots (`slots`; None: nothing is stored).  `update_state` (only where every
    request of the step brings exactly one token; `context_lens` [B] says which requests are padding): the ring takes
    each token's projected row in the same kernel, so `conv_state` need not run."""
    dev = _dev(q_out, proj, taps_w, state, state_slots, token_seq, positions, cu_seqlens, slots, k_pool, v_pool, context_lens)
    n = proj.shape[0]
    channels = cq + k_heads * dk + v_heads * dv
    if proj.dim() != 2 or proj.dtype != torch.float32 or proj.stride(1) != 1 or proj.shape[1] != channels:
        raise ValueError(f"proj must be float32 [N, {channels}] with unit inner stride")
    _rows(q_out, "q_out", cq)
    if q_out.shape[0] != n:
        raise ValueError("q_out and proj differ in rows")
    taps = 0
    if taps_w is not None:
        _f32(taps_w, "taps_w")
        if taps_w.dim() != 2 or taps_w.shape[0] != channels:
            raise ValueError(f"taps_w must be [{channels}, taps]")
        taps = taps_w.shape[1]
    if taps > 0:
        _i32(token_seq, "token_seq", n)
        _i32(positions, "positions", n)
        _i32(cu_seqlens, "cu_seqlens")
    if taps > 1:
        if state is None or state.dtype != torch.float32 or not state.is_contiguous() or \
                tuple(state.shape[1:]) != (taps - 1, channels):
            raise ValueError(f"state must be a contiguous float32 [slots, {taps - 1}, {channels}] tensor")
        _i32(state_slots, "state_slots", cu_seqlens.numel() - 1)
    if slots is not None:
        _i32(slots, "slots", n)
        pages = k_pool.shape[0]
        if tuple(k_pool.shape) != (pages, k_heads, block_size, dk) or not k_pool.is_contiguous():
            raise ValueError(f"k_pool shape {tuple(k_pool.shape)} is not [pages,{k_heads},{block_size},{dk}]")
        if tuple(v_pool.shape) != (pages, v_heads, dv, block_size) or not v_pool.is_contiguous():
            raise ValueError(f"v_pool shape {tuple(v_pool.shape)} is not [pages,{v_heads},{dv},{block_size}]")
        if k_pool.dtype != q_out.dtype or v_pool.dtype != q_out.dtype:
            raise ValueError("pools and q_out differ in dtype")
    fused_state = bool(update_state and taps > 1)
    if fused_state:
        if cu_seqlens.numel() - 1 != n:
            raise ValueError("update_state needs every request to bring exactly one token")
        _i32(context_lens, "context_lens", n)
    if n == 0:
        return q_out
    _check(load("attention_composed").llms_conv_store(
        c_int(_code(q_out)), _ptr(q_out), c_int(q_out.stride(0)), _ptr(proj), c_int(proj.stride(0)), _ptr(taps_w),
        c_int(taps), _ptr(state), ctypes.c_size_t(state.stride(0) if state is not None else 0), _ptr(state_slots),
        _ptr(token_seq), _ptr(positions), _ptr(cu_seqlens), _ptr(slots), _ptr(k_pool), _ptr(v_pool), c_int(n), c_int(cq),
        c_int(k_heads * dk), c_int(v_heads * dv), c_int(k_heads), c_int(dk), c_int(v_heads), c_int(dv),
        c_int(block_size), _ptr(state if fused_state else None), _ptr(context_lens if fused_state else None),
        _stream(dev)), "conv_store")
    return q_out


def conv_state(state: torch.Tensor, proj: torch.Tensor, state_slots: torch.Tensor, cu_seqlens: torch.Tensor,
               context_lens: torch.Tensor) -> None:
    """The ring `state` [slots, taps-1, channels] takes the last taps-1 rows of `proj` of every request of the step
    (request b owns rows cu_seqlens[b] .. cu_seqlens[b+1] and is context_lens[b] long after the step; a request
    of length 0 is padding and left alone)."""
    dev = _dev(state, proj, state_slots, cu_seqlens, context_lens)
    if state.dtype != torch.float32 or state.dim() != 3 or not state.is_contiguous():
        raise ValueError("state must be a contiguous float32 [slots, taps-1, channels] tensor")
    channels = state.shape[2]
    if proj.dim() != 2 or proj.dtype != torch.float32 or proj.stride(1) != 1 or proj.shape[1] != channels:
        raise ValueError(f"proj must be float32 [N, {channels}] with unit inner stride")
    _i32(cu_seqlens, "cu_seqlens")
    b = cu_seqlens.numel() - 1
    _i32(context_lens, "context_lens", b)
    _i32(state_slots, "state_slots", b)
    if b <= 0 or proj.shape[0] == 0:
        return
    _check(load("attention_composed").llms_conv_state(
        _ptr(state), ctypes.c_size_t(state.stride(0)), _ptr(state_slots), _ptr(proj), c_int(proj.stride(0)),
        _ptr(cu_seqlens), _ptr(context_lens), c_int(b), c_int(state.shape[1] + 1), c_int(channels), _stream(dev)),
        "conv_state")


def _check_dist_bias_and_gate(dist_bias, gate, heads: int, dv: int, n: int) -> None:
    if dist_bias is not None and (dist_bias.dtype != torch.float32 or dist_bias.dim() != 2 or dist_bias.shape[0] != heads
                                  or dist_bias.shape[1] < 1 or not dist_bias.is_contiguous()):
        raise ValueError(f"dist_bias must be a contiguous float32 [{heads}, R + 1] tensor")
    if gate is not None and (gate.dtype != torch.float32 or gate.dim() != 2 or gate.stride(1) != 1 or gate.shape[0] != n
                             or gate.shape[1] < heads * dv):
        raise ValueError(f"gate must be float32 [{n}, >= {heads * dv}] with unit inner stride")


def norm_store(q_out: torch.Tensor, proj: torch.Tensor, *, q_heads: int, k_heads: int, dk: int, v_heads: int, dv: int,
               q_norm: torch.Tensor | None = None, k_norm: torch.Tensor | None = None, eps: float = 0.0,
               temp_coef: float = 0.0, temp_every: int = 0, positions: torch.Tensor | None = None,
               slots: torch.Tensor | None = None, k_pool: torch.Tensor | None = None, v_pool: torch.Tensor | None = None,
               block_size: int = 0, freq: torch.Tensor | None = None, unit_norm: bool = False) -> torch.Tensor:
    """proj float32 [N, >= q_heads*dk + k_heads*dk + v_heads*dv] (q, k, v side by side; unit inner stride): with
    `freq` (float32 [rot_dims / 2]) the first rot_dims numbers of every head of q and k are first turned by the
    token's position (dimension i with dimension i + rot_dims / 2, angle position * freq[i]); `unit_norm`: every head
    of q and k is divided by its root mean square with no weight; otherwise every
    head of q and of k is divided by its root mean square (eps inside the root) and multiplied by `q_norm` / `k_norm`
    (float32 [dk], shared by the heads; None: the head passes as it is); q is multiplied by
    1 + temp_coef * ln(floor((p + 1) / temp_every) + 1) at position p (temp_every 0: no factor); rounded once: queries
    to q_out [N, q_heads*dk], keys and values to the tokens' cache slots (`slots`; None: nothing is stored)."""
    dev = _dev(q_out, proj, q_norm, k_norm, positions, slots, k_pool, v_pool, freq)
    n = proj.shape[0]
    rot_dims = 0
    if freq is not None:
        _f32(freq, "freq")
        rot_dims = 2 * freq.numel()
        if rot_dims > dk:
            raise ValueError(f"{rot_dims} turned dimensions in a head of {dk}")
        _i32(positions, "positions", n)
    channels = (q_heads + k_heads) * dk + v_heads * dv
    if proj.dim() != 2 or proj.dtype != torch.float32 or proj.stride(1) != 1 or proj.shape[1] < channels:
        raise ValueError(f"proj must be float32 [N, >= {channels}] with unit inner stride")
    _rows(q_out, "q_out", q_heads * dk)
    if q_out.shape[0] != n:
        raise ValueError("q_out and proj differ in rows")
    for t, name in ((q_norm, "q_norm"), (k_norm, "k_norm")):
        if t is not None:
            _f32(t, name, dk)
    if temp_every < 0:
        raise ValueError("temp_every must not be negative")
    if temp_every > 0:
        _i32(positions, "positions", n)
    if slots is not None:
        _i32(slots, "slots", n)
        pages = k_pool.shape[0]
        if tuple(k_pool.shape) != (pages, k_heads, block_size, dk) or not k_pool.is_contiguous():
            raise ValueError(f"k_pool shape {tuple(k_pool.shape)} is not [pages,{k_heads},{block_size},{dk}]")
        if tuple(v_pool.shape) != (pages, v_heads, dv, block_size) or not v_pool.is_contiguous():
            raise ValueError(f"v_pool shape {tuple(v_pool.shape)} is not [pages,{v_heads},{dv},{block_size}]")
        if k_pool.dtype != q_out.dtype or v_pool.dtype != q_out.dtype:
            raise ValueError("pools and q_out differ in dtype")
    if n == 0:
        return q_out
    _check(load("attention_composed").llms_norm_store(
        c_int(_code(q_out)), _ptr(q_out), c_int(q_out.stride(0)), _ptr(proj), c_int(proj.stride(0)), _ptr(q_norm),
        _ptr(k_norm), c_float(eps), c_float(temp_coef), c_int(temp_every), _ptr(positions), _ptr(slots), _ptr(k_pool),
        _ptr(v_pool), c_int(n), c_int(q_heads), c_int(k_heads), c_int(dk), c_int(v_heads), c_int(dv), c_int(block_size),
        _ptr(freq), c_int(rot_dims), c_int(1 if unit_norm else 0), _stream(dev)), "norm_store")
    return q_out


ATTEND_COMPOSED_LDS = 160 * 1024


def attend_composed_lds_bytes(heads: int, maps: int, dk: int, dv: int, talk: bool) -> int:
    """LDS one workgroup of `attend_composed` takes."""
    s = heads * maps
    floats = s * dk + 2 * s + s * 64 + s * dv + ((heads * 64 + heads * heads) if talk else 0)
    return floats * 4 + 2 * 64 * 4


def attend_composed(out: torch.Tensor, q: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                    block_tables: torch.Tensor, token_seq: torch.Tensor, positions: torch.Tensor, *, heads: int,
                    kv_heads: int, dk: int, dv: int, block_size: int, scale: float, maps: int = 1, window: int = 0,
                    keep_first: int = 0, chunk: int = 0, slopes: torch.Tensor | None = None,
                    talk: torch.Tensor | None = None, lam: float = 0.0, head_norm: bool = False, eps: float = 0.0,
                    out_scale: float = 1.0, table_rows: torch.Tensor | None = None,
                    context_lens: torch.Tensor | None = None, dist_bias: torch.Tensor | None = None,
                    gate: torch.Tensor | None = None, sink: bool = False) -> torch.Tensor:
    """Attention of N new tokens over the paged cache, one workgroup per token (all its heads), float32 or bfloat16
    storage, 32-bit arithmetic.  q [N, heads*maps*dk] (head by head, a head's maps side by side); k_pool
    [pages, kv_heads*maps, block, dk]; v_pool [pages, kv_heads, dv, block]; out [N, heads*dv].  A query at
    position i sees j <= i with j >= its chunk's start (chunk > 0) and (i - j < window or j < keep_first) (window >
    0).  `slopes` float32 [heads]: slope_h * (i - j) is taken off the scores.  `talk` float32 [heads, heads]: the
    heads' normalised weights are mixed, w_h = sum_g talk[h, g] w_g (maps = 1).  maps = 2: a_1 - lam * a_2.
    `head_norm`: each head's result is divided by its root mean square (eps inside the root) and multiplied by
    out_scale.  `context_lens` [B]: rows of a request of length 0 are padding and give zeros.  `dist_bias` float32
    [heads, R + 1]: dist_bias[h, min(i - j, R)] is added to the scores.  `gate` float32 [N, >= heads*dv] (unit inner
    stride): the result is multiplied by sigmoid(gate).  `sink`: the softmax's denominator holds one more term,
    exp(0), a key of score zero without a value."""
    dev = _dev(out, q, k_pool, v_pool, block_tables, token_seq, positions, slopes, talk, table_rows, context_lens,
               dist_bias, gate)
    _check_dist_bias_and_gate(dist_bias, gate, heads, dv, q.shape[0])
    n = q.shape[0]
    if q.dim() != 2 or q.stride(1) != 1 or q.shape[1] < heads * maps * dk:
        raise ValueError("q must be [N, >= heads*maps*dk] with unit inner stride")
    _rows(out, "out", heads * dv)
    if out.shape[0] != n or out.dtype != q.dtype:
        raise ValueError("out and q disagree")
    pages = k_pool.shape[0]
    if tuple(k_pool.shape) != (pages, kv_heads * maps, block_size, dk) or not k_pool.is_contiguous():
        raise ValueError(f"k_pool shape {tuple(k_pool.shape)} is not [pages,{kv_heads * maps},{block_size},{dk}]")
    if tuple(v_pool.shape) != (pages, kv_heads, dv, block_size) or not v_pool.is_contiguous():
        raise ValueError(f"v_pool shape {tuple(v_pool.shape)} is not [pages,{kv_heads},{dv},{block_size}]")
    if k_pool.dtype != q.dtype or v_pool.dtype != q.dtype:
        raise ValueError("pools and q differ in dtype")
    if block_tables.dim() != 2 or block_tables.dtype != torch.int32 or not block_tables.is_contiguous():
        raise ValueError("block_tables must be a contiguous int32 [B, M] tensor")
    if heads % kv_heads or maps not in (1, 2) or (talk is not None and maps != 1):
        raise ValueError("heads must be a multiple of kv_heads, maps 1 or 2, and talk goes with maps = 1")
    _i32(token_seq, "token_seq", n)
    _i32(positions, "positions", n)
    if table_rows is not None:
        _i32(table_rows, "table_rows")
    if context_lens is not None:
        _i32(context_lens, "context_lens")
    if slopes is not None:
        _f32(slopes, "slopes", heads)
    if talk is not None:
        _f32(talk, "talk", heads * heads)
    if attend_composed_lds_bytes(heads, maps, dk, dv, talk is not None) > ATTEND_COMPOSED_LDS:
        raise ValueError("heads times sizes do not fit the 160 KB of LDS a workgroup has")
    if n == 0:
        return out
    _check(load("attention_composed").llms_attend_composed(
        c_int(_code(q)), _ptr(out), c_int(out.stride(0)), _ptr(q), c_int(q.stride(0)), _ptr(k_pool), _ptr(v_pool),
        _ptr(block_tables), _ptr(table_rows), c_int(block_tables.shape[1]), _ptr(token_seq), _ptr(positions),
        _ptr(context_lens), c_int(n), c_int(heads), c_int(kv_heads), c_int(maps), c_int(dk), c_int(dv),
        c_int(block_size), c_int(window), c_int(keep_first), c_int(chunk), c_float(scale), _ptr(slopes), _ptr(talk),
        c_float(lam), c_int(1 if head_norm else 0), c_float(eps), c_float(out_scale), _ptr(dist_bias),
        c_int(dist_bias.shape[1] - 1 if dist_bias is not None else 0), _ptr(gate),
        c_int(gate.stride(0) if gate is not None else 0), c_int(1 if sink else 0), _stream(dev)),
        "attend_composed")
    return out


def attend_composed_mfma_supported(dtype: torch.dtype, heads: int, kv_heads: int, dk: int, dv: int, block_size: int,
                                    talk: bool) -> bool:
    """Whether the matrix-core kernel takes this attention (else `attend_composed` does)."""
    if dtype != torch.bfloat16 or heads % kv_heads or heads // kv_heads > 16:
        return False
    if dk % 16 or dv % 16 or not (0 < dk <= 128 and 0 < dv <= 128) or block_size % 4:
        return False
    if talk:
        tok = max(1, 32 // kv_heads) * (16 // (heads // kv_heads))
        return kv_heads <= 32 and (tok * heads * 16 + heads * heads) * 4 <= ATTEND_COMPOSED_LDS
    return True


def attend_composed_mfma_tokens(heads: int, kv_heads: int, dk: int, dv: int, max_new: int) -> int:
    """Tokens one workgroup of `attend_composed_mfma` takes when heads are mixed (0: sizes it does not take)."""
    return int(load("attention_composed_mfma").llms_attend_composed_mfma_tokens(
        c_int(heads), c_int(kv_heads), c_int(dk), c_int(dv), c_int(max_new)))


def attend_composed_mfma(out: torch.Tensor, q: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                         block_tables: torch.Tensor, cu_seqlens: torch.Tensor, context_lens: torch.Tensor,
                         seq_begin: int, n_seqs: int, max_new: int, *, heads: int, kv_heads: int, dk: int, dv: int,
                         block_size: int, scale: float, maps: int = 1, window: int = 0, keep_first: int = 0,
                         chunk: int = 0, slopes: torch.Tensor | None = None, talk: torch.Tensor | None = None,
                         lam: float = 0.0, head_norm: bool = False, eps: float = 0.0, out_scale: float = 1.0,
                         table_rows: torch.Tensor | None = None, shares: int = 1, dist_bias: torch.Tensor | None = None,
                         gate: torch.Tensor | None = None, sink: bool = False) -> torch.Tensor:
    """`attend_composed` on the matrix cores (bfloat16) for requests [seq_begin, seq_begin + n_seqs) of a step: request
    b owns rows cu_seqlens[b] .. cu_seqlens[b+1] of q and out, brings at most `max_new` tokens and is context_lens[b]
    long after the step (0: padding, left alone).  Same arguments and arithmetic otherwise; the weights are rounded
    to bfloat16 as the operand of the value product.  `shares` > 1 (where the heads' weights are mixed): the keys
    of every block of tokens are shared out to that many workgroups in two launches (maxima and sums; weights and
    values), their 32-bit parts added up by a third."""
    dev = _dev(out, q, k_pool, v_pool, block_tables, cu_seqlens, context_lens, slopes, talk, table_rows, dist_bias, gate)
    if not attend_composed_mfma_supported(q.dtype, heads, kv_heads, dk, dv, block_size, talk is not None):
        raise ValueError("attend_composed_mfma does not take these sizes; see attend_composed_mfma_supported")
    if q.dim() != 2 or q.stride(1) != 1 or q.shape[1] < heads * maps * dk or q.stride(0) % 4 or q.data_ptr() % 8:
        raise ValueError("q must be [N, >= heads*maps*dk] with unit inner stride and 8-byte aligned rows")
    _rows(out, "out", heads * dv)
    if out.shape[0] != q.shape[0] or out.dtype != q.dtype or out.data_ptr() % 8:
        raise ValueError("out and q disagree")
    pages = k_pool.shape[0]
    if tuple(k_pool.shape) != (pages, kv_heads * maps, block_size, dk) or not k_pool.is_contiguous():
        raise ValueError(f"k_pool shape {tuple(k_pool.shape)} is not [pages,{kv_heads * maps},{block_size},{dk}]")
    if tuple(v_pool.shape) != (pages, kv_heads, dv, block_size) or not v_pool.is_contiguous():
        raise ValueError(f"v_pool shape {tuple(v_pool.shape)} is not [pages,{kv_heads},{dv},{block_size}]")
    if k_pool.dtype != q.dtype or v_pool.dtype != q.dtype or k_pool.data_ptr() % 8 or v_pool.data_ptr() % 8:
        raise ValueError("pools and q differ in dtype, or a pool is not 8-byte aligned")
    if block_tables.dim() != 2 or block_tables.dtype != torch.int32 or not block_tables.is_contiguous():
        raise ValueError("block_tables must be a contiguous int32 [B, M] tensor")
    if maps not in (1, 2) or (talk is not None and maps != 1):
        raise ValueError("maps is 1 or 2, and talk goes with maps = 1")
    _i32(cu_seqlens, "cu_seqlens")
    b = cu_seqlens.numel() - 1
    _i32(context_lens, "context_lens", b)
    if table_rows is not None:
        _i32(table_rows, "table_rows", b)
    elif block_tables.shape[0] < b:
        raise ValueError("block_tables has fewer rows than there are requests")
    if not (0 <= seq_begin and n_seqs >= 0 and seq_begin + n_seqs <= b):
        raise ValueError("request range is outside the batch")
    if slopes is not None:
        _f32(slopes, "slopes", heads)
    if talk is not None:
        _f32(talk, "talk", heads * heads)
    if dist_bias is not None and (dist_bias.dtype != torch.float32 or dist_bias.dim() != 2 or dist_bias.shape[0] != heads
                                  or dist_bias.shape[1] < 1 or not dist_bias.is_contiguous()):
        raise ValueError("dist_bias must be a contiguous float32 [heads, reach + 1] tensor")
    if gate is not None and (talk is not None or gate.dtype != torch.float32 or gate.dim() != 2 or gate.stride(1) != 1
                             or gate.shape[0] != q.shape[0] or gate.shape[1] < heads * dv or gate.stride(0) % 4
                             or gate.data_ptr() % 16):
        raise ValueError("gate must be float32 [N, >= heads*dv] with unit inner stride and 16-byte aligned rows (and no mixed heads)")
    if n_seqs == 0 or max_new <= 0 or q.shape[0] == 0:
        return out
    ws_stats = ws_o = None
    if not (shares > 1 and talk is not None):
        shares = 1
    else:
        shares = min(int(shares), 16)
        ws_stats = torch.empty((q.shape[0], heads, shares, 2), dtype=torch.float32, device=dev)
        ws_o = torch.empty((shares, q.shape[0], heads * dv), dtype=torch.float32, device=dev)
    _check(load("attention_composed_mfma").llms_attend_composed_mfma(
        _ptr(out), c_int(out.stride(0)), _ptr(q), c_int(q.stride(0)), _ptr(k_pool), _ptr(v_pool), _ptr(block_tables),
        _ptr(table_rows), c_int(block_tables.shape[1]), _ptr(cu_seqlens), _ptr(context_lens), c_int(seq_begin),
        c_int(n_seqs), c_int(max_new), c_int(heads), c_int(kv_heads), c_int(maps), c_int(dk), c_int(dv),
        c_int(block_size), c_int(window), c_int(keep_first), c_int(chunk), c_float(scale), _ptr(slopes), _ptr(talk),
        c_float(lam), c_int(1 if head_norm else 0), c_float(eps), c_float(out_scale), c_int(shares), _ptr(ws_stats),
        _ptr(ws_o), c_int(q.shape[0]), _ptr(dist_bias), c_int(dist_bias.shape[1] - 1 if dist_bias is not None else 0),
        _ptr(gate), c_int(gate.stride(0) if gate is not None else 0), c_int(1 if sink else 0), _stream(dev)),
        "attend_composed_mfma")
    return out


# ------------------------------------------------------------------------------ sampling


def sample_rows(out: torch.Tensor, logits: torch.Tensor, temperature: torch.Tensor | None = None,
                top_k: torch.Tensor | None = None, top_p: torch.Tensor | None = None,
                uniform: torch.Tensor | None = None) -> torch.Tensor:
    """out[r] = chosen token of logits[r] (float32 [R,V]); all-None options mean greedy."""
    dev = _dev(out, logits, temperature, top_k, top_p, uniform)
    if logits.dim() != 2 or logits.dtype != torch.float32 or logits.stride(1) != 1:
        raise ValueError("logits must be float32 [R, V] with unit inner stride")
    r, v = logits.shape
    _i32(out, "out", r)
    if temperature is not None:
        _f32(temperature, "temperature", r)
        if uniform is None:
            raise ValueError("temperature sampling needs uniform numbers")
    if top_k is not None:
        _i32(top_k, "top_k", r)
    if top_p is not None:
        _f32(top_p, "top_p", r)
    if uniform is not None:
        _f32(uniform, "uniform", r)
    if r == 0:
        return out
    _check(load("sampling").llms_sample_rows(
        _ptr(out), _ptr(logits), c_int(logits.stride(0)), c_int(r), c_int(v), _ptr(temperature), _ptr(top_k),
        _ptr(top_p), _ptr(uniform), _stream(dev)), "sample_rows")
    return out


# ------------------------------------------------------------------------------ streams of residuals, layer norm

STREAMS_MAX = 8


def streams_norm(out: torch.Tensor | None, x: torch.Tensor, weight: torch.Tensor | None, eps: float, *,
                 source: torch.Tensor | None = None, y: torch.Tensor | None = None, mix: torch.Tensor | None = None,
                 write: torch.Tensor | None = None, read: torch.Tensor | None = None,
                 rows: torch.Tensor | None = None, center: bool = True) -> torch.Tensor | None:
    """A residual stream of S copies x [N, S, hidden] (float32), in one kernel:
    with `y` [N, hidden] the streams become new_t = sum_s mix[s, t] x_s + write[t] y, all at once (stored into x
    unless `rows` picks rows); u = sum_t read[t] new_t (`read` None: the plain sum); out = layer norm of u with
    `weight`, no bias, rounded once to out's dtype (`center` False: the mean is not taken off, an RMS norm).  `source` [N, hidden]: the streams are read as S copies of it
    (and stored into x).  `rows`: out[r] is worked out from row rows[r], nothing is stored.  `out` None: only the
    streams are brought up to date."""
    dev = _dev(out, x, weight, source, y, mix, write, read, rows)
    if x.dim() != 3 or x.dtype != torch.float32 or not x.is_contiguous():
        raise ValueError(f"x must be a contiguous float32 [N, S, hidden] tensor, got {tuple(x.shape)} {x.dtype}")
    n, s, hidden = x.shape
    if not 1 <= s <= STREAMS_MAX:
        raise ValueError(f"1 to {STREAMS_MAX} streams, got {s}")
    if hidden * 4 > 96 * 1024:
        raise ValueError("rows of up to 24,576 elements")
    for t, name, numel in ((mix, "mix", s * s), (write, "write", s), (read, "read", s)):
        if t is not None:
            _f32(t, name, numel)
    if (mix is None) != (write is None) or (y is None and mix is not None):
        raise ValueError("mix and write come together, with y")
    if y is not None:
        _f32(y, "y", n * hidden)
    if source is not None:
        _f32(source, "source", n * hidden)
    store = rows is None
    if rows is not None:
        _i32(rows, "rows")
        n_out = rows.numel()
    else:
        n_out = n
    if out is not None:
        _rows(out, "out", hidden)
        if out.shape[0] != n_out:
            raise ValueError(f"out has {out.shape[0]} rows, expected {n_out}")
        _f32(weight, "weight", hidden)
    elif not store or (y is None and source is None):
        raise ValueError("nothing to do: no output and nothing to store")
    if n_out == 0:
        return out
    src = source if source is not None else x
    _check(load("stream32").llms_streams_norm(
        c_int(_code(out) if out is not None else 0), _ptr(out), _ptr(x), _ptr(src), c_int(source is not None), _ptr(y),
        _ptr(mix), _ptr(write), _ptr(read), _ptr(weight), _ptr(rows), c_int(n_out), c_int(s), c_int(hidden), c_float(eps),
        c_int(1 if store and (y is not None or source is not None) else 0), c_int(1 if center else 0), _stream(dev)),
        "streams_norm")
    return out


# ------------------------------------------------------------------------------ attention through a latent


def _pairing(pairing: str) -> int:
    if pairing not in ("neighbours", "half"):
        raise ValueError(f"pairing {pairing!r}; choose 'neighbours' (2i, 2i+1) or 'half' (i, i + dims/2)")
    return 1 if pairing == "half" else 0


def _latent_rotation(freq: torch.Tensor | None, dr: int) -> int:
    if freq is None:
        return 0
    _f32(freq, "freq")
    dims = 2 * freq.numel()
    if dims > dr:
        raise ValueError(f"{dims} turned dimensions in a part of {dr}")
    return dims


def latent_prepare(z: torch.Tensor, *, col_q: int, q_rank: int, col_c: int | None, r: int, dr: int, wq: torch.Tensor,
                   wc: torch.Tensor | None, freq: torch.Tensor | None, positions: torch.Tensor, eps: float,
                   cq: torch.Tensor, pool: torch.Tensor | None = None, slots: torch.Tensor | None = None,
                   pairing: str = "neighbours") -> torch.Tensor:
    """From the 32-bit input products z [N, columns]: cq [N, q_rank] = z[:, col_q:][:q_rank] over its root mean
    square times wq; with `col_c`, the cache rows pool[slots[n]] = [z_c over its root mean square times wc ; the dr
    columns behind it with their first 2 len(freq) dimensions turned by the token's position (pairs 2i, 2i+1; with
    `pairing` "half" pairs i, i + len(freq))].
    pool [pages, 1, block, r + dr] in the dtype of cq."""
    dev = _dev(z, wq, wc, freq, positions, cq, pool, slots)
    if z.dim() != 2 or z.dtype != torch.float32 or z.stride(1) != 1:
        raise ValueError("z must be a float32 matrix with unit inner stride")
    n = z.shape[0]
    _rows(cq, "cq", q_rank)
    _f32(wq, "wq", q_rank)
    _i32(positions, "positions", n)
    dims = _latent_rotation(freq, dr)
    if col_q < 0 or col_q + q_rank > z.shape[1]:
        raise ValueError("the query latent's columns lie outside z")
    if col_c is not None:
        if col_c < 0 or col_c + r + dr > z.shape[1]:
            raise ValueError("the latent's columns lie outside z")
        _f32(wc, "wc", r)
        if pool is None or slots is None or pool.dtype != cq.dtype or not pool.is_contiguous() or pool.shape[-1] != r + dr:
            raise ValueError("a layer that keeps a latent needs its pool [.., r + dr] in cq's dtype and the tokens' slots")
        _i32(slots, "slots", n)
    if cq.shape[0] != n:
        raise ValueError("cq and z differ in rows")
    if n == 0:
        return cq
    _check(load("latent").llms_latent_prepare(
        c_int(_code(cq)), _ptr(cq), _ptr(pool if col_c is not None else None), _ptr(z), c_int(z.stride(0)), c_int(col_q),
        c_int(q_rank), c_int(-1 if col_c is None else col_c), c_int(r), c_int(dr), _ptr(wq), _ptr(wc), _ptr(freq), c_int(dims),
        _ptr(positions), _ptr(slots if col_c is not None else None), c_float(eps), c_int(n), c_int(_pairing(pairing)),
        _stream(dev)), "latent_prepare")
    return cq


def latent_query(plain: torch.Tensor, folded: torch.Tensor, q: torch.Tensor, *, heads: int, dn: int, dr: int, r: int,
                 freq: torch.Tensor | None, positions: torch.Tensor, pairing: str = "neighbours") -> None:
    """q [N, heads * (dn + dr)] float32 -> plain [N, heads * dn] (the unrotated parts) and folded[n, h, r:] (the
    rotated parts, turned); folded [N, heads * (r + dr)]."""
    dev = _dev(plain, folded, q, freq, positions)
    n = q.shape[0]
    _f32(q, "q", n * heads * (dn + dr))
    _rows(plain, "plain", heads * dn)
    _rows(folded, "folded", heads * (r + dr))
    _i32(positions, "positions", n)
    if plain.dtype != folded.dtype or plain.shape[0] != n or folded.shape[0] != n:
        raise ValueError("plain and folded share one dtype and q's rows")
    dims = _latent_rotation(freq, dr)
    if n == 0:
        return
    _check(load("latent").llms_latent_query(
        c_int(_code(plain)), _ptr(plain), _ptr(folded), _ptr(q), c_int(heads), c_int(dn), c_int(dr), c_int(r), _ptr(freq),
        c_int(dims), _ptr(positions), c_int(n), c_int(_pairing(pairing)), _stream(dev)), "latent_query")


LATENT_ROW_MAX = 1024


def attend_latent(out: torch.Tensor, q: torch.Tensor, pool: torch.Tensor, block_tables: torch.Tensor,
                  token_seq: torch.Tensor, positions: torch.Tensor, context_lens: torch.Tensor, *, heads: int, r: int,
                  dr: int, block_size: int, window: int, scale: float, table_rows: torch.Tensor | None = None) -> torch.Tensor:
    """out[n, h] = sum_j softmax_j(scale q[n, h] . row_j) row_j[:r] over the cache rows j of token n's request with
    0 <= position - j < window (window 0: every j <= position); q [N, heads * (r + dr)], out [N, heads * r], pool
    [pages, 1, block, r + dr]."""
    dev = _dev(out, q, pool, block_tables, token_seq, positions, context_lens, table_rows)
    n = q.shape[0]
    _rows(q, "q", heads * (r + dr))
    _rows(out, "out", heads * r)
    if out.shape[0] != n or out.dtype != q.dtype or pool.dtype != q.dtype:
        raise ValueError("out, q and pool share one dtype; out and q their rows")
    if not pool.is_contiguous() or pool.dim() != 4 or pool.shape[1] != 1 or pool.shape[2] != block_size or pool.shape[3] != r + dr:
        raise ValueError(f"pool must be [pages, 1, {block_size}, {r + dr}], got {tuple(pool.shape)}")
    if r + dr > LATENT_ROW_MAX:
        raise ValueError(f"a cache row of up to {LATENT_ROW_MAX} numbers")
    if block_tables.dtype != torch.int32 or block_tables.dim() != 2 or not block_tables.is_contiguous():
        raise ValueError("block_tables must be a contiguous int32 matrix")
    _i32(token_seq, "token_seq", n)
    _i32(positions, "positions", n)
    _i32(context_lens, "context_lens")
    if table_rows is not None:
        _i32(table_rows, "table_rows", context_lens.numel())
    elif block_tables.shape[0] < context_lens.numel():
        raise ValueError("fewer block tables than requests")
    if window < 0:
        raise ValueError("window must be >= 0")
    if n == 0:
        return out
    _check(load("latent").llms_attend_latent(
        c_int(_code(q)), _ptr(out), _ptr(q), _ptr(pool), _ptr(block_tables), c_int(block_tables.shape[1]), _ptr(table_rows),
        _ptr(token_seq), _ptr(positions), _ptr(context_lens), c_int(n), c_int(heads), c_int(r), c_int(dr), c_int(block_size),
        c_int(window), c_float(scale), _stream(dev)), "attend_latent")
    return out


LATENT_MFMA = os.environ.get("LLMSERVE_LATENT_ATTENTION", "") != "plain"  # "plain": keep the matrix-core kernel out
LATENT_MFMA_PAIRS = 128  # (token, head) pairs of a workgroup of the matrix-core kernel
LATENT_MFMA_KEYS = 32  # keys of one of its tiles


def attend_latent_mfma_supported(dtype: torch.dtype, r: int, dr: int) -> bool:
    """Whether the matrix-core kernel takes these sizes: bfloat16, r a multiple of 16 up to 512, r + dr a multiple of
    8 that fits r's size class."""
    if not LATENT_MFMA or dtype != torch.bfloat16 or r % 16 or (r + dr) % 8 or r > 512:
        return False
    padded = -(-(r + dr) // 32) * 32
    return any(r <= 16 * rt and padded <= 32 * (rt // 2 + 2) for rt in (8, 16, 32))


def attend_latent_mfma(out: torch.Tensor, q: torch.Tensor, pool: torch.Tensor, block_tables: torch.Tensor,
                       cu_seqlens: torch.Tensor, context_lens: torch.Tensor, *, n_seqs: int, max_count: int, heads: int,
                       r: int, dr: int, block_size: int, window: int, scale: float, splits: int = 1,
                       table_rows: torch.Tensor | None = None) -> torch.Tensor:
    """`attend_latent` on the matrix cores for the requests [0, n_seqs) of a step: request b owns the rows
    cu_seqlens[b] .. cu_seqlens[b + 1] of q and out, which are its last tokens (positions context_lens[b] - count ..).
    `max_count`: no request brings more rows.  `splits`: workgroups that share the keys of one block of rows."""
    dev = _dev(out, q, pool, block_tables, cu_seqlens, context_lens, table_rows)
    n = q.shape[0]
    _rows(q, "q", heads * (r + dr))
    _rows(out, "out", heads * r)
    if not attend_latent_mfma_supported(q.dtype, r, dr):
        raise ValueError(f"the matrix-core kernel does not take {q.dtype} rows of {r} + {dr}")
    if out.shape[0] != n or out.dtype != q.dtype or pool.dtype != q.dtype:
        raise ValueError("out, q and pool share one dtype; out and q their rows")
    if not pool.is_contiguous() or pool.dim() != 4 or pool.shape[1] != 1 or pool.shape[2] != block_size or pool.shape[3] != r + dr:
        raise ValueError(f"pool must be [pages, 1, {block_size}, {r + dr}], got {tuple(pool.shape)}")
    if block_tables.dtype != torch.int32 or block_tables.dim() != 2 or not block_tables.is_contiguous():
        raise ValueError("block_tables must be a contiguous int32 matrix")
    _i32(cu_seqlens, "cu_seqlens")
    _i32(context_lens, "context_lens")
    if cu_seqlens.numel() < n_seqs + 1 or context_lens.numel() < n_seqs or n_seqs < 1 or max_count < 1:
        raise ValueError("cu_seqlens and context_lens do not cover the requests")
    if table_rows is not None:
        _i32(table_rows, "table_rows")
        if table_rows.numel() < n_seqs:
            raise ValueError("table_rows does not cover the requests")
    elif block_tables.shape[0] < n_seqs:
        raise ValueError("fewer block tables than requests")
    if window < 0 or not 1 <= splits <= 16:
        raise ValueError("window must be >= 0 and splits 1 to 16")
    if n == 0:
        return out
    ws = torch.empty(n * heads * splits * (r + 2), dtype=torch.float32, device=dev) if splits > 1 else None
    _check(load("latent_mfma").llms_attend_latent_mfma(
        _ptr(out), _ptr(q), _ptr(pool), _ptr(block_tables), c_int(block_tables.shape[1]), _ptr(table_rows), _ptr(cu_seqlens),
        _ptr(context_lens), _ptr(ws), c_int(n_seqs), c_int(n), c_int(max_count), c_int(heads), c_int(r), c_int(dr),
        c_int(block_size), c_int(window), c_float(scale), c_int(splits), _stream(dev)), "attend_latent_mfma")
    return out


# ------------------------------------------------------------------------------ products with a weight per group

c_long = ctypes.c_long
GROUPED_TILE = 64  # rows of a tile of the multiply-add kernel
GROUPED_TILE_MFMA = 128  # and of the matrix-core kernel
PAIRED_BLOCK = 32  # units per block of a paired weight: 32 rows of the first projection, then 32 of the second
_EPILOGUES = {"plain": 0, "paired": 1, "gated": 2}
_GATED_UNITS = {"clamped": 0, "silu": 1}
GROUPED_KERNEL = os.environ.get("LLMSERVE_GROUPED_GEMM", "")  # "fma": keep the matrix-core kernel out


def stack_paired(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """[.., units, K] twice -> [.., 64 * ceil(units / 32), K]: blocks of 32 rows of a followed by the 32 rows of b of
    the same units (rows of units that do not exist are zero): the weight of the "paired" epilogue."""
    units, k = a.shape[-2:]
    blocks = -(-units // PAIRED_BLOCK)
    pad = blocks * PAIRED_BLOCK - units
    if pad:
        zeros = torch.zeros((*a.shape[:-2], pad, k), dtype=a.dtype, device=a.device)
        a, b = torch.cat([a, zeros], dim=-2), torch.cat([b, zeros], dim=-2)
    a = a.reshape(*a.shape[:-2], blocks, PAIRED_BLOCK, k)
    b = b.reshape(*b.shape[:-2], blocks, PAIRED_BLOCK, k)
    return torch.cat([a, b], dim=-2).reshape(*a.shape[:-3], blocks * 2 * PAIRED_BLOCK, k).contiguous()


def _grouped_on_matrix_cores(x: torch.Tensor, w: torch.Tensor, x_ld: int, x_gs: int) -> bool:
    return (GROUPED_KERNEL != "fma" and x.dtype == torch.bfloat16 and w.shape[2] % 8 == 0 and x_ld % 8 == 0
            and x_gs % 8 == 0 and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


def grouped_product(out: torch.Tensor, x: torch.Tensor, w: torch.Tensor, *, epilogue: str = "plain",
                    segments: "tuple[torch.Tensor, torch.Tensor] | None" = None, gate: torch.Tensor | None = None,
                    gate_column: int = 0, limit: float = 0.0, units: int = 0, k_parts: int = 1,
                    unit: str = "clamped") -> torch.Tensor:
    """w [G, N, K].  Without `segments` every row meets every group: x [M, G, K] and out [M, G, N'] (views whose
    last axis has unit stride; the strides of the other two are free), out[m, g] = x[m, g] w[g]^T.  With `segments`
    = (seg [G + 1], tile_start [2, G + 1]) on the device (what `moe_sort` returns), x [M, K] and out [M, N'] hold rows
    sorted by group, rows seg[g] .. seg[g + 1] belonging to group g.
    Epilogues: "plain" (N' = N); "paired" (N' = `units`: w is `stack_paired(a, b)`,
    out = min(a, limit) sigmoid(1.702 min(a, limit)) (clamp(b, +-limit) + 1), or with `unit` "silu"
    out = a sigmoid(a) b); "gated" (out times
    sigmoid(gate[m, gate_column + g N + n]), gate float32 [M, columns]).
    bfloat16 operands with K and the strides of x in multiples of 8 go to the matrix cores, all else to the 32-bit
    multiply-add kernel.  `k_parts` > 1 (as `grouped_k_parts` allows): out is float32 [k_parts, M, N] and holds partial
    sums over shares of K, for the caller to add up."""
    parts_out = None
    if k_parts > 1:
        if out.dim() != 3 or out.shape[0] != k_parts or not out.is_contiguous() or out.dtype != torch.float32:
            raise ValueError("partial sums go to a contiguous float32 [k_parts, M, N] tensor")
        parts_out, out = out, out[0]
    dev = _dev(out, x, w, gate, *(segments or ()))
    if w.dim() != 3 or not w.is_contiguous():
        raise ValueError("w must be a contiguous [G, N, K] tensor")
    g, n, k = w.shape
    if epilogue not in _EPILOGUES:
        raise ValueError(f"epilogue {epilogue!r}")
    if unit not in _GATED_UNITS:
        raise ValueError(f"unit {unit!r}; choose from {sorted(_GATED_UNITS)}")
    if epilogue == "paired" and (n % (2 * PAIRED_BLOCK) or not 0 < units <= n // 2):
        raise ValueError(f"a paired weight of {n} rows does not hold {units} units")
    n_out = units if epilogue == "paired" else n
    if x.dtype != w.dtype or (x.dtype, out.dtype) not in ((torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16),
                                                         (torch.bfloat16, torch.float32)):
        raise ValueError(f"grouped_product does not take {x.dtype} x {w.dtype} -> {out.dtype}")
    if segments is None:
        if x.dim() != 3 or out.dim() != 3 or x.stride(2) != 1 or out.stride(2) != 1:
            raise ValueError("x and out must be [M, G, .] views with unit inner stride")
        if tuple(x.shape[1:]) != (g, k) or tuple(out.shape) != (x.shape[0], g, n_out):
            raise ValueError(f"x {tuple(x.shape)} and out {tuple(out.shape)} do not fit w {tuple(w.shape)}")
        m = x.shape[0]
        x_ld, x_gs, out_ld, out_gs = x.stride(0), x.stride(1), out.stride(0), out.stride(1)
    else:
        seg, tiles = segments
        _i32(seg, "seg", g + 1)
        _i32(tiles, "tile_start", 2 * (g + 1))
        if x.dim() != 2 or out.dim() != 2 or x.stride(1) != 1 or out.stride(1) != 1:
            raise ValueError("x and out must be matrices with unit inner stride")
        if x.shape[1] != k or tuple(out.shape) != (x.shape[0], n_out):
            raise ValueError(f"x {tuple(x.shape)} and out {tuple(out.shape)} do not fit w {tuple(w.shape)}")
        m = x.shape[0]
        x_ld, x_gs, out_ld, out_gs = x.stride(0), 0, out.stride(0), 0
    mfma = _grouped_on_matrix_cores(x, w, x_ld, x_gs)
    if k_parts > 1 and not (mfma and segments is not None and epilogue == "plain"):
        raise ValueError("K is shared out only by the matrix-core kernel, with segments and the plain epilogue")
    seg_ptr = tiles_ptr = None
    max_tiles = 0
    if segments is not None:
        tile = GROUPED_TILE_MFMA if mfma else GROUPED_TILE
        seg_ptr, tiles_ptr = seg, tiles.view(2, g + 1)[1 if mfma else 0]
        max_tiles = -(-m // tile) + g
    z_ld = z_gs = 0
    z = None
    if epilogue == "gated":
        if gate is None or gate.dtype != torch.float32 or gate.dim() != 2 or gate.stride(1) != 1 or gate.shape[0] != m:
            raise ValueError("the gated epilogue needs float32 gate products [M, columns]")
        if gate_column < 0 or gate_column + g * n > gate.shape[1]:
            raise ValueError("the gate's columns lie outside the gate products")
        z, z_ld, z_gs = gate[:, gate_column:], gate.stride(0), n
    if m == 0:
        return out
    common = (_ptr(out), c_long(out_ld), c_long(out_gs), _ptr(x), c_long(x_ld), c_long(x_gs), _ptr(w), c_int(m), c_int(n),
              c_int(k), c_int(g), _ptr(seg_ptr), _ptr(tiles_ptr), c_int(max_tiles), _ptr(z), c_long(z_ld), c_long(z_gs),
              c_float(limit), c_int(_GATED_UNITS[unit]), c_int(units), _stream(dev))
    lib = load("grouped_gemm")
    if mfma:
        _check(lib.llms_grouped_mfma(c_int(_code(out)), c_int(_EPILOGUES[epilogue]), *common[:-1], c_int(k_parts),
                                     c_long(out.numel() if k_parts > 1 else 0), common[-1]), "grouped_product")
    else:
        _check(lib.llms_grouped_fma(c_int(_code(x)), c_int(_code(out)), c_int(_EPILOGUES[epilogue]), *common), "grouped_product")
    return out if parts_out is None else parts_out


def grouped_k_parts(x: torch.Tensor, w: torch.Tensor, cus: int = 256) -> int:
    """Into how many shares a product over segments of few rows (x [M, K] against w [G, N, K]) splits its K: while the
    weights' tiles alone leave compute units idle and each would walk a long K with one load in flight, up to 4 shares
    of 512 numbers at least.  1 where the matrix-core kernel does not apply or the rows are many."""
    g, n, k = w.shape
    if x.shape[0] > 256 or not _grouped_on_matrix_cores(x, w, x.stride(0), 0):
        return 1
    tiles = g * -(-n // GROUPED_TILE_MFMA)
    return max(1, min(4, cus // max(tiles, 1), k // 512))


# ------------------------------------------------------------------------------ routing to experts

MOE_MAX_TOP = 16


def moe_router(chosen: torch.Tensor, weight: torch.Tensor, h: torch.Tensor, w_router: torch.Tensor, *,
               renormalize: bool = False, scores: str = "sigmoid", groups: int = 1, keep: int = 1,
               renorm_eps: float = 0.0, bias: torch.Tensor | None = None, extra_out: torch.Tensor | None = None) -> None:
    """Per row of h [N, hidden]: scores sigmoid(W_router h), or with `scores` "softmax" the softmax over all experts,
    in 32-bit; the `top` largest in descending order (the lower expert wins a tie) into chosen int32 [N, top], their
    scores (over their sum + `renorm_eps` with `renormalize`) into weight float32 [N, top].  `groups` > 1: the experts
    form that many equal groups of neighbours, a group's score is its largest, and only experts of the `keep` best
    groups can be chosen.  `bias` float32 [experts] is added to z.  `extra_out` float32 [N, extra]: w_router holds
    `extra` more rows behind the experts', whose products with h are stored there as they are."""
    dev = _dev(chosen, weight, h, w_router, bias, extra_out)
    _rows(h, "h")
    _rows(w_router, "w_router", h.shape[1])
    n, top = h.shape[0], chosen.shape[-1]
    _i32(chosen, "chosen", n * top)
    _f32(weight, "weight", n * top)
    extra = 0
    if extra_out is not None:
        if extra_out.dim() != 2 or extra_out.shape[0] != n:
            raise ValueError("extra_out is [N, extra]")
        extra = extra_out.shape[1]
        _f32(extra_out, "extra_out", n * extra)
    experts = w_router.shape[0] - extra
    if experts < 1:
        raise ValueError("w_router holds no experts' rows")
    if bias is not None:
        _f32(bias, "bias", experts)
    if h.dtype != w_router.dtype:
        raise ValueError("h and w_router differ in dtype")
    if not 1 <= top <= min(MOE_MAX_TOP, experts):
        raise ValueError(f"1 to {MOE_MAX_TOP} choices among {experts} experts, got {top}")
    if scores not in ("sigmoid", "softmax"):
        raise ValueError(f"scores {scores!r}; choose 'sigmoid' or 'softmax'")
    if groups < 1 or experts % groups or not 1 <= keep <= groups or (groups > 1 and top > keep * (experts // groups)):
        raise ValueError(f"{groups} groups of which {keep} are kept do not fit {experts} experts and {top} choices")
    if n == 0:
        return
    _check(load("moe").llms_moe_router(
        c_int(_code(h)), _ptr(chosen), _ptr(weight), _ptr(h), _ptr(w_router), c_int(n), c_int(h.shape[1]), c_int(experts),
        c_int(top), c_int(1 if renormalize else 0), c_int(1 if scores == "softmax" else 0), c_int(groups), c_int(keep),
        c_float(renorm_eps), _ptr(bias), c_int(extra), _ptr(extra_out), _stream(dev)), "moe_router")


def moe_sort(chosen: torch.Tensor, experts: int):
    """(rank [pairs], seg [E + 1], tile_start [2, E + 1]) of the pairs (token, choice) sorted by expert, stably: pair
    p's row is seg[chosen[p]] + rank[p]; tile_start counts the tiles of rows of all experts before each, once for the
    tiles of the multiply-add kernel and once for those of the matrix-core kernel."""
    dev = _dev(chosen)
    _i32(chosen, "chosen")
    pairs = chosen.numel()
    work = torch.empty(pairs + 4 * experts + 3, dtype=torch.int32, device=dev)
    count, rank = work[:experts], work[experts: experts + pairs]
    seg = work[experts + pairs: 2 * experts + pairs + 1]
    tiles = work[2 * experts + pairs + 1:]
    if pairs:
        _check(load("moe").llms_moe_sort(_ptr(count), _ptr(rank), _ptr(seg), _ptr(tiles), _ptr(chosen), c_int(pairs),
                                         c_int(experts), c_int(GROUPED_TILE), c_int(GROUPED_TILE_MFMA), _stream(dev)), "moe_sort")
    return rank, seg, tiles


MOE_FEW_PAIRS = 512  # pairs (token, choice) up to which `moe_place_few` sorts and scatters in one launch


def moe_place_few(xs: torch.Tensor, place: torch.Tensor, h: torch.Tensor, chosen: torch.Tensor, weight: torch.Tensor | None,
                  experts: int):
    """`moe_sort` and `moe_scatter` in one launch for few pairs: returns (seg [E + 1], tile_start [2, E + 1]) and fills
    xs and place as they do (the same rows: sorted by expert, stably)."""
    dev = _dev(xs, place, h, chosen, weight)
    _rows(h, "h")
    _i32(chosen, "chosen")
    pairs = chosen.numel()
    _rows(xs, "xs", h.shape[1])
    top = pairs // max(h.shape[0], 1)
    if xs.shape[0] != pairs or xs.dtype != h.dtype or top * h.shape[0] != pairs:
        raise ValueError("xs has a row per pair, in h's dtype")
    if not 0 < pairs <= 2048:
        raise ValueError("1 to 2,048 pairs")
    _i32(place, "place", pairs)
    if weight is not None:
        _f32(weight, "weight", pairs)
    work = torch.empty(3 * experts + 3, dtype=torch.int32, device=dev)
    seg, tiles = work[: experts + 1], work[experts + 1:]
    _check(load("moe").llms_moe_place_few(c_int(_code(h)), _ptr(xs), _ptr(place), _ptr(seg), _ptr(tiles), _ptr(h), _ptr(chosen),
                                          _ptr(weight), c_int(pairs), c_int(h.shape[1]), c_int(top), c_int(experts),
                                          c_int(GROUPED_TILE), c_int(GROUPED_TILE_MFMA), _stream(dev)), "moe_place_few")
    return seg, tiles


def moe_scatter(xs: torch.Tensor, place: torch.Tensor, h: torch.Tensor, chosen: torch.Tensor,
                weight: torch.Tensor | None, rank: torch.Tensor, seg: torch.Tensor) -> None:
    """xs[seg[chosen[p]] + rank[p]] = weight[p] * h[p // top] (rounded to xs's dtype; `weight` None: the row as it
    is); place[p] = that row."""
    dev = _dev(xs, place, h, chosen, weight, rank, seg)
    _rows(h, "h")
    pairs = chosen.numel()
    _rows(xs, "xs", h.shape[1])
    top = pairs // max(h.shape[0], 1)
    if xs.shape[0] != pairs or xs.dtype != h.dtype or top * h.shape[0] != pairs:
        raise ValueError("xs has a row per pair, in h's dtype")
    _i32(place, "place", pairs)
    _i32(chosen, "chosen", pairs)
    _i32(rank, "rank", pairs)
    _i32(seg, "seg")
    if weight is not None:
        _f32(weight, "weight", pairs)
    if pairs == 0:
        return
    _check(load("moe").llms_moe_scatter(c_int(_code(h)), _ptr(xs), _ptr(place), _ptr(h), _ptr(chosen), _ptr(weight), _ptr(rank),
                                        _ptr(seg), c_int(pairs), c_int(h.shape[1]), c_int(top), _stream(dev)), "moe_scatter")


def moe_combine(y: torch.Tensor, rows: torch.Tensor, place: torch.Tensor, weight: torch.Tensor | None = None, *,
                always: torch.Tensor | None = None, always_gate: torch.Tensor | None = None) -> torch.Tensor:
    """y[n] = sum_k rows[place[n, k]] in the order of k (times weight[n, k] where `weight`, float32 [N, top], is
    given); y float32 [N, hidden], rows float32 [pairs, hidden] or [parts, pairs, hidden] (partial sums of each row,
    added in the order of the parts).  `always` float32 [N, hidden]: a result that every token adds last, times
    sigmoid(always_gate[n]) where `always_gate` float32 [N] is given."""
    dev = _dev(y, rows, place, weight, always, always_gate)
    n, hidden = y.shape
    _f32(y, "y")
    _f32(rows, "rows")
    parts = rows.shape[0] if rows.dim() == 3 else 1
    pairs = rows.shape[-2]
    _i32(place, "place", pairs)
    top = pairs // max(n, 1)
    if rows.shape[-1] != hidden or top * n != pairs:
        raise ValueError("rows has top rows of y's width per row of y")
    if weight is not None:
        _f32(weight, "weight", pairs)
    if always is not None:
        _f32(always, "always", n * hidden)
    if always_gate is not None:
        if always is None:
            raise ValueError("always_gate comes with always")
        _f32(always_gate, "always_gate", n)
    if n == 0:
        return y
    _check(load("moe").llms_moe_combine(_ptr(y), _ptr(rows), _ptr(place), c_int(n), c_int(hidden), c_int(top), c_int(parts),
                                        c_long(pairs * hidden), _ptr(weight), _ptr(always), _ptr(always_gate), _stream(dev)),
           "moe_combine")
    return y


# ------------------------------------------------------------------------------ linear attention with a decay per head

DECAY_MAX_KEY = 256  # numbers of a key that `decay_scan` takes
_ACTIVATIONS = {None: 0, "none": 0, "silu": 1, "sigmoid": 2}


def _decay_proj(proj: torch.Tensor, col_q: int, col_k: int, col_v: int, heads: int, dk: int, dv: int) -> None:
    if proj.dim() != 2 or proj.dtype != torch.float32 or proj.stride(1) != 1:
        raise ValueError("proj must be a float32 [N, columns] tensor with unit inner stride")
    for col, width, name in ((col_q, heads * dk, "q"), (col_k, heads * dk, "k"), (col_v, heads * dv, "v")):
        if col < 0 or col + width > proj.shape[1]:
            raise ValueError(f"the columns of {name} ({col} .. {col + width}) lie outside proj's {proj.shape[1]}")


def decay_prepare(proj: torch.Tensor, *, col_q: int, col_k: int, col_v: int, heads: int, dk: int, dv: int,
                  activation: str | None = None, freq: torch.Tensor | None = None, rot_dims: int = 0,
                  positions: torch.Tensor | None = None, key_scale: float = 1.0) -> torch.Tensor:
    """In place on proj float32 [N, columns] (q, k and v of `heads` heads from the given columns on): `activation`
    ("silu" or None) on q, k and v; with `freq` float32 [rot_dims / 2], dimension i < rot_dims / 2 of every head of q and
    k is turned together with dimension i + rot_dims / 2 by the angle positions[n] * freq[i]; k times `key_scale`."""
    dev = _dev(proj, freq, positions)
    _decay_proj(proj, col_q, col_k, col_v, heads, dk, dv)
    if activation not in (None, "none", "silu"):
        raise ValueError(f"activation {activation!r}; choose 'silu' or None")
    if rot_dims:
        if rot_dims % 2 or not 0 < rot_dims <= dk:
            raise ValueError(f"{rot_dims} turned dimensions of {dk}")
        _f32(freq, "freq", rot_dims // 2)
        _i32(positions, "positions", proj.shape[0])
    if proj.shape[0] == 0:
        return proj
    _check(load("decay_attention").llms_decay_prepare(
        _ptr(proj), c_int(proj.stride(0)), c_int(col_q), c_int(col_k), c_int(col_v), _ptr(positions if rot_dims else None),
        _ptr(freq if rot_dims else None), c_int(rot_dims), c_int(proj.shape[0]), c_int(heads), c_int(dk), c_int(dv),
        c_int(_ACTIVATIONS[activation]), c_float(key_scale), _stream(dev)), "decay_prepare")
    return proj


def _decay_state(state, state_slots, cu_seqlens, context_lens, decay, heads, dk, dv) -> int:
    if state.dtype != torch.float32 or not state.is_contiguous() or tuple(state.shape[1:]) != (heads, dk, dv):
        raise ValueError(f"state must be a contiguous float32 [slots, {heads}, {dk}, {dv}] tensor")
    _i32(cu_seqlens, "cu_seqlens")
    b = cu_seqlens.numel() - 1
    _i32(state_slots, "state_slots", b)
    _i32(context_lens, "context_lens", b)
    _f32(decay, "decay", heads)
    return b


def _decay_prepare_args(prepare: dict | None, proj: torch.Tensor, dk: int) -> tuple:
    """The trailing arguments of the kernels that prepare q, k and v on their way in: (whether, positions, freq,
    rot_dims, activation, key_scale) from the keyword arguments of `decay_prepare` (None: nothing to prepare)."""
    if prepare is None:
        return c_int(0), None, None, c_int(0), c_int(0), c_float(1.0)
    if prepare.get("activation") not in (None, "none", "silu"):
        raise ValueError(f"activation {prepare.get('activation')!r}")
    rot = int(prepare.get("rot_dims") or 0)
    if rot % 2 or not 0 <= rot <= dk:
        raise ValueError("rot_dims must be even and at most dk")
    positions = freq = None
    if rot:
        positions, freq = prepare.get("positions"), prepare.get("freq")
        _f32(freq, "freq", rot // 2)
        _i32(positions, "positions", proj.shape[0])
        _dev(proj, freq, positions)
    return (c_int(1), _ptr(positions), _ptr(freq), c_int(rot), c_int(_ACTIVATIONS[prepare.get("activation")]),
            c_float(float(prepare.get("key_scale", 1.0))))


def decay_scan(out: torch.Tensor, proj: torch.Tensor, state: torch.Tensor, state_slots: torch.Tensor,
               cu_seqlens: torch.Tensor, context_lens: torch.Tensor, decay: torch.Tensor, *, col_q: int, col_k: int,
               col_v: int, heads: int, dk: int, dv: int, prepare: dict | None = None) -> torch.Tensor:
    """The recurrence S_t = decay_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t over the new tokens of every request, token by
    token: request b owns rows cu_seqlens[b] .. cu_seqlens[b+1] of proj (float32; q, k, v from the given columns on),
    starts from state[state_slots[b]] (float32 [slots, heads, dk, dv]; from zero when its portion starts at position 0,
    which context_lens[b], its length after the step, tells) and leaves its last state there.  out float32 [N, heads*dv].
    A request of length 0 is padding: its rows give zeros and no state is touched.  `prepare` (the keyword arguments of
    `decay_prepare`: activation, freq, rot_dims, positions, key_scale): proj is as the projection left it, and what
    `decay_prepare` would do to q, k and v is done on their way in, with the same arithmetic (proj is not written)."""
    dev = _dev(out, proj, state, state_slots, cu_seqlens, context_lens, decay)
    _decay_proj(proj, col_q, col_k, col_v, heads, dk, dv)
    prep_args = _decay_prepare_args(prepare, proj, dk)
    if out.dtype != torch.float32 or out.dim() != 2 or out.stride(1) != 1 or tuple(out.shape) != (proj.shape[0], heads * dv):
        raise ValueError(f"out must be float32 [{proj.shape[0]}, {heads * dv}] with unit inner stride")
    if dk > DECAY_MAX_KEY:
        raise ValueError(f"keys of up to {DECAY_MAX_KEY} numbers, got {dk}")
    b = _decay_state(state, state_slots, cu_seqlens, context_lens, decay, heads, dk, dv)
    if b <= 0 or proj.shape[0] == 0:
        return out
    _check(load("decay_attention").llms_decay_scan(
        _ptr(out), c_int(out.stride(0)), _ptr(proj), c_int(proj.stride(0)), c_int(col_q), c_int(col_k), c_int(col_v),
        _ptr(state), _ptr(state_slots), _ptr(cu_seqlens), _ptr(context_lens), _ptr(decay), c_int(b), c_int(heads), c_int(dk),
        c_int(dv), *prep_args, _stream(dev)), "decay_scan")
    return out


DECAY_CHUNKS_MAX_KEY = 128  # numbers of a key that `decay_chunks` takes
DECAY_CHUNKS_SLAB = 64  # columns of v that one of its workgroups takes


def decay_chunks(out: torch.Tensor, proj: torch.Tensor, state: torch.Tensor, state_slots: torch.Tensor,
                 cu_seqlens: torch.Tensor, context_lens: torch.Tensor, decay: torch.Tensor, max_new: int, *, col_q: int,
                 col_k: int, col_v: int, heads: int, dk: int, dv: int, prepare: dict | None = None) -> torch.Tensor:
    """What `decay_scan` computes, for portions of many tokens (`max_new`: the most one request brings): runs of 64
    tokens gather their own sums of k v^T, a scan over the runs gives the state before each and the request's last
    state, and every run adds what its tokens see of each other to what they see of that state; all products on the
    32-bit matrix instruction.  Same arguments (also `prepare`), and the same result up to the order of the sums."""
    dev = _dev(out, proj, state, state_slots, cu_seqlens, context_lens, decay)
    _decay_proj(proj, col_q, col_k, col_v, heads, dk, dv)
    if out.dtype != torch.float32 or out.dim() != 2 or out.stride(1) != 1 or tuple(out.shape) != (proj.shape[0], heads * dv):
        raise ValueError(f"out must be float32 [{proj.shape[0]}, {heads * dv}] with unit inner stride")
    if dk > DECAY_CHUNKS_MAX_KEY:
        raise ValueError(f"keys of up to {DECAY_CHUNKS_MAX_KEY} numbers, got {dk}")
    b = _decay_state(state, state_slots, cu_seqlens, context_lens, decay, heads, dk, dv)
    if b <= 0 or proj.shape[0] == 0 or max_new <= 0:
        return out
    prep_args = _decay_prepare_args(prepare, proj, dk)
    lib = load("decay_attention")
    lib.llms_decay_chunks_workspace.restype = ctypes.c_longlong
    floats = int(lib.llms_decay_chunks_workspace(c_int(proj.shape[0]), c_int(b), c_int(heads), c_int(dk), c_int(dv)))
    ws = torch.empty(floats, dtype=torch.float32, device=dev)
    _check(lib.llms_decay_chunks(
        _ptr(out), c_int(out.stride(0)), _ptr(proj), c_int(proj.stride(0)), c_int(col_q), c_int(col_k), c_int(col_v),
        _ptr(state), _ptr(state_slots), _ptr(cu_seqlens), _ptr(context_lens), _ptr(decay), _ptr(ws), c_int(b), c_int(max_new),
        c_int(heads), c_int(dk), c_int(dv), *prep_args, _stream(dev)), "decay_chunks")
    return out


def decay_finish(out: torch.Tensor, o: torch.Tensor, *, heads: int, dv: int, eps: float, weight: torch.Tensor | None = None,
                 gate: torch.Tensor | None = None, gate_activation: str | None = None) -> torch.Tensor:
    """out[n] = norm(o[n]) * activation(gate[n]), rounded once to out's dtype.  o float32 [N, heads*dv].  `weight` None:
    every head is divided by its own root mean square (eps inside the root); `weight` float32 [heads*dv]: all heads
    together are RMS-normed and multiplied by it.  `gate` float32 [N, >= heads*dv] (unit inner stride) with
    `gate_activation` "sigmoid" or "silu"."""
    dev = _dev(out, o, weight, gate)
    width = heads * dv
    if o.dtype != torch.float32 or o.dim() != 2 or o.stride(1) != 1 or o.shape[1] != width:
        raise ValueError(f"o must be float32 [N, {width}] with unit inner stride")
    _rows(out, "out", width)
    n = o.shape[0]
    if out.shape[0] != n:
        raise ValueError("out and o differ in rows")
    if weight is not None:
        _f32(weight, "weight", width)
    if gate_activation not in (None, "none", "silu", "sigmoid"):
        raise ValueError(f"gate_activation {gate_activation!r}")
    act = _ACTIVATIONS[gate_activation]
    if act:
        if gate is None or gate.dtype != torch.float32 or gate.dim() != 2 or gate.stride(1) != 1 or gate.shape[0] != n \
                or gate.shape[1] < width:
            raise ValueError(f"gate must be float32 [{n}, >= {width}] with unit inner stride")
    if width * 4 > 128 * 1024:
        raise ValueError("heads times value size up to 32,768")
    if n == 0:
        return out
    _check(load("decay_attention").llms_decay_finish(
        c_int(_code(out)), _ptr(out), c_int(out.stride(0)), _ptr(o), c_int(o.stride(0)), _ptr(gate if act else None),
        c_int(gate.stride(0) if act else 0), _ptr(weight), c_int(n), c_int(heads), c_int(dv), c_int(1 if weight is not None else 0),
        c_int(act), c_float(eps), _stream(dev)), "decay_finish")
    return out


def weighted_sum(out: torch.Tensor, a: torch.Tensor, b: torch.Tensor, scale_a: float, scale_b: float) -> torch.Tensor:
    """out = scale_a * a + scale_b * b, element by element in 32-bit (out may be a or b)."""
    dev = _dev(out, a, b)
    for t, name in ((out, "out"), (a, "a"), (b, "b")):
        _f32(t, name, out.numel())
    if out.numel():
        _check(load("stream32").llms_weighted_sum(_ptr(out), _ptr(a), _ptr(b), c_float(scale_a), c_float(scale_b),
                                                  ctypes.c_size_t(out.numel()), _stream(dev)), "weighted_sum")
    return out


# ------------------------------------------------------------------------------ a stream that sublayers join through a norm


def normed_add_norm(out: torch.Tensor | None, x: torch.Tensor, weight: torch.Tensor | None, eps: float, *,
                    y: torch.Tensor | None = None, y_weight: torch.Tensor | None = None, y_eps: float = 0.0,
                    rows: torch.Tensor | None = None) -> torch.Tensor | None:
    """x float32 [N, hidden], in one kernel: with `y` float32 [N, hidden], x += y / sqrt(mean(y^2) + y_eps) * y_weight
    (stored into x unless `rows` picks rows); out = x / sqrt(mean(x^2) + eps) * weight, rounded once to out's dtype.
    `rows` int32 [R]: out[r] comes from row rows[r] and nothing is stored.  `out` None: only the sum."""
    dev = _dev(out, x, weight, y, y_weight, rows)
    if x.dim() != 2 or x.dtype != torch.float32 or not x.is_contiguous():
        raise ValueError(f"x must be a contiguous float32 [N, hidden] tensor, got {tuple(x.shape)} {x.dtype}")
    n, hidden = x.shape
    if hidden * 4 > 128 * 1024:
        raise ValueError("rows of up to 32,768 elements")
    if y is not None:
        _f32(y, "y", n * hidden)
        _f32(y_weight, "y_weight", hidden)
    n_out = n
    if rows is not None:
        _i32(rows, "rows")
        n_out = rows.numel()
    if out is not None:
        _rows(out, "out", hidden)
        if out.shape[0] != n_out:
            raise ValueError(f"out has {out.shape[0]} rows, expected {n_out}")
        _f32(weight, "weight", hidden)
    elif y is None or rows is not None:
        raise ValueError("nothing to do: no output and nothing to store")
    if n_out == 0:
        return out
    _check(load("stream32").llms_normed_add_norm(
        c_int(_code(out) if out is not None else 0), _ptr(out), _ptr(x), _ptr(y), _ptr(y_weight), _ptr(weight), _ptr(rows),
        c_int(n_out), c_int(hidden), c_float(y_eps), c_float(eps), c_int(1 if rows is None else 0), _stream(dev)),
        "normed_add_norm")
    return out


def add_vector(x: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """x[..., :] += v for a contiguous float32 x whose last dimension is v's length."""
    dev = _dev(x, v)
    hidden = v.numel()
    _f32(v, "v")
    if x.dtype != torch.float32 or not x.is_contiguous() or x.shape[-1] != hidden:
        raise ValueError("x must be contiguous float32 with rows of v's length")
    n = x.numel() // max(hidden, 1)
    if n:
        _check(load("stream32").llms_add_vector(_ptr(x), _ptr(v), c_int(n), c_int(hidden), _stream(dev)), "add_vector")
    return x


# ------------------------------------------------------------------------------ recurrences over a state of fixed size

c_size_t = ctypes.c_size_t


def _state_rows(state: torch.Tensor, state_slots: torch.Tensor, need: int, offset: int, what: str) -> int:
    """state float32 [slots, numbers]: the stride between slots, after checking that [offset, offset + need) lies inside."""
    if state.dim() != 2 or state.dtype != torch.float32 or not state.is_contiguous():
        raise ValueError("state must be a contiguous float32 [slots, numbers] tensor")
    if offset < 0 or offset + need > state.shape[1]:
        raise ValueError(f"{what}: {need} numbers at {offset} do not fit a slot of {state.shape[1]}")
    _i32(state_slots, "state_slots")
    return state.shape[1]


def _f32_matrix(t: torch.Tensor, name: str, rows: int, min_cols: int) -> None:
    if t.dtype != torch.float32 or t.dim() != 2 or t.stride(1) != 1 or t.shape[0] != rows or t.shape[1] < min_cols:
        raise ValueError(f"{name} must be float32 [{rows}, >= {min_cols}] with unit inner stride")


def conv_act(u: torch.Tensor, u_col: int, channels: int, taps_w: torch.Tensor, *, bias: torch.Tensor | None = None,
             state: torch.Tensor | None = None, ring_offset: int = 0, batch=None, out32: torch.Tensor | None = None,
             out16: torch.Tensor | None = None, activation: str | None = "silu") -> None:
    """A causal convolution per channel over time on columns u_col .. u_col + channels of u (float32 [N, >=]):
    y_t = act(bias + sum_j taps_w[c, j] u_(t - taps + 1 + j)), zeros before the sequence; taps_w float32 [channels,
    taps] with the last column for the present token.  A request's last taps - 1 rows are a ring [taps - 1, channels]
    at `ring_offset` of its slot of `state` (float32 [slots, numbers]), indexed by position and brought up to date here.
    The result goes to out32 (float32 [N, channels]) and/or out16 ([N, channels] in any kernel dtype).  `batch` brings
    token_seq, positions, cu_seqlens, context_lens, state_slots, num_seqs and max_count."""
    dev = _dev(u, taps_w, bias, state, out32, out16)
    n = u.shape[0]
    _f32_matrix(u, "u", n, u_col + channels)
    taps = taps_w.shape[1]
    _f32(taps_w, "taps_w", channels * taps)
    if bias is not None:
        _f32(bias, "bias", channels)
    if activation not in (None, "silu"):
        raise ValueError(f"activation {activation!r}")
    slot_stride = 0
    if taps > 1:
        slot_stride = _state_rows(state, batch.state_slots, (taps - 1) * channels, ring_offset, "conv_act")
    for t, name in ((out32, "out32"), (out16, "out16")):
        if t is not None and (t.dim() != 2 or t.stride(1) != 1 or t.shape[0] != n or t.shape[1] != channels):
            raise ValueError(f"{name} must be [N, {channels}] with unit inner stride")
    if out32 is not None and out32.dtype != torch.float32:
        raise ValueError("out32 is float32")
    if out32 is None and out16 is None:
        raise ValueError("nothing to store")
    for t, name in ((batch.token_seq, "token_seq"), (batch.positions, "positions")):
        _i32(t, name, n)
    _i32(batch.cu_seqlens, "cu_seqlens")
    _i32(batch.context_lens, "context_lens")
    if n == 0:
        return
    lib = load("recurrent")
    single = taps > 1 and batch.max_count == 1 and batch.num_seqs == n  # every request brings one token
    _check(lib.llms_conv_act(
        c_int(_code(out16) if out16 is not None else 0), _ptr(out32), c_int(out32.stride(0) if out32 is not None else 0),
        _ptr(out16), c_int(out16.stride(0) if out16 is not None else 0), _ptr(u), c_int(u.stride(0)), c_int(u_col),
        _ptr(taps_w), _ptr(bias), c_int(taps), c_int(channels), _ptr(state), c_size_t(slot_stride), c_size_t(ring_offset),
        _ptr(batch.state_slots), _ptr(batch.token_seq), _ptr(batch.positions), _ptr(batch.cu_seqlens),
        _ptr(batch.context_lens), c_int(n), c_int(1 if activation == "silu" else 0), c_int(1 if single else 0),
        _stream(dev)), "conv_act")
    if taps > 1 and not single:
        _check(lib.llms_conv_ring(_ptr(state), c_size_t(slot_stride), c_size_t(ring_offset), _ptr(batch.state_slots), _ptr(u),
                                  c_int(u.stride(0)), c_int(u_col), _ptr(batch.cu_seqlens), _ptr(batch.context_lens),
                                  c_int(batch.num_seqs), c_int(taps), c_int(channels), _stream(dev)), "conv_ring")


def conv_heads(u: torch.Tensor, u_col: int, channels: int, taps_w: torch.Tensor, out32: torch.Tensor, *, q_heads: int, k_heads: int,
               dk: int, eps: float, q_factor: float = 1.0, bias: torch.Tensor | None = None, state: torch.Tensor | None = None,
               ring_offset: int = 0, batch=None, activation: str | None = "silu", gates: dict | None = None) -> torch.Tensor:
    """`conv_act` into out32 (float32 [N, channels]) and, in the same launch, `unit_heads` on its result: the first
    q_heads + k_heads heads of dk channels (q first) are divided by sqrt(their sum of squares + eps), q also multiplied by
    q_factor; `gates` as in `unit_heads`.  Heads of up to 256 numbers."""
    dev = _dev(u, taps_w, bias, state, out32)
    n = u.shape[0]
    _f32_matrix(u, "u", n, u_col + channels)
    taps = taps_w.shape[1]
    _f32(taps_w, "taps_w", channels * taps)
    if bias is not None:
        _f32(bias, "bias", channels)
    if activation not in (None, "silu"):
        raise ValueError(f"activation {activation!r}")
    if not 1 <= dk <= 256 or (q_heads + k_heads) * dk > channels:
        raise ValueError("heads of 1 to 256 numbers within the channels")
    slot_stride = _state_rows(state, batch.state_slots, (taps - 1) * channels, ring_offset, "conv_heads") if taps > 1 else 0
    _f32_matrix(out32, "out32", n, channels)
    for t, name in ((batch.token_seq, "token_seq"), (batch.positions, "positions")):
        _i32(t, name, n)
    _i32(batch.cu_seqlens, "cu_seqlens")
    _i32(batch.context_lens, "context_lens")
    g = gates or {}
    if gates is not None:
        _f32_matrix(g["gates"], "gates", n, max(g["a_col"], g["b_col"]) + g["heads"])
        _f32(g["a_log"], "a_log", g["heads"])
        _f32(g["dt_bias"], "dt_bias", g["heads"])
    if n == 0:
        return out32
    lib = load("recurrent")
    single = taps > 1 and batch.max_count == 1 and batch.num_seqs == n  # every request brings one token
    _check(lib.llms_conv_heads(
        _ptr(out32), c_int(out32.stride(0)), _ptr(u), c_int(u.stride(0)), c_int(u_col), _ptr(taps_w), _ptr(bias), c_int(taps),
        c_int(channels), _ptr(state), c_size_t(slot_stride), c_size_t(ring_offset), _ptr(batch.state_slots), _ptr(batch.token_seq),
        _ptr(batch.positions), _ptr(batch.cu_seqlens), _ptr(batch.context_lens), c_int(n), c_int(1 if activation == "silu" else 0),
        c_int(1 if single else 0), c_int(q_heads), c_int(k_heads), c_int(dk), c_float(eps), c_float(q_factor), _ptr(g.get("gates")),
        c_int(g["gates"].stride(0) if gates else 0), c_int(g.get("a_col", 0)), c_int(g.get("b_col", 0)), _ptr(g.get("a_log")),
        _ptr(g.get("dt_bias")), c_int(g.get("heads", 0)), _stream(dev)), "conv_heads")
    if taps > 1 and not single:
        _check(lib.llms_conv_ring(_ptr(state), c_size_t(slot_stride), c_size_t(ring_offset), _ptr(batch.state_slots), _ptr(u),
                                  c_int(u.stride(0)), c_int(u_col), _ptr(batch.cu_seqlens), _ptr(batch.context_lens),
                                  c_int(batch.num_seqs), c_int(taps), c_int(channels), _stream(dev)), "conv_ring")
    return out32


SCAN_MAX_STATES = 256


def step_sizes(dt: torch.Tensor, low: torch.Tensor, low_col: int, w_t: torch.Tensor, bias: torch.Tensor, *,
               z: torch.Tensor | None = None, z_col: int = 0) -> torch.Tensor:
    """dt[n, c] = softplus(sum_r low[n, low_col + r] w_t[r, c] + bias[c]), all 32-bit: low float32 [N, >=], w_t float32
    [rank, channels] (the weight transposed), dt float32 [N, channels].  With `z` (float32 [N, >= z_col + channels]) the same
    launch turns z's columns into silu(z), in place."""
    dev = _dev(dt, low, w_t, bias, z)
    n, channels = dt.shape
    if w_t.dim() != 2 or w_t.shape[1] != channels:
        raise ValueError("w_t is [rank, channels]")
    rank = w_t.shape[0]
    _f32(w_t, "w_t", rank * channels)
    _f32(bias, "bias", channels)
    _f32_matrix(dt, "dt", n, channels)
    _f32_matrix(low, "low", n, low_col + rank)
    if z is not None:
        _f32_matrix(z, "z", n, z_col + channels)
    if n:
        _check(load("recurrent").llms_step_sizes(
            _ptr(dt), c_int(dt.stride(0)), _ptr(low), c_int(low.stride(0)), c_int(low_col), c_int(rank), _ptr(w_t), _ptr(bias),
            _ptr(z), c_int(z.stride(0) if z is not None else 0), c_int(z_col), c_int(channels), c_int(n), _stream(dev)), "step_sizes")
    return dt


def selective_scan(out: torch.Tensor, x: torch.Tensor, z: torch.Tensor, z_col: int, low: torch.Tensor, b_col: int, c_col: int,
                   dt: torch.Tensor, a_neg: torch.Tensor, d_skip: torch.Tensor, state: torch.Tensor, scan_offset: int, batch,
                   z_prepared: bool = False) -> torch.Tensor:
    """Per request, token by token, per channel c and state n:  S[c, n] <- exp(dt_c a_neg[c, n]) S[c, n] + dt_c x_c B_n,
    y_c = sum_n S[c, n] C_n + d_skip[c] x_c; out[t, c] = y_c silu(z_c), rounded once.  x float32 [N, channels]; z float32
    [N, >= z_col + channels] (`z_prepared`: it already holds silu(z), see `step_sizes`); low float32 [N, >=] with B at
    b_col and C at c_col (`states` numbers each); dt float32 [N, channels], the step sizes; S float32 [channels, states]
    at `scan_offset` of the request's slot of `state`, read before the first token and left behind the last."""
    dev = _dev(out, x, z, low, dt, a_neg, d_skip, state)
    n, channels = x.shape
    if a_neg.dim() != 2 or a_neg.shape[0] != channels:
        raise ValueError("a_neg is [channels, states]")
    states = a_neg.shape[1]
    if not 1 <= states <= SCAN_MAX_STATES:
        raise ValueError(f"1 to {SCAN_MAX_STATES} states per channel, got {states}")
    _f32_matrix(x, "x", n, channels)
    _f32_matrix(z, "z", n, z_col + channels)
    _f32_matrix(low, "low", n, max(b_col, c_col) + states)
    _f32_matrix(dt, "dt", n, channels)
    _f32(a_neg, "a_neg", channels * states)
    _f32(d_skip, "d_skip", channels)
    if out.dim() != 2 or out.stride(1) != 1 or out.shape != (n, channels):
        raise ValueError(f"out must be [N, {channels}] with unit inner stride")
    slot_stride = _state_rows(state, batch.state_slots, channels * states, scan_offset, "selective_scan")
    _i32(batch.cu_seqlens, "cu_seqlens")
    _i32(batch.context_lens, "context_lens")
    if n == 0:
        return out
    _check(load("recurrent").llms_selective_scan(
        c_int(_code(out)), _ptr(out), c_int(out.stride(0)), _ptr(x), c_int(x.stride(0)), _ptr(z), c_int(z.stride(0)),
        c_int(z_col), _ptr(low), c_int(low.stride(0)), c_int(b_col), c_int(c_col), _ptr(dt), c_int(dt.stride(0)),
        _ptr(None), _ptr(a_neg), _ptr(d_skip), c_int(channels), c_int(states), _ptr(state), c_size_t(slot_stride),
        c_size_t(scan_offset), _ptr(batch.state_slots), _ptr(batch.cu_seqlens), _ptr(batch.context_lens),
        c_int(batch.num_seqs), c_int(1 if z_prepared else 0), _stream(dev)), "selective_scan")
    return out


def unit_heads(x: torch.Tensor, *, q_col: int, k_col: int, q_heads: int, k_heads: int, dk: int, eps: float,
               q_factor: float = 1.0, gates: dict | None = None) -> torch.Tensor:
    """In place on x (float32 [N, >=]): every head of dk numbers among the q_heads at q_col and the k_heads at k_col is
    divided by sqrt(its sum of squares + eps); the q heads are also multiplied by q_factor.  `gates` (the arguments
    gates, a_col, b_col, a_log, dt_bias, heads of `delta_scan`): the same launch turns the gates' products into the
    decay exp(-exp(a_log) softplus(. + dt_bias)) and the step sigmoid(.), in place, for `delta_scan(prepared=True)`."""
    dev = _dev(x)
    n = x.shape[0]
    _f32_matrix(x, "x", n, max(q_col + q_heads * dk, k_col + k_heads * dk))
    g = gates or {}
    if gates is not None:
        _f32_matrix(g["gates"], "gates", n, max(g["a_col"], g["b_col"]) + g["heads"])
        _f32(g["a_log"], "a_log", g["heads"])
        _f32(g["dt_bias"], "dt_bias", g["heads"])
    if n:
        _check(load("recurrent").llms_unit_heads(
            _ptr(x), c_int(x.stride(0)), c_int(q_col), c_int(k_col), c_int(q_heads), c_int(k_heads), c_int(dk), c_float(eps),
            c_float(q_factor), c_int(n), _ptr(g.get("gates")), c_int(g["gates"].stride(0) if gates else 0), c_int(g.get("a_col", 0)),
            c_int(g.get("b_col", 0)), _ptr(g.get("a_log")), _ptr(g.get("dt_bias")), c_int(g.get("heads", 0)), _stream(dev)),
            "unit_heads")
    return x


DELTA_MAX_KEY = 256


def delta_scan(o: torch.Tensor, qkv: torch.Tensor, *, q_col: int, k_col: int, v_col: int, gates: torch.Tensor, a_col: int,
               b_col: int, a_log: torch.Tensor, dt_bias: torch.Tensor, heads: int, kv_heads: int, dk: int, dv: int,
               state: torch.Tensor, scan_offset: int, batch, prepared: bool = False) -> torch.Tensor:
    """The gated delta rule per request, token by token, per head h over S [dk, dv] (q and k from head h / (heads /
    kv_heads)):  S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q, with beta = sigmoid(gates[:, b_col + h])
    and g = exp(-exp(a_log[h]) softplus(gates[:, a_col + h] + dt_bias[h])).  qkv float32 [N, >=] holds the prepared q
    (kv_heads * dk at q_col), k (at k_col) and v (heads * dv at v_col); o float32 [N, heads * dv]; S float32 [heads, dv,
    dk] (a head's state column by column) at `scan_offset` of the request's slot of `state`.  `prepared`: the gates' columns already hold decay and beta
    (`unit_heads` with gates)."""
    dev = _dev(o, qkv, gates, a_log, dt_bias, state)
    n = qkv.shape[0]
    if heads % kv_heads or not 1 <= dk <= DELTA_MAX_KEY:
        raise ValueError(f"heads must be a multiple of kv_heads and keys hold 1 to {DELTA_MAX_KEY} numbers")
    _f32_matrix(qkv, "qkv", n, max(q_col + kv_heads * dk, k_col + kv_heads * dk, v_col + heads * dv))
    _f32_matrix(gates, "gates", n, max(a_col, b_col) + heads)
    _f32_matrix(o, "o", n, heads * dv)
    _f32(a_log, "a_log", heads)
    _f32(dt_bias, "dt_bias", heads)
    slot_stride = _state_rows(state, batch.state_slots, heads * dk * dv, scan_offset, "delta_scan")
    _i32(batch.cu_seqlens, "cu_seqlens")
    _i32(batch.context_lens, "context_lens")
    if n == 0:
        return o
    _check(load("recurrent").llms_delta_scan(
        _ptr(o), c_int(o.stride(0)), _ptr(qkv), c_int(qkv.stride(0)), c_int(q_col), c_int(k_col), c_int(v_col), _ptr(gates),
        c_int(gates.stride(0)), c_int(a_col), c_int(b_col), _ptr(a_log), _ptr(dt_bias), c_int(heads), c_int(kv_heads),
        c_int(dk), c_int(dv), _ptr(state), c_size_t(slot_stride), c_size_t(scan_offset), _ptr(batch.state_slots),
        _ptr(batch.cu_seqlens), _ptr(batch.context_lens), c_int(batch.num_seqs), c_int(1 if prepared else 0), _stream(dev)),
        "delta_scan")
    return o


def delta_finish(out: torch.Tensor, o: torch.Tensor, gate: torch.Tensor, gate_col: int, weight: torch.Tensor, *, heads: int,
                 dv: int, eps: float) -> torch.Tensor:
    """out[n, h] = o[n, h] / sqrt(mean(o[n, h]^2) + eps) * weight * silu(gate[n, gate_col + h dv ..]), rounded once;
    o float32 [N, heads * dv], weight float32 [dv] shared by the heads, gate float32 [N, >=]."""
    dev = _dev(out, o, gate, weight)
    n = o.shape[0]
    _f32_matrix(o, "o", n, heads * dv)
    _f32_matrix(gate, "gate", n, gate_col + heads * dv)
    _f32(weight, "weight", dv)
    if out.dim() != 2 or out.stride(1) != 1 or out.shape != (n, heads * dv):
        raise ValueError(f"out must be [N, {heads * dv}] with unit inner stride")
    if n:
        _check(load("recurrent").llms_delta_finish(
            c_int(_code(out)), _ptr(out), c_int(out.stride(0)), _ptr(o), c_int(o.stride(0)), _ptr(gate), c_int(gate.stride(0)),
            c_int(gate_col), _ptr(weight), c_int(heads), c_int(dv), c_float(eps), c_int(n), _stream(dev)), "delta_finish")
    return out
