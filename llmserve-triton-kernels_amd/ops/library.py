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


def ensure_built(dtype_name: str, verbose: bool = True) -> None:
    """Compile (if missing) and load every library a model of this dtype uses."""
    names = _build.GROUPS[dtype_name]
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
