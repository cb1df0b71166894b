"""Python face of the HIP kernels: checks shapes on the host, then launches on
torch's current stream.  Tensors are torch tensors used as device memory; no
torch operator computes anything here.

The reference's façade (python/lyapunov_engine/ops.py:12-216) falls back to
eager PyTorch when its extension is missing.  There is no fallback here: a
library that cannot be loaded, or an input on the wrong device, is an error.
"""
from __future__ import annotations

import ctypes
import math
import os
from ctypes import c_float, c_int, c_longlong, c_void_p

import torch

from . import build

F32, BF16 = 0, 1
_CODE = {torch.float32: F32, torch.bfloat16: BF16}

STORE_ACT, STORE_F32, ACCUM_F32 = 0, 1, 2


class KernelError(RuntimeError):
    pass


def _load(path) -> ctypes.CDLL:
    try:
        return ctypes.CDLL(str(path))
    except OSError as e:
        raise KernelError(f"cannot load the kernel library {path}: {e}") from None


_core = None
_attn: dict[int, ctypes.CDLL] = {}


def core() -> ctypes.CDLL:
    global _core
    if _core is None:
        lib = _load(build.core_library())
        lib.lyp_last_error.restype = ctypes.c_char_p
        lib.lyp_embedding.argtypes = [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_void_p]
        lib.lyp_table_load.argtypes = [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_void_p]
        lib.lyp_rmsnorm.argtypes = [c_void_p, c_void_p, c_int, c_longlong, c_void_p, c_int, c_void_p, c_int, c_void_p,
                                    c_int, c_int, c_float, c_void_p]
        lib.lyp_rmsnorm_act.argtypes = [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_float, c_void_p]
        lib.lyp_rope_kv_write.argtypes = [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                          c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p]
        lib.lyp_swiglu.argtypes = [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p]
        lib.lyp_gemm_parts_hint.argtypes = [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int]
        lib.lyp_gemm_nt_parts.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                          c_int, c_void_p]
        lib.lyp_gemm_swiglu.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                        c_int, c_void_p]
        lib.lyp_gemm_rope_kv.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                         c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                         c_int, c_int, c_int, c_void_p]
        lib.lyp_gemm_residual_parts.argtypes = [c_int, c_int, c_int]
        lib.lyp_gemm_residual.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                          c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p]
        lib.lyp_gemm_swiglu_normed.argtypes = [c_void_p, c_int, c_void_p, c_int, c_int, c_float, c_void_p, c_void_p,
                                               c_int, c_int, c_int, c_int, c_int, c_int, c_void_p]
        lib.lyp_gemm_rope_kv_normed.argtypes = [c_void_p, c_int, c_void_p, c_int, c_int, c_float, c_void_p, c_void_p,
                                                c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p,
                                                c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                                c_void_p]
        lib.lyp_cast.argtypes = [c_void_p, c_int, c_void_p, c_int, c_longlong, c_void_p]
        lib.lyp_sum_parts.argtypes = [c_void_p, c_int, c_longlong, c_void_p, c_int, c_void_p]
        lib.lyp_gemm_nt.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                                    c_int, c_void_p]
        lib.lyp_sample.argtypes = [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                   c_void_p, c_void_p, c_void_p]
        lib.lyp_sample_cand.argtypes = [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                        c_int, c_void_p, c_void_p, c_void_p]
        lib.lyp_lm_head.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                                    c_void_p, c_int, c_void_p]
        lib.lyp_sample_workspace.argtypes = [c_int]
        lib.lyp_sample_workspace.restype = c_longlong
        lib.lyp_norm_threads_override.argtypes = [c_int]
        lib.lyp_skinny_row_tiles_override.argtypes = [c_int]
        lib.lyp_skinny_workgroups.argtypes = [c_int, c_int, c_int, c_int]
        lib.lyp_skinny_slices.argtypes = [c_int, c_int]
        lib.lyp_stream_read.argtypes = [c_void_p, c_longlong, c_int, c_void_p, c_void_p]
        lib.lyp_stream_rows.argtypes = [c_void_p, c_longlong, c_int, c_int, c_int, c_void_p, c_void_p]
        _core = lib
    return _core


def attention_lib(head_dim: int) -> ctypes.CDLL:
    lib = _attn.get(head_dim)
    if lib is None:
        lib = _load(build.attention_library(head_dim))
        lib.lyp_last_error.restype = ctypes.c_char_p
        if lib.lyp_attn_head_dim() != head_dim:
            raise KernelError(f"attention library for head size {head_dim} reports {lib.lyp_attn_head_dim()}")
        lib.lyp_attn_prefill.argtypes = [c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int,
                                         c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                                         c_float, c_int, c_void_p, c_void_p, c_int, c_void_p]
        lib.lyp_attn_prefill_plan.argtypes = [c_int, c_int, c_int, c_int, c_int, c_int]
        lib.lyp_attn_decode.argtypes = [c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int,
                                        c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int,
                                        c_int, c_int, c_int, c_float, c_void_p]
        lib.lyp_attn_decode_plan.argtypes = [c_int, c_int, c_int, c_int]
        _attn[head_dim] = lib
    return lib


def require_gpu() -> None:
    """The kernels are built for one architecture; say so before the first
    launch rather than after a failed one."""
    if not torch.cuda.is_available():
        raise KernelError("no GPU: this package has no CPU path")
    name = torch.cuda.get_device_properties(0).gcnArchName.split(":")[0]
    if name != build.GPU_ARCH:
        raise KernelError(f"the kernels are built for {build.GPU_ARCH}, this device is {name}")


# torch's current stream as a raw handle.  torch.cuda.current_stream() builds a
# Stream object on every call (several microseconds, a tenth of the host's time
# in an eager step); the two private accessors below, where this torch has
# them, give the same handle directly.
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_current_device = getattr(torch._C, "_cuda_getDevice", None)


# Addresses go to the libraries as plain integers: every function declares its pointer arguments,
# so ctypes converts them, and no c_void_p object is built per argument.
def _stream() -> int:
    if _raw_stream is not None and _current_device is not None:
        return _raw_stream(_current_device())
    return torch.cuda.current_stream().cuda_stream


def _p(t) -> int:
    return 0 if t is None else t.data_ptr()


def _check(rc: int, lib: ctypes.CDLL) -> None:
    if rc != 0:
        raise KernelError(lib.lyp_last_error().decode())


def _dev(*ts) -> None:
    for t in ts:
        if t is not None and (not t.is_cuda or not t.is_contiguous()):
            raise KernelError(f"kernel operand must be a contiguous GPU tensor, got {tuple(t.shape)} on {t.device} "
                              f"contiguous={t.is_contiguous()}")


def _code(dt: torch.dtype) -> int:
    try:
        return _CODE[dt]
    except KeyError:
        raise KernelError(f"kernels take float32 or bfloat16, not {dt}") from None


# ------------------------------------------------------------------ row kernels
def embedding(ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[t, :] = table[ids[t], :] as float (the residual stream)."""
    _dev(ids, table, out)
    T, H = out.shape
    if ids.dtype != torch.int32 or ids.numel() != T or table.shape[1] != H or out.dtype != torch.float32:
        raise KernelError(f"embedding: ids {tuple(ids.shape)} {ids.dtype}, table {tuple(table.shape)}, out {tuple(out.shape)} {out.dtype}")
    lib = core()
    _check(lib.lyp_embedding(_p(ids), _p(table), _code(table.dtype), _p(out), T, H, _stream()), lib)
    return out


# ------------------------------------------------- work handed on to a consumer
# A step with few rows is bound by the number of kernels, so two kinds of work
# may be passed on as a description for the next kernel to fold in, instead of
# being run on their own:
#   PendingLinear  a projection whose output is only ever added to the residual
#                  stream (``linear(..., pending=True)``): the adding kernel is
#                  the product itself (``linear_residual``);
#   PendingNorm    RMS-normed rows of the residual stream (``rmsnorm_pending``):
#                  the kernel that added to the stream also left the rows times
#                  the norm's weights and their sums of squares; ``linear_rope_kv``
#                  and ``linear_swiglu`` multiply those rows and divide by the
#                  rms at the end.
# Whoever cannot fold one in calls its ``run()`` and gets the plain tensor.
PENDING_MAX_ROWS = 16


class PendingLinear:
    def __init__(self, x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype):
        self.x, self.w, self.out_dtype = x, w, out_dtype

    def run(self) -> torch.Tensor:
        """The product, as ``linear(..., may_split=True)`` gives it."""
        return linear(self.x, self.w, out_dtype=self.out_dtype, may_split=True)


class PendingNorm:
    """Rows of the residual stream ``h`` (already holding the sum) that are to be
    RMS-normed.  ``xs`` is h * weight in the activations' type and ``ssq_part``
    [parts, 16] the rows' sums of squares in parts: what the kernel that
    added to h left behind for the product that comes next."""

    def __init__(self, h: torch.Tensor, weight: torch.Tensor, eps: float, dtype: torch.dtype, xs: torch.Tensor,
                 ssq_part: torch.Tensor):
        self.h, self.weight, self.eps, self.dtype = h, weight, float(eps), dtype
        self.xs, self.ssq_part = xs, ssq_part
        self.shape = h.shape

    def run(self) -> torch.Tensor:
        out = torch.empty(self.h.shape, dtype=self.dtype, device=self.h.device)
        return rmsnorm(self.h, self.weight, self.eps, out)


def as_delta(delta, dtype: torch.dtype):
    """What a mixer or feed-forward returned, as one plain tensor [T, H] of
    ``dtype`` (for a norm that adds it by itself)."""
    if delta is None:
        return None
    if isinstance(delta, PendingLinear):
        delta = delta.run()
    return sum_parts(delta, dtype)


def _few_rows_product(M: int, w: torch.Tensor, act_dtype: torch.dtype) -> bool:
    """Whether x [M, K] @ w.T runs in the weight-streaming kernel of this package."""
    return (M <= 64 and w.dtype == act_dtype and w.shape[1] % 64 == 0 and w.stride(1) == 1
            and not _library_product(M, w.shape[0], w.shape[1], act_dtype))


def linear_residual(h: torch.Tensor, p: PendingLinear, next_weight: torch.Tensor | None = None):
    """h += p.x @ p.w.T on the float residual stream, in the product's kernel.
    With ``next_weight`` (the weights of the RMS norm that follows) the kernel
    also leaves what a PendingNorm carries, and (xs, ssq_part) is returned;
    without it, True.  False (nothing done) when that kernel does not apply."""
    x, w = p.x, p.w
    M, K = x.shape
    N = w.shape[0]
    if h.dtype != torch.float32 or tuple(h.shape) != (M, N) or w.shape[1] != K or not _few_rows_product(M, w, x.dtype):
        return False
    _dev(h, x, w, next_weight)
    lib = core()
    xs = ssq = None
    if next_weight is not None:
        if M > PENDING_MAX_ROWS or next_weight.numel() != N:
            return False
        xs = torch.empty((M, N), dtype=x.dtype, device=h.device)
        ssq = torch.empty((lib.lyp_gemm_residual_parts(M, N, K), 16), dtype=torch.float32, device=h.device)
    rc = lib.lyp_gemm_residual(_p(x), _p(w), _p(h), _code(x.dtype), M, N, K, x.stride(0), w.stride(0), h.stride(0),
                               _p(next_weight), _code(next_weight.dtype) if next_weight is not None else 0, _p(xs), N,
                               _p(ssq), _stream())
    if rc < 0:
        _check(rc, lib)
    if rc != 0:
        return False
    return (xs, ssq) if next_weight is not None else True


def rmsnorm_pending(h: torch.Tensor, weight: torch.Tensor, eps: float, dtype: torch.dtype, delta=None):
    """Add ``delta`` to h and describe the normed rows instead of computing
    them.  Returns (PendingNorm, None), or (None, delta) when the rows had
    better be normed by ``rmsnorm``: ``delta`` is then what still has to be
    added.  Only a delta that is a product still to be run can be folded: its
    kernel is the one that prepares the norm."""
    if (not isinstance(delta, PendingLinear) or h.shape[0] > PENDING_MAX_ROWS or h.dtype != torch.float32
            or delta.x.dtype != dtype):
        return None, delta
    done = linear_residual(h, delta, weight)
    if done is False:
        return None, delta
    return PendingNorm(h, weight, eps, dtype, *done), None


def rmsnorm(h: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor, delta: torch.Tensor | None = None,
            rows: torch.Tensor | None = None) -> torch.Tensor:
    """out = rmsnorm(h [+ delta]) * weight.  h is the float residual stream and
    takes the sum, unless ``rows`` picks the rows to norm.  ``delta`` is [T, H]
    in out's dtype, float partial sums [S, T, H], or a product still to be run
    (see ``linear``)."""
    if isinstance(delta, PendingLinear):
        delta = delta.run()
    _dev(h, weight, out, delta, rows)
    H = h.shape[1]
    n = out.shape[0]
    if h.dtype != torch.float32 or weight.numel() != H or out.shape[1] != H:
        raise KernelError(f"rmsnorm: h {tuple(h.shape)} {h.dtype}, weight {tuple(weight.shape)}, out {tuple(out.shape)}")
    parts, stride = 0, 0
    if delta is not None:
        if delta.dim() == 3:
            if delta.dtype != torch.float32 or tuple(delta.shape[1:]) != tuple(h.shape):
                raise KernelError(f"rmsnorm: partial sums {tuple(delta.shape)} {delta.dtype} against h {tuple(h.shape)}")
            parts, stride = delta.shape[0], delta.shape[1] * delta.shape[2]
        elif delta.shape != h.shape or delta.dtype != out.dtype:
            raise KernelError(f"rmsnorm: delta {tuple(delta.shape)} {delta.dtype} against h {tuple(h.shape)}, out {out.dtype}")
    if rows is not None:
        if rows.dtype != torch.int32 or rows.numel() != n:
            raise KernelError("rmsnorm: rows must be int32, one per output row")
    elif n != h.shape[0]:
        raise KernelError("rmsnorm: output rows differ from input rows")
    lib = core()
    _check(lib.lyp_rmsnorm(_p(h), _p(delta), parts, stride, _p(weight), _code(weight.dtype), _p(out), _code(out.dtype),
                           _p(rows), n, H, float(eps), _stream()), lib)
    return out


def stream_read(src: torch.Tensor, sink: torch.Tensor, blocks: int) -> None:
    """Read all of ``src`` once with ``blocks`` workgroups (a yardstick for the
    kernels that stream weights); ``sink``: int32, blocks * 4 values."""
    _dev(src, sink)
    nbytes = src.numel() * src.element_size()
    if sink.dtype != torch.int32 or sink.numel() < blocks * 4:
        raise KernelError("stream_read: the sink must hold four int32 values per workgroup")
    lib = core()
    _check(lib.lyp_stream_read(_p(src), nbytes, blocks, _p(sink), _stream()), lib)


def stream_rows(src: torch.Tensor, sink: torch.Tensor, blocks: int, row_bytes: int, whole_lines: bool = False) -> None:
    """Read all of ``src`` once as a matrix of rows of ``row_bytes``, the way the
    weight-streaming products do (16 rows a wave, 64 bytes of each per load; with
    ``whole_lines`` 8 rows a wave and 128 bytes of each)."""
    _dev(src, sink)
    nbytes = src.numel() * src.element_size()
    if sink.dtype != torch.int32 or sink.numel() < blocks * 4:
        raise KernelError("stream_rows: the sink must hold four int32 values per workgroup")
    lib = core()
    _check(lib.lyp_stream_rows(_p(src), nbytes, row_bytes, int(whole_lines), blocks, _p(sink), _stream()), lib)


def norm_threads_override(threads: int) -> None:
    """Threads per row of the two-pass norm kernels (0: the built-in rule); for measurements."""
    lib = core()
    _check(lib.lyp_norm_threads_override(threads), lib)


def skinny_row_tiles_override(row_tiles: int) -> None:
    """Row tiles (of 16 rows of the weights) per workgroup of the weight-streaming product in steps
    of more than 16 rows (0: the built-in rule); for measurements."""
    lib = core()
    _check(lib.lyp_skinny_row_tiles_override(row_tiles), lib)


def rmsnorm_act(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor) -> torch.Tensor:
    _dev(x, weight, out)
    n, H = x.shape
    if out.shape != x.shape or out.dtype != x.dtype or weight.numel() != H:
        raise KernelError("rmsnorm_act: shapes or dtypes differ")
    lib = core()
    _check(lib.lyp_rmsnorm_act(_p(x), _p(weight), _code(weight.dtype), _p(out), _code(x.dtype), n, H, float(eps),
                               _stream()), lib)
    return out


def _rope_check(T: int, dtype: torch.dtype, positions, cos_sin, slots, kpool, vpool, num_kv_heads: int,
                head_dim: int, page_size: int, has_kv: bool) -> int:
    """Checks the operands that the rotation and the page write share; returns the rotary size."""
    if positions.numel() != T or positions.dtype != torch.int32:
        raise KernelError(f"rope_kv_write: positions {tuple(positions.shape)} {positions.dtype} for {T} tokens")
    rot = 0
    if cos_sin is not None:
        rot = cos_sin.shape[1]
        if cos_sin.dtype != torch.float32 or rot > head_dim or rot % 2:
            raise KernelError(f"rope_kv_write: table {tuple(cos_sin.shape)} {cos_sin.dtype} for heads of {head_dim}")
    if has_kv:
        n_pages = kpool.shape[0]
        if (slots is None or slots.numel() != T or slots.dtype != torch.int32
                or tuple(kpool.shape) != (n_pages, num_kv_heads, page_size, head_dim)
                or tuple(vpool.shape) != (n_pages, num_kv_heads, head_dim, page_size)
                or kpool.dtype != dtype or vpool.dtype != dtype):
            raise KernelError(f"rope_kv_write: pools {tuple(kpool.shape)} / {tuple(vpool.shape)} {kpool.dtype} do not "
                              f"fit {num_kv_heads} heads of {head_dim}, pages of {page_size}, dtype {dtype}")
    return rot


def rope_kv_write(qkv: torch.Tensor, positions: torch.Tensor, cos_sin: torch.Tensor | None,
                  slots: torch.Tensor | None, kpool: torch.Tensor | None, vpool: torch.Tensor | None, *, num_heads: int,
                  num_kv_heads: int, head_dim: int, page_size: int, has_kv: bool = True) -> None:
    """Rotate the query (and key) heads of ``qkv`` in place by each token's
    position and store keys and values in the token's cache slot."""
    _dev(qkv, positions, cos_sin, slots, kpool, vpool)
    T = qkv.shape[0]
    width = (num_heads + 2 * num_kv_heads) * head_dim if has_kv else num_heads * head_dim
    if qkv.shape[1] != width:
        raise KernelError(f"rope_kv_write: qkv {tuple(qkv.shape)} against width {width}")
    rot = _rope_check(T, qkv.dtype, positions, cos_sin, slots, kpool, vpool, num_kv_heads, head_dim, page_size, has_kv)
    lib = core()
    _check(lib.lyp_rope_kv_write(_p(qkv), _code(qkv.dtype), _p(positions), _p(cos_sin), _p(slots), _p(kpool),
                                 _p(vpool), T, num_heads, num_kv_heads, head_dim, rot, page_size, int(has_kv),
                                 _stream()), lib)


def swiglu(gate_up: torch.Tensor, out: torch.Tensor, interleave: int = 0) -> torch.Tensor:
    """out = silu(gate) * up.  interleave 0: gate_up[:, :I] are the gates and
    gate_up[:, I:] the ups; interleave 8: columns come in tiles of 16, eight
    gates then the eight ups that go with them."""
    _dev(gate_up, out)
    T, I = out.shape
    if tuple(gate_up.shape) != (T, 2 * I) or gate_up.dtype != out.dtype:
        raise KernelError(f"swiglu: {tuple(gate_up.shape)} -> {tuple(out.shape)}")
    lib = core()
    _check(lib.lyp_swiglu(_p(gate_up), _p(out), _code(out.dtype), T, I, interleave, _stream()), lib)
    return out


def linear_rope_kv(x: torch.Tensor, w: torch.Tensor, positions: torch.Tensor, cos_sin: torch.Tensor | None,
                   slots: torch.Tensor | None, kpool: torch.Tensor | None, vpool: torch.Tensor | None, *,
                   num_heads: int, num_kv_heads: int, head_dim: int, page_size: int,
                   has_kv: bool = True) -> torch.Tensor:
    """The fused q/k/v projection of x (w: query heads, then key heads, then
    value heads; query heads alone without ``has_kv``), query and key heads
    rotated by position, keys and values stored in the tokens' cache slots.
    Returns a tensor whose first ``num_heads * head_dim`` columns are the
    rotated query heads.  With few rows this is one kernel; its results equal
    ``linear`` followed by ``rope_kv_write`` bit for bit."""
    M, K = x.shape
    N = w.shape[0]
    width = (num_heads + 2 * num_kv_heads) * head_dim if has_kv else num_heads * head_dim
    if N != width or w.shape[1] != K:
        raise KernelError(f"linear_rope_kv: weight {tuple(w.shape)} for {width} features of {K}")
    if isinstance(x, PendingNorm):
        p = x
        if _few_rows_product(M, w, p.dtype):
            _dev(p.xs, p.ssq_part, w, positions, cos_sin, slots, kpool, vpool)
            rot = _rope_check(M, p.dtype, positions, cos_sin, slots, kpool, vpool, num_kv_heads, head_dim, page_size,
                              has_kv)
            out = torch.empty((M, num_heads * head_dim), dtype=p.dtype, device=w.device)
            lib = core()
            rc = lib.lyp_gemm_rope_kv_normed(_p(p.xs), p.xs.stride(0), _p(p.ssq_part), p.ssq_part.shape[0],
                                             p.h.shape[1], p.eps,
                                             _p(w), _p(out), _code(p.dtype), M, K, w.stride(0), out.stride(0),
                                             _p(positions), _p(cos_sin), _p(slots), _p(kpool), _p(vpool), num_heads,
                                             num_kv_heads, head_dim, rot, page_size, int(has_kv), _stream())
            if rc == 0:
                return out
            if rc < 0:
                _check(rc, lib)
        x = p.run()
    if w.dtype == x.dtype and M <= 64 and not _library_product(M, N, K, x.dtype):
        _dev(x, w, positions, cos_sin, slots, kpool, vpool)
        rot = _rope_check(M, x.dtype, positions, cos_sin, slots, kpool, vpool, num_kv_heads, head_dim, page_size,
                          has_kv)
        out = torch.empty((M, num_heads * head_dim), dtype=x.dtype, device=x.device)
        lib = core()
        rc = lib.lyp_gemm_rope_kv(_p(x), _p(w), _p(out), _code(x.dtype), M, K, x.stride(0), w.stride(0),
                                  out.stride(0), _p(positions), _p(cos_sin), _p(slots), _p(kpool), _p(vpool),
                                  num_heads, num_kv_heads, head_dim, rot, page_size, int(has_kv), _stream())
        if rc == 0:
            return out
        if rc < 0:
            _check(rc, lib)
    qkv = linear(x, w, out_dtype=x.dtype)
    rope_kv_write(qkv, positions, cos_sin, slots, kpool, vpool, num_heads=num_heads, num_kv_heads=num_kv_heads,
                  head_dim=head_dim, page_size=page_size, has_kv=has_kv)
    return qkv


def linear_swiglu(x: torch.Tensor, w: torch.Tensor, interleave: int) -> torch.Tensor:
    """silu(x @ Wgate.T) * (x @ Wup.T) for the fused matrix w [2 I, K] laid out
    as ``swiglu`` describes.  With few rows and interleave 8 it is one kernel."""
    I = w.shape[0] // 2
    if isinstance(x, PendingNorm):
        p, M = x, x.shape[0]
        if interleave == 8 and p.h.shape[1] == w.shape[1] and _few_rows_product(M, w, p.dtype):
            _dev(p.xs, p.ssq_part, w)
            out = torch.empty((M, I), dtype=p.dtype, device=w.device)
            lib = core()
            rc = lib.lyp_gemm_swiglu_normed(_p(p.xs), p.xs.stride(0), _p(p.ssq_part), p.ssq_part.shape[0],
                                            p.h.shape[1], p.eps, _p(w), _p(out), _code(p.dtype), M, w.shape[0],
                                            w.shape[1], w.stride(0), I, _stream())
            if rc == 0:
                return out
            if rc < 0:
                _check(rc, lib)
        x = p.run()
    if w.dtype != x.dtype:
        if w.dtype != torch.float32:
            raise KernelError(f"linear_swiglu: weight {w.dtype} against activations {x.dtype}")
        return cast(linear_swiglu(cast(x, torch.float32), w, interleave), x.dtype)
    out = torch.empty((x.shape[0], I), dtype=x.dtype, device=x.device)
    if interleave == 8 and x.shape[0] <= 64 and not _library_product(x.shape[0], w.shape[0], w.shape[1], x.dtype):
        _dev(x, w)
        lib = core()
        rc = lib.lyp_gemm_swiglu(_p(x), _p(w), _p(out), _code(x.dtype), x.shape[0], w.shape[0], w.shape[1],
                                 x.stride(0), w.stride(0), I, _stream())
        if rc == 0:
            return out
        if rc < 0:
            _check(rc, lib)
    gate_up = torch.empty((x.shape[0], 2 * I), dtype=x.dtype, device=x.device)
    gemm_nt(x, w, gate_up)
    return swiglu(gate_up, out, interleave)


def cast(x: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    if x.dtype == dtype:
        return x
    _dev(x)
    out = torch.empty_like(x, dtype=dtype)
    lib = core()
    _check(lib.lyp_cast(_p(x), _code(x.dtype), _p(out), _code(dtype), x.numel(), _stream()), lib)
    return out


# ------------------------------------------------------------------------ GEMM
# Large bfloat16 products go to the vendor's matrix library (hipBLASLt, called
# directly with the plan of every shape kept), as the reference's projections go
# to cuBLAS (nn.Linear, models/llama.py:45-48, 112-117, 177).  Products with few
# rows (decode steps), every float product (true 32-bit) and everything when
# LYAPUNOV_AMD_GEMM=own use the kernels of this package.
LIBRARY_GEMM_MODE = os.environ.get("LYAPUNOV_AMD_GEMM", "library")
if LIBRARY_GEMM_MODE not in ("library", "own"):
    raise KernelError(f"LYAPUNOV_AMD_GEMM is 'library' or 'own', not {LIBRARY_GEMM_MODE!r}")
LIBRARY_GEMM = LIBRARY_GEMM_MODE != "own"
LIBRARY_WORKSPACE_BYTES = 76 << 20    # what the library may use beside the operands (stream-K partial tiles)
LIBRARY_GEMM_MIN_ROWS = 65
# Between 17 and 64 rows the weight-streaming kernel is one burst of loads per workgroup: every
# workgroup reads the step's activations over its share of K, asks for all of its weights at once,
# sums its waves' parts and is done.  That beats the library's tiled kernels while the whole matrix
# is taken in one round of workgroups on the machine (as many workgroups as compute units, at most),
# and loses to them when the launch needs several rounds (``_library_product``).  Measured cold on
# 256 compute units at 64 rows, this kernel against the library (with the passes the library cannot
# fold in): q/k/v 3072x2048 14.7 against 18.3 us (192 workgroups), o 2048x2048 7.8 against 13.4 (256),
# down 2048x8192 16.8 against 22.8 (256), gate/up 16384x2048 28.4 against 21.9 (512: the library's).
# The burst also has to stay small: a workgroup reads its rows of the matrix and the step's
# activations over all of its share of K; past about 64 KiB of weights or 192 KiB of activations per
# workgroup the library's tiles are ahead again.  Whole decode steps at context 2,304, this package's
# kernel for every product that fits one round against the library for every product of 17 to 64 rows:
# 1B shape, batch 24 / 32 / 48 / 64: 15,510 / 19,430 / 24,630 / 29,280 against 14,820 / 18,870 / 24,250 /
# 29,680 tokens a second (64 rows of 2,048 values are 256 KiB of activations; the gains are the q/k/v and
# o products'); 8B shape, whose products of one round have 128 KiB and more of weights per workgroup:
# 4,030 / 4,930 / 6,040 / 7,410 against 4,130 / 5,090 / 6,180 / 7,760.
# (LYAPUNOV_AMD_LIBRARY_ROUNDS sets the number of rounds this package's kernel may take: 0 sends every
# product of 17 to 64 rows to the library, a large number none.)
LIBRARY_ROUNDS = float(os.environ.get("LYAPUNOV_AMD_LIBRARY_ROUNDS", "1"))
LIBRARY_ACTIVATION_BYTES = 192 << 10
LIBRARY_WEIGHT_BYTES = 64 << 10
# In an engine's warm-up step and in the run before a graph is captured, a library product's algorithm is
# chosen by measurement among this many of the library's candidates (at the shape's first call).
# Which candidate wins a timing may differ from process to process, and with it the last bits of
# bfloat16 results; LYAPUNOV_AMD_GEMM_TUNE=0 leaves every choice to the library's own heuristic, which
# gives the same bits in every run.
LIBRARY_TUNE_CANDIDATES = int(os.environ.get("LYAPUNOV_AMD_GEMM_TUNE", "16"))


_blas_lib = None
_blas_workspace: dict = {}
_blas_tuning = (0, 0)   # (candidates, without a workspace): the library's setting, kept here while it is not loaded


def blas() -> ctypes.CDLL:
    global _blas_lib
    if _blas_lib is None:
        require_gpu()
        try:
            lib = _load(build.blas_library())
        except (RuntimeError, KernelError) as e:
            raise KernelError(f"{e}\n(LYAPUNOV_AMD_GEMM=own runs every product in this package's kernels)") from None
        lib.lyp_last_error.restype = ctypes.c_char_p
        lib.lyp_library_gemm_nt.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                            c_int, c_void_p, c_longlong, c_void_p]
        lib.lyp_library_gemm_plans.restype = c_int
        lib.lyp_library_gemm_rejected.restype = c_int
        lib.lyp_library_gemm_solution.argtypes = [c_int] * 8
        lib.lyp_library_gemm_tuning.argtypes = [c_int, c_int]
        lib.lyp_library_gemm_tuning(*_blas_tuning)   # what a tuning context asked for before the library was there
        _blas_lib = lib
    return _blas_lib


class library_gemm_tuning:
    """While this context is open, a library product of a shape not seen before
    in this process is given the fastest of the library's first ``candidates``
    algorithms, found by running them on the call's operands (which waits for
    the stream); shapes seen before keep their plan.  Meant for a warm-up step."""

    def __init__(self, candidates: int | None = None, for_graph: bool = False):
        """``for_graph``: the products are about to be recorded into a graph;
        only algorithms that need no workspace are taken (one with a workspace
        may clear it with a memset node, which replayed graphs must not hold)."""
        self.candidates = LIBRARY_TUNE_CANDIDATES if candidates is None else candidates
        self.for_graph = for_graph
        self.before = None

    def __enter__(self):
        if LIBRARY_GEMM_MODE == "library" and (self.candidates > 1 or self.for_graph):
            self.before = _blas_tuning
            _set_blas_tuning(self.candidates, int(self.for_graph))
        return self

    def __exit__(self, *exc):
        if self.before is not None:
            _set_blas_tuning(*self.before)
        return False


def _set_blas_tuning(candidates: int, no_workspace: int) -> None:
    """The library is loaded by the first product that needs it (a 32-bit
    engine never does); until then the setting waits here."""
    global _blas_tuning
    _blas_tuning = (candidates, no_workspace)
    if _blas_lib is not None:
        _blas_lib.lyp_library_gemm_tuning(candidates, no_workspace)


def library_gemm_nt(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out [M, N] (bfloat16 or float) = a [M, K] @ w [N, K].T for bfloat16
    operands, by the vendor's library."""
    M, K = a.shape
    N = w.shape[0]
    if (a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or w.shape[1] != K or tuple(out.shape) != (M, N)
            or out.dtype not in (torch.bfloat16, torch.float32) or a.stride(1) != 1 or w.stride(1) != 1
            or out.stride(1) != 1 or not (a.is_cuda and w.is_cuda and out.is_cuda)):
        raise KernelError(f"library gemm: a {tuple(a.shape)} {a.dtype}, w {tuple(w.shape)} {w.dtype}, "
                          f"out {tuple(out.shape)} {out.dtype}")
    lib = blas()
    ws = _blas_workspace.get(a.device)
    if ws is None:
        ws = _blas_workspace[a.device] = torch.empty(LIBRARY_WORKSPACE_BYTES, dtype=torch.uint8, device=a.device)
    _check(lib.lyp_library_gemm_nt(_p(a), _p(w), _p(out), _code(out.dtype), M, N, K, a.stride(0), w.stride(0),
                                   out.stride(0), _p(ws), ws.numel(), _stream()), lib)
    return out


def library_gemm_rejected() -> int:
    """Candidates that tuning measured and turned down because their output was off the
    heuristic's first choice by more than rounding, so far in this process."""
    return blas().lyp_library_gemm_rejected()


def library_gemm_solution(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, for_graph: bool = False) -> int:
    """The library's number for the algorithm kept for this product, -1 if the shape has no plan yet."""
    return blas().lyp_library_gemm_solution(a.shape[0], w.shape[0], a.shape[1], a.stride(0), w.stride(0), out.stride(0),
                                            _code(out.dtype), int(for_graph))


_compute_units: dict = {}


def compute_units(device=None) -> int:
    """Compute units of the device (asked once)."""
    index = torch.cuda.current_device() if device is None or torch.device(device).index is None else torch.device(device).index
    n = _compute_units.get(index)
    if n is None:
        n = _compute_units[index] = torch.cuda.get_device_properties(index).multi_processor_count
    return n


def _library_product(M: int, N: int, K: int, dtype: torch.dtype, sliced: bool = False) -> bool:
    """Whether a bfloat16 product of M rows with a matrix [N, K] goes to the vendor's library.
    ``sliced``: the caller takes partial sums over slices of K (which gives this package's kernel
    more workgroups to spread a matrix of few rows over)."""
    if not LIBRARY_GEMM or dtype != torch.bfloat16:
        return False
    if M >= LIBRARY_GEMM_MIN_ROWS:
        return True
    if M <= PENDING_MAX_ROWS:
        return False
    lib = core()
    workgroups = lib.lyp_skinny_workgroups(M, N, K, int(sliced))
    if workgroups == 0 or workgroups > LIBRARY_ROUNDS * compute_units():
        return True
    slices = lib.lyp_skinny_slices(N, K) if sliced else 1
    k_per_workgroup = K // slices
    rows_per_workgroup = -(-N // (workgroups // slices))
    return (-(-M // 16) * 16 * k_per_workgroup * 2 > LIBRARY_ACTIVATION_BYTES
            or rows_per_workgroup * k_per_workgroup * 2 > LIBRARY_WEIGHT_BYTES)


def gemm_nt(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, accumulate: bool = False) -> torch.Tensor:
    """out = a @ w.T (or out += ...).  a [M, K], w [N, K] of one dtype; out
    [M, N] of that dtype or float.  Rows may lie further apart than they are
    long (column ranges of wider tensors); a row's values must be neighbours."""
    M, K = a.shape
    N = w.shape[0]
    if w.shape[1] != K or tuple(out.shape) != (M, N) or a.dtype != w.dtype:
        raise KernelError(f"gemm: a {tuple(a.shape)} {a.dtype}, w {tuple(w.shape)} {w.dtype}, out {tuple(out.shape)}")
    for name, t in (("a", a), ("w", w), ("out", out)):
        if not t.is_cuda or t.dim() != 2 or t.stride(1) != 1 or t.stride(0) < t.shape[1]:
            raise KernelError(f"gemm: {name} {tuple(t.shape)} with strides {t.stride()} on {t.device}: the values of "
                              f"a row must be neighbours in GPU memory")
    if out.dtype == torch.bfloat16 and not accumulate and _library_product(M, N, K, a.dtype):
        return library_gemm_nt(a, w, out)
    if accumulate:
        if out.dtype != torch.float32:
            raise KernelError("gemm: accumulation needs a float output")
        mode = ACCUM_F32
    elif out.dtype == torch.float32:
        mode = STORE_F32
    elif out.dtype == a.dtype:
        mode = STORE_ACT
    else:
        raise KernelError(f"gemm: output dtype {out.dtype} for operands of {a.dtype}")
    lib = core()
    _check(lib.lyp_gemm_nt(_p(a), _p(w), _p(out), _code(a.dtype), mode, M, N, K, a.stride(0), w.stride(0),
                           out.stride(0), _stream()), lib)
    return out


def linear(x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype | None = None,
           may_split: bool = False, pending: bool = False):
    """x @ w.T for a projection weight [out_features, in_features].  A weight
    kept in 32-bit is multiplied in 32-bit whatever the activations are.

    With ``may_split`` the result may come back as float partial sums
    [S, rows, out_features] instead (few rows, few output features: the inner
    dimension is then cut into S slices so that every compute unit has work);
    ``rmsnorm`` takes such a delta and adds the slices up, ``sum_parts`` does it
    for any other consumer.  With ``pending`` (the result will only be added to
    the residual stream) a product of few rows is not run at all but handed on
    as a ``PendingLinear``."""
    out_dtype = out_dtype or x.dtype
    if pending and x.shape[0] <= PENDING_MAX_ROWS and _few_rows_product(x.shape[0], w, x.dtype):
        return PendingLinear(x, w, out_dtype)
    if w.dtype != x.dtype:
        if w.dtype != torch.float32:
            raise KernelError(f"linear: weight {w.dtype} against activations {x.dtype}")
        x = cast(x, torch.float32)
    if may_split and x.shape[0] <= 64 and not _library_product(x.shape[0], w.shape[0], w.shape[1], x.dtype, sliced=True):
        _dev(x, w)
        lib = core()
        M, K, N = x.shape[0], x.shape[1], w.shape[0]
        slices = lib.lyp_gemm_parts_hint(_p(x), _p(w), _code(x.dtype), M, N, K, x.stride(0), w.stride(0))
        if slices > 1:
            parts = torch.empty((slices, M, N), dtype=torch.float32, device=x.device)
            _check(lib.lyp_gemm_nt_parts(_p(x), _p(w), _p(parts), _code(x.dtype), slices, M, N, K, x.stride(0),
                                         w.stride(0), _stream()), lib)
            return parts
    if out_dtype == torch.float32 and _library_product(x.shape[0], w.shape[0], w.shape[1], x.dtype):
        _dev(x, w)   # the library's float accumulators written out as they are
        return library_gemm_nt(x, w, torch.empty((x.shape[0], w.shape[0]), dtype=torch.float32, device=x.device))
    if out_dtype in (x.dtype, torch.float32):
        out = torch.empty((x.shape[0], w.shape[0]), dtype=out_dtype, device=x.device)
        return gemm_nt(x, w, out)
    out = torch.empty((x.shape[0], w.shape[0]), dtype=torch.float32, device=x.device)
    return cast(gemm_nt(x, w, out), out_dtype)


LM_HEAD_MAX_ROWS = 32     # what the output-head kernels may take (the library call says no where the general products are ahead)
LM_HEAD_BLOCKS = 1024     # most workgroups of the output-head kernels (the library says how many it used)


def lm_head(x: torch.Tensor, w: torch.Tensor) -> tuple:
    """-> (float logits x @ w.T for the output head [vocab, hidden], row maxima
    or None).  Few rows (a decode step's) take a kernel of their own that reads
    the matrix with few long-lived waves and leaves, beside the logits, every
    workgroup's largest logit per row: an int32 tensor [rows, workgroups, 2] of
    (value bits, index) pairs, which ``sample`` takes as ``row_maxima`` instead
    of a pass over the row.  Anything else goes through ``linear``."""
    M, K = x.shape
    if M <= LM_HEAD_MAX_ROWS and w.dtype == x.dtype and w.shape[1] == K and w.stride(1) == 1 and x.stride(1) == 1:
        _dev(x)
        lib = core()
        V = w.shape[0]
        out = torch.empty((M, V), dtype=torch.float32, device=x.device)
        cand = torch.empty((M, LM_HEAD_BLOCKS, 2), dtype=torch.int32, device=x.device)
        rc = lib.lyp_lm_head(_p(x), _p(w), _p(out), _code(x.dtype), M, V, K, x.stride(0), w.stride(0), out.stride(0),
                             _p(cand), LM_HEAD_BLOCKS, _stream())
        if rc < 0:
            _check(rc, lib)
        if rc > 0:
            return out, (cand if rc == LM_HEAD_BLOCKS else cand.view(-1)[:M * rc * 2].view(M, rc, 2))
    return linear(x, w, out_dtype=torch.float32), None


def sum_parts(parts: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """Add up the partial sums ``linear(..., may_split=True)`` may return (slice
    by slice, in 32-bit), as a tensor [rows, features] of ``dtype``."""
    if parts.dim() == 2:
        return parts if parts.dtype == dtype else cast(parts, dtype)
    if parts.dim() != 3 or parts.dtype != torch.float32:
        raise KernelError(f"sum_parts: float partial sums [slices, rows, features], not {tuple(parts.shape)} {parts.dtype}")
    _dev(parts)
    out = torch.empty(parts.shape[1:], dtype=dtype, device=parts.device)
    lib = core()
    _check(lib.lyp_sum_parts(_p(parts), parts.shape[0], out.numel(), _p(out), _code(dtype), _stream()), lib)
    return out


# ------------------------------------------------------------------- attention
def attn_decode_plan(n_seqs: int, max_ctx: int, num_heads: int, num_kv_heads: int, head_dim: int) -> int:
    """Keys per workgroup (the partition size) for a decode launch of this size."""
    return attention_lib(head_dim).lyp_attn_decode_plan(n_seqs, max_ctx, num_heads, num_kv_heads)


def attn_prefill_plan(n_tiles: int, max_keys: int, num_heads: int, num_kv_heads: int, head_dim: int,
                      dtype: torch.dtype, page_size: int) -> int:
    """Into how many runs a prefill launch had better cut every tile's keys
    (1: not at all) when one of its ``n_tiles`` tiles sees ``max_keys`` keys."""
    return attention_lib(head_dim).lyp_attn_prefill_plan(n_tiles, max_keys, num_heads, num_kv_heads, _code(dtype),
                                                         page_size)


def _attn_check(q, out, kpool, vpool, block_tables, nh, nkv, hd):
    _dev(out, kpool, vpool, block_tables)
    n_pages, bs = kpool.shape[0], kpool.shape[2]
    if (tuple(kpool.shape) != (n_pages, nkv, bs, hd) or tuple(vpool.shape) != (n_pages, nkv, hd, bs)
            or kpool.dtype != q.dtype or vpool.dtype != q.dtype or out.dtype != q.dtype):
        raise KernelError(f"attention: pools {tuple(kpool.shape)} / {tuple(vpool.shape)} {kpool.dtype} do not fit "
                          f"{nkv} heads of {hd} and queries of {q.dtype}")
    if q.stride(1) != 1 or q.stride(0) < nh * hd or tuple(out.shape) != (q.shape[0], nh * hd):
        raise KernelError(f"attention: q {tuple(q.shape)} strides {q.stride()}, out {tuple(out.shape)}")
    if block_tables.dtype != torch.int32 or block_tables.dim() != 2:
        raise KernelError("attention: block tables must be a 2-d int32 tensor")
    return bs


def attn_prefill(q: torch.Tensor, out: torch.Tensor, kpool: torch.Tensor, vpool: torch.Tensor,
                 block_tables: torch.Tensor, q_start: torch.Tensor, ctx_len: torch.Tensor, tile_seq: torch.Tensor,
                 tile_q0: torch.Tensor, n_tiles: int, *, num_heads: int, num_kv_heads: int, head_dim: int,
                 window: int = 0, scale: float | None = None, pair: bool | None = None,
                 split: bool = True, parts: int = 1, part_o: torch.Tensor | None = None,
                 part_ml: torch.Tensor | None = None) -> torch.Tensor:
    """Attention of the step's new tokens over the paged cache (which already
    holds their own keys).  q is a view [T, >= nh * hd] whose first nh * hd
    columns are the query heads; a tile is 64 new tokens of one request, and
    the tiles are best listed in rising order of the keys they see.  ``pair``
    says whether the first tiles see far fewer keys than the last (then a
    workgroup may take one of each); None leaves it to the kernel's launcher.
    ``split=False`` keeps a small launch from sharing a tile's keys between
    two sets of waves (a different order of additions, for tests).  ``parts``
    > 1 (see ``attn_prefill_plan``) cuts every tile's keys into that many runs
    for workgroups of their own; it needs float workspaces ``part_o`` of
    n_tiles * 64 * heads * parts * head_dim and ``part_ml`` of n_tiles * 64 *
    heads * parts * 2 elements."""
    if not q.is_cuda or q.dim() != 2:
        raise KernelError("attention: q must be a 2-d GPU tensor")
    bs = _attn_check(q, out, kpool, vpool, block_tables, num_heads, num_kv_heads, head_dim)
    _dev(q_start, ctx_len, tile_seq, tile_q0, part_o, part_ml)
    if parts > 1:
        need = n_tiles * 64 * num_heads * parts
        if part_o is None or part_ml is None or part_o.dtype != torch.float32 or part_ml.dtype != torch.float32 or \
                part_o.numel() < need * head_dim or part_ml.numel() < need * 2:
            raise KernelError("attention: the workspace for the parts of the keys is missing or too small")
    lib = attention_lib(head_dim)
    scale = 1.0 / math.sqrt(head_dim) if scale is None else scale
    _check(lib.lyp_attn_prefill(_p(q), q.stride(0), _p(out), out.stride(0), _p(kpool), _p(vpool), _code(q.dtype),
                                _p(block_tables), block_tables.shape[1], _p(q_start), _p(ctx_len), _p(tile_seq),
                                _p(tile_q0), n_tiles, num_heads, num_kv_heads, bs, window, scale,
                                (1 if pair is None else int(bool(pair))) | (0 if split else 2), _p(part_o),
                                _p(part_ml), parts, _stream()), lib)
    return out


def attn_decode(q: torch.Tensor, out: torch.Tensor, kpool: torch.Tensor, vpool: torch.Tensor,
                block_tables: torch.Tensor, q_start: torch.Tensor, ctx_len: torch.Tensor,
                dec_seqs: torch.Tensor | None, n_seqs: int, part_o: torch.Tensor, part_ml: torch.Tensor,
                max_parts: int, part_keys: int, *, num_heads: int, num_kv_heads: int, head_dim: int, window: int = 0,
                scale: float | None = None) -> torch.Tensor:
    """Attention of requests that bring one new token each, split over
    partitions of the context and merged.  ``part_keys`` comes from
    ``attn_decode_plan``; the caller guarantees that no request's context
    exceeds ``max_parts * part_keys`` (the contexts live on the device and are
    not read here: keys beyond that many partitions would silently be left
    out).  ``PagedAttention.decode_launch`` derives both from the step's bound."""
    if not q.is_cuda or q.dim() != 2:
        raise KernelError("attention: q must be a 2-d GPU tensor")
    bs = _attn_check(q, out, kpool, vpool, block_tables, num_heads, num_kv_heads, head_dim)
    _dev(q_start, ctx_len, dec_seqs, part_o, part_ml)
    if part_o.dtype != torch.float32 or part_ml.dtype != torch.float32 or \
            part_o.numel() < n_seqs * num_heads * max_parts * head_dim or \
            part_ml.numel() < n_seqs * num_heads * max_parts * 2:
        raise KernelError("attention: partition workspace too small")
    lib = attention_lib(head_dim)
    scale = 1.0 / math.sqrt(head_dim) if scale is None else scale
    _check(lib.lyp_attn_decode(_p(q), q.stride(0), _p(out), out.stride(0), _p(kpool), _p(vpool), _code(q.dtype),
                               _p(block_tables), block_tables.shape[1], _p(q_start), _p(ctx_len), _p(dec_seqs),
                               n_seqs, _p(part_o), _p(part_ml), max_parts, part_keys, num_heads, num_kv_heads, bs,
                               window, scale, _stream()), lib)
    return out


# -------------------------------------------------------------------- sampling
def sample_workspace(rows: int, device) -> torch.Tensor:
    return torch.empty(max(1, core().lyp_sample_workspace(rows)), dtype=torch.uint8, device=device)


def _pinned(t: torch.Tensor, dtype: torch.dtype, what: str) -> None:
    if t.is_cuda or not t.is_pinned() or t.dtype != dtype or not t.is_contiguous():
        raise KernelError(f"{what} must be a contiguous pinned host tensor of {dtype}")


def table_load(src: torch.Tensor, dst: torch.Tensor, patch: torch.Tensor | None = None, patch_at: int = 0) -> None:
    """dst (int32, device) = the first dst.numel() words of src (int32, pinned
    host memory, read by the kernel itself: no copy engine, no second launch);
    ``patch`` (int32, device) replaces the words from ``patch_at`` on."""
    _pinned(src, torch.int32, "table_load: the source")
    _dev(dst, patch)
    if dst.dtype != torch.int32 or dst.numel() > src.numel() or not dst.is_contiguous():
        raise KernelError("table_load: the destination must be a contiguous int32 tensor no longer than the source")
    n_patch = 0
    if patch is not None:
        n_patch = patch.numel()
        if patch.dtype != torch.int32 or not patch.is_contiguous() or patch_at < 0 or patch_at + n_patch > dst.numel():
            raise KernelError("table_load: the patch does not fit")
    lib = core()
    _check(lib.lyp_table_load(src.data_ptr(), _p(dst), dst.numel(), _p(patch), patch_at, n_patch, _stream()), lib)


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
           uniform: torch.Tensor, out: torch.Tensor, workspace: torch.Tensor | None = None,
           mirror: torch.Tensor | None = None, row_maxima: torch.Tensor | None = None) -> torch.Tensor:
    """One token per row of logits.  With a ``workspace`` (``sample_workspace``)
    the search for each row's maximum is spread over the chip; with
    ``row_maxima`` (what ``lm_head`` returns beside these very logits) there is
    no search.  ``mirror``: pinned host memory (int32, a row each) that receives
    the tokens as well, readable once the work on the stream up to here is done."""
    _dev(temperature, top_k, top_p, uniform, out, workspace)
    if not logits.is_cuda or logits.dim() != 2 or logits.stride(1) != 1:
        raise KernelError("sample: logits must be a 2-d GPU tensor whose rows are contiguous")
    if mirror is not None:
        _pinned(mirror, torch.int32, "sample: the mirror")
        if mirror.numel() != out.numel():
            raise KernelError("sample: one mirrored token per row")
    R, V = logits.shape
    if logits.dtype != torch.float32 or temperature.dtype != torch.float32 or top_k.dtype != torch.int32 or \
            top_p.dtype != torch.float32 or uniform.dtype != torch.float32 or out.dtype != torch.int32:
        raise KernelError("sample: logits, temperature, top_p, uniform float32; top_k, out int32")
    if any(t.numel() != R for t in (temperature, top_k, top_p, uniform, out)):
        raise KernelError("sample: one parameter per row")
    lib = core()
    cand = row_maxima
    if cand is not None:   # the head's kernel left the row maxima in pieces: no pass over the row for them
        if cand.dtype != torch.int32 or cand.dim() != 3 or cand.shape[0] < R or cand.shape[2] != 2 or \
                not cand.is_contiguous() or cand.device != logits.device:
            raise KernelError("sample: the row maxima must be a contiguous int32 tensor [rows, pieces, 2]")
        _check(lib.lyp_sample_cand(_p(logits), logits.stride(0), R, V, _p(temperature), _p(top_k), _p(top_p),
                                   _p(uniform), _p(cand), cand.shape[1], _p(out),
                                   mirror.data_ptr() if mirror is not None else None, _stream()), lib)
        return out
    if workspace is not None and workspace.numel() < lib.lyp_sample_workspace(R):
        raise KernelError("sample: workspace too small")
    _check(lib.lyp_sample(_p(logits), logits.stride(0), R, V, _p(temperature), _p(top_k), _p(top_p), _p(uniform),
                          _p(workspace), _p(out), mirror.data_ptr() if mirror is not None else None, _stream()), lib)
    return out
