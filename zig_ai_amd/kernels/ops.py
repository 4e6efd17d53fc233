"""Python bindings of the HIP kernels: argument checks on the host, then one
launch on torch's current stream.  Nothing here computes on the CPU and nothing
falls back to a library: if a kernel library cannot be built or loaded the call
raises.

Shapes and dtypes are verified before every launch so that a kernel never sees
operands other than the ones its indexing assumes.
"""

from __future__ import annotations

import ctypes
import os
from typing import Optional, Tuple

import torch

from . import build

c_int, c_float, c_void_p, c_longlong = ctypes.c_int, ctypes.c_float, ctypes.c_void_p, ctypes.c_longlong
c_size_t = ctypes.c_size_t

_DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 1}

_SIGNATURES = {
    ("norm", "za_add_rmsnorm"): [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p,
                                 c_int, c_int, c_float, c_int, c_int, c_longlong, c_void_p],
    ("norm", "za_embed_gather"): [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_void_p],
    ("gemm", "za_gemm_f32"): [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                              c_int, c_void_p],
    ("gemm", "za_gemm_bf16"): [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                               c_int, c_void_p],
    ("rope_kv", "za_qk_norm_rope_kv_write"): [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                              c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                              c_int, c_int, c_int, c_int, c_float, c_int, c_int,
                                              c_void_p],
    ("attention", "za_paged_attention"): [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                                          c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p,
                                          c_void_p, c_int, c_int, c_int, c_int, c_int, c_float,
                                          c_int, c_int, c_int, c_void_p],
    ("attention", "za_paged_attention_mfma"): [c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                                               c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                                               c_int, c_void_p, c_void_p, c_int, c_int, c_int,
                                               c_int, c_float, c_int, c_int, c_int, c_int, c_void_p],
    ("attention", "za_paged_attention_decode_mfma"): [c_void_p, c_void_p, c_void_p, c_void_p,
                                                      c_int, c_void_p, c_void_p, c_void_p,
                                                      c_void_p, c_int, c_int, c_void_p, c_void_p,
                                                      c_int, c_int, c_int, c_int, c_float, c_int,
                                                      c_int, c_int, c_void_p],
    ("attention", "za_paged_attention_decode_mfma_rope"): [
        c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
        c_void_p, c_float, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_float, c_int,
        c_int, c_int, c_int, c_void_p],
    ("attention", "za_attention_combine"): [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                            c_void_p],
    ("gemm", "za_gemm_bf16_rows16_merged"): [c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p,
                                             c_int, c_int, c_int, c_int, c_int, c_void_p],
    ("shortconv", "za_short_conv"): [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                     c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                                     c_longlong, c_void_p],
    ("activation", "za_swiglu"): [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p],
    ("activation", "za_cast"): [c_void_p, c_int, c_void_p, c_int, c_longlong, c_void_p],
    ("activation", "za_copy_columns"): [c_void_p, c_int, c_int, c_int, c_void_p, c_int, c_int, c_int,
                                        c_int, c_int, c_void_p],
    ("sampling", "za_argmax"): [c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_int,
                                c_void_p],
    ("gemm", "za_gemm_bf16_rows16"): [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                      c_int, c_int, c_int, c_void_p],
    ("gemm", "za_gemm_bf16_rows16_stream"): [c_void_p, c_void_p, c_void_p, c_void_p, c_float,
                                             c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                             c_int, c_int, c_int, c_void_p],
    ("gemm", "za_gemm_bf16_rows16_swiglu"): [c_void_p, c_void_p, c_void_p, c_void_p, c_float,
                                             c_void_p, c_void_p, c_int, c_int, c_int, c_void_p],
    ("gemm", "za_gemm_bf16_rows16_gated_conv"): [c_void_p, c_void_p, c_void_p, c_float, c_void_p,
                                                 c_void_p, c_void_p, c_void_p, c_longlong,
                                                 c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                                 c_int, c_void_p],
    ("gemm_rows64", "za_gemm_bf16_rows64"): [c_void_p, c_void_p, c_void_p, c_void_p, c_float,
                                             c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                                             c_void_p],
    ("sampling", "za_sample"): [c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                                c_void_p, c_int, c_void_p],
    ("sampling", "za_repetition_penalty"): [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int,
                                            c_void_p],
    ("calibrate", "za_read_stream"): [c_void_p, c_size_t, c_int, c_void_p, c_void_p],
    ("calibrate", "za_mfma_loop"): [c_int, c_int, c_void_p, c_void_p],
    ("blaslt", "za_lt_matmul"): [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                                 c_int, c_void_p, c_size_t, c_void_p],
}
_functions = {}


class KernelError(RuntimeError):
    pass


# Diagnostics: when this is a list, every projection and attention call appends a record
# of the form it took (which of several equivalent kernels ran, and so where values were
# rounded to the storage type on the way): ``{"op", "M", "N", "K", ...}``.  Steps replayed
# from a HIP graph call nothing here and leave no records.
form_log: Optional[list] = None


def _note(op: str, **fields) -> None:
    if form_log is not None:
        fields["op"] = op
        form_log.append(fields)


def _fn(lib: str, name: str):
    key = (lib, name)
    f = _functions.get(key)
    if f is None:
        f = getattr(build.load(lib), name)
        f.argtypes = _SIGNATURES[key]
        f.restype = c_int
        _functions[key] = f
    return f


def _check(rc: int, name: str, detail: str = "") -> None:
    if rc == 0:
        return
    if rc == -1:
        why = "bad argument"
    elif rc == -2:
        why = "size or dtype the kernel does not support"
    else:
        why = f"HIP error {rc}"
    raise KernelError(f"{name}: {why}" + (f" ({detail})" if detail else ""))


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()      # an int converts to void*, None to NULL


# The current stream's handle, asked for before every launch: torch's binding that
# returns the raw handle costs a fraction of a microsecond, building a Stream object
# some eight; the latter is the fallback where the binding is missing.
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream():
    if _raw_stream is not None and _raw_device is not None:
        return _raw_stream(_raw_device())
    return torch.cuda.current_stream().cuda_stream


def _code(dtype: torch.dtype) -> int:
    if dtype not in _DTYPE_CODE:
        raise KernelError(f"kernels take float32 or bfloat16, not {dtype}")
    return _DTYPE_CODE[dtype]


def _need(t: torch.Tensor, name: str, dtype=None, shape: Optional[Tuple[int, ...]] = None) -> None:
    if not isinstance(t, torch.Tensor):
        raise KernelError(f"{name} is not a tensor")
    if not t.is_cuda:
        raise KernelError(f"{name} is on {t.device}; the kernels run on the GPU only")
    if not t.is_contiguous():
        raise KernelError(f"{name} is not contiguous")
    if dtype is not None:
        ok = t.dtype in dtype if isinstance(dtype, (tuple, list)) else t.dtype == dtype
        if not ok:
            raise KernelError(f"{name} has dtype {t.dtype}, expected {dtype}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise KernelError(f"{name} has shape {tuple(t.shape)}, expected {tuple(shape)}")


# --------------------------------------------------------------------- norms
def add_rmsnorm(residual: Optional[torch.Tensor], delta: Optional[torch.Tensor],
                weight: torch.Tensor, eps: float, out_dtype: torch.dtype,
                rows: Optional[torch.Tensor] = None, write_residual: bool = True) -> torch.Tensor:
    """``out = rmsnorm(residual + delta) * weight``; see csrc/norm.hip.  ``delta`` may
    be a stack ``[P, rows, width]`` of 32-bit partial sums, which are added up."""
    if residual is None and delta is None:
        raise KernelError("add_rmsnorm needs residual or delta")
    n_partials, partial_stride = 1, 0
    if delta is not None and delta.dim() == 3:
        _need(delta, "delta", torch.float32)
        n_partials = delta.shape[0]
        partial_stride = delta.shape[1] * delta.shape[2]
        shape2 = tuple(delta.shape[1:])
    else:
        shape2 = tuple((residual if residual is not None else delta).shape)
    if len(shape2) != 2:
        raise KernelError(f"add_rmsnorm takes [rows, width], got {shape2}")
    n, width = shape2
    if residual is not None:
        _need(residual, "residual", torch.float32, (n, width))
    if delta is not None and delta.dim() == 2:
        _need(delta, "delta", (torch.float32, torch.bfloat16), (n, width))
    _need(weight, "weight", torch.float32, (width,))
    n_out = n
    if rows is not None:
        _need(rows, "rows", torch.int32)
        n_out = rows.numel()
    ref = residual if residual is not None else delta
    out = torch.empty((n_out, width), dtype=out_dtype, device=ref.device)
    rc = _fn("norm", "za_add_rmsnorm")(
        _ptr(residual), _ptr(delta), _code(delta.dtype) if delta is not None else 0, _ptr(weight),
        _ptr(out), _code(out_dtype), _ptr(rows), n_out, width, float(eps),
        1 if (write_residual and residual is not None and delta is not None and rows is None) else 0,
        n_partials, partial_stride, _stream())
    _check(rc, "add_rmsnorm")
    return out


def embed_gather(tokens: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    """Rows of ``table`` as 32-bit floats: the start of the residual stream."""
    _need(tokens, "tokens", torch.int32)
    _need(table, "table", (torch.float32, torch.bfloat16))
    if tokens.dim() != 1 or table.dim() != 2:
        raise KernelError("embed_gather takes tokens [T] and table [vocab, width]")
    vocab, width = table.shape
    out = torch.empty((tokens.numel(), width), dtype=torch.float32, device=table.device)
    rc = _fn("norm", "za_embed_gather")(_ptr(tokens), _ptr(table), _code(table.dtype), _ptr(out),
                                        tokens.numel(), width, vocab, _stream())
    _check(rc, "embed_gather")
    return out


class NormedRows:
    """An RMSNorm that has not run yet: rows of the 32-bit residual stream (``rows``
    selects and orders them; all of them without it) with the norm's weight and eps.
    ``linear`` and ``linear_swiglu`` take it in place of activations and, for a decode
    batch, let the projection's kernel normalise the rows on its way; everywhere else
    ``materialise`` runs the norm kernel."""

    __slots__ = ("residual", "weight", "eps", "dtype", "rows")

    def __init__(self, residual: torch.Tensor, weight: torch.Tensor, eps: float,
                 dtype: torch.dtype, rows: Optional[torch.Tensor] = None):
        _need(residual, "residual", torch.float32)
        if residual.dim() != 2:
            raise KernelError(f"NormedRows takes [rows, width], got {tuple(residual.shape)}")
        _need(weight, "weight", torch.float32, (residual.shape[1],))
        if rows is not None:
            _need(rows, "rows", torch.int32)
        self.residual, self.weight, self.eps, self.dtype, self.rows = \
            residual, weight, float(eps), dtype, rows

    @property
    def shape(self) -> Tuple[int, int]:
        n = self.residual.shape[0] if self.rows is None else self.rows.numel()
        return (n, self.residual.shape[1])

    @property
    def device(self) -> torch.device:
        return self.residual.device

    def materialise(self) -> torch.Tensor:
        return add_rmsnorm(self.residual, None, self.weight, self.eps, self.dtype, rows=self.rows,
                           write_residual=False)


# The fused forms exist for a decode batch of bfloat16 products whose K one workgroup
# covers in slices of 512, a wave's share.
NORMED_ROWS_MAX_K = 4096
NORMED_ROWS_K_MULTIPLE = 512
NORMED_ROWS_MAX_ROWS = 16


def normed_rows_fusable(rows: int, width: int) -> bool:
    return rows <= NORMED_ROWS_MAX_ROWS and width <= NORMED_ROWS_MAX_K \
        and width % NORMED_ROWS_K_MULTIPLE == 0


def _takes_normed_rows(x, weight: torch.Tensor, M: int, K: int) -> bool:
    """Whether the product's kernel runs the norm itself: every workgroup then reads the
    step's rows in 32-bit (whole lines, staged through LDS) and a kernel is saved.  Measured
    at K = 2048 against the norm kernel followed by the product: 2 to 2.5 us saved per
    product at every row count up to 16."""
    return (isinstance(x, NormedRows) and x.dtype == torch.bfloat16
            and weight.dtype == torch.bfloat16 and normed_rows_pay(M, weight.shape[0], K))


def normed_rows_pay(M: int, N: int, K: int) -> bool:
    return normed_rows_fusable(M, K)


class MergedRows:
    """An attention's output ``[T, heads * head_dim]`` while it still lies in the partial
    results of its context ranges (``acc [T, heads, ranges, head_dim]``, ``ml [T, heads,
    ranges, 2]``: accumulator, maximum on the base-2 scale and sum).  ``linear`` merges them
    on the product's way in where that pays (a kernel less); ``materialise`` runs the merge
    as a kernel of its own.  The same bits either way."""

    def __init__(self, acc: torch.Tensor, ml: torch.Tensor):
        _need(acc, "acc", torch.float32)
        T, nh, nsplit, d = acc.shape
        _need(ml, "ml", torch.float32, (T, nh, nsplit, 2))
        self.acc, self.ml = acc, ml
        self.rows, self.heads, self.ranges, self.head_dim = T, nh, nsplit, d
        self.shape = (T, nh * d)
        self.dtype = torch.bfloat16

    @property
    def device(self) -> torch.device:
        return self.acc.device

    def materialise(self) -> torch.Tensor:
        out = torch.empty(self.shape, dtype=torch.bfloat16, device=self.acc.device)
        rc = _fn("attention", "za_attention_combine")(
            _ptr(self.acc), _ptr(self.ml), _ptr(out), self.rows * self.heads, self.head_dim,
            self.ranges, _stream())
        _check(rc, "attention_combine")
        _note("attention_combine", rows=self.rows, ranges=self.ranges)
        return out


MERGED_ROWS_MAX_ROWS = 8
MERGED_ROWS_MAX_RANGES = 16


def merged_rows_pay(rows: int, ranges: int) -> bool:
    """Whether the output projection should merge the ranges itself.  Measured against the
    combine kernel followed by the projection, hidden 2048 (1024): one row in 8 ranges 4.6
    (3.4) against 8.0 (6.7) us, four rows in 8 ranges 6.7 (5.3) against 8.1 (6.7), eight rows
    in 2 ranges 5.5 (4.6) against 6.8 (5.3), eight rows in 4 ranges 7.1 (5.9) against 7.3
    (5.8): every workgroup of the projection merges its slice of every row.  In a decode step
    of the 1.2B shape: batch 1 (12 ranges) 0.731 -> 0.704 ms, batch 2 0.735 -> 0.716, batch 4
    (8 ranges) 0.750 -> 0.762: up to 24 rows x ranges."""
    return (1 < ranges <= MERGED_ROWS_MAX_RANGES and 0 < rows <= MERGED_ROWS_MAX_ROWS
            and rows * ranges <= 24)


# --------------------------------------------------------------------- gemm
# Above this many rows a bfloat16 projection without bias goes to the library
# (measured: the decode kernel wins up to 16 rows, the library from there on).
LIBRARY_GEMM_ROWS = 16
# Up to this many rows the library is given K in ranges when the consumer takes
# partial sums (too few tiles of M x N to fill the chip when N is small).
LIBRARY_SPLIT_ROWS = 1024


def check_projection_weight(weight: torch.Tensor, what: str) -> None:
    """Refuse, when a part is built, a weight the GEMM kernels cannot take."""
    if weight.dtype == torch.bfloat16 and weight.shape[1] % 8:
        raise KernelError(
            f"{what}: a bfloat16 projection needs an input width that is a multiple of 8 "
            f"(rows start on 16-byte boundaries), got {weight.shape[1]}; store the weight in "
            "32-bit or run with float32")


def _k_splits(M: int, N: int, K: int) -> int:
    """Into how many ranges K is cut when the consumer accepts partial sums:
    enough to give every compute unit work when N alone is too small.  Measured
    together with the norm that adds the stack up, N = 2048:

    * up to 16 rows (the decode kernel): 4 ranges from K = 4096 on (8192: 15 us
      instead of 19.5), 2 ranges from 2048 on (8.3 instead of 8.9);
    * more rows (the library, as one batched product over the ranges, its algorithm
      timed at first use): from K = 4096 on 8 ranges up to 256 rows and 4 up to
      ``LIBRARY_SPLIT_ROWS`` (K = 8192 with the norm that adds the stack, 64 rows: 16.5 us
      instead of 19.9; 512 rows: 32.9 instead of 42.0; 1,024 rows: 47.7 instead of 59.9; the
      same order at N = 1024, K = 4608 and N = 2560, K = 10752; a whole step of the 1.2B
      shape: 640 rows 2.72 -> 2.56 ms, 768 rows 3.28 -> 3.14, 1,024 rows 3.40 -> 3.29; with 2
      ranges 1,280 rows 3.98 -> 3.95, 1,536 rows 4.32 -> 4.37, 2,048 rows 5.17 -> 5.14: left
      as one product), and
      from K = 2048 on 4 ranges up to 128 rows (64 rows: 11.4 instead of 11.7, 8 ranges
      12.6; 128 rows: 13.5 instead of 15.8; from 192 rows on one product is fastest)."""
    if N > 4096:
        return 1
    if M <= 16:
        if K >= 4096:
            choices = (4, 2)
        elif K >= 2048 and N <= 2048:
            choices = (2,)
        else:
            return 1
        for split in choices:
            if K % (split * 32) == 0:
                return split
        return 1
    choices = ()
    if K >= 4096 and M <= LIBRARY_SPLIT_ROWS:
        choices = (8, 4, 2) if M <= 256 else (4, 2)
    elif K >= 2048 and M <= 128:
        choices = (4, 2)
    for split in choices:
        if K % (split * 128) == 0:
            return split
    return 1


LIBRARY_WORKSPACE_BYTES = 64 << 20
_library_workspace = {}
# Whether the GEMM library's candidates for a shape of many rows are timed at the shape's
# first call (csrc/blaslt.hip), for calls that do not say (``linear(..., tune=None)``).
# Which candidate wins can differ from run to run; a model that promises the same bits run
# after run passes ``tune=False`` with every product (``Runtime.tune``), and
# ZIG_AI_GEMM_TUNE=0 switches the default off for a whole process.
library_tuning = os.environ.get("ZIG_AI_GEMM_TUNE", "1") != "0"


def _library_matmul(x: torch.Tensor, weight: torch.Tensor, out_dtype: torch.dtype,
                    splits: int, tune: Optional[bool] = None,
                    added_to: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """``x @ weight^T`` through the GEMM library (csrc/blaslt.hip): ``[M, N]``, or the
    stack ``[splits, M, N]`` of 32-bit partial sums over ranges of K, or, with ``added_to``
    (32-bit ``[M, N]``), that tensor with the product added to it.  ``None`` when
    the library names no algorithm for the shape (nothing was launched)."""
    M, K = x.shape
    N = weight.shape[0]
    device = x.device.index or 0
    work = _library_workspace.get(device)
    if work is None:
        work = torch.empty((LIBRARY_WORKSPACE_BYTES,), dtype=torch.uint8, device=x.device)
        _library_workspace[device] = work
    f32 = splits > 1 or out_dtype == torch.float32
    if added_to is not None:
        out, kind = added_to, 2
    else:
        shape = (splits, M, N) if splits > 1 else (M, N)
        out = torch.empty(shape, dtype=torch.float32 if f32 else torch.bfloat16, device=x.device)
        kind = 1 if f32 else 0
    rc = _fn("blaslt", "za_lt_matmul")(_ptr(x), _ptr(weight), _ptr(out), M, N, K, kind,
                                       splits, 1 if (library_tuning if tune is None else tune) else 0,
                                       _ptr(work),
                                       LIBRARY_WORKSPACE_BYTES, _stream())
    if rc == -2:
        return None
    if rc != 0:
        why = build.load("blaslt").za_lt_last_error
        why.restype = ctypes.c_char_p
        raise KernelError(f"library matmul M={M} N={N} K={K} splits={splits}: "
                          f"{why().decode('utf-8', 'replace')}")
    return out


ROWS16_MAX_K_PER_WORKGROUP = 8192      # what one workgroup of the decode kernel covers


def _accumulate_splits(N: int, K: int) -> int:
    """Into how many ranges K is cut when a decode batch's product is added to the
    stream with atomics: until some 512 workgroups stream the weight, and at least so
    many that one workgroup's range fits the kernel.  0: no cut fits (the caller then
    takes the ordinary path and lets the next norm add the product)."""
    groups = (N + 15) // 16
    for split in (8, 4, 2):
        if groups * split <= 640 and K % (split * 32) == 0 and K // split >= 512 \
                and K // split <= ROWS16_MAX_K_PER_WORKGROUP:
            return split
    if K <= ROWS16_MAX_K_PER_WORKGROUP:
        return 1
    # a wide model: more workgroups than the chip wants, rather than a range too long
    for split in (2, 4, 8, 16):
        if K % (split * 32) == 0 and (K + split - 1) // split <= ROWS16_MAX_K_PER_WORKGROUP:
            return split
    return 0


def _merged_splits(N: int, K: int) -> int:
    """The same for rows that are merged on the way in: a workgroup's range of K is then a
    multiple of a wave's 512 and at most 4096.  0: no such cut."""
    groups = (N + 15) // 16
    for split in (8, 4, 3, 2, 1):
        if K % (split * 512) == 0 and K // split <= 4096 and (groups * split <= 640 or split == 1):
            return split
    return 0


LIBRARY_ADDS_MIN_K = 4096


def library_adds(M: int, N: int, K: int) -> bool:
    """Whether a product of this shape, asked to add itself to the 32-bit stream, does so
    through the GEMM library (its beta = 1).

    Many rows (beyond those whose K the library gets in ranges): with K long enough that
    reading and writing the stream in the product's epilogue costs less than the next norm
    saves by not adding (measured at 2,048 rows: [2048, 8192] 75 us against 79 into bfloat16,
    the norm after it 4.8 us against 7.7; [2048, 2048] 25.5 against 22.2, which the norm does
    not win back).

    Few rows (a decode batch beyond this package's kernels for 16 rows): a mixer's closing
    product, K short, where the stream of width N is then complete for a feed-forward whose
    first product runs the norm itself (``rows64_swiglu_fusable``).  Added by the library,
    [2048, 2048] takes 6.5 us at 24 rows and 7.8 at 32 (its partial sums 6.0 to 6.2, which the
    norm kernel would have to add; this package's kernel adding with atomics 9.0 and 9.5),
    [1024, 1024] 5.6 to 7.4 us at 24 to 64 rows, as its partial sums do.  A long K (the
    feed-forward's own closing product) stays in ranges: [2048, 8192] at 24 rows 13.2 us
    added against 10.4 in ranges."""
    if K % 8:
        return False
    if M > LIBRARY_SPLIT_ROWS:
        return K >= LIBRARY_ADDS_MIN_K
    return M > LIBRARY_GEMM_ROWS and K < LIBRARY_ADDS_MIN_K and rows64_swiglu_fusable(M, N)


def accumulate_plan(M: int, N: int, K: int, normed: bool) -> int:
    """How a decode batch's product reaches the stream: the number of ranges of K whose
    partial products are added there with atomics, or 0 when the kernel that adds takes
    no such product (the product then comes back and the caller adds it)."""
    if M > 16 or K % 8:
        return 0
    if normed:
        return 1            # the kernel that runs the norm covers K with one workgroup
    return _accumulate_splits(N, K)


def linear(x, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
           out_dtype: Optional[torch.dtype] = None, force_tiled: bool = False,
           partial_ok: bool = False,
           accumulate: Optional[torch.Tensor] = None,
           tune: Optional[bool] = None) -> Optional[torch.Tensor]:
    """``x [M, K] @ weight[N, K]^T + bias`` with 32-bit accumulation.

    bfloat16 weights use the matrix-core kernels of csrc/gemm.hip up to
    ``LIBRARY_GEMM_ROWS`` rows (a decode batch), and always when a bias is asked
    for; larger plain products go to the GEMM library, with bfloat16 or 32-bit
    output.  32-bit weights use the all-32-bit kernel (``x`` may be either type and
    is widened): no library, no reduced-precision matrix mode.

    With ``partial_ok`` the result may come back as a stack ``[P, M, N]`` of 32-bit
    partial sums (K cut into ranges, for more workgroups, when N is small and M is
    at most ``LIBRARY_SPLIT_ROWS``); ``add_rmsnorm`` adds such a stack up while it
    reads it.

    ``x`` may be a ``NormedRows``: a decode batch is then normalised by the product's
    own kernel.  With ``accumulate`` (the 32-bit ``[M, N]`` residual stream) a decode
    batch's product is added to that tensor with atomics and ``None`` comes back (the
    additions of the ranges of K arrive in the hardware's order: reproducible to
    rounding only); otherwise the product comes back as usual and the caller adds it.

    ``tune``: whether the GEMM library may time its candidates at this shape's first call
    (``None``: the process's default, ``library_tuning``)."""
    if len(x.shape) != 2 or weight.dim() != 2:
        raise KernelError(f"linear takes x [M, K] and weight [N, K], got {tuple(x.shape)} and "
                          f"{tuple(weight.shape)}")
    M, K = x.shape
    N = weight.shape[0]
    if isinstance(x, MergedRows):
        splits = 0
        if accumulate is not None and bias is None and weight.dtype == torch.bfloat16 \
                and not force_tiled and merged_rows_pay(M, x.ranges):
            splits = _merged_splits(N, K)
        if not splits:
            x = x.materialise()
        else:
            _need(weight, "weight", torch.bfloat16, (N, K))
            _need(accumulate, "accumulate", torch.float32, (M, N))
            rc = _fn("gemm", "za_gemm_bf16_rows16_merged")(
                _ptr(x.acc), _ptr(x.ml), x.ranges, x.head_dim, _ptr(weight), _ptr(accumulate),
                M, N, K, splits, 1, _stream())
            _check(rc, "gemm_bf16_rows16_merged", f"M={M} N={N} K={K} splits={splits}")
            _note("linear", M=M, N=N, K=K, norm_in_product=False, added_to_stream=True,
                  partial_sums=1, out=accumulate.dtype, merged_ranges=x.ranges)
            return None
    normed = None
    if isinstance(x, NormedRows):
        if _takes_normed_rows(x, weight, M, K) and not force_tiled:
            normed = x
        else:
            x = x.materialise()
    if normed is not None and accumulate is not None \
            and normed.residual.untyped_storage().data_ptr() == accumulate.untyped_storage().data_ptr():
        # workgroups would read rows of the stream while others add to them
        normed, x = None, x.materialise()
    splits = 1
    if accumulate is not None and library_adds(M, N, K) and normed is None and bias is None \
            and weight.dtype == torch.bfloat16 and x.dtype == torch.bfloat16 and not force_tiled:
        # the library adds its product to the stream itself (many rows and a long K, or
        # the closing product of a mixer in a step of 17 to 64 rows)
        _need(weight, "weight", torch.bfloat16, (N, K))
        _need(accumulate, "accumulate", torch.float32, (M, N))
        if _library_matmul(x, weight, torch.float32, 1, tune, added_to=accumulate) is not None:
            _note("linear", M=M, N=N, K=K, norm_in_product=False, added_to_stream=True,
                  partial_sums=1, out=accumulate.dtype, kernel="library")
            return None
    if accumulate is not None and NORMED_ROWS_MAX_ROWS < M <= ROWS64_SWIGLU_ROWS and normed is None \
            and bias is None and weight.dtype == torch.bfloat16 and x.dtype == torch.bfloat16 \
            and not force_tiled and rows64_add_splits(N, K):
        # such a step for which the library has no algorithm: the closing product
        # of a mixer adds itself to the stream with this package's kernel
        # (so that the feed-forward's first product can run the norm, see above)
        ks = rows64_add_splits(N, K)
        linear_rows64(x, weight, ROWS64_ADD, accumulate, ks)
        _note("linear", M=M, N=N, K=K, norm_in_product=False, added_to_stream=True,
              partial_sums=1, out=accumulate.dtype, kernel="rows64")
        return None
    if accumulate is not None:
        if weight.dtype == torch.bfloat16 and not force_tiled \
                and (normed is not None or x.dtype == torch.bfloat16):
            splits = accumulate_plan(M, N, K, normed is not None)
        else:
            splits = 0
        if splits == 0:
            accumulate, splits = None, 1
    if normed is not None or accumulate is not None:
        _need(weight, "weight", torch.bfloat16, (N, K))
        if bias is not None:
            _need(bias, "bias", torch.float32, (N,))
        if normed is None:
            _need(x, "x", torch.bfloat16)
        if accumulate is not None:
            _need(accumulate, "accumulate", torch.float32, (M, N))
            out, out_code = accumulate, 0
        else:
            out_dtype = out_dtype or normed.dtype
            out = torch.empty((M, N), dtype=out_dtype, device=weight.device)
            out_code = _code(out_dtype)
        rc = _fn("gemm", "za_gemm_bf16_rows16_stream")(
            None if normed is not None else _ptr(x),
            _ptr(normed.residual) if normed is not None else None,
            _ptr(normed.rows) if normed is not None else None,
            _ptr(normed.weight) if normed is not None else None,
            normed.eps if normed is not None else 0.0,
            _ptr(weight), _ptr(bias), _ptr(out), out_code, M, N, K, splits,
            1 if accumulate is not None else 0, _stream())
        _check(rc, "gemm_bf16_rows16_stream", f"M={M} N={N} K={K} splits={splits}")
        _note("linear", M=M, N=N, K=K, norm_in_product=normed is not None,
              added_to_stream=accumulate is not None, partial_sums=1, out=out.dtype)
        return None if accumulate is not None else out
    _need(x, "x", (torch.float32, torch.bfloat16))
    _need(weight, "weight", (torch.float32, torch.bfloat16), (N, K))
    if bias is not None:
        _need(bias, "bias", torch.float32, (N,))
    out_dtype = out_dtype or x.dtype
    if weight.dtype == torch.float32:
        out = torch.empty((M, N), dtype=out_dtype, device=x.device)
        rc = _fn("gemm", "za_gemm_f32")(_ptr(x), _code(x.dtype), _ptr(weight), _ptr(bias), _ptr(out),
                                        _code(out_dtype), M, N, K, _stream())
        _check(rc, "gemm_f32", f"M={M} N={N} K={K}")
        _note("linear", M=M, N=N, K=K, norm_in_product=False, added_to_stream=False,
              partial_sums=1, out=out.dtype)
        return out
    if x.dtype != torch.bfloat16:
        raise KernelError("a bfloat16 weight needs bfloat16 activations")
    if K % 8:
        raise KernelError(f"the bfloat16 GEMM needs K to be a multiple of 8, got K={K}")
    # Many rows: the vendor's GEMM library, as the reference does for every
    # projection (/root/reference/src/matmul/root.zig:292-313 calls cuBLAS).
    library = M > LIBRARY_GEMM_ROWS and bias is None and not force_tiled \
        and out_dtype in (torch.bfloat16, torch.float32)
    splits = 1
    if partial_ok and not force_tiled and K <= 8192 * 4 and (M <= 16 or library):
        splits = _k_splits(M, N, K)
    if splits > 1 and M <= 16:
        stack = torch.empty((splits, M, N), dtype=torch.float32, device=x.device)
        rc = _fn("gemm", "za_gemm_bf16_rows16")(_ptr(x), _ptr(weight), _ptr(bias), _ptr(stack),
                                                0, M, N, K, splits, 0, _stream())
        _check(rc, "gemm_bf16_rows16", f"M={M} N={N} K={K} splits={splits}")
        _note("linear", M=M, N=N, K=K, norm_in_product=False, added_to_stream=False,
              partial_sums=splits, out=stack.dtype)
        return stack
    if library:
        # (with ranges of K: one batched product, [P, M, K/P] x [P, K/P, N])
        out = _library_matmul(x, weight, out_dtype, splits, tune)
        if out is not None:
            _note("linear", M=M, N=N, K=K, norm_in_product=False, added_to_stream=False,
                  partial_sums=splits, out=out.dtype)
            return out
    out = torch.empty((M, N), dtype=out_dtype, device=x.device)
    rc = _fn("gemm", "za_gemm_bf16")(_ptr(x), _ptr(weight), _ptr(bias), _ptr(out),
                                     _code(out_dtype), M, N, K, 1 if force_tiled else 0,
                                     _stream())
    _check(rc, "gemm_bf16", f"M={M} N={N} K={K}")
    _note("linear", M=M, N=N, K=K, norm_in_product=False, added_to_stream=False, partial_sums=1,
          out=out.dtype)
    return out


def linear_swiglu(x, gate_up_weight: torch.Tensor) -> torch.Tensor:
    """``silu(x Wg^T) * (x Wu^T)`` for ``gate_up_weight = [Wg; Wu]`` of shape ``[2I, K]``
    and at most 16 rows of bfloat16 ``x`` (or a ``NormedRows``): the gate is applied to
    the 32-bit accumulators, the ``[M, 2I]`` intermediate is never stored.  17 to
    ``ROWS64_SWIGLU_ROWS`` rows are taken as ``NormedRows`` only (``rows64_swiglu_fusable``)."""
    if len(x.shape) != 2 or gate_up_weight.dim() != 2 or gate_up_weight.shape[0] % 2 \
            or gate_up_weight.shape[1] != x.shape[1]:
        raise KernelError(f"linear_swiglu takes x [M, K] and a weight [2I, K], got "
                          f"{tuple(x.shape)} and {tuple(gate_up_weight.shape)}")
    M, K = x.shape
    I = gate_up_weight.shape[0] // 2
    _need(gate_up_weight, "gate_up_weight", torch.bfloat16)
    if M > NORMED_ROWS_MAX_ROWS:
        if not (isinstance(x, NormedRows) and x.dtype == torch.bfloat16
                and rows64_swiglu_fusable(M, K)):
            raise KernelError(f"linear_swiglu takes a step of {M} rows only as rows awaiting "
                              f"their norm, up to {ROWS64_SWIGLU_ROWS} rows, got K={K}")
        out = linear_rows64(x, gate_up_weight, ROWS64_SWIGLU)
        _note("linear_swiglu", M=M, N=2 * I, K=K, norm_in_product=True, kernel="rows64")
        return out
    normed = None
    if isinstance(x, NormedRows):
        if _takes_normed_rows(x, gate_up_weight, M, K):
            normed = x
        else:
            x = x.materialise()
    if normed is None:
        _need(x, "x", torch.bfloat16)
    if M > 16 or K % 8 or K > 8192:
        raise KernelError(f"linear_swiglu takes at most 16 rows and K <= 8192 in multiples of "
                          f"8, got M={M} K={K}")
    out = torch.empty((M, I), dtype=torch.bfloat16, device=gate_up_weight.device)
    rc = _fn("gemm", "za_gemm_bf16_rows16_swiglu")(
        None if normed is not None else _ptr(x),
        _ptr(normed.residual) if normed is not None else None,
        _ptr(normed.rows) if normed is not None else None,
        _ptr(normed.weight) if normed is not None else None,
        normed.eps if normed is not None else 0.0,
        _ptr(gate_up_weight), _ptr(out), M, I, K, _stream())
    _check(rc, "linear_swiglu", f"M={M} I={I} K={K}")
    _note("linear_swiglu", M=M, N=2 * I, K=K, norm_in_product=normed is not None)
    return out


# ------------------------------------------ products of 17 to 64 rows, fused forms
ROWS64_MAX_ROWS = 64
ROWS64_K_MULTIPLE = 512        # a workgroup's range of K: spans of 512, at least two
ROWS64_STORE, ROWS64_SWIGLU, ROWS64_ADD = 0, 1, 2


def rows64_takes(M: int, K: int, ksplit: int = 1) -> bool:
    """Whether ``linear_rows64`` takes a product of ``M`` rows over ``K`` in ``ksplit`` ranges."""
    return (1 <= M <= ROWS64_MAX_ROWS and ksplit >= 1 and K % ksplit == 0
            and (K // ksplit) % ROWS64_K_MULTIPLE == 0 and K // ksplit >= 2 * ROWS64_K_MULTIPLE)


# Where the kernel of csrc/gemm_rows64.hip is taken, by measurement (one MI355X, replayed
# from graphs, weights from memory, against the norm kernel + the library's product + the
# SwiGLU kernel): the fused norm + gate|up + SwiGLU of 2 x 8192 x 2048 takes 19.5-19.9 us at
# 17 to 32 rows against 24.8-25.8, 22.8-23.9 at 40-48 rows against 25.6, 25.5 at 64 rows
# against 25.9; the plain forms lose (norm + in_proj 15.3 against 13.2 at 24 rows, w2 added
# to the stream 12.7-14.5 against the library's 10.3).  So it serves the feed-forward's
# first product up to ROWS64_SWIGLU_ROWS rows (64 on a narrow stream), which needs the stream complete before it,
# and therefore the mixer's closing product of such a step, added to the stream with
# atomics (2048 x 2048: 8.6-9.4 us against the library's 6.6-8.8, without the stack of
# partial sums that the norm kernel would have to add).
ROWS64_SWIGLU_ROWS = 48
ROWS64_NARROW_WIDTH = 1024
ROWS64_ADD_MAX_K = 4096
ROWS64_ADD_MIN_WORKGROUPS = 48


def rows64_add_splits(N: int, K: int) -> int:
    """Into how many ranges K is cut when a product of 17 to 64 rows is added to the stream
    by the kernel of csrc/gemm_rows64.hip: as many as keep a range at 1,024 elements or
    more (two spans).  0: the kernel is not taken (no cut fits, too few workgroups to pay,
    or a K beyond what was measured to pay)."""
    if K > ROWS64_ADD_MAX_K:
        return 0
    tiles = (N + 63) // 64
    best = 0
    for split in (1, 2, 3, 4):
        if rows64_takes(1, K, split):
            best = split
    if best == 0 or tiles * best < ROWS64_ADD_MIN_WORKGROUPS:
        return 0
    return best


def rows64_swiglu_fusable(rows: int, width: int) -> bool:
    """Whether a step of ``rows`` rows takes the fused norm + gate|up + SwiGLU kernel for
    17 to 64 rows (``linear_swiglu`` with a ``NormedRows``): up to 48 rows, and up to 64
    where the stream is narrow (every workgroup reads all of the step's rows: at width 1024
    the fused form takes 13.7 us at 40 and 48 rows and 15.3 at 64, [9216, 1024], against
    18.4 to 18.6 for norm, library product and SwiGLU kernel; at width 2048, [16384, 2048],
    22.8 to 23.9 at 40 to 48 rows against 25.6, and at 64 rows it only equals them: a decode
    step of the 1.2B shape at batch 40 1.50 -> 1.47 ms, at batch 48 1.53 -> 1.49, at batch 64
    1.562 -> 1.557)."""
    most = ROWS64_MAX_ROWS if width <= ROWS64_NARROW_WIDTH else ROWS64_SWIGLU_ROWS
    return (NORMED_ROWS_MAX_ROWS < rows <= most and width <= NORMED_ROWS_MAX_K
            and rows64_takes(rows, width))


def linear_rows64(x, weight: torch.Tensor, mode: int = ROWS64_STORE,
                  accumulate: Optional[torch.Tensor] = None, ksplit: int = 1) -> Optional[torch.Tensor]:
    """A product of at most 64 rows on the kernel of csrc/gemm_rows64.hip.  ``x``: bfloat16
    ``[M, K]`` or a ``NormedRows`` (the kernel then runs the norm).  ``mode``:
    ``ROWS64_STORE`` (``x W^T`` as bfloat16), ``ROWS64_SWIGLU`` (``weight = [Wg; Wu]``:
    ``silu(x Wg^T) * (x Wu^T)`` as bfloat16) or ``ROWS64_ADD`` (``x W^T`` added to the 32-bit
    ``accumulate [M, N]`` with atomics, K in ``ksplit`` ranges; returns ``None``)."""
    if len(x.shape) != 2 or weight.dim() != 2 or weight.shape[1] != x.shape[1]:
        raise KernelError(f"linear_rows64 takes x [M, K] and a weight [N, K], got {tuple(x.shape)} "
                          f"and {tuple(weight.shape)}")
    M, K = x.shape
    _need(weight, "weight", torch.bfloat16)
    N = weight.shape[0]
    if mode == ROWS64_SWIGLU:
        if N % 2:
            raise KernelError("a fused gate|up weight has an even number of rows")
        N //= 2
    if not rows64_takes(M, K, ksplit) or (ksplit > 1 and mode != ROWS64_ADD):
        raise KernelError(f"linear_rows64 takes at most {ROWS64_MAX_ROWS} rows and ranges of K that "
                          f"are multiples of {ROWS64_K_MULTIPLE}, got M={M} K={K} in {ksplit} ranges")
    normed = x if isinstance(x, NormedRows) else None
    if normed is not None:
        if mode == ROWS64_ADD or normed.dtype != torch.bfloat16:
            raise KernelError("the kernel runs the norm only for bfloat16 products that it stores")
        if normed.residual.numel() >= 1 << 31:
            raise KernelError("the kernel addresses the stream's rows with 32-bit offsets")
    else:
        _need(x, "x", torch.bfloat16)
    if mode == ROWS64_ADD:
        _need(accumulate, "accumulate", torch.float32, (M, N))
        out = accumulate
    else:
        out = torch.empty((M, N), dtype=torch.bfloat16, device=weight.device)
    rc = _fn("gemm_rows64", "za_gemm_bf16_rows64")(
        None if normed is not None else _ptr(x),
        _ptr(normed.residual) if normed is not None else None,
        _ptr(normed.rows) if normed is not None else None,
        _ptr(normed.weight) if normed is not None else None,
        normed.eps if normed is not None else 0.0,
        _ptr(weight), _ptr(out), int(mode), M, N, K, int(ksplit), _stream())
    _check(rc, "gemm_bf16_rows64", f"M={M} N={N} K={K} mode={mode} ksplit={ksplit}")
    return None if mode == ROWS64_ADD else out


# ------------------------------------------------------------ rope + kv write
def qk_norm_rope_kv_write(qkv: torch.Tensor, positions: torch.Tensor,
                          slots: Optional[torch.Tensor], q_norm_w: Optional[torch.Tensor],
                          k_norm_w: Optional[torch.Tensor], inv_freq: Optional[torch.Tensor],
                          kv_cache: Optional[torch.Tensor], num_heads: int, num_kv_heads: int,
                          head_dim: int, rotary_dim: int, adjacent_pairs: bool, eps: float,
                          write_kv: bool = True) -> torch.Tensor:
    """Returns the normalised, rotated queries ``[T, num_heads, head_dim]`` and
    scatters keys/values into ``kv_cache [pages, 2, kv_heads, page_size, head_dim]``
    (keys as ``[offset][head_dim]``; the values' half of a page holds
    ``[head_dim][offset]``)."""
    T = qkv.shape[0]
    total = num_heads + 2 * num_kv_heads
    _need(qkv, "qkv", (torch.float32, torch.bfloat16), (T, total * head_dim))
    _need(positions, "positions", torch.int32, (T,))
    if head_dim > 256:
        raise KernelError(f"head_dim {head_dim} exceeds the kernel's limit of 256")
    if rotary_dim % 2 or not 0 <= rotary_dim <= head_dim:
        raise KernelError(f"rotary_dim {rotary_dim} must be even and at most head_dim {head_dim}")
    for name, w in (("q_norm_w", q_norm_w), ("k_norm_w", k_norm_w)):
        if w is not None:
            _need(w, name, torch.float32, (head_dim,))
    if rotary_dim:
        _need(inv_freq, "inv_freq", torch.float32, (rotary_dim // 2,))
    page_size = 0
    if write_kv:
        if kv_cache is None or slots is None:
            raise KernelError("write_kv needs kv_cache and slots")
        _need(slots, "slots", torch.int32, (T,))
        _need(kv_cache, "kv_cache", qkv.dtype)
        if kv_cache.dim() != 5 or kv_cache.shape[1] != 2 or kv_cache.shape[2] != num_kv_heads \
                or kv_cache.shape[4] != head_dim:
            raise KernelError(f"kv_cache has shape {tuple(kv_cache.shape)}, expected "
                              f"[pages, 2, {num_kv_heads}, page_size, {head_dim}]")
        page_size = kv_cache.shape[3]
    q_out = torch.empty((T, num_heads, head_dim), dtype=qkv.dtype, device=qkv.device)
    rc = _fn("rope_kv", "za_qk_norm_rope_kv_write")(
        _ptr(qkv), _ptr(positions), _ptr(slots) if write_kv else None, _ptr(q_norm_w),
        _ptr(k_norm_w), _ptr(inv_freq) if rotary_dim else None, _ptr(q_out),
        _ptr(kv_cache) if write_kv else None, _code(qkv.dtype), T, num_heads, num_kv_heads,
        head_dim, rotary_dim, 1 if adjacent_pairs else 0, float(eps), page_size,
        1 if write_kv else 0, _stream())
    _check(rc, "qk_norm_rope_kv_write")
    return q_out


# ----------------------------------------------------------------- attention
ATTENTION_MAX_ROWS = 32


def paged_attention(q: torch.Tensor, kv_cache: torch.Tensor, block_table: torch.Tensor,
                    positions: torch.Tensor, item_seq: torch.Tensor, item_row0: torch.Tensor,
                    item_count: torch.Tensor, n_items: int, scale: float, window: int = 0,
                    keys_per_split: int = 0, nsplit: int = 1,
                    workspace: Optional[Tuple[torch.Tensor, torch.Tensor]] = None) -> torch.Tensor:
    """Causal attention of ``q [T, heads, head_dim]`` over the cache; see
    csrc/attention.hip.  ``item_*`` list the work items: the request (row of
    ``block_table``), the first query row and the number of consecutive query
    rows, at most ``ATTENTION_MAX_ROWS // (heads // kv_heads)`` each."""
    if q.dim() != 3:
        raise KernelError(f"q must be [T, heads, head_dim], got {tuple(q.shape)}")
    T, nh, d = q.shape
    _need(q, "q", (torch.float32, torch.bfloat16))
    _need(kv_cache, "kv_cache", q.dtype)
    if kv_cache.dim() != 5 or kv_cache.shape[1] != 2 or kv_cache.shape[4] != d:
        raise KernelError(f"kv_cache has shape {tuple(kv_cache.shape)}, expected "
                          f"[pages, 2, kv_heads, page_size, {d}]")
    nkv, page_size = kv_cache.shape[2], kv_cache.shape[3]
    if nh % nkv:
        raise KernelError(f"{nh} heads do not divide into {nkv} key/value heads")
    if nh // nkv > ATTENTION_MAX_ROWS:
        raise KernelError(f"{nh // nkv} query heads per key/value head exceed the kernel's "
                          f"limit of {ATTENTION_MAX_ROWS}")
    if d % 8 or d > 256:
        raise KernelError(f"head_dim {d} must be a multiple of 8 and at most 256")
    _need(block_table, "block_table", torch.int32)
    if block_table.dim() != 2:
        raise KernelError("block_table must be [requests, max_pages]")
    _need(positions, "positions", torch.int32, (T,))
    for name, t in (("item_seq", item_seq), ("item_row0", item_row0), ("item_count", item_count)):
        _need(t, name, torch.int32)
        if t.numel() < n_items:
            raise KernelError(f"{name} holds {t.numel()} entries, fewer than {n_items} items")
    out = torch.empty_like(q)
    part_acc = part_ml = None
    if nsplit > 1:
        if keys_per_split <= 0 or keys_per_split % 64:
            raise KernelError("keys_per_split must be a positive multiple of 64")
        if workspace is not None:
            part_acc, part_ml = workspace
            _need(part_acc, "part_acc", torch.float32)
            _need(part_ml, "part_ml", torch.float32)
            if part_acc.numel() < T * nh * nsplit * d or part_ml.numel() < T * nh * nsplit * 2:
                raise KernelError("attention workspace is too small")
        else:
            part_acc = torch.empty((T, nh, nsplit, d), dtype=torch.float32, device=q.device)
            part_ml = torch.empty((T, nh, nsplit, 2), dtype=torch.float32, device=q.device)
    rc = _fn("attention", "za_paged_attention")(
        _ptr(q), _ptr(out), _ptr(kv_cache), _ptr(block_table), block_table.shape[1],
        _ptr(positions), _ptr(item_seq), _ptr(item_row0), _ptr(item_count), n_items, T,
        _ptr(part_acc), _ptr(part_ml), _code(q.dtype), nh, nkv, d, page_size, float(scale),
        int(window), int(keys_per_split), int(nsplit), _stream())
    _check(rc, "paged_attention")
    _note("attention", kernel="plain", rows=T, dtype=q.dtype, nsplit=int(nsplit))
    return out


ATTENTION_MFMA_ROWS = 128


def attention_mfma_supported(dtype: torch.dtype, num_heads: int, num_kv_heads: int,
                             head_dim: int, page_size: int = 4, scale: float = 1.0) -> bool:
    """Whether the matrix-core attention kernels (the one for prompt portions and
    the one for decoding) take these sizes."""
    group = num_heads // num_kv_heads
    return (dtype == torch.bfloat16 and head_dim in (64, 128) and group <= 16
            and page_size % 4 == 0 and scale > 0.0)


def paged_attention_mfma(q: torch.Tensor, kv_cache: torch.Tensor, block_table: torch.Tensor,
                         positions: torch.Tensor, item_seq: torch.Tensor,
                         item_row0: torch.Tensor, item_count: torch.Tensor, n_items: int,
                         scale: float, window: int = 0, keys_per_split: int = 0,
                         nsplit: int = 1, tile_keys: int = 64) -> torch.Tensor:
    """The same attention on the matrix cores (bfloat16, head_dim 64 or 128, at most
    16 query heads per key/value head, a page size that is a multiple of 4, a
    positive scale).  Work items hold at most
    ``ATTENTION_MFMA_ROWS // (heads // kv_heads)`` query tokens; long contexts may be
    cut into ``nsplit`` ranges of ``keys_per_split`` keys (a portion of a prompt far
    into its request yields few work items).  ``tile_keys``: 64, or 128 for long contexts
    (head_dim 64 only; head_dim 128 always takes 64)."""
    if tile_keys not in (64, 128):
        raise KernelError(f"tile_keys must be 64 or 128, got {tile_keys}")
    if q.dim() != 3:
        raise KernelError(f"q must be [T, heads, head_dim], got {tuple(q.shape)}")
    T, nh, d = q.shape
    _need(q, "q", torch.bfloat16)
    _need(kv_cache, "kv_cache", torch.bfloat16)
    if kv_cache.dim() != 5 or kv_cache.shape[1] != 2 or kv_cache.shape[4] != d:
        raise KernelError(f"kv_cache has shape {tuple(kv_cache.shape)}, expected "
                          f"[pages, 2, kv_heads, page_size, {d}]")
    nkv, page_size = kv_cache.shape[2], kv_cache.shape[3]
    if nh % nkv or not attention_mfma_supported(q.dtype, nh, nkv, d, page_size, scale):
        raise KernelError(f"the matrix-core attention kernel does not take {nh} heads, {nkv} "
                          f"key/value heads, head_dim {d}, page size {page_size}, scale {scale}")
    _need(block_table, "block_table", torch.int32)
    if block_table.dim() != 2:
        raise KernelError("block_table must be [requests, max_pages]")
    _need(positions, "positions", torch.int32, (T,))
    for name, t in (("item_seq", item_seq), ("item_row0", item_row0), ("item_count", item_count)):
        _need(t, name, torch.int32)
        if t.numel() < n_items:
            raise KernelError(f"{name} holds {t.numel()} entries, fewer than {n_items} items")
    out = torch.empty_like(q)
    part_acc = part_ml = None
    if nsplit > 1:
        if keys_per_split <= 0 or keys_per_split % 64:
            raise KernelError("keys_per_split must be a positive multiple of 64")
        part_acc = torch.empty((T, nh, nsplit, d), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((T, nh, nsplit, 2), dtype=torch.float32, device=q.device)
    rc = _fn("attention", "za_paged_attention_mfma")(
        _ptr(q), _ptr(out), _ptr(kv_cache), _ptr(block_table), block_table.shape[1],
        _ptr(positions), _ptr(item_seq), _ptr(item_row0), _ptr(item_count), n_items, T,
        _ptr(part_acc), _ptr(part_ml), nh, nkv, d, page_size, float(scale), int(window),
        int(keys_per_split), int(nsplit), int(tile_keys), _stream())
    _check(rc, "paged_attention_mfma")
    _note("attention", kernel="mfma", rows=T, dtype=q.dtype, nsplit=int(nsplit))
    return out


ATTENTION_MFMA_DECODE_ROWS = 16


def paged_attention_decode_mfma(q: torch.Tensor, kv_cache: torch.Tensor,
                                block_table: torch.Tensor, positions: torch.Tensor,
                                item_seq: Optional[torch.Tensor],
                                item_row0: Optional[torch.Tensor],
                                item_count: Optional[torch.Tensor], n_items: int, scale: float,
                                window: int = 0, keys_per_split: int = 0,
                                nsplit: int = 1) -> torch.Tensor:
    """The matrix-core kernel for decoding: work items of at most
    ``ATTENTION_MFMA_DECODE_ROWS // (heads // kv_heads)`` query tokens, long contexts
    optionally cut into ``nsplit`` ranges of ``keys_per_split`` keys.  With
    ``item_seq=None`` row ``i`` of ``q`` is the single token of request ``i``."""
    if q.dim() != 3:
        raise KernelError(f"q must be [T, heads, head_dim], got {tuple(q.shape)}")
    T, nh, d = q.shape
    _need(q, "q", torch.bfloat16)
    _need(kv_cache, "kv_cache", torch.bfloat16)
    if kv_cache.dim() != 5 or kv_cache.shape[1] != 2 or kv_cache.shape[4] != d:
        raise KernelError(f"kv_cache has shape {tuple(kv_cache.shape)}, expected "
                          f"[pages, 2, kv_heads, page_size, {d}]")
    nkv, page_size = kv_cache.shape[2], kv_cache.shape[3]
    if nh % nkv or not attention_mfma_supported(q.dtype, nh, nkv, d, page_size, scale):
        raise KernelError(f"the matrix-core attention kernel does not take {nh} heads, {nkv} "
                          f"key/value heads, head_dim {d}, page size {page_size}, scale {scale}")
    _need(block_table, "block_table", torch.int32)
    if block_table.dim() != 2:
        raise KernelError("block_table must be [requests, max_pages]")
    _need(positions, "positions", torch.int32, (T,))
    if item_seq is None:
        if n_items != T or block_table.shape[0] < T:
            raise KernelError("without work items every request brings exactly one token")
    else:
        for name, t in (("item_seq", item_seq), ("item_row0", item_row0),
                        ("item_count", item_count)):
            _need(t, name, torch.int32)
            if t.numel() < n_items:
                raise KernelError(f"{name} holds {t.numel()} entries, fewer than {n_items} items")
    out = torch.empty_like(q)
    part_acc = part_ml = None
    if nsplit > 1:
        if keys_per_split <= 0 or keys_per_split % 64:
            raise KernelError("keys_per_split must be a positive multiple of 64")
        part_acc = torch.empty((T, nh, nsplit, d), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((T, nh, nsplit, 2), dtype=torch.float32, device=q.device)
    rc = _fn("attention", "za_paged_attention_decode_mfma")(
        _ptr(q), _ptr(out), _ptr(kv_cache), _ptr(block_table), block_table.shape[1],
        _ptr(positions), _ptr(item_seq), _ptr(item_row0), _ptr(item_count), n_items, T,
        _ptr(part_acc), _ptr(part_ml), nh, nkv, d, page_size, float(scale), int(window),
        int(keys_per_split), int(nsplit), _stream())
    _check(rc, "paged_attention_decode_mfma")
    _note("attention", kernel="decode_mfma", rows=T, dtype=q.dtype, nsplit=int(nsplit))
    return out


def decode_rope_fusable(qkv, num_heads: int, num_kv_heads: int, head_dim: int, rotary_dim: int,
                        adjacent_pairs: bool, page_size: int, scale: float) -> bool:
    """Whether ``rope_attention_decode`` takes the step: bfloat16, the rotation over the whole
    head with half pairing, and what the matrix-core decode kernel takes."""
    return (qkv.dtype == torch.bfloat16 and rotary_dim == head_dim and not adjacent_pairs
            and attention_mfma_supported(qkv.dtype, num_heads, num_kv_heads, head_dim, page_size,
                                         scale)
            and num_heads // num_kv_heads <= ATTENTION_MFMA_DECODE_ROWS)


def rope_attention_decode(qkv: torch.Tensor, positions: torch.Tensor, slots: torch.Tensor,
                          q_norm_w: Optional[torch.Tensor], k_norm_w: Optional[torch.Tensor],
                          inv_freq: torch.Tensor, kv_cache: torch.Tensor,
                          block_table: torch.Tensor, num_heads: int, eps: float, scale: float,
                          window: int = 0, keys_per_split: int = 0,
                          nsplit: int = 1, combine: bool = True):
    """A step in which request ``i`` brings the one token of row ``i``: what
    ``qk_norm_rope_kv_write`` followed by ``paged_attention_decode_mfma`` does, in the
    attention's kernel (its prologue normalises and rotates the token's queries and key;
    the workgroup that meets the token's own position stores key and value to the cache).
    The same bits in the result and in the cache, one kernel and one trip through memory
    less.  Returns the attention's output ``[T, heads, head_dim]``, or, with ``nsplit`` > 1 and
    ``combine=False``, the ranges' partial results unmerged as ``MergedRows``."""
    if kv_cache.dim() != 5 or kv_cache.shape[1] != 2:
        raise KernelError(f"kv_cache has shape {tuple(kv_cache.shape)}, expected "
                          f"[pages, 2, kv_heads, page_size, head_dim]")
    nkv, page_size, d = kv_cache.shape[2], kv_cache.shape[3], kv_cache.shape[4]
    T = qkv.shape[0]
    nh = int(num_heads)
    _need(qkv, "qkv", torch.bfloat16, (T, (nh + 2 * nkv) * d))
    _need(kv_cache, "kv_cache", torch.bfloat16)
    if nh % nkv or not decode_rope_fusable(qkv, nh, nkv, d, d, False, page_size, scale):
        raise KernelError(f"rope_attention_decode does not take {nh} heads, {nkv} key/value "
                          f"heads, head_dim {d}, page size {page_size}, scale {scale}")
    _need(block_table, "block_table", torch.int32)
    if block_table.dim() != 2 or block_table.shape[0] < T:
        raise KernelError("block_table must be [requests, max_pages] with a row per token")
    _need(positions, "positions", torch.int32, (T,))
    _need(slots, "slots", torch.int32, (T,))
    _need(inv_freq, "inv_freq", torch.float32, (d // 2,))
    for name, w in (("q_norm_w", q_norm_w), ("k_norm_w", k_norm_w)):
        if w is not None:
            _need(w, name, torch.float32, (d,))
    unmerged = nsplit > 1 and not combine
    out = None if unmerged else torch.empty((T, nh, d), dtype=torch.bfloat16, device=qkv.device)
    part_acc = part_ml = None
    if nsplit > 1:
        if keys_per_split <= 0 or keys_per_split % 64:
            raise KernelError("keys_per_split must be a positive multiple of 64")
        part_acc = torch.empty((T, nh, nsplit, d), dtype=torch.float32, device=qkv.device)
        part_ml = torch.empty((T, nh, nsplit, 2), dtype=torch.float32, device=qkv.device)
    rc = _fn("attention", "za_paged_attention_decode_mfma_rope")(
        _ptr(qkv), _ptr(out), _ptr(kv_cache), _ptr(block_table), block_table.shape[1],
        _ptr(positions), _ptr(slots), _ptr(q_norm_w), _ptr(k_norm_w), _ptr(inv_freq), float(eps),
        T, _ptr(part_acc), _ptr(part_ml), nh, nkv, d, page_size, float(scale), int(window),
        int(keys_per_split), int(nsplit), 0 if unmerged else 1, _stream())
    _check(rc, "rope_attention_decode")
    _note("attention", kernel="decode_mfma_rope", rows=T, dtype=qkv.dtype, nsplit=int(nsplit),
          combine_kernel=nsplit > 1 and not unmerged)
    return MergedRows(part_acc, part_ml) if unmerged else out


# ---------------------------------------------------------------- short conv
GATED_CONV_MAX_ROWS = 16


def gated_conv_fusable(x, w_in: torch.Tensor, taps: torch.Tensor) -> bool:
    """Whether ``in_proj_gated_conv`` takes these operands: rows that still await their
    norm, at most sixteen of them, bfloat16 weights whose K the fused norm covers, and a
    width that is a multiple of 16."""
    if not isinstance(x, NormedRows) or x.dtype != torch.bfloat16 or w_in.dtype != torch.bfloat16:
        return False
    M, K = x.shape
    L, width = taps.shape
    return (0 < M <= GATED_CONV_MAX_ROWS and normed_rows_fusable(M, K) and width % 16 == 0
            and L <= 8 and tuple(w_in.shape) == (3 * width, K))


def in_proj_gated_conv(x: "NormedRows", w_in: torch.Tensor, taps: torch.Tensor,
                       bias: Optional[torch.Tensor], state: torch.Tensor,
                       slot_id: torch.Tensor, channels: int = 0) -> torch.Tensor:
    """The ShortConv mixer from the residual stream to the convolution's output for a
    decode batch in which every request brings ONE token (row m belongs to the request
    with state slot ``slot_id[m]``): the norm, ``in_proj`` (no bias) and ``short_conv``
    in one kernel, with the bits that the three kernels give one after the other.
    Operands as ``linear`` and ``short_conv`` take them; see ``gated_conv_fusable``.
    ``channels`` (4, 8 or 16; 0 leaves it to the launcher): channels per workgroup."""
    if not gated_conv_fusable(x, w_in, taps):
        raise KernelError("in_proj_gated_conv: operands outside what the fused kernel takes")
    M, K = x.shape
    L, width = taps.shape
    _need(w_in, "w_in", torch.bfloat16, (3 * width, K))
    _need(taps, "taps", torch.float32)
    if bias is not None:
        _need(bias, "bias", torch.float32, (width,))
    if not (isinstance(state, torch.Tensor) and state.is_cuda and state.dtype == torch.float32):
        raise KernelError("state must be a float32 tensor on the GPU")
    if state.dim() != 3 or tuple(state.shape[1:]) != (width, L):
        raise KernelError(f"state has shape {tuple(state.shape)}, expected [slots, {width}, {L}]")
    if state.stride(2) != 1 or state.stride(1) != L or state.stride(0) < width * L:
        raise KernelError(f"state has strides {state.stride()}; a slot must be laid out "
                          f"[{width}, {L}] contiguously")
    _need(slot_id, "slot_id", torch.int32)
    if slot_id.numel() < M:
        raise KernelError(f"{M} rows but {slot_id.numel()} state slots")
    y = torch.empty((M, width), dtype=torch.bfloat16, device=w_in.device)
    rc = _fn("gemm", "za_gemm_bf16_rows16_gated_conv")(
        _ptr(x.residual), _ptr(x.rows), _ptr(x.weight), x.eps, _ptr(w_in), _ptr(taps), _ptr(bias),
        _ptr(state), state.stride(0), _ptr(slot_id), _ptr(y), M, width, K, L, channels, _stream())
    _check(rc, "gemm_bf16_rows16_gated_conv", f"M={M} width={width} K={K} L={L}")
    _note("linear", M=M, N=3 * width, K=K, norm_in_product=True, added_to_stream=False,
          partial_sums=1, out=torch.bfloat16)
    return y


def short_conv(z: torch.Tensor, taps: torch.Tensor, bias: Optional[torch.Tensor],
               state: torch.Tensor, token_seq: torch.Tensor, seq_start: torch.Tensor,
               slot_id: torch.Tensor) -> torch.Tensor:
    """Gated causal depth-wise convolution with carried state; see
    csrc/shortconv.hip.  ``z [T, 3*width]``; ``taps [L, width]``, the filter tap by
    tap (a checkpoint's ``[width, L]`` turned round, so that a thread's channels lie
    side by side); ``state [slots, width, L]`` (updated in place; slots may be spaced
    further apart than ``width * L`` floats)."""
    T = z.shape[0]
    if taps.dim() != 2:
        raise KernelError(f"taps must be [L, width], got {tuple(taps.shape)}")
    L, width = taps.shape
    _need(z, "z", (torch.float32, torch.bfloat16), (T, 3 * width))
    _need(taps, "taps", torch.float32)
    if L > 8:
        raise KernelError(f"convolution length {L} exceeds the kernel's limit of 8")
    if bias is not None:
        _need(bias, "bias", torch.float32, (width,))
    if not (isinstance(state, torch.Tensor) and state.is_cuda and state.dtype == torch.float32):
        raise KernelError("state must be a float32 tensor on the GPU")
    if state.dim() != 3 or tuple(state.shape[1:]) != (width, L):
        raise KernelError(f"state has shape {tuple(state.shape)}, expected [slots, {width}, {L}]")
    if state.stride(2) != 1 or state.stride(1) != L or state.stride(0) < width * L:
        raise KernelError(f"state has strides {state.stride()}; a slot must be laid out "
                          f"[{width}, {L}] contiguously")
    _need(token_seq, "token_seq", torch.int32, (T,))
    _need(seq_start, "seq_start", torch.int32)
    _need(slot_id, "slot_id", torch.int32)
    y = torch.empty((T, width), dtype=z.dtype, device=z.device)
    rc = _fn("shortconv", "za_short_conv")(_ptr(z), _ptr(taps), _ptr(bias), _ptr(state),
                                           _ptr(token_seq), _ptr(seq_start), _ptr(slot_id), _ptr(y),
                                           _code(z.dtype), T, slot_id.numel(), width, L,
                                           state.stride(0), _stream())
    _check(rc, "short_conv")
    return y


# ---------------------------------------------------------------- activation
def swiglu(gate_up: torch.Tensor) -> torch.Tensor:
    """``silu(gate) * up`` for ``gate_up = [gate | up]`` of shape ``[T, 2*I]``."""
    _need(gate_up, "gate_up", (torch.float32, torch.bfloat16))
    if gate_up.dim() != 2 or gate_up.shape[1] % 2:
        raise KernelError(f"swiglu takes [T, 2*I], got {tuple(gate_up.shape)}")
    T, two_i = gate_up.shape
    out = torch.empty((T, two_i // 2), dtype=gate_up.dtype, device=gate_up.device)
    rc = _fn("activation", "za_swiglu")(_ptr(gate_up), _ptr(out), _code(gate_up.dtype), T,
                                        two_i // 2, _stream())
    _check(rc, "swiglu")
    return out


def cast(x: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """Element-wise conversion between float32 and bfloat16 (round to nearest even)."""
    _need(x, "x", (torch.float32, torch.bfloat16))
    if x.dtype == dtype:
        return x
    out = torch.empty(x.shape, dtype=dtype, device=x.device)
    rc = _fn("activation", "za_cast")(_ptr(x), _code(x.dtype), _ptr(out), _code(dtype), x.numel(),
                                      _stream())
    _check(rc, "cast")
    return out


def copy_columns(src: torch.Tensor, col0: int, ncols: int, out: Optional[torch.Tensor] = None,
                 out_col0: int = 0, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """Columns ``[col0, col0 + ncols)`` of every row of ``src [rows, width]``, as a new
    ``[rows, ncols]`` tensor of ``dtype`` (the source's by default), or into columns
    ``[out_col0, out_col0 + ncols)`` of ``out [rows, any width]``; converted between
    float32 and bfloat16 on the way where the two differ."""
    _need(src, "src", (torch.float32, torch.bfloat16))
    if src.dim() != 2:
        raise KernelError(f"copy_columns takes [rows, width], got {tuple(src.shape)}")
    rows, width = src.shape
    if out is None:
        out = torch.empty((rows, ncols), dtype=dtype or src.dtype, device=src.device)
        out_col0 = 0
    _need(out, "out", (torch.float32, torch.bfloat16))
    if out.dim() != 2 or out.shape[0] != rows:
        raise KernelError(f"out has shape {tuple(out.shape)}, expected [{rows}, width]")
    if not (0 <= col0 and col0 + ncols <= width and 0 <= out_col0
            and out_col0 + ncols <= out.shape[1] and ncols >= 0):
        raise KernelError(f"columns [{col0}, {col0 + ncols}) of {width} into [{out_col0}, "
                          f"{out_col0 + ncols}) of {out.shape[1]}")
    rc = _fn("activation", "za_copy_columns")(_ptr(src), _code(src.dtype), width, int(col0), _ptr(out),
                                              _code(out.dtype), out.shape[1], int(out_col0), rows,
                                              int(ncols), _stream())
    _check(rc, "copy_columns")
    return out


# ------------------------------------------------------------------ sampling
def argmax(logits: torch.Tensor) -> torch.Tensor:
    """First index of each row's maximum."""
    _need(logits, "logits", torch.float32)
    if logits.dim() != 2:
        raise KernelError("argmax takes [rows, vocab]")
    R, V = logits.shape
    out = torch.empty((R,), dtype=torch.int32, device=logits.device)
    # few rows of a long vocabulary: cut each row so that some 512 workgroups run
    chunks = max(1, min((512 + R - 1) // R, 64, V // 4096))
    part_v = part_i = None
    if chunks > 1:
        part_v = torch.empty((R, chunks), dtype=torch.float32, device=logits.device)
        part_i = torch.empty((R, chunks), dtype=torch.int32, device=logits.device)
    rc = _fn("sampling", "za_argmax")(_ptr(logits), R, V, _ptr(out), _ptr(part_v), _ptr(part_i),
                                      chunks, _stream())
    _check(rc, "argmax")
    return out


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor,
           top_p: torch.Tensor, uniform: torch.Tensor, whole_row_only: bool = False) -> torch.Tensor:
    """One token per row: greedy where temperature <= 0, else temperature, top-k, top-p
    and a draw with the row's uniform number; see csrc/sampling.hip.  ``whole_row_only``
    makes the kernel search its thresholds the slow way only (tests compare the two)."""
    _need(logits, "logits", torch.float32)
    if logits.dim() != 2:
        raise KernelError("sample takes [rows, vocab]")
    R = logits.shape[0]
    _need(temperature, "temperature", torch.float32, (R,))
    _need(top_k, "top_k", torch.int32, (R,))
    _need(top_p, "top_p", torch.float32, (R,))
    _need(uniform, "uniform", torch.float32, (R,))
    out = torch.empty((R,), dtype=torch.int32, device=logits.device)
    rc = _fn("sampling", "za_sample")(_ptr(logits), R, logits.shape[1], _ptr(temperature),
                                      _ptr(top_k), _ptr(top_p), _ptr(uniform), _ptr(out),
                                      1 if whole_row_only else 0, _stream())
    _check(rc, "sample", f"rows={R} vocab={logits.shape[1]}")
    return out


def repetition_penalty_(logits: torch.Tensor, rows: torch.Tensor, tokens: torch.Tensor,
                        factors: torch.Tensor) -> None:
    """In place; each (row, token) pair may be listed once."""
    _need(logits, "logits", torch.float32)
    n = rows.numel()
    _need(rows, "rows", torch.int32, (n,))
    _need(tokens, "tokens", torch.int32, (n,))
    _need(factors, "factors", torch.float32, (n,))
    rc = _fn("sampling", "za_repetition_penalty")(_ptr(logits), logits.shape[1], _ptr(rows),
                                                  _ptr(tokens), _ptr(factors), n, _stream())
    _check(rc, "repetition_penalty")


# ------------------------------------------------------------ measured ceilings
def measured_read_bandwidth(n_bytes: int = 1 << 30, repeats: int = 5) -> float:
    """Bytes per second of a kernel that only reads ``n_bytes`` of device memory (more than
    any cache holds), the best of ``repeats`` runs; see csrc/calibrate.hip."""
    n_bytes = n_bytes // 16 * 16
    device = torch.device("cuda", torch.cuda.current_device())
    src = torch.zeros((n_bytes,), dtype=torch.uint8, device=device)
    sink = torch.zeros((1,), dtype=torch.float32, device=device)
    fn = _fn("calibrate", "za_read_stream")
    best = 0.0
    for i in range(repeats + 1):
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        _check(fn(_ptr(src), n_bytes, 256 * 16, _ptr(sink), _stream()), "read_stream")
        stop.record()
        stop.synchronize()
        if i:                                   # (the first run also loads the kernel)
            best = max(best, n_bytes / (start.elapsed_time(stop) * 1e-3))
    return best


def measured_mfma_rate(repeats: int = 3) -> float:
    """bfloat16 flop per second of matrix-core instructions issued back to back from
    registers by every compute unit; see csrc/calibrate.hip."""
    device = torch.device("cuda", torch.cuda.current_device())
    sink = torch.zeros((1,), dtype=torch.float32, device=device)
    fn = _fn("calibrate", "za_mfma_loop")
    blocks, iters = 256 * 8, 20000
    flops = blocks * 4 * iters * 8 * 16384.0
    best = 0.0
    for i in range(repeats + 1):
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        _check(fn(blocks, iters, _ptr(sink), _stream()), "mfma_loop")
        stop.record()
        stop.synchronize()
        if i:
            best = max(best, flops / (start.elapsed_time(stop) * 1e-3))
    return best
