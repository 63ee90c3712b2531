"""Python face of the HIP kernels: checks shapes, dtypes and devices on the host, then launches
on the current HIP stream.  Tensors are torch tensors used as plain device buffers.

There is no CPU path and no library fallback: a tensor that is not on the GPU, or a shape a
kernel does not take, raises.
"""

from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_int64, c_void_p
from typing import Dict, List, Optional, Tuple

import torch

from . import jit

F32, BF16 = 0, 1


class KernelError(RuntimeError):
  pass


def dtype_code(dt: torch.dtype) -> int:
  if dt == torch.float32:
    return F32
  if dt == torch.bfloat16:
    return BF16
  raise KernelError(f"dtype {dt} is not supported by the HIP kernels (float32 and bfloat16 are)")


def _ptr(t: Optional[torch.Tensor]):
  return None if t is None else t.data_ptr()


# the current stream's handle, asked for by every launch: torch's raw accessor where it has one (a tenth of the cost
# of building a Stream object: a prompt's step of 28 layers asks 145 times)
_RAW_STREAM = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream():
  if _RAW_STREAM is not None:
    return _RAW_STREAM(torch.cuda.current_device())
  return torch.cuda.current_stream().cuda_stream


def _dev(*tensors):
  for t in tensors:
    if t is not None and not t.is_cuda:
      raise KernelError("miniinfer_amd kernels run on the GPU only; got a tensor on " + str(t.device))


def _contig(name, t):
  if t is not None and not t.is_contiguous():
    raise KernelError(f"{name} must be contiguous")


def _i32(name, t, n=None):
  if t is None:
    return
  if t.dtype != torch.int32:
    raise KernelError(f"{name} must be int32, got {t.dtype}")
  _contig(name, t)
  if n is not None and t.numel() < n:
    raise KernelError(f"{name} has {t.numel()} elements, {n} are needed")


def _f32(name, t, n=None):
  if t is None:
    return
  if t.dtype != torch.float32:
    raise KernelError(f"{name} must be float32, got {t.dtype}")
  _contig(name, t)
  if n is not None and t.numel() != n:
    raise KernelError(f"{name} has {t.numel()} elements, {n} are expected")


_SIGS = {
  "elementwise": {
    "mi_embed": [c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_int, c_float, c_void_p,
                 c_void_p, c_int, c_void_p],
    "mi_logit_transform": [c_void_p, c_int64, c_int, c_int, c_float, c_float, c_void_p],
    "mi_add_rmsnorm": [c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_float, c_int,
                       c_void_p],
    "mi_silu_mul": [c_int, c_void_p, c_void_p, c_int, c_int, c_void_p],
    "mi_silu_mul_scaled": [c_int, c_void_p, c_void_p, c_int, c_int, c_void_p, c_int, c_int, c_float, c_int, c_void_p],
    "mi_add_bias": [c_int, c_void_p, c_int64, c_void_p, c_int, c_int, c_void_p],
    "mi_qk_norm_rope_cache": [c_int, c_void_p, c_int64, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_float,
                              c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p],
  },
  "gemm": {
    "mi_gemm_nt": [c_int, c_int, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int, c_int, c_int,
                   c_void_p],
  },
  "attention": {
    "mi_paged_attention": [c_int, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int,
                           c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int,
                           c_int, c_void_p, c_void_p, c_void_p],
  },
}

_SIGS["attention_mfma"] = {
  "mi_attn_prefill": [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int,
                      c_void_p, c_void_p, c_int, c_int, c_int, c_float, c_int, c_int, c_void_p],
  "mi_attn_decode": [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                     c_int, c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_float, c_int, c_int, c_int, c_void_p],
  "mi_attn_decode_front": [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                           c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_float, c_int,
                           c_int, c_int, c_void_p, c_void_p, c_float, c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p],
  "mi_attn_prefill_tokens_per_block": [c_int, c_int],
  "mi_attn_prefill_tokens_per_block_wide": [c_int, c_int],
}

_SIGS["gemm_skinny"] = {
  "mi_gemm_skinny": [c_int, c_int, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int, c_int, c_int,
                     c_void_p],
}

_SIGS["gemm_skinny"]["mi_gemm_skinny_ex"] = [c_int, c_int, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int,
                                             c_int, c_int, c_void_p, c_int, c_float, c_void_p, c_void_p, c_void_p,
                                             c_void_p, c_void_p]
_SIGS["gemm_skinny"]["mi_gemm_skinny_groups"] = [c_int, c_int, c_int]
_SIGS["gemm_skinny"]["mi_gemm_skinny_v"] = [c_int, c_int, c_int, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64,
                                            c_int, c_int, c_int, c_void_p, c_int, c_float, c_void_p, c_void_p, c_void_p,
                                            c_void_p, c_void_p, c_int64, c_void_p]
_SIGS["gemm_skinny"]["mi_gemm_skinny_plan"] = [c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p]
_SIGS["gemm_skinny"]["mi_gemm_skinny_ss_row"] = [c_int]
_SIGS["gemm_skinny"]["mi_gemm_skinny_waves"] = [c_int, c_int, c_int, c_int, c_int]
_SIGS["gemm_skinny"]["mi_norm_gemm_skinny"] = [c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_float,
                                               c_void_p, c_int64, c_void_p, c_int64, c_int, c_int, c_int, c_void_p]

_SIGS["sampling"] = {
  "mi_sample": [c_void_p, c_int64, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p],
  "mi_sample_simple": [c_void_p, c_int64, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                       c_void_p],
  "mi_sample_parts_count": [c_int],
}

_SIGS["probes"] = {
  "mi_probe_stream_read": [c_void_p, c_int64, c_void_p, c_void_p],
  "mi_probe_mfma": [c_int, c_int, c_void_p, c_void_p, c_void_p],
}

_libs = {}


def _lib(name: str, defines=()):
  key = (name, tuple(sorted(defines)))
  lib = _libs.get(key)
  if lib is None:
    lib = jit.load_module(name, defines)
    for fn, sig in _SIGS.get(name, {}).items():
      f = getattr(lib, fn)
      f.argtypes = sig
      f.restype = c_int
    _libs[key] = lib
  return lib


def _check(lib, rc):
  if rc != 0:
    raise KernelError(lib.mi_last_error().decode())



def _check_pages(what, k_pages, v_pages, nkv, d, dtype):
  """Key pages [pages, nkv, P, d]; value pages transposed [pages, nkv, d, P]."""
  if k_pages.dim() != 4 or v_pages.dim() != 4:
    raise KernelError(f"{what}: pages must have 4 dims")
  n, h, P, dd = k_pages.shape
  if h != nkv or dd != d or tuple(v_pages.shape) != (n, nkv, d, P):
    raise KernelError(f"{what}: key pages {tuple(k_pages.shape)} / value pages {tuple(v_pages.shape)} are not "
                      f"[pages, {nkv}, P, {d}] / [pages, {nkv}, {d}, P]")
  if k_pages.dtype != dtype or v_pages.dtype != dtype:
    raise KernelError(f"{what}: pages are {k_pages.dtype}/{v_pages.dtype}, activations {dtype}")
  _contig("k_pages", k_pages)
  _contig("v_pages", v_pages)


# ----------------------------------------------------------------------------- embedding

def embed(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor, future: Optional[torch.Tensor] = None,
          scale: float = 1.0, pos_table: Optional[torch.Tensor] = None,
          positions: Optional[torch.Tensor] = None) -> torch.Tensor:
  """out[t, :] = float32(table[ids[t], :]) * scale (+ pos_table[positions[t], :]).  An id or a position outside
  its table gives a row of NaN.  With `future` (int32), an id -(r + 1) is replaced by future[r] as it stands when
  the kernel runs."""
  _dev(table, ids, out, future, pos_table, positions)
  _i32("future", future)
  V, H = table.shape
  T = ids.numel()
  _contig("table", table)
  _i32("ids", ids)
  _f32("out", out, T * H)
  max_pos = 0
  if pos_table is not None:
    _contig("pos_table", pos_table)
    if pos_table.dtype != table.dtype or pos_table.dim() != 2 or pos_table.shape[1] != H:
      raise KernelError(f"embed: the position table {tuple(pos_table.shape)} {pos_table.dtype} does not fit rows "
                        f"of {H} {table.dtype}")
    _i32("positions", positions, T)
    max_pos = pos_table.shape[0]
  lib = _lib("elementwise")
  _check(lib, lib.mi_embed(dtype_code(table.dtype), _ptr(table), _ptr(ids), _ptr(out), T, H, V, _ptr(future),
                           0 if future is None else future.numel(), float(scale), _ptr(pos_table),
                           _ptr(positions) if pos_table is not None else None, max_pos, _stream()))
  return out


def logit_transform(logits: torch.Tensor, scale: float = 1.0, softcap: float = 0.0) -> torch.Tensor:
  """In place on float32 logits [R, V]: x = x * scale, then (softcap > 0) x = softcap * tanh(x / softcap)."""
  _dev(logits)
  if logits.dtype != torch.float32 or logits.dim() != 2 or (logits.shape[1] > 1 and logits.stride(1) != 1):
    raise KernelError("logit_transform: logits must be float32 [R, V] with dense rows")
  R, V = logits.shape
  lib = _lib("elementwise")
  _check(lib, lib.mi_logit_transform(_ptr(logits), logits.stride(0) if R > 1 else V, R, V, float(scale),
                                     float(softcap), _stream()))
  return logits


# ----------------------------------------------------------------------------- norms

def add_rmsnorm(x: Optional[torch.Tensor], residual: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                out: torch.Tensor, rows: Optional[torch.Tensor] = None, write_back: bool = False) -> torch.Tensor:
  """out[i] = rmsnorm(residual[s] + x[s]) * weight with s = rows[i] (or i); 32-bit arithmetic.
  x [M, N] in float32 or bfloat16 (may be None), residual [M, N] float32 (may be None; updated in
  place to the sum when `write_back`)."""
  _dev(x, residual, weight, out, rows)
  N = weight.numel()
  _f32("weight", weight)
  src = x if x is not None else residual
  if src is None:
    raise KernelError("add_rmsnorm needs x or a residual")
  if src.shape[-1] != N:
    raise KernelError(f"add_rmsnorm: rows of {src.shape[-1]} elements, weight of {N}")
  M_src = src.numel() // N
  for name, t in (("x", x), ("residual", residual)):
    if t is not None:
      _contig(name, t)
      if t.numel() != M_src * N:
        raise KernelError(f"add_rmsnorm: {name} has another shape than its partner")
  if residual is not None and residual.dtype != torch.float32:
    raise KernelError("add_rmsnorm: the residual stream is float32")
  if rows is not None:
    _i32("rows", rows)
    M = rows.numel()
  else:
    M = M_src
  _contig("out", out)
  if out.numel() != M * N:
    raise KernelError(f"add_rmsnorm: out has {out.numel()} elements, {M * N} are expected")
  lib = _lib("elementwise")
  _check(lib, lib.mi_add_rmsnorm(dtype_code(x.dtype) if x is not None else F32, dtype_code(out.dtype), _ptr(x),
                                 _ptr(residual), _ptr(weight), _ptr(out), _ptr(rows), M, N, float(eps),
                                 1 if write_back else 0, _stream()))
  return out


def add_bias(y: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
  """y[m, :] += bias, in place; y [M, N] with dense rows, bias [N] of y's dtype (bfloat16 or float32)."""
  _dev(y, bias)
  if y.dim() != 2 or (y.shape[1] > 1 and y.stride(1) != 1) or bias.dim() != 1 or bias.numel() != y.shape[1]:
    raise KernelError(f"add_bias: y {tuple(y.shape)} and bias {tuple(bias.shape)} do not fit")
  if bias.dtype != y.dtype:
    raise KernelError(f"add_bias: y is {y.dtype}, the bias {bias.dtype}")
  _contig("bias", bias)
  M, N = y.shape
  lib = _lib("elementwise")
  _check(lib, lib.mi_add_bias(dtype_code(y.dtype), _ptr(y), y.stride(0) if M > 1 else N, _ptr(bias), M, N, _stream()))
  return y


def silu_mul(gate_up: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
  """out[m, c] = silu(gate_up[m, c]) * gate_up[m, I + c]."""
  _dev(gate_up, out)
  _contig("gate_up", gate_up)
  _contig("out", out)
  M, I2 = gate_up.shape
  if I2 % 2 or out.shape != (M, I2 // 2) or out.dtype != gate_up.dtype:
    raise KernelError(f"silu_mul: gate_up {tuple(gate_up.shape)} and out {tuple(out.shape)} do not fit")
  lib = _lib("elementwise")
  _check(lib, lib.mi_silu_mul(dtype_code(gate_up.dtype), _ptr(gate_up), _ptr(out), M, I2 // 2, _stream()))
  return out


def silu_mul_scaled(gate_up: torch.Tensor, out: torch.Tensor, row_ss: torch.Tensor, eps: float, k: int) -> torch.Tensor:
  """`silu_mul` of a product whose left operand was the first half of an RMS norm (`gemm_skinny_into_norm`): row m of
  gate and up is first scaled by rsqrt(sum_p row_ss[p, m] / k + eps), the norm's missing factor (k: the length of
  the normed rows).  row_ss float32 [parts, rows per part]; the columns I a multiple of 4."""
  _dev(gate_up, out, row_ss)
  _contig("gate_up", gate_up)
  _contig("out", out)
  M, I2 = gate_up.shape
  if I2 % 8 or out.shape != (M, I2 // 2) or out.dtype != gate_up.dtype:
    raise KernelError(f"silu_mul_scaled: gate_up {tuple(gate_up.shape)} and out {tuple(out.shape)} do not fit")
  if row_ss.dtype != torch.float32 or row_ss.dim() != 2 or row_ss.shape[1] < M or not row_ss.is_contiguous():
    raise KernelError(f"silu_mul_scaled: row_ss must be a contiguous float32 [parts, >= {M}]")
  lib = _lib("elementwise")
  _check(lib, lib.mi_silu_mul_scaled(dtype_code(gate_up.dtype), _ptr(gate_up), _ptr(out), M, I2 // 2, _ptr(row_ss),
                                     row_ss.shape[0], row_ss.shape[1], float(eps), int(k), _stream()))
  return out


def qk_norm_rope_cache(qkv: torch.Tensor, nq: int, nkv: int, d: int, q_weight: Optional[torch.Tensor],
                       k_weight: Optional[torch.Tensor], eps: float, cos_sin: Optional[torch.Tensor],
                       positions: Optional[torch.Tensor], k_pages: Optional[torch.Tensor],
                       v_pages: Optional[torch.Tensor], slots: Optional[torch.Tensor], page_size: int) -> None:
  """In place on qkv [T, (nq + 2 nkv) d]: per-head RMS norm of q and k (if weights), rotation of q and k
  (if cos_sin [max_pos, rotary_dim]), and a copy of the new k rows into key pages [num_pages, nkv, page_size, d]
  and of the new v rows into the transposed value pages [num_pages, nkv, d, page_size], at
  slots[t] = page * page_size + offset."""
  _dev(qkv, q_weight, k_weight, cos_sin, positions, k_pages, v_pages, slots)
  if qkv.dim() != 2 or qkv.stride(1) != 1 or qkv.shape[1] != (nq + 2 * nkv) * d:
    raise KernelError(f"qk_norm_rope_cache: qkv {tuple(qkv.shape)} does not hold {nq}+2*{nkv} heads of {d}")
  T = qkv.shape[0]
  _f32("q_weight", q_weight, d)
  _f32("k_weight", k_weight, d)
  rotary_dim, max_pos = 0, 0
  if cos_sin is not None:
    _f32("cos_sin", cos_sin)
    max_pos, rotary_dim = cos_sin.shape
    _i32("positions", positions, T)
  if k_pages is not None:
    _check_pages("qk_norm_rope_cache", k_pages, v_pages, nkv, d, qkv.dtype)
    if k_pages.shape[2] != page_size:
      raise KernelError(f"qk_norm_rope_cache: pages of {k_pages.shape[2]} tokens, page_size={page_size}")
    _i32("slots", slots, T)
  lib = _lib("elementwise")
  _check(lib, lib.mi_qk_norm_rope_cache(dtype_code(qkv.dtype), _ptr(qkv), qkv.stride(0), T, nq, nkv, d,
                                        _ptr(q_weight), _ptr(k_weight), float(eps), _ptr(cos_sin), rotary_dim,
                                        max_pos, _ptr(positions), _ptr(k_pages), _ptr(v_pages), _ptr(slots),
                                        page_size, _stream()))


# ----------------------------------------------------------------------------- matrix product

def gemm_nt(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
  """out[M, N] = a[M, K] @ w[N, K]^T with 32-bit FMA accumulation (no matrix instruction).
  a and w share a dtype; out is that dtype or float32.  Rows may be strided, columns are dense."""
  _dev(a, w, out)
  if a.dim() != 2 or w.dim() != 2 or out.dim() != 2:
    raise KernelError("gemm_nt takes matrices")
  M, K = a.shape
  N, K2 = w.shape
  if K != K2 or tuple(out.shape) != (M, N):
    raise KernelError(f"gemm_nt: a {tuple(a.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)} do not fit")
  if a.dtype != w.dtype:
    raise KernelError(f"gemm_nt: a is {a.dtype}, w is {w.dtype}")
  for name, t in (("a", a), ("w", w), ("out", out)):
    if t.stride(1) != 1:
      raise KernelError(f"gemm_nt: {name} must have dense rows")
  lib = _lib("gemm")
  _check(lib, lib.mi_gemm_nt(dtype_code(a.dtype), dtype_code(out.dtype), _ptr(a), a.stride(0) if M > 1 else K,
                             _ptr(w), w.stride(0) if N > 1 else K, _ptr(out), out.stride(0) if M > 1 else N,
                             M, N, K, _stream()))
  return out


SKINNY_MAX_ROWS = 64
SKINNY_OWN_ROWS = 16                 # without a measurement: up to here the weight-streaming kernel for every matrix,
SKINNY_OWN_ELEMENTS = 8 << 20        # and for more rows (up to SKINNY_MAX_ROWS) while the matrix is smaller than this
TUNE_ROWS = (1, 4, 8, 16, 32, 48, 64)   # row counts at which `tuning.tune_products` times the candidates
# (rows point, matrix rows, k, gate|up) -> the quickest: LIBRARY, or this library's kernel in which every workgroup
# owns whole rows of the result (OWN_ROWS; OWN_ROWS_STAGED: with the left operand staged through LDS; OWN_ROWS_LINES,
# OWN_ROWS_STAGED_LINES: the same two with the weights fetched in whole memory lines; OWN_ROWS_BOTH_STAGED: both
# operands through LDS, for up to 16 rows; OWN_ROWS_SHARED_OUT: for more than 16 rows, the rows of the left operand
# shared out across workgroups too, 16 to each, both operands staged), or the one that splits k across workgroups
# (OWN_KSPLIT).  An own kernel's choice is its variant number + 1.
(LIBRARY, OWN_ROWS, OWN_KSPLIT, OWN_ROWS_STAGED, OWN_ROWS_LINES, OWN_ROWS_STAGED_LINES, OWN_ROWS_BOTH_STAGED,
 OWN_ROWS_SHARED_OUT) = range(8)
BOTH_STAGED_MAX_ROWS = 16
BOTH_STAGED_ANY_ELEMENTS = 16 << 20  # without a measurement: both operands are staged for matrices of this size,
BOTH_STAGED_MIN_K = 2048             # or with rows of at least this many columns where no activation follows
KSPLIT_MIN_ROWS = 17                 # without a measurement: k is split for more than 16 rows
KSPLIT_MIN_K = 2048                  # of at least this many columns (the left operand is then 64 KB and more)
KSPLIT_OVER_LIBRARY_K = 16384        # and for large matrices too, instead of the library, when the rows are this long
STAGED_MIN_ROWS = 4                  # without a measurement: the left operand is staged from this many rows
STAGED_MIN_ELEMENTS = 12 << 10       # and this many elements (4 rows of 3,072 columns, 8 of 1,536)
LINES_MIN_ELEMENTS = 40 << 20        # without a measurement: the weights come in whole lines for matrices of this size
LINES_MIN_K = 16384                  # with rows of at least this many columns (a multiple of 64)


class ProductChoices:
  """Where products of few rows go: a table of timed choices, keyed by (rows point, matrix rows, k, gate|up), over a
  rule, with switches that set the table aside.  An engine owns one and makes it the current one around its steps
  (`with choices:`), so two engines in a process never share timings; code that runs outside any engine (tests,
  tools) uses the module's default table, which starts empty, i.e. by rule.

  force: None, or LIBRARY / an OWN_... constant that every product goes to which can (for tests and measurements);
  rule_only: the table is never consulted; own_only: nothing goes to the library."""

  def __init__(self, rule_only: bool = False):
    self.table: Dict[tuple, int] = {}
    self.rule_only = bool(rule_only)
    self.own_only = False
    self.force: Optional[int] = None
    self.stream_weights = False        # every matrix is read with nontemporal loads (set by the runner, step by step)
    self.library_products = [0, 0]     # (all, avoidable) products that went to the library
    self.off_rule = 0                  # products sent, by measurement, elsewhere than the rule would have
    self._outer: List["ProductChoices"] = []

  def __enter__(self):
    self._outer.append(_CURRENT[0])
    _CURRENT[0] = self
    return self

  def __exit__(self, *exc):
    _CURRENT[0] = self._outer.pop()
    return False

  def set(self, rows_point: int, matrix_rows: int, k: int, gate_up: bool, choice) -> None:
    self.table[(rows_point, matrix_rows, k, bool(gate_up))] = int(choice)

  def known(self, matrix_rows: int, k: int, gate_up: bool) -> bool:
    return all((p, matrix_rows, k, bool(gate_up)) in self.table for p in TUNE_ROWS)

  def clear(self) -> None:
    self.table.clear()

  def measured(self, num_rows: int, matrix_rows: int, k: int, gate_up: bool) -> Optional[int]:
    if self.force is not None:
      can_split = not (gate_up and (matrix_rows // 2) % 4)
      if self.force == OWN_KSPLIT and not can_split:
        return OWN_ROWS
      if self.force == OWN_ROWS_BOTH_STAGED and not (num_rows <= BOTH_STAGED_MAX_ROWS and k % 32 == 0):
        return OWN_ROWS
      if self.force == OWN_ROWS_SHARED_OUT and k % 32:
        return OWN_ROWS
      if self.force in (OWN_ROWS_LINES, OWN_ROWS_STAGED_LINES) and k % 64:
        return OWN_ROWS
      return self.force
    if self.table and not self.rule_only:
      for p in TUNE_ROWS:
        if p >= num_rows:
          return self.table.get((p, matrix_rows, k, bool(gate_up)))
    return None


_DEFAULT_CHOICES = ProductChoices()
_CURRENT: List[ProductChoices] = [_DEFAULT_CHOICES]


def current_choices() -> ProductChoices:
  return _CURRENT[0]


def set_product_choice(rows_point: int, matrix_rows: int, k: int, gate_up: bool, choice) -> None:
  """In the current table.  choice: LIBRARY or one of the OWN_... constants (False and True stand for LIBRARY and
  OWN_ROWS)."""
  _CURRENT[0].set(rows_point, matrix_rows, k, gate_up, choice)


def product_choice_known(matrix_rows: int, k: int, gate_up: bool) -> bool:
  return _CURRENT[0].known(matrix_rows, k, gate_up)


def clear_product_choices() -> None:
  _CURRENT[0].clear()


_COMPUTE_UNITS: Dict[int, int] = {}


def compute_units(device=None) -> int:
  """Compute units of the device (256 on an MI355X, which is also what is assumed where there is no GPU to ask, as in
  host-only tests of the launch rules).  The launch rules derive from it how many workgroups or waves fill the chip."""
  if not torch.cuda.is_available():
    return 256
  index = torch.device(device).index if device is not None else None
  if index is None:
    index = torch.cuda.current_device()
  if index not in _COMPUTE_UNITS:
    _COMPUTE_UNITS[index] = int(torch.cuda.get_device_properties(index).multi_processor_count) or 256
  return _COMPUTE_UNITS[index]


_SIDE_STREAMS: Dict[int, "torch.cuda.Stream"] = {}


def side_stream(device=None) -> "torch.cuda.Stream":
  """One stream per device beside the current one, for warm-up runs before a graph capture.  It is made once:
  every further stream a process has used has cost later decode steps time here (a step of 32 requests ran 10%
  slower after eight streams had been used once), so nothing in this package makes streams freely."""
  index = torch.device(device).index if device is not None else None
  if index is None:
    index = torch.cuda.current_device()
  if index not in _SIDE_STREAMS:
    _SIDE_STREAMS[index] = torch.cuda.Stream(device=index)
  return _SIDE_STREAMS[index]


class own_products_only:
  """While active, `skinny_preferred` sends every product of up to SKINNY_MAX_ROWS rows to this library's kernel."""

  def __enter__(self):
    self.table = _CURRENT[0]
    self.was, self.table.own_only = self.table.own_only, True
    return self

  def __exit__(self, *exc):
    self.table.own_only = self.was
    return False


class rule_products_only:
  """While active, measurements are set aside: every product of few rows goes where the rule sends it."""

  def __enter__(self):
    self.table = _CURRENT[0]
    self.was, self.table.rule_only = self.table.rule_only, True
    return self

  def __exit__(self, *exc):
    self.table.rule_only = self.was
    return False


def off_rule_products_run() -> int:
  """How many products have so far been sent, by measurement, elsewhere than the rule would have sent them."""
  return _CURRENT[0].off_rule


def library_products_run() -> Tuple[int, int]:
  """(all, avoidable): how many products have gone to the library so far, and how many of them this library's
  weight-streaming kernel could have run instead (`linear` counts them with `note_library_product`)."""
  c = _CURRENT[0]
  return c.library_products[0], c.library_products[1]


def note_library_product(avoidable: bool = False) -> None:
  c = _CURRENT[0]
  c.library_products[0] += 1
  if avoidable:
    c.library_products[1] += 1


def skinny_preferred(num_rows: int, matrix_rows: int, k: int, gate_up: bool = False) -> bool:
  """Whether a product of `num_rows` rows with a [matrix_rows, k] matrix (a fused gate|up matrix counts its 2 I
  rows) goes to `gemm_skinny` rather than to the library: what `tuning.tune_products` measured for this shape at
  the next row count of TUNE_ROWS, else a rule.  The rule: each wave of that kernel reads the left operand's rows
  for its own slice of k again, so beyond 16 rows its loads are mostly left operand; on matrices of tens of MB the
  library's kernels (which split k across workgroups) then stream the weights about twice as fast, which
  outweighs the norm and activation kernels that fusing saved."""
  if num_rows > SKINNY_MAX_ROWS:
    return False
  cur = _CURRENT[0]
  if cur.own_only:
    return True
  c = cur.measured(num_rows, matrix_rows, k, gate_up)
  rule = rule_choice(num_rows, matrix_rows, k, gate_up)
  if c is not None:
    if c != rule:
      cur.off_rule += 1
    return c != LIBRARY
  return rule != LIBRARY


def _measured_choice(num_rows: int, matrix_rows: int, k: int, gate_up: bool) -> Optional[int]:
  return _CURRENT[0].measured(num_rows, matrix_rows, k, gate_up)


def skinny_variant(num_rows: int, matrix_rows: int, k: int, gate_up: bool = False) -> int:
  """Which of this library's kernels runs a product that `skinny_preferred` keeps: 0 = every workgroup owns whole
  rows of the result and reads the whole left operand (which is what its time grows with beyond 16 rows); 2 = the
  same with the left operand staged through LDS (read in whole memory lines, which costs a little when the operand
  is small and saves much when it is not; the same sums bit for bit); 3, 4 = 0 and 2 with the weights fetched in
  whole memory lines too (two steps of k at a time, put in place by an exchange between lanes: large matrices
  stream faster that way); 5 = both operands staged through LDS, every request for whole lines (up to 16 rows;
  the same sums as 0 bit for bit); 1 = k is split across workgroups, which read a slice of the left operand each and
  leave 32-bit partial results that a second kernel adds in a fixed order; 6 = for more than 16 rows, the rows of the
  left operand are shared out across workgroups too, 16 to each (see `shared_out_offered`).
  Measured where `tuning.tune_products` has been; else by rule."""
  c = _measured_choice(num_rows, matrix_rows, k, gate_up)
  can_split = not (gate_up and (matrix_rows // 2) % 4)
  if c is not None and c != LIBRARY and (c != OWN_KSPLIT or can_split):
    return c - 1
  return _rule_variant(num_rows, matrix_rows, k, gate_up)


SHARED_OUT_MAX_WORKGROUPS_PER_UNIT = 1.5   # without a measurement: the rows of the left operand are shared out while
                                           # (row blocks of the matrix) x (blocks of 16 rows) stay within this


def shared_out_offered(num_rows: int, matrix_rows: int, k: int, gate_up: bool) -> bool:
  """Whether the form that shares out the rows of the left operand too is a candidate: more than 16 rows, and so few
  rows of the matrix that whole blocks of 16 of them leave compute units idle (a [1024, 2048] matrix at 64 rows: 64
  workgroups otherwise; 5.0 us this way against 7.9 with the left operand staged, 8.4 with k split and 8.3 in the
  library; [1024, 3072]: 5.9 against 10.4, 9.5 and 10.0).  Every workgroup reads its rows of the matrix once per
  block of 16 rows, out of its XCD's L2, so matrices of many rows gain nothing ([4096, 1024] at 64 rows: 6.5 against
  6.4) and a gate|up matrix loses (9.8 against 7.9)."""
  if num_rows <= 16 or k % 32 or gate_up:
    return False
  groups = -(-matrix_rows // 16) * -(-num_rows // 16)
  return groups <= SHARED_OUT_MAX_WORKGROUPS_PER_UNIT * compute_units()


def _rule_variant(num_rows: int, matrix_rows: int, k: int, gate_up: bool) -> int:
  can_split = not (gate_up and (matrix_rows // 2) % 4)
  if shared_out_offered(num_rows, matrix_rows, k, gate_up):
    return 6
  if can_split and num_rows >= KSPLIT_MIN_ROWS and k >= KSPLIT_MIN_K:
    return 1
  large = matrix_rows * k >= LINES_MIN_ELEMENTS
  if num_rows >= STAGED_MIN_ROWS and large and k >= LINES_MIN_K and k % 64 == 0 and not gate_up:
    return 4
  if both_staged_offered(num_rows, matrix_rows, k, gate_up):
    return 5
  # (a matrix of very many rows, the output head, has as many workgroups re-reading the left operand: staged too)
  if num_rows >= STAGED_MIN_ROWS and (num_rows * k >= STAGED_MIN_ELEMENTS or large):
    return 2
  return 0


def both_staged_offered(num_rows: int, matrix_rows: int, k: int, gate_up: bool) -> bool:
  """Whether the form with both operands staged through LDS is a candidate.  A small gate|up matrix, or one with
  short rows, is none: timed alone it is as quick or quicker that way, but inside a decode step (Qwen3-0.6B's
  [4096, 1024] and gate|up [6144, 1024], 1 to 16 rows) the step takes a quarter of a microsecond more per product."""
  return (num_rows <= BOTH_STAGED_MAX_ROWS and k % 32 == 0
          and (matrix_rows * k >= BOTH_STAGED_ANY_ELEMENTS or (not gate_up and k >= BOTH_STAGED_MIN_K)))


def rule_choice(num_rows: int, matrix_rows: int, k: int, gate_up: bool = False) -> int:
  """What runs a product of up to SKINNY_MAX_ROWS rows when nothing has been measured: LIBRARY, or an OWN_... kernel."""
  if num_rows <= SKINNY_OWN_ROWS or matrix_rows * k < SKINNY_OWN_ELEMENTS:
    return _rule_variant(num_rows, matrix_rows, k, gate_up) + 1
  # more than 16 rows of a large matrix: the library, but for very long rows (its kernels split k too little for
  # them: [5120, 25600] at 64 rows 168 us against 81 with k split here; at 12,288 columns and 32 rows the library
  # is still the quicker one inside a step)
  if k >= KSPLIT_OVER_LIBRARY_K and not (gate_up and (matrix_rows // 2) % 4):
    return OWN_KSPLIT
  return LIBRARY


_KSPLIT_SCRATCH: Dict[tuple, torch.Tensor] = {}


def _ksplit_scratch(device, floats: int) -> torch.Tensor:
  """Partial results of the k-split kernel.  Buffers are kept for good, one per device and size class: a captured
  step holds the address of the one it was recorded with."""
  size = max(1 << 16, 1 << (int(floats) - 1).bit_length())
  key = (torch.device(device).index, size)
  t = _KSPLIT_SCRATCH.get(key)
  if t is None:
    t = torch.empty(size, dtype=torch.float32, device=device)
    _KSPLIT_SCRATCH[key] = t
  return t


_SKINNY_PLANS: Dict[tuple, Tuple[int, int]] = {}


def _skinny_plan(lib, variant: int, gate_up: bool, M: int, N: int, K: int) -> Tuple[int, int]:
  """(rows of the table of partial sums of squares, floats of scratch) of a launch of the chosen kernel."""
  key = (variant, bool(gate_up), M, N, K)
  plan = _SKINNY_PLANS.get(key)
  if plan is None:
    parts, floats = ctypes.c_int(0), ctypes.c_int64(0)
    _check(lib, lib.mi_gemm_skinny_plan(variant, 1 if gate_up else 0, M, N, K, ctypes.byref(parts),
                                        ctypes.byref(floats)))
    plan = _SKINNY_PLANS[key] = (parts.value, floats.value)
  return plan


def gemm_skinny_supported(a: torch.Tensor, w: torch.Tensor) -> bool:
  K = w.shape[1]
  return (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and a.shape[0] <= SKINNY_MAX_ROWS and K % 8 == 0
          and a.stride(1) == 1 and w.stride(1) == 1 and (a.shape[0] <= 1 or a.stride(0) % 8 == 0)
          and (w.shape[0] <= 1 or w.stride(0) % 8 == 0) and a.shape[1] == K
          and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


def _skinny_call(lib, variant: int, out_f32: bool, gate_up: bool, a, w, c_ptr, ldc: int, M: int, N: int, K: int,
                 row_ss=None, eps: float = 0.0, residual=None, norm_weight=None, a_out=None, ss_out=None) -> None:
  scratch, floats = None, 0
  if variant == 1:
    _, floats = _skinny_plan(lib, 1, gate_up, M, N, K)
    scratch = _ksplit_scratch(a.device, floats)
  _check(lib, lib.mi_gemm_skinny_v(variant, 1 if out_f32 else 0, 1 if gate_up else 0, _ptr(a),
                                   a.stride(0) if M > 1 else a.shape[1], _ptr(w), w.stride(0), c_ptr, ldc, M, N, K,
                                   _ptr(row_ss), row_ss.shape[0] if row_ss is not None else 0, float(eps),
                                   _ptr(residual), _ptr(norm_weight), _ptr(a_out), _ptr(ss_out), _ptr(scratch),
                                   scratch.numel() if scratch is not None else 0, _stream()))


def gemm_skinny(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, gate_up: bool = False,
                variant: Optional[int] = None) -> torch.Tensor:
  """out[M, N] = a[M, K] @ w[N, K]^T on the matrix cores for M <= 64 rows, bfloat16 operands, bfloat16 or float32
  result.  With `gate_up`, w is a fused gate|up matrix [2 N, K] (gate rows first) and
  out = silu(a @ w_gate^T) * (a @ w_up^T), made from the 32-bit sums.  variant: see `skinny_variant` (default: its
  answer for this shape)."""
  _dev(a, w, out)
  if not gemm_skinny_supported(a, w):
    raise KernelError(f"gemm_skinny does not take a {tuple(a.shape)} {a.dtype}, w {tuple(w.shape)} {w.dtype}")
  M = a.shape[0]
  N, K = w.shape
  if gate_up:
    if N % 2:
      raise KernelError("gemm_skinny: a gate|up matrix has an even number of rows")
    N //= 2
  if tuple(out.shape) != (M, N) or out.stride(1) != 1 or out.dtype not in (torch.bfloat16, torch.float32):
    raise KernelError(f"gemm_skinny: out {tuple(out.shape)} {out.dtype} does not fit [{M}, {N}]")
  lib = _skinny_lib(w)
  if variant is None:
    variant = skinny_variant(M, w.shape[0], K, gate_up)
  _skinny_call(lib, variant, out.dtype == torch.float32, gate_up, a, w, _ptr(out), out.stride(0) if M > 1 else N,
               M, N, K)
  return out


# A matrix from this size on is read with nontemporal loads (a build of the kernels of its own): it is read once a
# step and is larger than what the caches keep from one step to the next, so all it does there is push out what
# could stay.  Measured on an MI355X, 8 rows: [151936, 1024] 56.4 -> 50.5 us, [151936, 4096] 213 -> 190,
# gate|up [24576, 4096] 35.9 -> 31.9, [4096, 12288] 22.4 -> 20.4, gate|up [12288, 2048] 13.9 -> 12.9; matrices of
# 34 MB and less lose (gate|up [6144, 1024] 5.4 -> 5.6, [4096, 4096] 8.5 -> 8.6, [8192, 2048] 9.8 -> 10.0).
STREAMED_MATRIX_MIN_BYTES = 48 << 20

# The last-level cache of an MI355X (256 MB) keeps the keys and values of a step for the next one if they fit and the
# weights, which never do, are kept out of it: the current table's `stream_weights` then sends every matrix to the
# nontemporal build.  Whole decode steps of the 0.6B shape, all weights nontemporal against only the large ones: one
# request of 1,024 tokens (117 MB of keys and values in all layers) 0.992 against 1.036 ms, 2,048 tokens (235 MB) 1.010
# against 1.050, 3,000 (344 MB) 1.035 against 1.050, 4,000 (459 MB) 1.066 against 1.050, 8,192 1.200 against 1.194;
# 2 x 1,024 / 4 x 512 / 8 x 256 tokens 1.008 / 1.035 / 1.074 against 1.051 / 1.064 / 1.092; 2 x 2,048 1.077 against 1.067.
# A step's count of cached tokens is an upper bound (decode graphs are made for tables of up to twice the pages in
# use), so weights are streamed while the bound stays within twice the cache.
LAST_LEVEL_CACHE_BYTES = 256 << 20


def weights_stream_past_cache(cached_bytes_bound: int) -> bool:
  """Whether a step that reads at most `cached_bytes_bound` bytes of keys and values (all layers) should keep its
  weights out of the last-level cache, so that those keys and values are still there at the next step."""
  return 0 < cached_bytes_bound <= 2 * LAST_LEVEL_CACHE_BYTES


def _skinny_lib(w: torch.Tensor):
  if w.numel() * w.element_size() >= STREAMED_MATRIX_MIN_BYTES or _CURRENT[0].stream_weights:
    return _lib("gemm_skinny", (("SKINNY_NT", 1),))
  return _lib("gemm_skinny")


def gemm_skinny_waves(variant: int, num_rows: int, matrix_rows: int, k: int, gate_up: bool = False) -> int:
  """Waves per workgroup of `gemm_skinny` in a form that owns whole rows of the result (variant 0, 2 to 5); the waves
  share out k, so forms with the same number add the same products in the same order."""
  n = matrix_rows // 2 if gate_up else matrix_rows
  return int(_lib("gemm_skinny").mi_gemm_skinny_waves(variant, 1 if gate_up else 0, num_rows, n, k))


def gemm_skinny_scaled(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, row_ss: torch.Tensor, eps: float,
                       gate_up: bool = False, variant: Optional[int] = None) -> torch.Tensor:
  """`gemm_skinny` whose rows are scaled by rsqrt(sum_p row_ss[p, m] / K + eps) before they are stored (and, with
  `gate_up`, before the activation): the second half of an RMS norm whose first half `gemm_skinny_into_norm` did.
  row_ss float32 [parts, 16] for up to 16 rows, [parts, 64] for more."""
  _dev(a, w, out, row_ss)
  if not gemm_skinny_supported(a, w):
    raise KernelError(f"gemm_skinny does not take a {tuple(a.shape)} {a.dtype}, w {tuple(w.shape)} {w.dtype}")
  M = a.shape[0]
  N, K = w.shape
  if gate_up:
    if N % 2:
      raise KernelError("gemm_skinny: a gate|up matrix has an even number of rows")
    N //= 2
  if tuple(out.shape) != (M, N) or out.stride(1) != 1 or out.dtype not in (torch.bfloat16, torch.float32):
    raise KernelError(f"gemm_skinny: out {tuple(out.shape)} {out.dtype} does not fit [{M}, {N}]")
  lib = _skinny_lib(w)
  ss_row = lib.mi_gemm_skinny_ss_row(M)
  if row_ss.dtype != torch.float32 or row_ss.dim() != 2 or row_ss.shape[1] != ss_row or not row_ss.is_contiguous():
    raise KernelError(f"gemm_skinny_scaled: row_ss must be a contiguous float32 [parts, {ss_row}] for {M} rows")
  if variant is None:
    variant = skinny_variant(M, w.shape[0], K, gate_up)
  _skinny_call(lib, variant, out.dtype == torch.float32, gate_up, a, w, _ptr(out), out.stride(0) if M > 1 else N,
               M, N, K, row_ss=row_ss, eps=eps)
  return out


def gemm_skinny_into_norm_supported(a: torch.Tensor, w: torch.Tensor, residual: torch.Tensor,
                                    norm_weight: torch.Tensor) -> bool:
  N = w.shape[0]
  return (gemm_skinny_supported(a, w) and residual.dtype == torch.float32 and residual.is_contiguous()
          and tuple(residual.shape) == (a.shape[0], N) and norm_weight.dtype == torch.float32
          and norm_weight.numel() == N and norm_weight.is_contiguous())


def gemm_skinny_into_norm(a: torch.Tensor, w: torch.Tensor, residual: torch.Tensor, norm_weight: torch.Tensor,
                          variant: Optional[int] = None):
  """residual += a @ w^T (in place, 32-bit), and the first half of the RMS norm of the new residual: returns
  (operand, row_ss) with operand[m, n] = bfloat16(residual[m, n] * norm_weight[n]) and row_ss float32 [parts, 16 or 64],
  the sum of squares of row m over each workgroup's columns.  `gemm_skinny_scaled` finishes the norm."""
  _dev(a, w, residual, norm_weight)
  if not gemm_skinny_into_norm_supported(a, w, residual, norm_weight):
    raise KernelError("gemm_skinny_into_norm does not take these operands")
  M = a.shape[0]
  N, K = w.shape
  lib = _skinny_lib(w)
  if variant is None:
    variant = skinny_variant(M, N, K)
  parts, _ = _skinny_plan(lib, variant, False, M, N, K)
  operand = torch.empty((M, N), dtype=torch.bfloat16, device=a.device)
  row_ss = torch.empty((parts, lib.mi_gemm_skinny_ss_row(M)), dtype=torch.float32, device=a.device)
  _skinny_call(lib, variant, False, False, a, w, None, N, M, N, K, residual=residual, norm_weight=norm_weight,
               a_out=operand, ss_out=row_ss)
  return operand, row_ss


NORM_GEMM_MAX_ROWS = 16


def norm_gemm_supported(num_rows: int, residual: torch.Tensor, x: Optional[torch.Tensor], w: torch.Tensor) -> bool:
  K = w.shape[1]
  return (w.dtype == torch.bfloat16 and num_rows <= NORM_GEMM_MAX_ROWS and K % 8 == 0 and residual.shape[-1] == K
          and residual.dtype == torch.float32 and residual.is_contiguous() and w.stride(1) == 1
          and w.stride(0) % 8 == 0 and w.data_ptr() % 16 == 0 and residual.data_ptr() % 16 == 0
          and (x is None or (x.dtype == torch.bfloat16 and x.is_contiguous() and x.shape == residual.shape
                             and x.data_ptr() % 16 == 0)))


def norm_gemm_skinny(residual: torch.Tensor, x: Optional[torch.Tensor], norm_weight: torch.Tensor, eps: float,
                     w: torch.Tensor, out: torch.Tensor, residual_out: Optional[torch.Tensor] = None,
                     rows: Optional[torch.Tensor] = None, gate_up: bool = False) -> torch.Tensor:
  """For up to 16 rows, in one kernel: r' = residual + x (x may be None); out = (rmsnorm(r') * norm_weight) @ w^T,
  or with `gate_up` silu(.. @ w_gate^T) * (.. @ w_up^T) for a fused gate|up matrix.  r' is written to
  `residual_out` (another buffer than `residual`) when given.  `rows` picks rows of residual and x instead."""
  _dev(residual, x, norm_weight, w, out, residual_out, rows)
  M = rows.numel() if rows is not None else residual.shape[0]
  if not norm_gemm_supported(M, residual, x, w):
    raise KernelError("norm_gemm_skinny does not take these operands")
  N, K = w.shape
  if gate_up:
    N //= 2
  _f32("norm_weight", norm_weight, K)
  _i32("rows", rows)
  if tuple(out.shape) != (M, N) or out.dtype != torch.bfloat16 or not out.is_contiguous():
    raise KernelError(f"norm_gemm_skinny: out {tuple(out.shape)} {out.dtype} does not fit [{M}, {N}] bfloat16")
  if residual_out is not None:
    if rows is not None or residual_out.shape != residual.shape or residual_out.dtype != torch.float32 \
        or not residual_out.is_contiguous() or residual_out.data_ptr() == residual.data_ptr():
      raise KernelError("norm_gemm_skinny: residual_out must be another float32 buffer of the residual's shape")
  lib = _skinny_lib(w)
  _check(lib, lib.mi_norm_gemm_skinny(1 if gate_up else 0, _ptr(residual), _ptr(x), _ptr(residual_out),
                                      _ptr(norm_weight), _ptr(rows), float(eps), _ptr(w), w.stride(0), _ptr(out), N,
                                      M, N, K, _stream()))
  return out


# ----------------------------------------------------------------------------- attention

def paged_attention(q: torch.Tensor, nq: int, nkv: int, d: int, out: torch.Tensor, k_pages: torch.Tensor,
                    v_pages: torch.Tensor, block_table: torch.Tensor, token_req: torch.Tensor, cu_q: torch.Tensor,
                    kv_len: torch.Tensor, scale: float, window: int = 0, num_splits: int = 1,
                    part_o: Optional[torch.Tensor] = None, part_ml: Optional[torch.Tensor] = None) -> torch.Tensor:
  """Causal attention of new tokens over their requests' paged keys and values.

  q: [T, >= nq*d] rows (the q part of a fused qkv buffer is fine), out [T, nq*d];
  key pages [num_pages, nkv, P, d], value pages [num_pages, nkv, d, P]; block_table [B, W] int32; token_req [T] = request of each token;
  cu_q [B+1] = first token of each request; kv_len [B] = keys per request including the new tokens.
  num_splits > 1 cuts every token's keys into that many parts that run side by side (for few tokens over many
  keys); then part_o float32 [>= T * nq * num_splits * d] and part_ml float32 [>= T * nq * num_splits * 2] are
  scratch."""
  _dev(q, out, k_pages, v_pages, block_table, token_req, cu_q, kv_len)
  T = q.shape[0]
  if num_splits > 1:
    need = T * nq * num_splits
    if part_o is None or part_ml is None or part_o.dtype != torch.float32 or part_ml.dtype != torch.float32 or \
        part_o.numel() < need * d or part_ml.numel() < need * 2:
      raise KernelError("paged_attention: partial buffers are missing, too small or not float32")
    _dev(part_o, part_ml)
  B = kv_len.numel()
  if q.stride(1) != 1 or q.shape[1] < nq * d or out.stride(1) != 1 or out.shape != (T, nq * d):
    raise KernelError(f"paged_attention: q {tuple(q.shape)} / out {tuple(out.shape)} do not hold {nq} heads of {d}")
  _check_pages("paged_attention", k_pages, v_pages, nkv, d, q.dtype)
  if q.dtype != out.dtype:
    raise KernelError("paged_attention: q and out must share a dtype")
  _i32("block_table", block_table)
  if block_table.dim() != 2 or block_table.shape[0] < B:
    raise KernelError(f"paged_attention: block_table {tuple(block_table.shape)} for {B} requests")
  _i32("token_req", token_req, T)
  _i32("cu_q", cu_q, B + 1)
  _i32("kv_len", kv_len, B)
  lib = _lib("attention")
  _check(lib, lib.mi_paged_attention(dtype_code(q.dtype), _ptr(q), q.stride(0), _ptr(out), out.stride(0),
                                     _ptr(k_pages), _ptr(v_pages), _ptr(block_table), block_table.shape[1],
                                     _ptr(token_req), _ptr(cu_q), _ptr(kv_len), T, B, nq, nkv, d,
                                     k_pages.shape[2], float(scale), int(window), int(num_splits),
                                     _ptr(part_o) if num_splits > 1 else None,
                                     _ptr(part_ml) if num_splits > 1 else None, _stream()))
  return out


# ----------------------------------------------------------------------------- sampling

def sample(logits: torch.Tensor, temperature: Optional[torch.Tensor], top_k: Optional[torch.Tensor],
           top_p: Optional[torch.Tensor], seeds: Optional[torch.Tensor], steps: Optional[torch.Tensor],
           out: torch.Tensor) -> torch.Tensor:
  """out[r] = next token of row r of float32 logits [R, V].  temperature[r] == 0 (or no temperatures) is
  argmax with the lowest index winning ties; otherwise a draw from softmax(logits / temperature), limited to
  the top_k[r] most probable tokens (0 = all) and then to the top_p[r] mass (1 = all), from the counter-based
  generator keyed by (seeds[r], steps[r], token index)."""
  _dev(logits, temperature, top_k, top_p, seeds, steps, out)
  if logits.dim() != 2 or logits.dtype != torch.float32 or logits.stride(1) != 1:
    raise KernelError("sample: logits must be float32 [R, V] with dense rows")
  R, V = logits.shape
  _f32("temperature", temperature, R)
  _i32("top_k", top_k, R)
  _f32("top_p", top_p, R)
  for name, t in (("seeds", seeds), ("steps", steps)):
    if t is not None and (t.dtype != torch.int64 or t.numel() != R or not t.is_contiguous()):
      raise KernelError(f"sample: {name} must be int64 [R]")
  _i32("out", out, R)
  lib = _lib("sampling")
  if top_k is None and top_p is None:
    # greedy and plain temperature rows: the vocabulary is searched in parts by many workgroups
    nparts = lib.mi_sample_parts_count(V)
    part_val = torch.empty(R * nparts, dtype=torch.float32, device=logits.device)
    part_idx = torch.empty(R * nparts, dtype=torch.int32, device=logits.device)
    _check(lib, lib.mi_sample_simple(_ptr(logits), logits.stride(0) if R > 1 else V, R, V, _ptr(temperature),
                                     _ptr(seeds), _ptr(steps), _ptr(part_val), _ptr(part_idx), _ptr(out), _stream()))
    return out
  _check(lib, lib.mi_sample(_ptr(logits), logits.stride(0) if R > 1 else V, R, V, _ptr(temperature), _ptr(top_k),
                            _ptr(top_p), _ptr(seeds), _ptr(steps), _ptr(out), _stream()))
  return out


def plain_attention_geometry(dtype: torch.dtype, nq: int, nkv: int, d: int, page_size: int) -> Tuple[int, int]:
  """(query heads one wave of the plain kernel takes, waves that are resident on a compute unit at once) for these
  sizes, as `mi_paged_attention` launches them: 32-bit caches with head sizes 64, 80, 96 or 128 and pages of 16 keys
  or more go to the kernel with four lanes a key, which holds a whole tile's loads in registers (8 waves a unit, up
  to 4 heads a wave); everything else to the kernel with one key a lane (16 waves, up to 8 heads)."""
  per_kv = nq // nkv
  quad = dtype == torch.float32 and d in (64, 80, 96, 128) and page_size >= 16
  rep = per_kv if per_kv in (2, 4, 8) else 1
  if quad and rep == 8:
    rep = 4
  return rep, (8 if quad else 16)


# ----------------------------------------------------------------------------- attention on the matrix cores

def mfma_attention_supported(dtype: torch.dtype, nq: int, nkv: int, d: int, page_size: int) -> bool:
  """The MFMA attention kernels take bfloat16, head sizes that are multiples of 16 up to 256, up to 16 query
  heads per kv head, and pages of at least 8 tokens; everything else runs on the plain kernel."""
  return (dtype == torch.bfloat16 and d % 16 == 0 and 16 <= d <= 256 and nq % nkv == 0 and nq // nkv <= 16
          and page_size >= 8)


def attn_prefill_tokens_per_block(nq: int, nkv: int, d: int, wide: bool = False) -> int:
  """Query tokens one work item of the prefill launch takes (the granule of its work list).  wide: of the variant
  "wide", whose waves take two blocks of query columns (0 where the head size has no such instance)."""
  lib = _lib("attention_mfma", (("HEAD_DIM", d),))
  return lib.mi_attn_prefill_tokens_per_block_wide(nq, nkv) if wide else lib.mi_attn_prefill_tokens_per_block(nq, nkv)


PREFILL_WIDE_WORKGROUPS_PER_UNIT = 4   # from this many workgroups for every compute unit on, the "wide" prefill variant pays


def attn_prefill_wide_pays(q_lens, nq: int, nkv: int, d: int) -> int:
  """The work granule of the "wide" prefill variant if the step's prompt portions make workgroups enough for it
  (long prompts: 672 against 619 TFLOP/s at 8,192 tokens, 789 against 665 at 32,768), else 0."""
  tpb = attn_prefill_tokens_per_block(nq, nkv, d, wide=True)
  if tpb <= 0:
    return 0
  items = sum(-(-n // tpb) for n in q_lens if n > 1)
  return tpb if items * nkv >= PREFILL_WIDE_WORKGROUPS_PER_UNIT * compute_units() else 0


def attn_decode_geometry(d: int, wide: bool = False):
  """(keys per macro tile, waves per workgroup) of the decode kernel for this head size; wide: of its launch with
  workgroups of twice the waves."""
  lib = _lib("attention_mfma", (("HEAD_DIM", d),))
  return lib.mi_attn_macro_tile_keys(), (lib.mi_attn_decode_waves_wide() if wide else lib.mi_attn_decode_waves())


def _attn_common(what, q, out, nq, nkv, d, k_pages, v_pages, block_table, cu_q, kv_len):
  _dev(q, out, k_pages, v_pages, block_table, cu_q, kv_len)
  T = q.shape[0]
  if q.dtype != torch.bfloat16 or out.dtype != torch.bfloat16:
    raise KernelError(f"{what}: bfloat16 only")
  if q.stride(1) != 1 or q.shape[1] < nq * d or out.stride(1) != 1 or tuple(out.shape) != (T, nq * d):
    raise KernelError(f"{what}: q {tuple(q.shape)} / out {tuple(out.shape)} do not hold {nq} heads of {d}")
  _check_pages(what, k_pages, v_pages, nkv, d, q.dtype)
  _i32("block_table", block_table)
  B = kv_len.numel()
  if block_table.dim() != 2 or block_table.shape[0] < B:
    raise KernelError(f"{what}: block_table {tuple(block_table.shape)} for {B} requests")
  _i32("cu_q", cu_q, B + 1)
  _i32("kv_len", kv_len, B)
  return B


_PREFILL_VARIANTS = {"auto": 0, "two_tiles": 1, "dense": 2, "wide": 3}


def attn_prefill(q: torch.Tensor, nq: int, nkv: int, d: int, out: torch.Tensor, k_pages: torch.Tensor,
                 v_pages: torch.Tensor, block_table: torch.Tensor, work: torch.Tensor, cu_q: torch.Tensor,
                 kv_len: torch.Tensor, scale: float, window: int = 0, variant: str = "auto") -> None:
  """MFMA attention of the entries named in `work` [n, 2] = (entry, block of `attn_prefill_tokens_per_block` query
  tokens within it).  Other arguments as `paged_attention`.  variant: "auto" (by the number of work items),
  "two_tiles" (8 waves a workgroup, for few work items), "dense" (4 waves, three waves a SIMD) or "wide" (4 waves
  with two blocks of query columns each, for long prompts; its work items count
  `attn_prefill_tokens_per_block(.., wide=True)` tokens)."""
  if variant not in _PREFILL_VARIANTS:
    raise KernelError(f"attn_prefill: variant {variant!r}; known: {sorted(_PREFILL_VARIANTS)}")
  _attn_common("attn_prefill", q, out, nq, nkv, d, k_pages, v_pages, block_table, cu_q, kv_len)
  _dev(work)
  _i32("work", work)
  if work.dim() != 2 or work.shape[1] != 2:
    raise KernelError("attn_prefill: work must be [n, 2]")
  lib = _lib("attention_mfma", (("HEAD_DIM", d),))
  _check(lib, lib.mi_attn_prefill(_ptr(q), q.stride(0), _ptr(out), out.stride(0), _ptr(k_pages), _ptr(v_pages),
                                  _ptr(block_table), block_table.shape[1], _ptr(work), work.shape[0], _ptr(cu_q),
                                  _ptr(kv_len), nq, nkv, k_pages.shape[2], float(scale), int(window),
                                  _PREFILL_VARIANTS[variant], _stream()))


# A decode launch whose keys and values may come to this many bytes reads them with nontemporal loads: they are read
# once a step and, with the weights, are many times what the caches hold, so ordinary loads only push out what could
# stay.  Whole decode steps of the 0.6B shape (28 layers) at 2,048 tokens, nontemporal against ordinary loads: 8
# requests (67 MB a layer) 1.325 against 1.304 ms, 16 the same, 24 (201 MB) 2.239 against 2.209, 32 (268 MB) 2.423
# against 2.517, 48 3.172 against 3.335, 64 (537 MB) 3.68 against 4.08; one layer of 8 requests of 32,768 tokens
# (1.07 GB) 178 against 194 us.  The caller's count of keys is an upper bound (a decode graph is made for tables of up
# to twice the pages in use), hence a threshold of twice the size from which streaming pays.
DECODE_STREAM_MIN_BYTES = 512 << 20


def decode_streams_keys(num_entries: int, nkv: int, d: int, max_keys: int, element_size: int = 2) -> bool:
  """Whether a decode attention launch over `num_entries` requests of up to `max_keys` keys should stream them."""
  return 2 * num_entries * nkv * d * max_keys * element_size >= DECODE_STREAM_MIN_BYTES


def attn_decode(q: torch.Tensor, nq: int, nkv: int, d: int, out: torch.Tensor, k_pages: torch.Tensor,
                v_pages: torch.Tensor, block_table: torch.Tensor, cu_q: torch.Tensor, kv_len: torch.Tensor,
                first_entry: int, num_entries: int, num_splits: int, part_o: torch.Tensor, part_ml: torch.Tensor,
                scale: float, window: int = 0, stream_keys: bool = False, wide: bool = False) -> None:
  """MFMA split-key attention of entries first_entry .. first_entry + num_entries - 1, each of which brings exactly
  one token.  part_o float32 [>= num_entries * nq * num_splits * d], part_ml float32 [>= num_entries * nq *
  num_splits * 2] are scratch.  stream_keys: read the keys and values with nontemporal loads (`decode_streams_keys`);
  wide: workgroups of twice the waves (`attn_decode_geometry(d, wide=True)`; see `decode_launch` of the attention part)."""
  B = _attn_common("attn_decode", q, out, nq, nkv, d, k_pages, v_pages, block_table, cu_q, kv_len)
  if first_entry < 0 or num_entries < 0 or first_entry + num_entries > B:
    raise KernelError(f"attn_decode: entries {first_entry}..{first_entry + num_entries} of {B}")
  _dev(part_o, part_ml)
  need = num_entries * nq * num_splits
  if part_o.dtype != torch.float32 or part_o.numel() < need * d or part_ml.dtype != torch.float32 \
      or part_ml.numel() < need * 2 or not part_o.is_contiguous() or not part_ml.is_contiguous():
    raise KernelError("attn_decode: partial buffers are too small or not float32")
  lib = _lib("attention_mfma", (("HEAD_DIM", d),))
  _check(lib, lib.mi_attn_decode(_ptr(q), q.stride(0), _ptr(out), out.stride(0), _ptr(k_pages), _ptr(v_pages),
                                 _ptr(block_table), block_table.shape[1], _ptr(cu_q), _ptr(kv_len), first_entry,
                                 num_entries, num_splits, _ptr(part_o), _ptr(part_ml), nq, nkv, k_pages.shape[2],
                                 float(scale), int(window), 1 if stream_keys else 0, 1 if wide else 0, _stream()))


def attn_decode_front(qkv: torch.Tensor, nq: int, nkv: int, d: int, out: torch.Tensor, k_pages: torch.Tensor,
                      v_pages: torch.Tensor, block_table: torch.Tensor, cu_q: torch.Tensor, kv_len: torch.Tensor,
                      first_entry: int, num_entries: int, num_splits: int, part_o: torch.Tensor,
                      part_ml: torch.Tensor, scale: float, window: int, q_weight: Optional[torch.Tensor],
                      k_weight: Optional[torch.Tensor], eps: float, cos_sin: Optional[torch.Tensor],
                      positions: torch.Tensor, slots: torch.Tensor, stream_keys: bool = False,
                      wide: bool = False) -> None:
  """`attn_decode` for entries whose fused projection qkv [T, (nq + 2 nkv) d] (rows q | k | v) is still raw: the
  kernel does the per-head RMS norm of q and k (if weights), their rotation (if a table [max_pos, rotary_dim]) and
  the write of the new key and value to `slots`, as `qk_norm_rope_cache` would, and attends.  qkv is left as it is.
  A table must rotate whole heads (rotary_dim == d)."""
  B = _attn_common("attn_decode_front", qkv, out, nq, nkv, d, k_pages, v_pages, block_table, cu_q, kv_len)
  T = qkv.shape[0]
  if qkv.shape[1] != (nq + 2 * nkv) * d:
    raise KernelError(f"attn_decode_front: qkv {tuple(qkv.shape)} does not hold {nq}+2*{nkv} heads of {d}")
  if first_entry < 0 or num_entries < 0 or first_entry + num_entries > B:
    raise KernelError(f"attn_decode_front: entries {first_entry}..{first_entry + num_entries} of {B}")
  _dev(part_o, part_ml, q_weight, k_weight, cos_sin, positions, slots)
  need = num_entries * nq * num_splits
  if part_o.dtype != torch.float32 or part_o.numel() < need * d or part_ml.dtype != torch.float32 \
      or part_ml.numel() < need * 2 or not part_o.is_contiguous() or not part_ml.is_contiguous():
    raise KernelError("attn_decode_front: partial buffers are too small or not float32")
  _f32("q_weight", q_weight, d)
  _f32("k_weight", k_weight, d)
  _i32("slots", slots, T)
  rotary_dim, max_pos = 0, 0
  if cos_sin is not None:
    if cos_sin.dtype != torch.float32 or cos_sin.dim() != 2 or not cos_sin.is_contiguous():
      raise KernelError("attn_decode_front: the rotation table must be a contiguous float32 [positions, rotary_dim]")
    max_pos, rotary_dim = cos_sin.shape
    if rotary_dim != d:
      raise KernelError(f"attn_decode_front: rotary_dim {rotary_dim}; this kernel rotates whole heads of {d} only")
    _i32("positions", positions, T)
  lib = _lib("attention_mfma", (("HEAD_DIM", d),))
  _check(lib, lib.mi_attn_decode_front(
    _ptr(qkv), qkv.stride(0), _ptr(out), out.stride(0), _ptr(k_pages), _ptr(v_pages), _ptr(block_table),
    block_table.shape[1], _ptr(cu_q), _ptr(kv_len), first_entry, num_entries, num_splits, _ptr(part_o), _ptr(part_ml),
    nq, nkv, k_pages.shape[2], float(scale), int(window), 1 if stream_keys else 0, 1 if wide else 0, _ptr(q_weight),
    _ptr(k_weight),
    float(eps), _ptr(cos_sin), rotary_dim, max_pos, _ptr(positions), _ptr(slots), _stream()))


# ----------------------------------------------------------------------------- what the device delivers

_MEASURED_PEAKS: Dict[int, Tuple[float, float]] = {}


def measured_peaks(device=None, stream_bytes: int = 1 << 31) -> Tuple[float, float]:
  """(GB/s of a kernel that only reads `stream_bytes` of device memory, TFLOP/s of a kernel that only runs dense
  bfloat16 matrix instructions on registers) on this device: the best of a few runs each, measured once per process
  and device (about 50 ms)."""
  index = torch.device(device).index if device is not None else None
  if index is None:
    index = torch.cuda.current_device()
  if index in _MEASURED_PEAKS:
    return _MEASURED_PEAKS[index]
  lib = _lib("probes")
  dev = torch.device("cuda", index)
  free, _ = torch.cuda.mem_get_info(dev)
  nbytes = max(1 << 24, min(stream_bytes, free // 4) // 16 * 16)
  buf = torch.empty(nbytes, dtype=torch.uint8, device=dev)
  buf.random_(0, 255)
  sink = torch.zeros(4, dtype=torch.float32, device=dev)
  start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
  flops = ctypes.c_double(0.0)
  cus = torch.cuda.get_device_properties(dev).multi_processor_count

  def best_ms(launch, reps):
    launch()
    torch.cuda.synchronize(dev)
    best = float("inf")
    for _ in range(reps):
      start.record()
      launch()
      end.record()
      torch.cuda.synchronize(dev)
      best = min(best, start.elapsed_time(end))
    return best

  with torch.cuda.device(dev):
    ms = best_ms(lambda: _check(lib, lib.mi_probe_stream_read(_ptr(buf), nbytes, _ptr(sink), _stream())), 5)
    gbs = nbytes / ms / 1e6
    ms = best_ms(lambda: _check(lib, lib.mi_probe_mfma(cus * 8, 4096, _ptr(sink), ctypes.byref(flops), _stream())), 3)
    tflops = flops.value / ms / 1e9
  del buf
  torch.cuda.empty_cache()      # the read buffer goes back to the driver: a cache sized from free memory must see it
  _MEASURED_PEAKS[index] = (gbs, tflops)
  return _MEASURED_PEAKS[index]
