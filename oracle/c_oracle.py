"""ctypes wrapper of oracle/libhstu_oracle.so (the plain-C restatement).

TEST INFRASTRUCTURE ONLY; see oracle/hstu_oracle.c.
"""

from __future__ import annotations

import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libhstu_oracle.so")


class OracleArgs(C.Structure):
  _fields_ = [
      ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("out", C.c_void_p),
      ("B", C.c_int), ("L", C.c_int), ("H", C.c_int), ("d_qk", C.c_int), ("d_v", C.c_int),
      ("seq_offsets", C.c_void_p), ("seq_lens", C.c_void_p),
      ("alpha", C.c_float), ("inv_n", C.c_float), ("causal", C.c_int),
      ("pos_tab", C.c_void_p), ("pos_heads", C.c_int),
      ("ts", C.c_void_p), ("ts_stride_b", C.c_int64),
      ("ts_tab", C.c_void_p), ("ts_heads", C.c_int), ("ts_nb", C.c_int),
      ("ts_bucket_size", C.c_float),
  ]


_lib = None


def load():
  global _lib
  if _lib is None:
    if not os.path.exists(LIB_PATH):
      raise RuntimeError(f"{LIB_PATH} is missing: run `make -C oracle`")
    _lib = C.CDLL(LIB_PATH)
    for fn in (_lib.hstu_oracle_fwd_f64, _lib.hstu_oracle_fwd_f32):
      fn.restype = C.c_int
      fn.argtypes = [C.POINTER(OracleArgs), C.c_int]
    _lib.hstu_oracle_max_threads.restype = C.c_int
  return _lib


def max_threads() -> int:
  return load().hstu_oracle_max_threads()


def hstu_attention_c(q, k, v, *, seq_lens=None, seq_offsets=None, max_len=None,
                     n=None, alpha=1.0, causal=True, pos_tab=None,
                     timestamps=None, ts_tab=None, ts_bucket_size=0.301,
                     acc="f64", nthreads=0):
  """Runs the C restatement.  q,k,v fp32 padded [B,L,H,d] or jagged [T,H,d]."""
  lib = load()
  keep = []

  def arr(x, dt):
    a = np.ascontiguousarray(x, dtype=dt)
    keep.append(a)
    return a.ctypes.data

  q = np.ascontiguousarray(q, dtype=np.float32)
  a = OracleArgs()
  if q.ndim == 3:
    T, H, d = q.shape
    off = np.ascontiguousarray(seq_offsets, dtype=np.int32)
    keep.append(off)
    B, L = len(off) - 1, int(max_len)
    a.seq_offsets = off.ctypes.data
  else:
    B, L, H, d = q.shape
    if seq_lens is not None:
      a.seq_lens = arr(seq_lens, np.int32)
  dv = np.shape(v)[-1]
  out = np.empty(q.shape[:-1] + (dv,), dtype=np.float32)
  a.q, a.k, a.v, a.out = arr(q, np.float32), arr(k, np.float32), arr(v, np.float32), out.ctypes.data
  a.B, a.L, a.H, a.d_qk, a.d_v = B, L, H, d, dv
  a.alpha = alpha
  a.inv_n = 1.0 / (L if n is None else n)
  a.causal = 1 if causal else 0
  if pos_tab is not None:
    pt = np.atleast_2d(np.asarray(pos_tab, dtype=np.float32))
    a.pos_tab, a.pos_heads = arr(pt, np.float32), pt.shape[0]
  if ts_tab is not None:
    tt = np.atleast_2d(np.asarray(ts_tab, dtype=np.float32))
    ts = np.asarray(timestamps)
    a.ts_tab, a.ts_heads, a.ts_nb = arr(tt, np.float32), tt.shape[0], tt.shape[1] - 1
    a.ts = arr(ts, np.int64)
    a.ts_stride_b = L if ts.ndim == 2 else 0
    a.ts_bucket_size = ts_bucket_size
  fn = lib.hstu_oracle_fwd_f64 if acc == "f64" else lib.hstu_oracle_fwd_f32
  rc = fn(C.byref(a), int(nthreads))
  if rc != 0:
    raise RuntimeError(f"C oracle failed: {rc}")
  return out
