"""ctypes binding of libhstu_block.so (the C ABI declared in include/hstu_block.h)."""

from __future__ import annotations

import ctypes as C
import os
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("RECML_AMD_BLOCK_LIB") or os.path.join(_HERE, "lib", "libhstu_block.so")

ABI_VERSION = 3

EXPORTS = (
    "hstu_block_abi_version",
    "hstu_block_last_error",
    "hstu_norm_gate_fwd",
    "hstu_norm_gate_bwd",
    "hstu_norm_gate_bwd_workspace_bytes",
    "hstu_gemm_silu_fwd",
    "hstu_gemm_silu_workspace_bytes",
    "hstu_embed_norm_fwd",
)


class HstuNormGateArgs(C.Structure):
  """Field-for-field image of `struct HstuNormGateArgs`."""

  _fields_ = [
      ("struct_size", C.c_uint32), ("version", C.c_uint32),
      ("rows", C.c_int64), ("width", C.c_int32), ("eps", C.c_float),
      ("a", C.c_void_p), ("u", C.c_void_p), ("out", C.c_void_p),
      ("a_stride", C.c_int64), ("u_stride", C.c_int64), ("out_stride", C.c_int64),
      ("gamma", C.c_void_p), ("beta", C.c_void_p),
  ]


class HstuNormGateBwdArgs(C.Structure):
  """Field-for-field image of `struct HstuNormGateBwdArgs`."""

  _fields_ = [
      ("struct_size", C.c_uint32), ("version", C.c_uint32),
      ("rows", C.c_int64), ("width", C.c_int32), ("eps", C.c_float),
      ("a", C.c_void_p), ("u", C.c_void_p), ("dout", C.c_void_p), ("da", C.c_void_p), ("du", C.c_void_p),
      ("a_stride", C.c_int64), ("u_stride", C.c_int64), ("dout_stride", C.c_int64),
      ("da_stride", C.c_int64), ("du_stride", C.c_int64),
      ("gamma", C.c_void_p), ("beta", C.c_void_p), ("dgamma", C.c_void_p), ("dbeta", C.c_void_p),
      ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t),
  ]


class HstuGemmSiluArgs(C.Structure):
  """Field-for-field image of `struct HstuGemmSiluArgs`."""

  _fields_ = [
      ("struct_size", C.c_uint32), ("version", C.c_uint32),
      ("M", C.c_int64), ("N", C.c_int32), ("K", C.c_int32),
      ("activation", C.c_int32), ("reserved0", C.c_int32),
      ("x", C.c_void_p), ("x_stride", C.c_int64),
      ("w", C.c_void_p), ("bias", C.c_void_p), ("out", C.c_void_p),
      ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t),
      ("c", C.c_void_p), ("c_stride", C.c_int64),
  ]


class HstuEmbedNormArgs(C.Structure):
  """Field-for-field image of `struct HstuEmbedNormArgs`."""

  _fields_ = [
      ("struct_size", C.c_uint32), ("version", C.c_uint32),
      ("rows", C.c_int64), ("width", C.c_int32), ("eps", C.c_float),
      ("scale", C.c_float), ("reserved0", C.c_int32),
      ("ids", C.c_void_p), ("table", C.c_void_p),
      ("vocab", C.c_int64), ("table_stride", C.c_int64),
      ("positions", C.c_void_p), ("pos_table", C.c_void_p), ("n_positions", C.c_int64),
      ("gamma", C.c_void_p), ("beta", C.c_void_p), ("out", C.c_void_p),
  ]


_lock = threading.Lock()
_lib = None


def load():
  """Loads the shared library; raises if it has not been built (there is no fallback in here)."""
  global _lib
  if _lib is not None:
    return _lib
  with _lock:
    if _lib is not None:
      return _lib
    if not os.path.exists(LIB_PATH):
      raise RuntimeError(
          f"{LIB_PATH} is missing: build it with `python -m recml_amd.build` (needs hipcc and hipBLASLt)")
    lib = C.CDLL(LIB_PATH)
    lib.hstu_block_abi_version.restype = C.c_int
    lib.hstu_block_abi_version.argtypes = []
    lib.hstu_block_last_error.restype = C.c_char_p
    lib.hstu_block_last_error.argtypes = []
    lib.hstu_norm_gate_fwd.restype = C.c_int
    lib.hstu_norm_gate_fwd.argtypes = [C.POINTER(HstuNormGateArgs), C.c_void_p]
    lib.hstu_norm_gate_bwd.restype = C.c_int
    lib.hstu_norm_gate_bwd.argtypes = [C.POINTER(HstuNormGateBwdArgs), C.c_void_p]
    lib.hstu_norm_gate_bwd_workspace_bytes.restype = C.c_size_t
    lib.hstu_norm_gate_bwd_workspace_bytes.argtypes = [C.c_int64, C.c_int32]
    lib.hstu_gemm_silu_fwd.restype = C.c_int
    lib.hstu_gemm_silu_fwd.argtypes = [C.POINTER(HstuGemmSiluArgs), C.c_void_p]
    lib.hstu_gemm_silu_workspace_bytes.restype = C.c_size_t
    lib.hstu_gemm_silu_workspace_bytes.argtypes = []
    lib.hstu_embed_norm_fwd.restype = C.c_int
    lib.hstu_embed_norm_fwd.argtypes = [C.POINTER(HstuEmbedNormArgs), C.c_void_p]
    ver = lib.hstu_block_abi_version()
    if ver != ABI_VERSION:
      raise RuntimeError(f"libhstu_block.so has ABI {ver}, expected {ABI_VERSION}")
    _lib = lib
  return _lib
