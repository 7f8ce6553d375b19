"""ctypes binding of libhstu_attn.so (the C ABI declared in include/hstu_attn.h)."""

from __future__ import annotations

import ctypes as C
import os
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("RECML_AMD_LIB") or os.path.join(_HERE, "lib", "libhstu_attn.so")

ABI_VERSION = 3

LAYOUT_PADDED, LAYOUT_JAGGED = 0, 1
DTYPE_FP32, DTYPE_BF16, DTYPE_FP8_E4M3FN = 0, 1, 2
FWD_WORKSPACE_PREPARED = 1
FWD_PREPARE_ONLY = 2
FWD_ONE_ITEM_PER_WORKGROUP = 4
FWD_RESIDENT_WORKGROUPS = 8
FWD_COMPILER_SCHEDULED_BLOCKS = 16
NOALLOC_SCRATCH_BYTES = 4 << 20   # HSTU_ATTN_NOALLOC_SCRATCH_BYTES
MASK_NONE, MASK_LENGTH, MASK_SEGMENT = 0, 1, 2

EXPORTS = (
    "hstu_attn_abi_version",
    "hstu_attn_fwd_workspace_bytes",
    "hstu_attn_fwd",
    "hstu_attn_fwd_noalloc",
    "hstu_attn_last_error",
    "hstu_attn_fwd_variant",
    "hstu_attn_bwd",
    "hstu_attn_bwd_variant",
    "hstu_attn_bucket_thresholds",
    "hstu_attn_dropout_keep",
)


class HstuAttnFwdArgs(C.Structure):
  """Field-for-field image of `struct HstuAttnFwdArgs`."""

  _fields_ = [
      ("struct_size", C.c_uint32), ("version", C.c_uint32),
      ("layout", C.c_int32), ("qk_dtype", C.c_int32),
      ("v_dtype", C.c_int32), ("out_dtype", C.c_int32),
      ("B", C.c_int32), ("L", C.c_int32), ("Lkv", C.c_int32),
      ("H", C.c_int32), ("d_qk", C.c_int32), ("d_v", C.c_int32),
      ("total_tokens", C.c_int64),
      ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p),
      ("out", C.c_void_p),
      ("q_stride_b", C.c_int64), ("q_stride_t", C.c_int64), ("q_stride_h", C.c_int64),
      ("k_stride_b", C.c_int64), ("k_stride_t", C.c_int64), ("k_stride_h", C.c_int64),
      ("v_stride_b", C.c_int64), ("v_stride_t", C.c_int64), ("v_stride_h", C.c_int64),
      ("o_stride_b", C.c_int64), ("o_stride_t", C.c_int64), ("o_stride_h", C.c_int64),
      ("alpha", C.c_float), ("inv_n", C.c_float),
      ("causal", C.c_int32), ("mask_mode", C.c_int32),
      ("window", C.c_int32), ("flags", C.c_int32),
      ("seq_lens", C.c_void_p), ("seq_offsets", C.c_void_p),
      ("q_segment_ids", C.c_void_p), ("kv_segment_ids", C.c_void_p),
      ("mask", C.c_void_p),
      ("mask_batched", C.c_int32), ("dense_bias_batched", C.c_int32),
      ("dense_bias", C.c_void_p),
      ("pos_tab", C.c_void_p),
      ("pos_heads", C.c_int32), ("ts_heads", C.c_int32),
      ("ts_tab", C.c_void_p), ("ts", C.c_void_p),
      ("ts_stride_b", C.c_int64),
      ("ts_num_buckets", C.c_int32), ("ts_bucket_size", C.c_float),
      ("q_scale", C.c_void_p), ("k_scale", C.c_void_p),
      ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t),
      ("dropout_p", C.c_float), ("reserved0", C.c_uint32), ("dropout_seed", C.c_uint64),
  ]


class HstuAttnBwdArgs(C.Structure):
  """Field-for-field image of `struct HstuAttnBwdArgs`."""

  _fields_ = [
      ("struct_size", C.c_uint32), ("version", C.c_uint32),
      ("fwd", HstuAttnFwdArgs),
      ("dout", C.c_void_p), ("dq", C.c_void_p), ("dk", C.c_void_p), ("dv", C.c_void_p),
      ("dpos_tab", C.c_void_p), ("dts_tab", C.c_void_p), ("ddense_bias", C.c_void_p),
  ]


_lock = threading.Lock()
_lib = None


def load():
  """Loads the shared library; raises if it has not been built.

  There is no fallback: without the HIP library the op does not run.
  """
  global _lib
  if _lib is not None:
    return _lib
  with _lock:
    if _lib is not None:
      return _lib
    if not os.path.exists(LIB_PATH):
      raise RuntimeError(
          f"{LIB_PATH} is missing: build it with `python -m recml_amd.build` "
          "(needs hipcc); this package has no CPU fallback")
    lib = C.CDLL(LIB_PATH)
    lib.hstu_attn_abi_version.restype = C.c_int
    lib.hstu_attn_abi_version.argtypes = []
    lib.hstu_attn_fwd_workspace_bytes.restype = C.c_size_t
    lib.hstu_attn_fwd_workspace_bytes.argtypes = [C.POINTER(HstuAttnFwdArgs)]
    lib.hstu_attn_fwd.restype = C.c_int
    lib.hstu_attn_fwd.argtypes = [C.POINTER(HstuAttnFwdArgs), C.c_void_p]
    lib.hstu_attn_fwd_noalloc.restype = C.c_int
    lib.hstu_attn_fwd_noalloc.argtypes = [C.POINTER(HstuAttnFwdArgs), C.c_void_p]
    lib.hstu_attn_last_error.restype = C.c_char_p
    lib.hstu_attn_last_error.argtypes = []
    lib.hstu_attn_fwd_variant.restype = C.c_char_p
    lib.hstu_attn_fwd_variant.argtypes = [C.POINTER(HstuAttnFwdArgs)]
    lib.hstu_attn_bwd.restype = C.c_int
    lib.hstu_attn_bwd.argtypes = [C.POINTER(HstuAttnBwdArgs), C.c_void_p]
    lib.hstu_attn_bwd_variant.restype = C.c_char_p
    lib.hstu_attn_bwd_variant.argtypes = [C.POINTER(HstuAttnBwdArgs)]
    lib.hstu_attn_bucket_thresholds.restype = C.c_int
    lib.hstu_attn_bucket_thresholds.argtypes = [C.c_float, C.POINTER(C.c_int32), C.c_int]
    lib.hstu_attn_dropout_keep.restype = C.c_int
    lib.hstu_attn_dropout_keep.argtypes = [C.c_uint64, C.c_float, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_int32]
    ver = lib.hstu_attn_abi_version()
    if ver != ABI_VERSION:
      raise RuntimeError(f"libhstu_attn.so has ABI {ver}, expected {ABI_VERSION}")
    _lib = lib
  return _lib


def new_args() -> HstuAttnFwdArgs:
  a = HstuAttnFwdArgs()
  a.struct_size = C.sizeof(HstuAttnFwdArgs)
  a.version = ABI_VERSION
  a.window = -1
  return a


def last_error() -> str:
  return load().hstu_attn_last_error().decode()
