"""The C ABI: the library loads, exports every declared symbol, and the ctypes
image of HstuAttnFwdArgs matches the C struct.  No GPU work is launched: every
call here returns from argument validation."""

import ctypes as C
import os
import re
import subprocess
import tempfile

import pytest

from recml_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "hstu_attn.h")


def _declared_functions():
  text = open(HEADER).read()
  return sorted(set(re.findall(r"\b(hstu_attn_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
  lib = _lib.load()
  names = _declared_functions()
  assert set(names) == set(_lib.EXPORTS)
  for n in names:
    assert getattr(lib, n) is not None
  assert lib.hstu_attn_abi_version() == _lib.ABI_VERSION


@pytest.mark.parametrize("name", ["HstuAttnFwdArgs", "HstuAttnBwdArgs"])
def test_struct_layout_matches_header(name):
  struct = getattr(_lib, name)
  fields = [f[0] for f in struct._fields_]
  prog = ['#include <stdio.h>', '#include <stddef.h>', '#include "hstu_attn.h"', "int main(void) {",
          f'  printf("%zu\\n", sizeof({name}));']
  prog += [f'  printf("%zu\\n", offsetof({name}, {f}));' for f in fields]
  prog += ["  return 0;", "}"]
  with tempfile.TemporaryDirectory() as d:
    src = os.path.join(d, "layout.c")
    exe = os.path.join(d, "layout")
    open(src, "w").write("\n".join(prog))
    subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), "-o", exe, src], check=True)
    out = subprocess.run([exe], check=True, capture_output=True, text=True).stdout.split()
  assert int(out[0]) == C.sizeof(struct)
  for f, off in zip(fields, out[1:]):
    assert getattr(struct, f).offset == int(off), f


def test_backward_validation_errors_without_gpu():
  lib = _lib.load()
  assert lib.hstu_attn_bwd(None, None) == -1
  b = _lib.HstuAttnBwdArgs()
  assert lib.hstu_attn_bwd(C.byref(b), None) == -2            # struct_size / version not filled in
  b.struct_size, b.version = C.sizeof(_lib.HstuAttnBwdArgs), _lib.ABI_VERSION
  b.fwd = _lib.new_args()
  f = b.fwd
  f.B, f.L, f.Lkv, f.H, f.d_qk, f.d_v = 1, 8, 8, 1, 32, 32
  f.q = f.k = f.v = 0x1000
  f.qk_dtype, f.v_dtype, f.out_dtype = _lib.DTYPE_FP8_E4M3FN, _lib.DTYPE_BF16, _lib.DTYPE_BF16
  b.dout = 0x1000
  assert lib.hstu_attn_bwd(C.byref(b), None) == -3            # no fp8 backward
  f.qk_dtype = f.v_dtype = f.out_dtype = _lib.DTYPE_BF16
  assert lib.hstu_attn_bwd(C.byref(b), None) == -1            # dq, dk, dv missing
  assert b"dq" in lib.hstu_attn_last_error()


def test_backward_variant_query():
  lib = _lib.load()
  b = _lib.HstuAttnBwdArgs()
  assert lib.hstu_attn_bwd_variant(C.byref(b)) == b"invalid"          # struct_size / version not filled in
  b.struct_size, b.version = C.sizeof(_lib.HstuAttnBwdArgs), _lib.ABI_VERSION
  b.fwd = _lib.new_args()
  f = b.fwd
  f.B, f.L, f.Lkv, f.H, f.d_qk, f.d_v = 2, 1024, 1024, 4, 64, 64
  f.q = f.k = f.v = 0x10000
  f.q_stride_t = f.k_stride_t = f.v_stride_t = f.o_stride_t = 4 * 64
  f.q_stride_h = f.k_stride_h = f.v_stride_h = f.o_stride_h = 64
  f.q_stride_b = f.k_stride_b = f.v_stride_b = f.o_stride_b = 1024 * 4 * 64
  f.alpha, f.inv_n, f.causal = 1.0, 1.0 / 1024, 1
  f.qk_dtype = f.v_dtype = f.out_dtype = _lib.DTYPE_BF16
  b.dout = b.dq = b.dk = b.dv = 0x20000
  # bf16 at a matrix-core head dim, but no workspace: the general pair (bf16 products: rows on 16-byte boundaries)
  assert lib.hstu_attn_bwd_variant(C.byref(b)) == b"hstu_bwd_general<bf16, bf16 products>"
  f.q = 0x10002                                                       # rows off a boundary: fp32 products
  assert lib.hstu_attn_bwd_variant(C.byref(b)) == b"hstu_bwd_general<bf16>"
  f.q = 0x10000
  f.out = 0x30000                                                     # the size query validates a forward call
  f.workspace, f.workspace_bytes = 0x40000, lib.hstu_attn_fwd_workspace_bytes(C.byref(f))
  f.out = None                                                        # the backward does not need it
  assert f.workspace_bytes > 0
  assert lib.hstu_attn_bwd_variant(C.byref(b)) == b"hstu_bwd_mfma_bf16"
  b.dq = 0x20004                                                      # gradient buffers must be 16-byte aligned for it
  assert lib.hstu_attn_bwd_variant(C.byref(b)) == b"hstu_bwd_general<bf16, bf16 products>"
  b.dq = 0x20000
  f.window = 8                                                        # a sliding window stays on the matrix cores
  assert lib.hstu_attn_bwd_variant(C.byref(b)) == b"hstu_bwd_mfma_bf16"
  f.window = -1
  f.mask = 0x50000                                                    # a dense keep-mask rides along tile by tile ...
  f.out = 0x30000
  plain_bytes = f.workspace_bytes
  f.workspace_bytes = lib.hstu_attn_fwd_workspace_bytes(C.byref(f))   # (its workspace also holds the tiles' step ranges)
  f.out = None
  assert f.workspace_bytes > 0
  assert lib.hstu_attn_bwd_variant(C.byref(b)) == b"hstu_bwd_mfma_bf16"
  f.dense_bias = 0x60000                                              # ... and so does a dense bias, with its gradient
  assert lib.hstu_attn_bwd_variant(C.byref(b)) == b"hstu_bwd_mfma_bf16"
  b.ddense_bias = 0x70000
  assert lib.hstu_attn_bwd_variant(C.byref(b)) == b"hstu_bwd_mfma_bf16"
  f.Lkv = f.L + 16                                                    # keys and queries of different lengths do not
  assert lib.hstu_attn_bwd_variant(C.byref(b)) == b"hstu_bwd_general<bf16, bf16 products>"
  f.Lkv = f.L
  b.ddense_bias = None
  f.dense_bias = None
  f.mask = None
  f.workspace_bytes = plain_bytes
  # a batch small enough to go without a work list, and no bias table: no workspace to ask for, the matrix cores all the same
  f.L = f.Lkv = 256
  f.workspace, f.workspace_bytes = None, 0
  f.out = 0x30000
  assert lib.hstu_attn_fwd_workspace_bytes(C.byref(f)) == 0
  f.out = None
  assert lib.hstu_attn_bwd_variant(C.byref(b)) == b"hstu_bwd_mfma_bf16"
  f.qk_dtype = f.v_dtype = f.out_dtype = _lib.DTYPE_FP32
  assert lib.hstu_attn_bwd_variant(C.byref(b)) == b"hstu_bwd_general<float>"


def test_validation_errors_without_gpu():
  lib = _lib.load()
  assert lib.hstu_attn_fwd(None, None) == -1                 # HSTU_ERR_NULL
  a = _lib.new_args()
  a.version = 99
  assert lib.hstu_attn_fwd(C.byref(a), None) == -2           # HSTU_ERR_VERSION
  assert b"version" in lib.hstu_attn_last_error()
  a = _lib.new_args()
  a.B, a.L, a.Lkv, a.H, a.d_qk, a.d_v = 1, 8, 8, 1, 32, 32
  assert lib.hstu_attn_fwd(C.byref(a), None) == -1           # q/k/v/out null
  a.q = a.k = a.v = a.out = 0x1000                           # never dereferenced: validation fails first
  a.d_qk = 512
  assert lib.hstu_attn_fwd(C.byref(a), None) == -4           # HSTU_ERR_SHAPE
  a.d_qk = 32
  a.flags = 64                                               # a bit no flag has
  assert lib.hstu_attn_fwd(C.byref(a), None) == -4
  assert b"flags" in lib.hstu_attn_last_error()
  a.flags = 0
  a.qk_dtype, a.v_dtype, a.out_dtype = 0, 1, 1
  assert lib.hstu_attn_fwd(C.byref(a), None) == -3           # HSTU_ERR_DTYPE
  a.qk_dtype = a.v_dtype = a.out_dtype = 1
  a.mask_mode = _lib.MASK_SEGMENT
  assert lib.hstu_attn_fwd(C.byref(a), None) == -1           # one-sided / missing segment ids
  assert b"segment" in lib.hstu_attn_last_error()
  a.mask_mode = _lib.MASK_LENGTH
  assert lib.hstu_attn_fwd(C.byref(a), None) == -1           # LENGTH needs seq_lens
  a.mask_mode = _lib.MASK_NONE
  a.layout = _lib.LAYOUT_JAGGED
  assert lib.hstu_attn_fwd(C.byref(a), None) == -1           # jagged needs offsets
  assert lib.hstu_attn_fwd_variant(C.byref(a)) == b"invalid"
  assert lib.hstu_attn_fwd_workspace_bytes(C.byref(a)) == 0


def test_variant_and_workspace_query():
  lib = _lib.load()
  a = _lib.new_args()
  a.B, a.L, a.Lkv, a.H, a.d_qk, a.d_v = 2, 256, 256, 4, 128, 128
  a.q = a.k = a.v = a.out = 0x10000
  a.q_stride_t = a.k_stride_t = a.v_stride_t = a.o_stride_t = 4 * 128
  a.q_stride_h = a.k_stride_h = a.v_stride_h = a.o_stride_h = 128
  a.q_stride_b = a.k_stride_b = a.v_stride_b = a.o_stride_b = 256 * 4 * 128
  a.alpha, a.inv_n, a.causal = 1.0, 1.0 / 256, 1
  a.qk_dtype = a.v_dtype = a.out_dtype = _lib.DTYPE_BF16
  assert lib.hstu_attn_fwd_variant(C.byref(a)) == b"hstu_fwd_mfma_bf16"
  # a batch this small (one workgroup per sequence, head and query tile fits the chip at once) goes without a work
  # list: nothing to prepare unless a table comes with it ...
  up = lambda x: (x + 255) // 256 * 256
  assert lib.hstu_attn_fwd_workspace_bytes(C.byref(a)) == 0
  # ... with a position table, its scaled and padded copy
  a.pos_tab, a.pos_heads = 0x20000, 4
  assert lib.hstu_attn_fwd_workspace_bytes(C.byref(a)) == up(4 * (2 * 256 - 1 + 512) * 4)
  a.pos_tab, a.pos_heads = None, 0
  # a larger batch: a work list of one int4 per query tile (200 sequences x 2 tiles here) behind a 16-byte header
  # and 16 counters behind that
  a.B = 200
  sched = up(16 + 16 * 200 * 2) + up(4 * 16)
  assert lib.hstu_attn_fwd_workspace_bytes(C.byref(a)) == sched
  a.pos_tab, a.pos_heads = 0x20000, 4
  assert lib.hstu_attn_fwd_workspace_bytes(C.byref(a)) == up(4 * (2 * 256 - 1 + 512) * 4) + sched
  a.B = 2
  # longer sequences can have query tiles whose key range is split over workgroups: room for the fp32
  # partial sums of up to 32 chunks per head, their arrival counters, and 32 more list entries
  a.pos_tab, a.pos_heads = None, 0
  a.L = a.Lkv = 1024
  a.q_stride_b = a.k_stride_b = a.v_stride_b = a.o_stride_b = 1024 * 4 * 128
  full = lib.hstu_attn_fwd_workspace_bytes(C.byref(a))
  assert full == up(16 + 16 * (2 * 8 + 32)) + up(4 * (16 + 32 * 4)) + 32 * 4 * 128 * 128 * 4
  a.L = a.Lkv = 256
  a.q_stride_b = a.k_stride_b = a.v_stride_b = a.o_stride_b = 256 * 4 * 128
  a.pos_tab, a.pos_heads = 0x20000, 4
  # general-kernel calls need none
  # a launch without the workspace is refused before anything is enqueued
  assert lib.hstu_attn_fwd(C.byref(a), None) == -5
  a.pos_tab = None
  a.qk_dtype = a.v_dtype = a.out_dtype = _lib.DTYPE_FP32
  assert lib.hstu_attn_fwd_variant(C.byref(a)) == b"hstu_fwd_general<float>"
  assert lib.hstu_attn_fwd_workspace_bytes(C.byref(a)) == 0
  a.qk_dtype = a.v_dtype = a.out_dtype = _lib.DTYPE_BF16
  a.window = 4                                         # a sliding window stays on the matrix cores
  assert lib.hstu_attn_fwd_variant(C.byref(a)) == b"hstu_fwd_mfma_bf16"
  a.window = -1
  a.dense_bias = 0x30000                               # so do a dense bias and an explicit mask ...
  a.mask = 0x50000
  assert lib.hstu_attn_fwd_variant(C.byref(a)) == b"hstu_fwd_mfma_bf16"
  a.dense_bias = 0x30004                               # ... unless their rows cannot be fetched 16 bytes at a time,
  assert lib.hstu_attn_fwd_variant(C.byref(a)) == b"hstu_fwd_general<bf16>"
  a.dense_bias = 0x30000
  a.pos_tab, a.pos_heads = 0x20000, 4                  # or a table bias comes on top
  assert lib.hstu_attn_fwd_variant(C.byref(a)) == b"hstu_fwd_general<bf16>"
  a.pos_tab, a.pos_heads = None, 0
  a.dense_bias = a.mask = None
  a.L = a.Lkv = 248                                    # 248 = 8 x 31: whole pieces of 4 floats, not of 16 mask bytes
  a.dense_bias = 0x30000
  assert lib.hstu_attn_fwd_variant(C.byref(a)) == b"hstu_fwd_mfma_bf16"
  a.mask = 0x50000
  assert lib.hstu_attn_fwd_variant(C.byref(a)) == b"hstu_fwd_general<bf16>"
  a.dense_bias = a.mask = None
  a.L = a.Lkv = 256
  a.d_qk = a.d_v = 48
  assert lib.hstu_attn_fwd_variant(C.byref(a)) == b"hstu_fwd_general<bf16>"
