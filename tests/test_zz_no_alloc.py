"""hstu_attn_fwd_noalloc (the entry point that brings its own scratch) against hstu_attn_fwd.

Both run the same kernels, so the outputs must be equal bit for bit.  Two calls in a row, the
second on a smaller batch: the scratch array is shared by every call on the GPU and keeps the
first call's contents.
"""

import ctypes as C

import numpy as np
import pytest
import torch

from recml_amd import _lib, hstu_ops, workloads
from oracle import hstu_oracle as O

pytestmark = pytest.mark.gpu


def _dev(x, dtype=None):
  if x is None:
    return None
  t = torch.from_numpy(np.ascontiguousarray(x)).to("cuda:0")
  return t if dtype is None else t.to(dtype)


def _both_ways(w):
  """The workload through hstu_attn_fwd (caller workspace) and through hstu_attn_fwd_noalloc."""
  lib = _lib.load()
  bf = torch.bfloat16
  q, k, v = (_dev(O.round_bf16(t), bf) for t in (w.q, w.k, w.v))
  kw = dict(n=w.n, alpha=w.alpha, pos_bias=_dev(w.pos_tab), ts_bias=_dev(w.ts_tab), timestamps=_dev(w.timestamps),
            seq_offsets=_dev(w.seq_offsets), max_len=w.L)
  stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
  out_ref = torch.full_like(v, float("nan"))
  args, keep = hstu_ops.build_args(q, k, v, out_ref, **kw)
  assert args.workspace_bytes > 0, "the case must be one that needs scratch"
  # the same amount of workspace as the built-in array holds: the library plans the split of long tiles
  # by the room for their partial sums, and equal room makes the two calls sum in the same order
  ws = torch.empty(_lib.NOALLOC_SCRATCH_BYTES, dtype=torch.uint8, device=q.device)
  keep.append(ws)
  args.workspace, args.workspace_bytes = ws.data_ptr(), ws.numel()
  assert lib.hstu_attn_fwd(C.byref(args), stream) == 0, _lib.last_error()
  out_new = torch.full_like(v, float("nan"))
  args2, keep2 = hstu_ops.build_args(q, k, v, out_new, **kw)
  need = min(args2.workspace_bytes, _lib.NOALLOC_SCRATCH_BYTES)
  args2.workspace, args2.workspace_bytes = None, 0      # the entry point must not need them
  del keep2[-1]                                         # drop the buffer build_args allocated
  assert lib.hstu_attn_fwd_noalloc(C.byref(args2), stream) == 0, _lib.last_error()
  torch.cuda.synchronize()
  return out_ref, out_new, need, (q, k, v)


def test_noalloc_matches_fwd_twice_second_call_smaller(gpu):
  from oracle import c_oracle
  big = workloads.config3()                                 # the headline batch: 64 sequences, both bias tables
  small = workloads.config3(seed=11, B=3, L=256, H=8, d=128)
  for w in (big, small):
    ref, new, need, (q, k, v) = _both_ways(w)
    assert need <= _lib.NOALLOC_SCRATCH_BYTES
    assert not torch.isnan(new.float()).any()
    assert torch.equal(ref, new), f"{w.B} sequences: outputs differ"
    # and the shared kernels are right: the C oracle on the same bf16 inputs, every sequence
    want = c_oracle.hstu_attention_c(q.float().cpu().numpy(), k.float().cpu().numpy(), v.float().cpu().numpy(),
                                     seq_offsets=w.seq_offsets, max_len=w.L, n=w.n, pos_tab=w.pos_tab,
                                     timestamps=w.timestamps, ts_tab=w.ts_tab)
    err = np.abs(new.float().cpu().numpy() - want).max() / np.abs(want).max()
    assert err <= 2e-2, err      # bf16 bound: max|out - ref| <= 2e-2 max|ref|


def test_noalloc_few_long_sequences_split_tiles(gpu):
  # two long sequences: the library splits the key range of the long tiles and sums fp32 partials from its scratch
  # (as many tiles as the scratch has room for)
  lens = np.asarray([1024, 700], np.int32)
  rng = np.random.Generator(np.random.PCG64(5))
  T = int(lens.sum())
  q, k, v = (rng.standard_normal((T, 2, 32), dtype=np.float32) * 0.1 for _ in range(3))
  off = np.zeros(3, np.int32)
  off[1:] = np.cumsum(lens)
  w = workloads.Workload("split", 2, 1024, 2, 32, "bf16", "jagged", lens, q, k, v, n=1024, seq_offsets=off)
  ref, new, need, _ = _both_ways(w)
  assert need <= _lib.NOALLOC_SCRATCH_BYTES
  assert torch.equal(ref, new)


def test_noalloc_rejects_calls_beyond_its_scratch(gpu):
  lib = _lib.load()
  a = _lib.new_args()
  B, L, H, d = 4096, 2048, 8, 128                         # int32 timestamps of 8 M tokens alone are 32 MB
  a.layout, a.qk_dtype, a.v_dtype, a.out_dtype = _lib.LAYOUT_PADDED, _lib.DTYPE_BF16, _lib.DTYPE_BF16, _lib.DTYPE_BF16
  a.B, a.L, a.Lkv, a.H, a.d_qk, a.d_v = B, L, L, H, d, d
  a.q = a.k = a.v = a.out = 0x100000                      # never dereferenced: the call is refused before any launch
  for n in ("q", "k", "v", "o"):
    setattr(a, f"{n}_stride_h", d)
    setattr(a, f"{n}_stride_t", H * d)
    setattr(a, f"{n}_stride_b", L * H * d)
  a.alpha, a.inv_n, a.causal, a.mask_mode = 1.0, 1.0 / L, 1, _lib.MASK_LENGTH
  a.seq_lens = 0x100000
  a.ts, a.ts_tab, a.ts_heads, a.ts_stride_b, a.ts_num_buckets, a.ts_bucket_size = 0x100000, 0x100000, 1, L, 128, 0.301
  assert lib.hstu_attn_fwd_workspace_bytes(C.byref(a)) > _lib.NOALLOC_SCRATCH_BYTES
  assert lib.hstu_attn_fwd_noalloc(C.byref(a), None) == -5
  assert b"scratch" in lib.hstu_attn_last_error()
