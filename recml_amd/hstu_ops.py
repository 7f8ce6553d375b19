"""HSTU pointwise-SiLU attention forward on MI355X: host-side operator.

Three entry points, each a thin argument check over one C call
(`hstu_attn_fwd`, include/hstu_attn.h):

  hstu_attention              the full op: padded or jagged Q/K/V, per-sequence
                              lengths, relative-position and timestamp bias
                              tables, normaliser N.
  pointwise_splash_attention  same names, argument meaning and errors as the
                              reference operator
                              (recml/core/ops/hstu_ops.py:829-851).
  pointwise_attention         the layer-side call with a dense mask and bias
                              (recml/layers/keras/hstu.py:356-390).

Tensors are torch tensors on the GPU; torch only supplies device memory and
the current HIP stream.  There is no CPU path.
"""

from __future__ import annotations

import ctypes as C
import enum
import math

import numpy as np
import torch

from recml_amd import _lib


class MaskType(str, enum.Enum):
  """Mask type of the operator (recml/core/ops/hstu_ops.py:41-45)."""

  CAUSAL = "causal"
  FULL = "full"


_DTYPES = {torch.float32: _lib.DTYPE_FP32, torch.bfloat16: _lib.DTYPE_BF16,
           torch.float8_e4m3fn: _lib.DTYPE_FP8_E4M3FN}


def _ptr(t):
  return None if t is None else C.c_void_p(t.data_ptr())


def _check_gpu(name, t):
  if not isinstance(t, torch.Tensor):
    raise TypeError(f"{name} must be a torch.Tensor, got {type(t).__name__}")
  if not t.is_cuda:
    raise ValueError(f"{name} must live on the GPU (got device {t.device}); "
                     "this operator has no CPU path")


def _inner_contiguous(t):
  return t if t.stride(-1) == 1 else t.contiguous()


def _as_table(name, t, H, width, device):
  """fp32 [heads, width] table with heads in {1, H}."""
  _check_gpu(name, t)
  if t.dim() == 1:
    t = t.unsqueeze(0)
  if t.dim() != 2 or t.shape[0] not in (1, H):
    raise ValueError(f"{name} must have shape [{width}] or [1|{H}, {width}], got {tuple(t.shape)}")
  if width is not None and t.shape[1] != width:
    raise ValueError(f"{name} must have {width} entries per head, got {t.shape[1]}")
  return t.to(device=device, dtype=torch.float32).contiguous()


def _attach_workspace(args, keep):
  """Allocates the device scratch the library asks for (once per argument set)."""
  ws = _lib.load().hstu_attn_fwd_workspace_bytes(C.byref(args))
  if ws:
    buf = torch.empty(ws, dtype=torch.uint8, device=keep[0].device)
    keep.append(buf)
    args.workspace = buf.data_ptr()
    args.workspace_bytes = ws


class AttentionBatch:
  """What the attention prepares from a batch before its kernel runs -- the work list, the timestamps
  as 32-bit offsets with their per-tile ranges, the scaled bias tables -- kept for every call on that
  batch: a model hands one of these to all its layers, and only the first call pays the preparation
  (`HSTU.forward` does).  It also keeps the device scratch, so no call after the first allocates.

  The preparation is reused when the call's shapes and options are the same and the tensors it was
  built from (`seq_lens` / `seq_offsets`, `timestamps`, `pos_bias`, `ts_bias`, a dense `mask`) are the same objects,
  unmodified since (torch's version counter); anything else prepares again.  q, k, v, `alpha` and `n`
  may differ from call to call.  Not for concurrent use on several streams.  Tensors created under
  `torch.inference_mode()` have no version counter: a change made to one of them in place is not noticed, so
  take a new AttentionBatch after such a change.
  """

  def __init__(self):
    self._buf = None
    self._prepared = None     # signature the workspace was prepared for
    self._pending = None
    self._tensors = ()        # keeps the signature's tensors alive (their addresses are part of it)
    self.prepared_calls = 0   # calls that skipped the preparation

  @staticmethod
  def _ident(t):
    if t is None:
      return None
    if not isinstance(t, torch.Tensor):
      return False            # not a tensor: never reused
    # (tensors made under torch.inference_mode() carry no version counter, and reading it raises)
    version = -1 if t.is_inference() else t._version
    return (t.data_ptr(), version, tuple(t.shape), tuple(t.stride()), t.dtype)

  def _attach(self, args, keep, sig, tensors):
    ws = _lib.load().hstu_attn_fwd_workspace_bytes(C.byref(args))
    if not ws:
      return
    dev = keep[0].device
    if self._buf is None or self._buf.numel() != ws or self._buf.device != dev:
      self._buf = torch.empty(ws, dtype=torch.uint8, device=dev)
      self._prepared = None
    keep.append(self._buf)
    args.workspace = self._buf.data_ptr()
    args.workspace_bytes = ws
    self._pending = None
    if sig is not None and sig == self._prepared:
      args.flags |= _lib.FWD_WORKSPACE_PREPARED
      self.prepared_calls += 1
    else:
      self._prepared = None
      self._pending = (sig, tensors)

  def _commit(self):
    if self._pending is not None:
      self._prepared, self._tensors = self._pending
      self._pending = None


def _passed_inputs(keep):
  """The q, k, v tensors whose pointers build_args put into the struct (after any copy)."""
  return keep[0], keep[1], keep[2]


def _run(args, keep):
  lib = _lib.load()
  stream = torch.cuda.current_stream(keep[0].device).cuda_stream
  rc = lib.hstu_attn_fwd(C.byref(args), C.c_void_p(stream))
  if rc != 0:
    msg = lib.hstu_attn_last_error().decode()
    if rc in (-3, -4, -1):
      raise ValueError(f"hstu_attn_fwd rejected the arguments ({rc}): {msg}")
    raise RuntimeError(f"hstu_attn_fwd failed ({rc}): {msg}")


def kernel_variant(args) -> str:
  return _lib.load().hstu_attn_fwd_variant(C.byref(args)).decode()


def build_args(q, k, v, out, *, seq_lens=None, seq_offsets=None, max_len=None,
               n=None, alpha=1.0, inv_n=None, causal=True, pos_bias=None,
               timestamps=None, ts_bias=None, ts_bucket_size=0.301,
               q_segment_ids=None, kv_segment_ids=None,
               sliding_window_size=None, mask=None, bias=None,
               q_scale=None, k_scale=None, batch=None, dropout_p=0.0, dropout_seed=0):
  """Validates the call and fills an HstuAttnFwdArgs.  Returns (args, keepalive)."""
  given = (seq_lens, seq_offsets, timestamps, pos_bias, ts_bias, mask)
  for name, t in (("q", q), ("k", k), ("v", v)):
    _check_gpu(name, t)
  if q.dtype not in _DTYPES:
    raise ValueError(f"unsupported dtype {q.dtype}: use float32, bfloat16 or float8_e4m3fn (q and k)")
  fp8 = q.dtype == torch.float8_e4m3fn
  if fp8:
    if k.dtype != q.dtype or v.dtype != torch.bfloat16:
      raise ValueError(f"float8_e4m3fn q needs float8_e4m3fn k and bfloat16 v, got {k.dtype}, {v.dtype}")
  elif k.dtype != q.dtype or v.dtype != q.dtype:
    raise ValueError(f"q, k, v must share one dtype, got {q.dtype}, {k.dtype}, {v.dtype}")
  if not fp8 and (q_scale is not None or k_scale is not None):
    raise ValueError("q_scale / k_scale belong to float8_e4m3fn q and k")
  keep = [q, k, v, out]
  a = _lib.new_args()
  dev = q.device
  jagged = q.dim() == 3
  if jagged:
    if seq_offsets is None or max_len is None:
      raise ValueError("jagged q/k/v ([T, H, d]) need seq_offsets and max_len")
    T, H, d = q.shape
    if k.shape != (T, H, d):
      raise ValueError(f"k shape {tuple(k.shape)} does not match q {tuple(q.shape)}")
    if v.shape[:2] != (T, H):
      raise ValueError(f"v shape {tuple(v.shape)} does not match q {tuple(q.shape)}")
    _check_gpu("seq_offsets", seq_offsets)
    if seq_offsets.dim() != 1 or seq_offsets.numel() < 1:
      raise ValueError("seq_offsets must have shape [B+1]")
    seq_offsets = seq_offsets.to(torch.int32).contiguous()
    keep.append(seq_offsets)
    B, L, Lkv = seq_offsets.numel() - 1, int(max_len), int(max_len)
    a.layout = _lib.LAYOUT_JAGGED
    a.total_tokens = T
    a.seq_offsets = seq_offsets.data_ptr()
    a.mask_mode = _lib.MASK_LENGTH
    if q_segment_ids is not None or kv_segment_ids is not None:
      raise ValueError("segment ids need the padded layout")
  else:
    if q.dim() != 4:
      raise ValueError(f"q must be [B, L, H, d] or [T, H, d], got {tuple(q.shape)}")
    B, L, H, d = q.shape
    if k.dim() != 4 or k.shape[0] != B or k.shape[2] != H or k.shape[3] != d:
      raise ValueError(f"k shape {tuple(k.shape)} does not match q {tuple(q.shape)}")
    Lkv = k.shape[1]
    if v.dim() != 4 or v.shape[:3] != (B, Lkv, H):
      raise ValueError(f"v shape {tuple(v.shape)} does not match k {tuple(k.shape)}")
    if max_len is not None and int(max_len) != L:
      raise ValueError(f"max_len={max_len} does not match the padded length {L}")
    a.layout = _lib.LAYOUT_PADDED
    if (q_segment_ids is None) != (kv_segment_ids is None):
      raise ValueError("Both or neither of `q_segment_ids` and `kv_segment_ids` must be provided.")
    if q_segment_ids is not None:
      if seq_lens is not None:
        raise ValueError("pass either seq_lens or segment ids, not both")
      _check_gpu("q_segment_ids", q_segment_ids)
      _check_gpu("kv_segment_ids", kv_segment_ids)
      if tuple(q_segment_ids.shape) != (B, L):
        raise ValueError(f"Invalid shape for q segment_ids: {tuple(q_segment_ids.shape)}. Expected: {(B, L)}")
      if tuple(kv_segment_ids.shape) != (B, Lkv):
        raise ValueError(f"Invalid shape for kv segment_ids: {tuple(kv_segment_ids.shape)}. Expected: {(B, Lkv)}")
      qs = q_segment_ids.to(torch.int32).contiguous()
      ks = kv_segment_ids.to(torch.int32).contiguous()
      keep += [qs, ks]
      a.q_segment_ids, a.kv_segment_ids = qs.data_ptr(), ks.data_ptr()
      a.mask_mode = _lib.MASK_SEGMENT
    elif seq_lens is not None:
      _check_gpu("seq_lens", seq_lens)
      if tuple(seq_lens.shape) != (B,):
        raise ValueError(f"seq_lens must have shape [{B}], got {tuple(seq_lens.shape)}")
      sl = seq_lens.to(torch.int32).contiguous()
      keep.append(sl)
      a.seq_lens = sl.data_ptr()
      a.mask_mode = _lib.MASK_LENGTH
    else:
      a.mask_mode = _lib.MASK_NONE
  d_v = v.shape[-1]
  exp_out = (q.shape[0], H, d_v) if jagged else (B, L, H, d_v)
  if tuple(out.shape) != exp_out or out.dtype != v.dtype or not out.is_cuda:
    raise ValueError(f"out must be a {v.dtype} GPU tensor of shape {exp_out}")

  q, k, v = (_inner_contiguous(t) for t in (q, k, v))
  if out.stride(-1) != 1:
    raise ValueError("out must be contiguous in its last dimension")
  keep[0:3] = [q, k, v]     # the tensors whose pointers go into the struct
  a.q, a.k, a.v, a.out = q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr()
  a.qk_dtype = _DTYPES[q.dtype]
  a.v_dtype = a.out_dtype = _DTYPES[v.dtype]
  for name, sc in (("q_scale", q_scale), ("k_scale", k_scale)):
    if sc is not None:
      _check_gpu(name, sc)
      if sc.numel() not in (1, H):
        raise ValueError(f"{name} must have 1 or {H} entries, got {tuple(sc.shape)}")
      sc = sc.to(torch.float32).reshape(-1).expand(H).contiguous()
      keep.append(sc)
      setattr(a, name, sc.data_ptr())
  for name, t in (("q", q), ("k", k), ("v", v), ("o", out)):
    if jagged:
      sb, st, sh = 0, t.stride(0), t.stride(1)
    else:
      sb, st, sh = t.stride(0), t.stride(1), t.stride(2)
    setattr(a, f"{name}_stride_b", sb)
    setattr(a, f"{name}_stride_t", st)
    setattr(a, f"{name}_stride_h", sh)
  a.B, a.L, a.Lkv, a.H, a.d_qk, a.d_v = B, L, Lkv, H, d, d_v

  a.alpha = float(alpha)
  if inv_n is None:
    n = L if n is None else n
    if not n > 0:
      raise ValueError(f"normaliser n must be positive, got {n}")
    inv_n = 1.0 / float(n)
  a.inv_n = float(inv_n)
  a.causal = 1 if causal else 0
  if sliding_window_size is not None:
    if int(sliding_window_size) < 0:
      raise ValueError("sliding_window_size must be >= 0")
    a.window = min(int(sliding_window_size), 2 ** 31 - 1)   # beyond the sequence it restricts nothing
  if not 0.0 <= float(dropout_p) < 1.0:
    raise ValueError(f"dropout_p must be in [0, 1), got {dropout_p}")
  a.dropout_p = float(dropout_p)
  a.dropout_seed = int(dropout_seed) & 0xFFFFFFFFFFFFFFFF

  if mask is not None:
    if isinstance(mask, np.ndarray):
      mask = torch.from_numpy(np.ascontiguousarray(mask)).to(dev)
    _check_gpu("mask", mask)
    if mask.dim() == 2:
      if tuple(mask.shape) != (L, Lkv):
        raise ValueError(f"Mask shape {tuple(mask.shape)} does not match query and key length ({L}, {Lkv}).")
      a.mask_batched = 0
    elif mask.dim() == 3 and tuple(mask.shape) == (B, L, Lkv):
      a.mask_batched = 1
    else:
      raise ValueError(f"mask must be [{L}, {Lkv}] or [{B}, {L}, {Lkv}], got {tuple(mask.shape)}")
    # the kernels keep a pair where the byte is non-zero: bool and uint8 masks go as they are
    if mask.dtype == torch.bool:
      m8 = mask.contiguous().view(torch.uint8)
    elif mask.dtype == torch.uint8:
      m8 = mask.contiguous()
    else:
      m8 = (mask != 0).to(torch.uint8).contiguous()
    keep.append(m8)
    a.mask = m8.data_ptr()
  if bias is not None:
    _check_gpu("bias", bias)
    if bias.dim() == 2:
      bias = bias.unsqueeze(0)
    if bias.dim() != 3 or tuple(bias.shape[1:]) != (L, Lkv) or bias.shape[0] not in (1, B):
      raise ValueError(f"bias must be [{L}, {Lkv}] or [1|{B}, {L}, {Lkv}], got {tuple(bias.shape)}")
    bf = bias.to(torch.float32).contiguous()
    keep.append(bf)
    a.dense_bias = bf.data_ptr()
    a.dense_bias_batched = 1 if bias.shape[0] == B and B > 1 else 0
  if pos_bias is not None:
    if L != Lkv:
      raise ValueError("relative-position bias needs q_len == kv_len")
    pt = _as_table("pos_bias", pos_bias, H, 2 * L - 1, dev)
    keep.append(pt)
    a.pos_tab, a.pos_heads = pt.data_ptr(), pt.shape[0]
  if (timestamps is None) != (ts_bias is None):
    raise ValueError("Both or neither of `timestamps` and `ts_bias` must be provided.")
  if ts_bias is not None:
    if L != Lkv:
      raise ValueError("timestamp bias needs q_len == kv_len")
    tt = _as_table("ts_bias", ts_bias, H, None, dev)
    _check_gpu("timestamps", timestamps)
    ts = timestamps.to(torch.int64).contiguous()
    if ts.dim() == 2 and tuple(ts.shape) == (B, L):
      a.ts_stride_b = L
    elif ts.dim() == 1 and jagged and ts.numel() == q.shape[0]:
      a.ts_stride_b = 0
    else:
      raise ValueError(f"timestamps must be [{B}, {L}]" + (f" or [{q.shape[0]}]" if jagged else "")
                       + f", got {tuple(ts.shape)}")
    keep += [tt, ts]
    a.ts_tab, a.ts_heads, a.ts = tt.data_ptr(), tt.shape[0], ts.data_ptr()
    a.ts_num_buckets = tt.shape[1] - 1
    a.ts_bucket_size = float(ts_bucket_size)
  if q.is_cuda:
    if batch is None:
      _attach_workspace(a, keep)
    else:
      # everything the preparation reads (the dense mask included: its key-step ranges) or the workspace
      # layout depends on; segment ids (not part of it, but of the choice of kernel) rule the reuse out
      sig = None
      idents = tuple(AttentionBatch._ident(t) for t in given)
      if q_segment_ids is None and False not in idents:
        sig = (tuple(q.shape), tuple(k.shape), int(v.shape[-1]), q.dtype, max_len, bool(causal),
               sliding_window_size, float(ts_bucket_size), bias is not None, idents)
      batch._attach(a, keep, sig, given)
  return a, keep


def hstu_attention(q, k, v, *, seq_lens=None, seq_offsets=None, max_len=None,
                   n=None, alpha=1.0, causal=True, pos_bias=None,
                   timestamps=None, ts_bias=None, ts_bucket_size=0.301,
                   q_segment_ids=None, kv_segment_ids=None,
                   sliding_window_size=None, mask=None, bias=None, out=None,
                   q_scale=None, k_scale=None, batch=None, dropout_p=0.0, dropout_seed=0):
  """out = (silu(alpha * q k^T + bias) / n, masked) v.

  Args:
    q, k, v: padded [B, L, H, d] or jagged [T, H, d] (with `seq_offsets`
      [B+1] and `max_len`); float32 or bfloat16 GPU tensors, or
      float8_e4m3fn q and k with bfloat16 v.
    q_scale, k_scale: per-head (or scalar) dequantisation scales of
      float8_e4m3fn q and k: the logits are alpha * q_scale * k_scale * q8.k8.
    seq_lens: int [B] valid lengths of an end-padded batch.  Rows and keys at
      or beyond the length are ignored and output rows there are exactly 0,
      as with make_causal_mask (recml/layers/keras/utils.py:39-41).
    n: the normaliser N; defaults to the padded length
      (recml/layers/keras/hstu.py:377-378).
    alpha: logit scale (1, or 1/sqrt(d) for the scaled variant, hstu.py:365-369).
    causal: keep j <= i.
    pos_bias: [2L-1] or [H, 2L-1] table; logit (i, j) gets
      pos_bias[(L-1) + j - i] (hstu.py:91-113).
    timestamps, ts_bias: int64 [B, L] (or jagged [T]) and [nb+1] or
      [H, nb+1]; logit (i, j) gets ts_bias[bucket(ts[i+1] - ts[j])]
      (hstu.py:190-221).  Jagged timestamps use the sequence's own last
      timestamp for its last row.
    q_segment_ids, kv_segment_ids: int [B, L] / [B, Lkv]; keep equal ids
      (recml/core/ops/hstu_ops.py:972-979).  Both or neither.
    sliding_window_size: keep |i - j| <= w (hstu_ops.py:940-945).
    mask: explicit keep-mask [L, Lkv] or [B, L, Lkv].
    bias: dense additive logit bias [L, Lkv] or [B, L, Lkv] shared by heads
      (hstu.py:373-374).
    out: optional preallocated output.
    dropout_p, dropout_seed: training-time dropout on the masked attention weights
      (hstu.py:386-387): each weight is dropped with probability dropout_p, the others are
      scaled by 1 / (1 - dropout_p).  Which pairs survive is a fixed function of
      (dropout_seed, sequence, head, i, j) -- `dropout_keep` gives it on the host -- so
      hstu_attention_bwd with the same two values differentiates exactly this output.
    batch: optional AttentionBatch shared by the calls on one batch (a model's layers): the first
      call prepares the work list, timestamps and tables, the later ones reuse them.

  Returns:
    Tensor shaped like q with v's head dim and v's dtype.
  """
  _check_gpu("q", q)
  _check_gpu("v", v)
  if out is None:
    shape = tuple(q.shape[:-1]) + (v.shape[-1],)
    out = torch.empty(shape, dtype=v.dtype, device=q.device)
  args, keep = build_args(
      q, k, v, out, seq_lens=seq_lens, seq_offsets=seq_offsets,
      max_len=max_len, n=n, alpha=alpha, causal=causal, pos_bias=pos_bias,
      timestamps=timestamps, ts_bias=ts_bias, ts_bucket_size=ts_bucket_size,
      q_segment_ids=q_segment_ids, kv_segment_ids=kv_segment_ids,
      sliding_window_size=sliding_window_size, mask=mask, bias=bias,
      q_scale=q_scale, k_scale=k_scale, batch=batch, dropout_p=dropout_p, dropout_seed=dropout_seed)
  with torch.cuda.device(q.device):
    _run(args, keep)
  if batch is not None:
    batch._commit()
  return out


def hstu_attention_bwd(q, k, v, dout, *, seq_lens=None, seq_offsets=None, max_len=None,
                       n=None, alpha=1.0, causal=True, pos_bias=None,
                       timestamps=None, ts_bias=None, ts_bucket_size=0.301,
                       q_segment_ids=None, kv_segment_ids=None,
                       sliding_window_size=None, mask=None, bias=None, dropout_p=0.0, dropout_seed=0,
                       table_grads=True, bias_grad=False, grads_out=None, _variant_out=None, _flags=0):
  """Gradients of sum(hstu_attention(q, k, v, ...) * dout).

  Same arguments as hstu_attention (fp32 or bf16; not fp8).  Returns
  (dq, dk, dv, dpos_bias, dts_bias): dq, dk, dv shaped and typed like q, k, v;
  the table gradients fp32 and shaped like the tables (None for a table that
  was not given, and for both with table_grads=False).  With bias_grad=True a
  sixth value: the gradient of the dense `bias`, fp32, shaped like it (summed
  over the heads, and over the batch when the bias is shared by it).
  `grads_out`: three tensors to take dq, dk, dv instead of new ones, each with
  the shape, dtype and strides of its input (the slices of the gradient of a
  fused projection, say).  Math of the reference's backward kernel
  (recml/core/ops/hstu_ops.py:417-548).
  """
  for name, t in (("q", q), ("k", k), ("v", v), ("dout", dout)):
    _check_gpu(name, t)
  if q.dtype not in (torch.float32, torch.bfloat16):
    raise ValueError(f"the backward takes float32 or bfloat16, got {q.dtype}")
  exp = tuple(q.shape[:-1]) + (v.shape[-1],)
  if tuple(dout.shape) != exp or dout.dtype != q.dtype:
    raise ValueError(f"dout must be a {q.dtype} tensor of shape {exp}")
  dout = dout if dout.stride(-1) == 1 else dout.contiguous()
  # (the forward struct's `out` is not read by the backward, which takes dout's strides from it: dout stands in)
  fa, keep = build_args(
      q, k, v, dout, seq_lens=seq_lens, seq_offsets=seq_offsets, max_len=max_len, n=n, alpha=alpha,
      causal=causal, pos_bias=pos_bias, timestamps=timestamps, ts_bias=ts_bias, ts_bucket_size=ts_bucket_size,
      q_segment_ids=q_segment_ids, kv_segment_ids=kv_segment_ids, sliding_window_size=sliding_window_size,
      mask=mask, bias=bias, dropout_p=dropout_p, dropout_seed=dropout_seed)
  # build_args may have made q, k, v contiguous in d: the gradients take the layout it passed on
  qi, ki, vi = _passed_inputs(keep)
  if grads_out is None:
    dq, dk, dv = _grad_buffers(qi, ki, vi)
  else:
    dq, dk, dv = grads_out
    for name, g, t in (("dq", dq, qi), ("dk", dk, ki), ("dv", dv, vi)):
      if g.shape != t.shape or g.dtype != t.dtype or g.stride() != t.stride() or g.device != t.device:
        raise ValueError(f"grads_out: {name} must have the shape, dtype and strides of its input as the kernels read it "
                         f"({tuple(t.shape)}, {t.dtype}, strides {t.stride()})")
  ba = _lib.HstuAttnBwdArgs()
  ba.struct_size = C.sizeof(_lib.HstuAttnBwdArgs)
  ba.version = _lib.ABI_VERSION
  fa.flags |= int(_flags)       # (comparison switches of the tests)
  ba.fwd = fa
  ba.dout, ba.dq, ba.dk, ba.dv = dout.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr()
  dpos = dts = None
  if pos_bias is not None and table_grads:
    dpos = torch.zeros((fa.pos_heads, 2 * fa.L - 1), dtype=torch.float32, device=q.device)
    ba.dpos_tab = dpos.data_ptr()
  if ts_bias is not None and table_grads:
    dts = torch.zeros((fa.ts_heads, fa.ts_num_buckets + 1), dtype=torch.float32, device=q.device)
    ba.dts_tab = dts.data_ptr()
  dbias = None
  if bias_grad:
    if bias is None:
      raise ValueError("bias_grad=True needs a dense `bias`")
    dbias = torch.zeros((fa.B if fa.dense_bias_batched else 1, fa.L, fa.Lkv), dtype=torch.float32, device=q.device)
    ba.ddense_bias = dbias.data_ptr()
  lib = _lib.load()
  if _variant_out is not None:
    _variant_out.append(lib.hstu_attn_bwd_variant(C.byref(ba)).decode())
  with torch.cuda.device(q.device):
    stream = torch.cuda.current_stream(q.device).cuda_stream
    rc = lib.hstu_attn_bwd(C.byref(ba), C.c_void_p(stream))
  if rc != 0:
    msg = lib.hstu_attn_last_error().decode()
    if rc in (-3, -4, -1):
      raise ValueError(f"hstu_attn_bwd rejected the arguments ({rc}): {msg}")
    raise RuntimeError(f"hstu_attn_bwd failed ({rc}): {msg}")
  del keep
  if dpos is not None:
    dpos = dpos.reshape(pos_bias.shape)
  if dts is not None:
    dts = dts.reshape(ts_bias.shape)
  if bias_grad:
    return dq, dk, dv, dpos, dts, dbias.reshape(bias.shape)
  return dq, dk, dv, dpos, dts


def dropout_keep(seed, p, b, h, H, i, j) -> bool:
  """Whether the weight of (sequence b, head h of H, query i, key j) survives dropout with this seed and
  rate: the library's own rule, evaluated on the host (no GPU needed)."""
  return bool(_lib.load().hstu_attn_dropout_keep(int(seed) & 0xFFFFFFFFFFFFFFFF, float(p), b, h, H, i, j))


def _grad_buffers(q, k, v):
  """dq, dk, dv with exactly the strides of q, k, v (the kernels write them so).  Slices of one fused
  projection (same storage, interleaved) get slices of ONE buffer laid out like that projection;
  mirrored one by one, each would span nearly the whole projection."""
  def extent(t):
    return sum((n - 1) * st for n, st in zip(t.shape, t.stride())) + 1 if t.numel() else 0
  ts = (q, k, v)
  if q.dtype == k.dtype == v.dtype and len({t.untyped_storage().data_ptr() for t in ts}) == 1 and all(t.numel() for t in ts):
    lo = min(t.storage_offset() for t in ts)
    hi = max(t.storage_offset() + extent(t) for t in ts)
    if hi - lo <= 2 * sum(t.numel() for t in ts):
      buf = torch.empty(hi - lo, dtype=q.dtype, device=q.device)
      return tuple(buf.as_strided(t.shape, t.stride(), t.storage_offset() - lo) for t in ts)
  # otherwise mirror each (empty_like would compact a view with gaps)
  return tuple(torch.empty_strided(t.shape, t.stride(), dtype=t.dtype, device=t.device) for t in ts)


class _HstuAttentionFn(torch.autograd.Function):
  """hstu_attention with gradients for q, k, v, the two bias tables and the dense bias."""

  @staticmethod
  def forward(ctx, q, k, v, pos_bias, ts_bias, bias, kwargs):
    ctx.kwargs = kwargs
    ctx.save_for_backward(q, k, v, *(t for t in (pos_bias, ts_bias, bias) if t is not None))
    ctx.has = (pos_bias is not None, ts_bias is not None, bias is not None)
    return hstu_attention(q, k, v, pos_bias=pos_bias, ts_bias=ts_bias, bias=bias, **kwargs)

  @staticmethod
  def backward(ctx, dout):
    saved = list(ctx.saved_tensors)
    q, k, v = saved[:3]
    rest = saved[3:]
    pos = rest.pop(0) if ctx.has[0] else None
    ts = rest.pop(0) if ctx.has[1] else None
    bias = rest.pop(0) if ctx.has[2] else None
    # needs_input_grad follows forward's arguments: q, k, v, pos_bias, ts_bias, bias, kwargs
    want_tables = (pos is not None and ctx.needs_input_grad[3]) or (ts is not None and ctx.needs_input_grad[4])
    want_bias = bias is not None and ctx.needs_input_grad[5]
    got = hstu_attention_bwd(q, k, v, dout.contiguous(), pos_bias=pos, ts_bias=ts, bias=bias,
                             table_grads=want_tables, bias_grad=want_bias, **ctx.kwargs)
    dq, dk, dv, dpos, dts = got[:5]
    cast = lambda g, t: None if g is None else g.to(t.dtype)
    return (dq, dk, dv, cast(dpos, pos) if pos is not None else None, cast(dts, ts) if ts is not None else None,
            cast(got[5], bias) if want_bias else None, None)


def _wants_grad(*tensors) -> bool:
  return torch.is_grad_enabled() and any(isinstance(t, torch.Tensor) and t.requires_grad for t in tensors)


def hstu_attention_autograd(q, k, v, *, pos_bias=None, ts_bias=None, bias=None, **kwargs):
  """hstu_attention as a differentiable torch op: gradients for q, k, v, the bias tables pos_bias
  and ts_bias, and a dense `bias` (its gradient is dS summed over the heads, and over the batch
  when the bias is shared by it)."""
  return _HstuAttentionFn.apply(q, k, v, pos_bias, ts_bias, bias, kwargs)


def pointwise_splash_attention(
    mask_type, q, k, v, *,
    q_segment_ids=None, kv_segment_ids=None, sliding_window_size=None,
    qkv_axis_names=(), segment_id_axis_names=(), scale=None,
    block_q=None, block_kv=None, block_kv_compute=None, block_q_dkv=None,
    block_kv_dkv=None, block_kv_dkv_compute=None, head_shards=1,
    q_seq_shards=1, downcast_smem_data=True, interpret=False):
  """Drop-in for recml/core/ops/hstu_ops.py:829-851 (forward).

  out = (silu(scale * q k^T) / q_len, masked) v with scale defaulting to
  1/sqrt(head_dim) (hstu_ops.py:909, 238).  `mask_type` is MaskType.CAUSAL,
  MaskType.FULL or an explicit boolean [q_len, kv_len] array.  The tile-size,
  sharding and interpret arguments belong to the TPU kernel and are accepted
  and ignored.  Differentiable like the reference's op (its custom_vjp,
  hstu_ops.py:417-548): when q, k or v asks for a gradient the call goes
  through the autograd function and the HIP backward kernels.
  """
  del qkv_axis_names, segment_id_axis_names, block_q, block_kv
  del block_kv_compute, block_q_dkv, block_kv_dkv, block_kv_dkv_compute
  del head_shards, q_seq_shards, downcast_smem_data, interpret
  _check_gpu("q", q)
  if q.dim() != 4:
    raise ValueError(f"q must be [batch, q_length, num_heads, head_dim], got {tuple(q.shape)}")
  bs, q_len, num_heads, head_dim = q.shape
  kv_len = v.shape[1] if v.dim() == 4 else -1
  for name, t in (("k", k), ("v", v)):
    if tuple(t.shape) != (bs, kv_len, num_heads, head_dim):
      raise ValueError(f"{name} shape {tuple(t.shape)} does not match {(bs, kv_len, num_heads, head_dim)}")
  explicit = None
  if isinstance(mask_type, (np.ndarray, torch.Tensor)):
    if tuple(mask_type.shape) != (q_len, kv_len):
      raise ValueError(
          f"Mask shape {tuple(mask_type.shape)} does not match query and key length ({q_len}, {kv_len}).")
    explicit, causal = mask_type, False
  elif mask_type == MaskType.CAUSAL:
    causal = True
  elif mask_type == MaskType.FULL:
    causal = False
  else:
    raise ValueError(f"Unsupported mask type: '{mask_type}'.")
  scale = scale if scale is not None else 1.0 / (head_dim**0.5)
  op = hstu_attention_autograd if _wants_grad(q, k, v) else hstu_attention
  return op(
      q, k, v, n=q_len, alpha=scale, causal=causal, mask=explicit,
      q_segment_ids=q_segment_ids, kv_segment_ids=kv_segment_ids,
      sliding_window_size=sliding_window_size)


def pointwise_attention(q, k, v, attention_mask, attention_bias=None, *,
                        scaled_pointwise_attn=False, seq_lens=None, batch=None,
                        dropout_p=0.0, dropout_seed=0):
  """Layer-side call, recml/layers/keras/hstu.py:356-390 (with dropout_p > 0 its training
  form: dropout on the masked weights, hstu.py:386-387).

  `attention_mask` is the [B, L, L] 0/1 mask the layer builds with
  make_causal_mask; `attention_bias` an optional [B or 1, L, L] additive bias
  shared by heads.  scaled_pointwise_attn=True divides q by sqrt(d) and skips
  the 1/L (hstu.py:365-378).  A caller that knows its batch is end-padded and
  causal can pass `seq_lens` with attention_mask=None: same result without
  ever building the [B, L, L] mask.  `batch`: an AttentionBatch shared by the
  calls that bring the same mask (the layers of a model): the mask is then
  scanned for its key-step ranges once, by the first of them (inference only).
  When q, k, v or the bias asks for a gradient the call goes through the
  autograd function (gradients by the HIP backward kernels, the bias's included).
  """
  d = q.shape[-1]
  alpha = 1.0 / math.sqrt(d) if scaled_pointwise_attn else 1.0
  n = 1.0 if scaled_pointwise_attn else q.shape[1]
  if attention_mask is None and seq_lens is None:
    raise ValueError("pass attention_mask or seq_lens")
  how = dict(seq_lens=seq_lens, causal=True) if attention_mask is None else dict(mask=attention_mask, causal=False)
  if _wants_grad(q, k, v, attention_bias):
    return hstu_attention_autograd(q, k, v, n=n, alpha=alpha, bias=attention_bias, dropout_p=dropout_p,
                                   dropout_seed=dropout_seed, **how)
  return hstu_attention(q, k, v, n=n, alpha=alpha, bias=attention_bias, batch=batch,
                        dropout_p=dropout_p, dropout_seed=dropout_seed, **how)
