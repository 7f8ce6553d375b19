"""Host side of the fused block steps (libhstu_block.so): torch tensors in, HIP kernels behind the C ABI.

  norm_gate(attn, u, gamma, beta, eps)     u * layer_norm(attn)       recml/layers/keras/hstu.py:471-472
  gemm_silu(x, w, bias, activation)        silu(x @ w + bias)          recml/layers/keras/hstu.py:444-449
  embed_norm(ids, table, ...)              layer_norm(scale * table[ids] + pos_table[positions])   hstu.py:593-601

bf16 on a GPU only; there is no other implementation behind these names.
"""

from __future__ import annotations

import ctypes as C

import torch

from recml_amd import _lib_block

_workspaces = {}


def _check(name, t, dtype=torch.bfloat16):
  if not isinstance(t, torch.Tensor) or not t.is_cuda:
    raise ValueError(f"{name} must be a GPU tensor")
  if t.dtype != dtype:
    raise ValueError(f"{name} must be {dtype}, got {t.dtype}")


def _raise(lib, rc, what):
  msg = lib.hstu_block_last_error().decode()
  if rc in (-1, -4):
    raise ValueError(f"{what} rejected the arguments ({rc}): {msg}")
  raise RuntimeError(f"{what} failed ({rc}): {msg}")


def norm_gate(attn, u, gamma, beta, eps: float = 1e-6):
  """u * layer_norm(attn) over the last axis.  attn, u: [..., W] bf16 whose last axis is contiguous
  and whose leading axes collapse to one row stride (a slice of a fused projection does);
  gamma, beta: [W]."""
  for n, t in (("attn", attn), ("u", u), ("gamma", gamma), ("beta", beta)):
    _check(n, t)
  if attn.shape != u.shape:
    raise ValueError(f"attn {tuple(attn.shape)} and u {tuple(u.shape)} differ in shape")
  W = attn.shape[-1]
  a2, u2 = _rows(attn, "attn"), _rows(u, "u")
  out = torch.empty(attn.shape, dtype=attn.dtype, device=attn.device)
  a = _lib_block.HstuNormGateArgs()
  a.struct_size, a.version = C.sizeof(_lib_block.HstuNormGateArgs), _lib_block.ABI_VERSION
  a.rows, a.width, a.eps = a2.shape[0], W, float(eps)
  a.a, a.u, a.out = a2.data_ptr(), u2.data_ptr(), out.data_ptr()
  a.a_stride, a.u_stride, a.out_stride = a2.stride(0), u2.stride(0), W
  g, b = gamma.reshape(-1).contiguous(), beta.reshape(-1).contiguous()
  if g.numel() != W or b.numel() != W:
    raise ValueError(f"gamma and beta must have {W} entries")
  a.gamma, a.beta = g.data_ptr(), b.data_ptr()
  lib = _lib_block.load()
  with torch.cuda.device(attn.device):
    rc = lib.hstu_norm_gate_fwd(C.byref(a), C.c_void_p(torch.cuda.current_stream(attn.device).cuda_stream))
  if rc != 0:
    _raise(lib, rc, "hstu_norm_gate_fwd")
  return out


def _rows(t, name):
  """[..., W] -> a [rows, W] view with one row stride (a copy when the layout does not allow it)."""
  W = t.shape[-1]
  if t.stride(-1) != 1:
    t = t.contiguous()
  try:
    return t.view(-1, W) if t.dim() != 2 else t
  except RuntimeError:
    pass
  # leading axes of a strided slice: [T, W] slices are 2-d already; anything else is flattened by a copy
  return t.reshape(-1, W)


def gemm_silu(x, w, bias=None, activation: bool = True):
  """silu(x @ w + bias) (or without the activation): x [M, K] bf16 (row stride free), w [K, N] contiguous,
  bias [N] or None -> [M, N] bf16."""
  _check("x", x)
  _check("w", w)
  if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[0]:
    raise ValueError(f"x [M, K] and w [K, N] expected, got {tuple(x.shape)} and {tuple(w.shape)}")
  # the library wants 16-byte aligned operands and a row stride that keeps rows so
  if x.stride(1) != 1 or x.stride(0) % 8 or x.data_ptr() % 16:
    x = x.contiguous()
  w = w.contiguous()
  if w.data_ptr() % 16:
    w = w.clone()
  M, K = x.shape
  N = w.shape[1]
  out = torch.empty((M, N), dtype=x.dtype, device=x.device)
  lib = _lib_block.load()
  key = (x.device.index, torch.cuda.current_stream(x.device).cuda_stream)
  ws = _workspaces.get(key)
  if ws is None:
    ws = torch.empty(lib.hstu_gemm_silu_workspace_bytes(), dtype=torch.uint8, device=x.device)
    _workspaces[key] = ws
  a = _lib_block.HstuGemmSiluArgs()
  a.struct_size, a.version = C.sizeof(_lib_block.HstuGemmSiluArgs), _lib_block.ABI_VERSION
  a.M, a.N, a.K, a.activation = M, N, K, 1 if activation else 0
  a.x, a.x_stride, a.w, a.out = x.data_ptr(), x.stride(0), w.data_ptr(), out.data_ptr()
  if bias is not None:
    _check("bias", bias)
    bias = bias.reshape(-1).contiguous()
    if bias.numel() != N:
      raise ValueError(f"bias must have {N} entries")
    if bias.data_ptr() % 16:
      bias = bias.clone()
    a.bias = bias.data_ptr()
  a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel()
  with torch.cuda.device(x.device):
    rc = lib.hstu_gemm_silu_fwd(C.byref(a), C.c_void_p(torch.cuda.current_stream(x.device).cuda_stream))
  if rc != 0:
    _raise(lib, rc, "hstu_gemm_silu_fwd")
  return out


def embed_norm(ids, table, gamma, beta, eps: float = 1e-6, *, scale: float = 1.0, positions=None, pos_table=None):
  """layer_norm(scale * table[ids] + pos_table[positions]) over the last axis: ids [...] int64 -> [..., W] bf16.
  table [V, W] bf16 (row stride free), pos_table [P, W] bf16 with positions shaped like ids, or neither."""
  _check("table", table)
  _check("gamma", gamma)
  _check("beta", beta)
  _check("ids", ids, torch.int64)
  if table.dim() != 2 or table.stride(1) != 1:
    raise ValueError("table must be [V, W] with a contiguous last axis")
  if (positions is None) != (pos_table is None):
    raise ValueError("positions and pos_table go together")
  V, W = table.shape
  flat = ids.reshape(-1).contiguous()
  out = torch.empty((flat.numel(), W), dtype=table.dtype, device=table.device)
  a = _lib_block.HstuEmbedNormArgs()
  a.struct_size, a.version = C.sizeof(_lib_block.HstuEmbedNormArgs), _lib_block.ABI_VERSION
  a.rows, a.width, a.eps, a.scale = flat.numel(), W, float(eps), float(scale)
  a.ids, a.table, a.vocab, a.table_stride = flat.data_ptr(), table.data_ptr(), V, table.stride(0)
  keep = [flat]
  if pos_table is not None:
    _check("pos_table", pos_table)
    _check("positions", positions, torch.int64)
    if positions.shape != ids.shape or pos_table.dim() != 2 or pos_table.shape[1] != W:
      raise ValueError("positions must be shaped like ids and pos_table [P, W]")
    pt, pf = pos_table.contiguous(), positions.reshape(-1).contiguous()
    keep += [pt, pf]
    a.positions, a.pos_table, a.n_positions = pf.data_ptr(), pt.data_ptr(), pt.shape[0]
  g, b = gamma.reshape(-1).contiguous(), beta.reshape(-1).contiguous()
  if g.numel() != W or b.numel() != W:
    raise ValueError(f"gamma and beta must have {W} entries")
  a.gamma, a.beta, a.out = g.data_ptr(), b.data_ptr(), out.data_ptr()
  lib = _lib_block.load()
  with torch.cuda.device(table.device):
    rc = lib.hstu_embed_norm_fwd(C.byref(a), C.c_void_p(torch.cuda.current_stream(table.device).cuda_stream))
  if rc != 0:
    _raise(lib, rc, "hstu_embed_norm_fwd")
  del keep
  return out.reshape(*ids.shape, W)
