"""Host side of the fused block steps (libhstu_block.so): torch tensors in, HIP kernels behind the C ABI.

  norm_gate(attn, u, gamma, beta, eps)     u * layer_norm(attn)       recml/layers/keras/hstu.py:471-472
  layer_norm(x, gamma, beta, eps)          the same kernels without the gate                     hstu.py:442
  norm_gate_bwd(...)                       their gradients (norm_gate and layer_norm are differentiable)
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


def _norm_gate_fwd(attn, u, gamma, beta, eps):
  """The forward kernel: u * layer_norm(attn), or layer_norm(attn) with u=None."""
  for n, t in (("attn", attn), ("gamma", gamma), ("beta", beta)) + ((("u", u),) if u is not None else ()):
    _check(n, t)
  if u is not None and attn.shape != u.shape:
    raise ValueError(f"attn {tuple(attn.shape)} and u {tuple(u.shape)} differ in shape")
  W = attn.shape[-1]
  a2 = _rows(attn, "attn")
  u2 = _rows(u, "u") if u is not None else None
  out = torch.empty(attn.shape, dtype=attn.dtype, device=attn.device)
  a = _lib_block.HstuNormGateArgs()
  a.struct_size, a.version = C.sizeof(_lib_block.HstuNormGateArgs), _lib_block.ABI_VERSION
  a.rows, a.width, a.eps = a2.shape[0], W, float(eps)
  a.a, a.out = a2.data_ptr(), out.data_ptr()
  a.a_stride, a.out_stride = a2.stride(0), W
  if u2 is not None:
    a.u, a.u_stride = u2.data_ptr(), u2.stride(0)
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


def norm_gate_bwd(attn, u, gamma, beta, dout, eps: float = 1e-6, *, du_out=None):
  """Gradients of u * layer_norm(attn) (of layer_norm(attn) with u=None) for the gradient `dout` of the
  result: (d_attn, d_u, d_gamma, d_beta); d_attn and d_u bf16 shaped like attn, d_gamma and d_beta fp32
  [W], summed over the rows in a fixed order.  `du_out`: where to write d_u (a slice of the gradient
  of a fused projection, say) instead of a new tensor.  W up to 2048."""
  for n, t in (("attn", attn), ("gamma", gamma), ("beta", beta), ("dout", dout)) + ((("u", u),) if u is not None else ()):
    _check(n, t)
  if dout.shape != attn.shape or (u is not None and u.shape != attn.shape):
    raise ValueError(f"attn {tuple(attn.shape)}, u and dout must have one shape")
  W = attn.shape[-1]
  a2, g2 = _rows(attn, "attn"), _rows(dout, "dout")
  da = torch.empty(attn.shape, dtype=attn.dtype, device=attn.device)
  a = _lib_block.HstuNormGateBwdArgs()
  a.struct_size, a.version = C.sizeof(_lib_block.HstuNormGateBwdArgs), _lib_block.ABI_VERSION
  a.rows, a.width, a.eps = a2.shape[0], W, float(eps)
  a.a, a.dout, a.da = a2.data_ptr(), g2.data_ptr(), da.data_ptr()
  a.a_stride, a.dout_stride, a.da_stride = a2.stride(0), g2.stride(0), W
  du = None
  if u is not None:
    u2 = _rows(u, "u")
    if du_out is None:
      du = torch.empty(attn.shape, dtype=attn.dtype, device=attn.device)
    else:
      _check("du_out", du_out)
      du = du_out
      if du.shape != attn.shape or du.stride(-1) != 1:
        raise ValueError("du_out must be shaped like attn with a contiguous last axis")
    d2 = du if du.dim() == 2 else du.view(-1, W)     # raises if the leading axes do not collapse: a copy would lose the writes
    a.u, a.u_stride, a.du, a.du_stride = u2.data_ptr(), u2.stride(0), d2.data_ptr(), d2.stride(0)
  g, b = gamma.reshape(-1).contiguous(), beta.reshape(-1).contiguous()
  if g.numel() != W or b.numel() != W:
    raise ValueError(f"gamma and beta must have {W} entries")
  a.gamma, a.beta = g.data_ptr(), b.data_ptr()
  dgb = torch.empty((2, W), dtype=torch.float32, device=attn.device)
  a.dgamma, a.dbeta = dgb[0].data_ptr(), dgb[1].data_ptr()
  lib = _lib_block.load()
  ws = torch.empty(max(lib.hstu_norm_gate_bwd_workspace_bytes(a2.shape[0], W), 16), dtype=torch.uint8, device=attn.device)
  a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel()
  with torch.cuda.device(attn.device):
    rc = lib.hstu_norm_gate_bwd(C.byref(a), C.c_void_p(torch.cuda.current_stream(attn.device).cuda_stream))
  if rc != 0:
    _raise(lib, rc, "hstu_norm_gate_bwd")
  return da, du, dgb[0], dgb[1]


class _NormGateFn(torch.autograd.Function):
  """u * layer_norm(attn) (u=None: layer_norm(attn)) with its gradients, both through the HIP kernels."""

  @staticmethod
  def forward(ctx, attn, u, gamma, beta, eps):
    ctx.eps = eps
    ctx.gated = u is not None
    ctx.save_for_backward(attn, gamma, beta, *((u,) if u is not None else ()))
    return _norm_gate_fwd(attn, u, gamma, beta, eps)

  @staticmethod
  def backward(ctx, dout):
    attn, gamma, beta, *rest = ctx.saved_tensors
    u = rest[0] if ctx.gated else None
    dout = dout if dout.stride(-1) == 1 else dout.contiguous()
    da, du, dg, db = norm_gate_bwd(attn, u, gamma, beta, dout, ctx.eps)
    return da, du, dg.to(gamma.dtype).reshape(gamma.shape), db.to(beta.dtype).reshape(beta.shape), None


def _wants_grad(*ts):
  return torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in ts)


NORM_GATE_BWD_MAX_WIDTH = 2048     # widest row hstu_norm_gate_bwd takes (the forward kernel: 8192)


def _check_grad_width(W):
  if W > NORM_GATE_BWD_MAX_WIDTH:
    raise ValueError(f"the gradient of the layer norm is there for rows of up to {NORM_GATE_BWD_MAX_WIDTH} elements, got {W}: "
                     "run the forward under torch.no_grad(), or use torch.nn.functional.layer_norm for this width")


def norm_gate(attn, u, gamma, beta, eps: float = 1e-6):
  """u * layer_norm(attn) over the last axis.  attn, u: [..., W] bf16 whose last axis is contiguous
  and whose leading axes collapse to one row stride (a slice of a fused projection does);
  gamma, beta: [W].  Differentiable in all four (W up to 2048 then: wider rows with a gradient wanted
  raise here, not at backward time)."""
  if _wants_grad(attn, u, gamma, beta):
    _check_grad_width(attn.shape[-1])
    return _NormGateFn.apply(attn, u, gamma, beta, eps)
  return _norm_gate_fwd(attn, u, gamma, beta, eps)


def layer_norm(x, gamma, beta, eps: float = 1e-6):
  """layer_norm(x) over the last axis (keras LayerNormalization as the block's input norm uses it,
  recml/layers/keras/hstu.py:442): the same kernels without the gate.  Differentiable in x, gamma, beta."""
  if _wants_grad(x, gamma, beta):
    _check_grad_width(x.shape[-1])
    return _NormGateFn.apply(x, None, gamma, beta, eps)
  return _norm_gate_fwd(x, None, gamma, beta, eps)


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


def gemm_silu(x, w, bias=None, activation: bool = True, residual=None):
  """silu(x @ w + bias) (or without the activation): x [M, K] bf16 (row stride free), w [K, N] contiguous,
  bias [N] or None -> [M, N] bf16.  `residual` [M, N] bf16 (row stride free) is added to the product as
  its C operand, before bias and activation: the block's `+ inputs` without a pass (or a copy) of its own."""
  _check("x", x)
  _check("w", w)
  if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[0]:
    raise ValueError(f"x [M, K] and w [K, N] expected, got {tuple(x.shape)} and {tuple(w.shape)}")
  # the library wants 16-byte aligned operands and a row stride that keeps rows so
  # (`contiguous()` returns a dense tensor as it is, misaligned or not: a view that starts off a 16-byte
  # boundary needs a copy of its own)
  if x.stride(1) != 1 or x.stride(0) % 8:
    x = x.contiguous()
  if x.data_ptr() % 16:
    x = x.clone(memory_format=torch.contiguous_format)
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
  if residual is not None:
    _check("residual", residual)
    if tuple(residual.shape) != (M, N):
      raise ValueError(f"residual must be [{M}, {N}], got {tuple(residual.shape)}")
    if residual.stride(1) != 1 or residual.stride(0) % 8:
      residual = residual.contiguous()
    if residual.data_ptr() % 16:
      residual = residual.clone(memory_format=torch.contiguous_format)
    a.c, a.c_stride = residual.data_ptr(), residual.stride(0)
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
