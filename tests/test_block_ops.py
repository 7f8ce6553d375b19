"""The fused block steps (libhstu_block.so): ABI checks on the CPU, parity on the GPU."""

import ctypes as C
import os
import re
import subprocess
import tempfile

import numpy as np
import pytest
import torch

from oracle import hstu_block_oracle as BO
from recml_amd import _lib_block

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "hstu_block.h")


def test_library_exports_every_declared_symbol():
  lib = _lib_block.load()
  text = open(HEADER).read()
  text = text[text.index("#ifdef __cplusplus"):]          # skip the prose at the top
  names = sorted(set(re.findall(r"\b(hstu_\w+)\s*\(", text)))
  assert set(names) == set(_lib_block.EXPORTS)
  for n in names:
    assert getattr(lib, n) is not None
  assert lib.hstu_block_abi_version() == _lib_block.ABI_VERSION


@pytest.mark.parametrize("name", ["HstuNormGateArgs", "HstuNormGateBwdArgs", "HstuGemmSiluArgs", "HstuEmbedNormArgs"])
def test_struct_layout_matches_header(name):
  struct = getattr(_lib_block, name)
  fields = [f[0] for f in struct._fields_]
  prog = ['#include <stdio.h>', '#include <stddef.h>', '#include "hstu_block.h"', "int main(void) {",
          f'  printf("%zu\\n", sizeof({name}));']
  prog += [f'  printf("%zu\\n", offsetof({name}, {f}));' for f in fields]
  prog += ["  return 0;", "}"]
  with tempfile.TemporaryDirectory() as d:
    src, exe = os.path.join(d, "layout.c"), os.path.join(d, "layout")
    open(src, "w").write("\n".join(prog))
    subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), "-o", exe, src], check=True)
    out = subprocess.run([exe], check=True, capture_output=True, text=True).stdout.split()
  assert int(out[0]) == C.sizeof(struct)
  for f, off in zip(fields, out[1:]):
    assert getattr(struct, f).offset == int(off), f


def test_validation_errors_without_gpu():
  lib = _lib_block.load()
  assert lib.hstu_norm_gate_fwd(None, None) == -1
  a = _lib_block.HstuNormGateArgs()
  assert lib.hstu_norm_gate_fwd(C.byref(a), None) == -2
  a.struct_size, a.version = C.sizeof(a), _lib_block.ABI_VERSION
  a.rows, a.width = 4, 12
  assert lib.hstu_norm_gate_fwd(C.byref(a), None) == -4          # width not a multiple of 8
  a.width = 64
  assert lib.hstu_norm_gate_fwd(C.byref(a), None) == -1          # null tensors
  a.a = a.u = a.out = a.gamma = a.beta = 0x1000
  a.a_stride, a.u_stride, a.out_stride = 64, 60, 64
  assert lib.hstu_norm_gate_fwd(C.byref(a), None) == -4          # row stride below the width
  assert b"stride" in lib.hstu_block_last_error()
  a.rows = 0
  assert lib.hstu_norm_gate_fwd(C.byref(a), None) == 0           # nothing to do
  nb = _lib_block.HstuNormGateBwdArgs()
  assert lib.hstu_norm_gate_bwd(None, None) == -1
  assert lib.hstu_norm_gate_bwd(C.byref(nb), None) == -2
  nb.struct_size, nb.version = C.sizeof(nb), _lib_block.ABI_VERSION
  nb.rows, nb.width = 4, 4096
  assert lib.hstu_norm_gate_bwd(C.byref(nb), None) == -4         # the backward stops at width 2048
  nb.width = 64
  assert lib.hstu_norm_gate_bwd(C.byref(nb), None) == -1         # null outputs
  nb.a = nb.dout = nb.da = nb.gamma = nb.beta = nb.dgamma = nb.dbeta = nb.u = 0x1000
  nb.a_stride = nb.dout_stride = nb.da_stride = nb.u_stride = nb.du_stride = 64
  assert lib.hstu_norm_gate_bwd(C.byref(nb), None) == -1         # a gate without a place for its gradient
  nb.du = 0x1000
  assert lib.hstu_norm_gate_bwd(C.byref(nb), None) == -5         # no workspace
  assert lib.hstu_norm_gate_bwd_workspace_bytes(4, 64) == 1 * 2 * 64 * 4
  assert lib.hstu_norm_gate_bwd_workspace_bytes(10 ** 6, 512) == 1024 * 2 * 512 * 4
  g = _lib_block.HstuGemmSiluArgs()
  assert lib.hstu_gemm_silu_fwd(C.byref(g), None) == -2
  g.struct_size, g.version = C.sizeof(g), _lib_block.ABI_VERSION
  g.M, g.N, g.K, g.x_stride = 8, 16, 32, 16
  assert lib.hstu_gemm_silu_fwd(C.byref(g), None) == -4          # row stride below K
  g.x_stride, g.activation = 32, 7
  assert lib.hstu_gemm_silu_fwd(C.byref(g), None) == -4
  g.activation = 1
  assert lib.hstu_gemm_silu_fwd(C.byref(g), None) == -1          # null tensors
  assert lib.hstu_gemm_silu_workspace_bytes() > 0


def test_oracle_compositions_on_a_hand_case():
  # one row [1, 2, 3, 4]: mean 2.5, biased variance 1.25; gate u = [2, 0, -1, 1]
  a = np.array([[1.0, 2.0, 3.0, 4.0]])
  u = np.array([[2.0, 0.0, -1.0, 1.0]])
  z = (a - 2.5) / np.sqrt(1.25)
  assert np.allclose(BO.norm_gate(a, u, np.ones(4), np.zeros(4), 0.0), u * z, atol=1e-15)
  x, w = np.array([[1.0, -2.0]]), np.array([[0.5, 1.0], [0.25, -1.0]])
  y = np.array([[0.0, 3.0]]) + np.array([0.5, -1.0])              # x w + bias = [0.5, 2.0]
  assert np.allclose(BO.gemm_silu(x, w, np.array([0.5, -1.0]), False), y, atol=1e-15)
  assert np.allclose(BO.gemm_silu(x, w, np.array([0.5, -1.0])), y / (1 + np.exp(-y)), atol=1e-15)
  assert np.allclose(BO.gemm_silu(x, w, np.array([0.5, -1.0]), False, residual=np.array([[10.0, 20.0]])), y + [10.0, 20.0], atol=1e-15)
  table = np.array([[0.0, 0.0, 0.0, 0.0], [1.0, 2.0, 3.0, 4.0]])
  pos = np.array([[0.0, 0.0, 0.0, 0.0], [1.0, 1.0, 1.0, 1.0]])    # a constant row shifts the mean only
  got = BO.embed_norm(np.array([1, 1]), table, np.ones(4), np.zeros(4), 0.0, 2.0, np.array([0, 1]), pos)
  assert np.allclose(got, np.stack([z[0], z[0]]), atol=1e-15)      # scale 2 and the shift both cancel in the norm


@pytest.mark.parametrize("gated", [True, False])
def test_oracle_norm_gate_gradients_by_central_differences(gated):
  """Pins oracle.norm_gate_bwd: every entry of each gradient against a central difference of the forward
  restatement in fp64 (a dropped mean term, a wrong sign or a missing gamma shows at 1e-3 or more)."""
  rng = np.random.default_rng(3)
  R, W, eps = 3, 8, 1e-3
  a, u, do = rng.normal(size=(R, W)), rng.normal(size=(R, W)), rng.normal(size=(R, W))
  gm, bt = 1 + 0.3 * rng.normal(size=W), 0.2 * rng.normal(size=W)
  f = lambda a_, u_, g_, b_: float(((BO.norm_gate(a_, u_, g_, b_, eps) if gated else BO.layer_norm(a_, g_, b_, eps)) * do).sum())
  da, du, dg, db = BO.norm_gate_bwd(a, u if gated else None, gm, bt, do, eps)
  h = 1e-6
  def fd(which):
    base = [a, u, gm, bt]
    out = np.zeros_like(base[which])
    for idx in np.ndindex(out.shape):
      hi = [t.copy() for t in base]; lo = [t.copy() for t in base]
      hi[which][idx] += h; lo[which][idx] -= h
      out[idx] = (f(*hi) - f(*lo)) / (2 * h)
    return out
  assert np.allclose(da, fd(0), rtol=1e-6, atol=1e-7)
  assert np.allclose(dg, fd(2), rtol=1e-6, atol=1e-7)
  assert np.allclose(db, fd(3), rtol=1e-6, atol=1e-7)
  if gated:
    assert np.allclose(du, fd(1), rtol=1e-6, atol=1e-7)
  else:
    assert du is None


def _rel(a, b):
  return float((a - b).abs().max() / b.abs().max().clamp_min(1e-30))


@pytest.mark.gpu
@pytest.mark.parametrize("rows,width", [(1, 8), (37, 64), (513, 512), (64, 1000), (9, 4096), (3, 8192)])
def test_norm_gate_parity(gpu, rows, width):
  """Against the fp64 oracle on the same bf16 inputs: the fused step rounds once, at the end."""
  from recml_amd import hstu_block_ops as B
  gen = torch.Generator().manual_seed(rows * 7 + width)
  dev, bf = "cuda:0", torch.bfloat16
  fused = (torch.randn((rows, 4, width), generator=gen) * 0.7).to(dev).to(bf)
  u = fused[:, 1]                                              # a strided slice, as in the block
  attn = (torch.randn((rows, width), generator=gen) * 3e-3 + 1e-3).to(dev).to(bf)
  gamma = (1 + 0.2 * torch.randn(width, generator=gen)).to(dev).to(bf)
  beta = (0.1 * torch.randn(width, generator=gen)).to(dev).to(bf)
  out = B.norm_gate(attn, u, gamma, beta, 1e-6)
  n = lambda t: t.float().cpu().numpy()
  ref = torch.from_numpy(BO.norm_gate(n(attn), n(u), n(gamma), n(beta), 1e-6))
  assert out.shape == attn.shape and out.dtype == bf
  assert _rel(out.double().cpu(), ref) <= 8e-3                 # bf16 rounding of the result: 2^-8


@pytest.mark.gpu
@pytest.mark.parametrize("rows,width,gated", [(1, 8, True), (37, 64, True), (5000, 512, True), (4099, 512, False),
                                              (64, 1000, True), (131, 2048, True), (9, 1536, False)])
def test_norm_gate_gradients_parity(gpu, rows, width, gated):
  """The backward kernel against the fp64 oracle on the same bf16 inputs; the column sums bit for bit
  the same on a second run; the plain layer norm as the kernel without a gate; and through autograd."""
  from recml_amd import hstu_block_ops as B
  gen = torch.Generator().manual_seed(rows * 11 + width)
  dev, bf = "cuda:0", torch.bfloat16
  fused = (torch.randn((rows, 4, width), generator=gen) * 0.7).to(dev).to(bf)
  u = fused[:, 1] if gated else None
  attn = (torch.randn((rows, width), generator=gen) * 3e-3 + 1e-3).to(dev).to(bf)
  dout = (torch.randn((rows, width), generator=gen) * 0.5).to(dev).to(bf)
  gamma = (1 + 0.2 * torch.randn(width, generator=gen)).to(dev).to(bf)
  beta = (0.1 * torch.randn(width, generator=gen)).to(dev).to(bf)
  dfused = torch.zeros_like(fused)
  da, du, dg, db = B.norm_gate_bwd(attn, u, gamma, beta, dout, 1e-6, du_out=dfused[:, 1] if gated else None)
  n = lambda t: t.float().cpu().numpy()
  rda, rdu, rdg, rdb = BO.norm_gate_bwd(n(attn), n(u) if gated else None, n(gamma), n(beta), n(dout), 1e-6)
  assert da.dtype == bf and dg.dtype == torch.float32 and dg.shape == (width,)
  assert _rel(da.double().cpu(), torch.from_numpy(rda)) <= 8e-3          # one bf16 rounding at the end
  assert _rel(dg.double().cpu(), torch.from_numpy(rdg)) <= 1e-4          # fp32 sums of fp32 products
  assert _rel(db.double().cpu(), torch.from_numpy(rdb)) <= 1e-4
  if gated:
    assert du.data_ptr() == dfused[:, 1].data_ptr()
    assert _rel(du.double().cpu(), torch.from_numpy(rdu)) <= 8e-3
    assert float(dfused[:, 0].abs().max()) == 0 and float(dfused[:, 2:].abs().max()) == 0   # only the slice is written
  else:
    assert du is None
  again = B.norm_gate_bwd(attn, u, gamma, beta, dout, 1e-6)
  assert torch.equal(again[2], dg) and torch.equal(again[3], db) and torch.equal(again[0], da)
  # the differentiable ops
  leaves = [t.clone().requires_grad_(True) for t in ((attn, u, gamma, beta) if gated else (attn, gamma, beta))]
  out = B.norm_gate(*leaves, 1e-6) if gated else B.layer_norm(*leaves, 1e-6)
  ref_out = BO.norm_gate(n(attn), n(u), n(gamma), n(beta), 1e-6) if gated else BO.layer_norm(n(attn), n(gamma), n(beta), 1e-6)
  assert _rel(out.detach().double().cpu(), torch.from_numpy(ref_out)) <= 8e-3
  out.backward(dout)
  assert torch.equal(leaves[0].grad, da)
  assert _rel(leaves[-2].grad.double().cpu(), torch.from_numpy(rdg)) <= 8e-3 and leaves[-2].grad.dtype == bf
  assert _rel(leaves[-1].grad.double().cpu(), torch.from_numpy(rdb)) <= 8e-3
  if gated:
    assert torch.equal(leaves[1].grad, du)


@pytest.mark.gpu
@pytest.mark.parametrize("M,K,N,bias,act", [(1, 64, 64, False, True), (300, 512, 2048, True, True),
                                            (4097, 512, 2048, False, True), (129, 256, 1024, True, False)])
def test_gemm_silu_parity(gpu, M, K, N, bias, act):
  from recml_amd import hstu_block_ops as B
  gen = torch.Generator().manual_seed(M + N)
  dev, bf = "cuda:0", torch.bfloat16
  x = (torch.randn((M, K), generator=gen) * 0.5).to(dev).to(bf)
  w = (torch.randn((K, N), generator=gen) * 0.05).to(dev).to(bf)
  b = (torch.randn(N, generator=gen) * 0.1).to(dev).to(bf) if bias else None
  out = B.gemm_silu(x, w, b, act)
  n = lambda t: t.float().cpu().numpy()
  ref = torch.from_numpy(BO.gemm_silu(n(x), n(w), n(b) if bias else None, act))
  assert out.shape == (M, N) and out.dtype == bf
  assert _rel(out.double().cpu(), ref) <= 8e-3
  # a strided x (row stride 2K) gives the same values
  wide = torch.zeros((M, 2 * K), device=dev, dtype=bf)
  wide[:, :K] = x
  assert torch.equal(B.gemm_silu(wide[:, :K], w, b, act), out)
  # a residual as the product's C operand (a strided one too): added before bias and activation, and left as it was
  res = (torch.randn((M, N), generator=gen) * 0.5).to(dev).to(bf)
  keep = res.clone()
  got = B.gemm_silu(x, w, b, act, residual=res)
  ref = torch.from_numpy(BO.gemm_silu(n(x), n(w), n(b) if bias else None, act, residual=n(res)))
  assert _rel(got.double().cpu(), ref) <= 8e-3 and torch.equal(res, keep)
  wide_res = torch.zeros((M, 2 * N), device=dev, dtype=bf)
  wide_res[:, :N] = res
  assert torch.equal(B.gemm_silu(x, w, b, act, residual=wide_res[:, :N]), got)


@pytest.mark.gpu
@pytest.mark.parametrize("shape,width,vocab,with_pos,scale", [((5,), 8, 3, False, 1.0), ((4, 33), 512, 1000, True, 512 ** 0.5),
                                                               ((700,), 1000, 50, True, 1.0), ((3, 2), 4096, 9, False, 2.0)])
def test_embed_norm_parity(gpu, shape, width, vocab, with_pos, scale):
  from recml_amd import hstu_block_ops as B
  gen = torch.Generator().manual_seed(width + vocab)
  dev, bf = "cuda:0", torch.bfloat16
  wide = (torch.randn((vocab, width + 8), generator=gen) * 0.02).to(dev).to(bf)
  table = wide[:, :width]                                      # a table with a row stride of its own
  ids = torch.randint(0, vocab, shape, generator=gen).to(dev)
  gamma = (1 + 0.2 * torch.randn(width, generator=gen)).to(dev).to(bf)
  beta = (0.1 * torch.randn(width, generator=gen)).to(dev).to(bf)
  pos_table = positions = None
  if with_pos:
    pos_table = (torch.randn((40, width), generator=gen) * 0.02).to(dev).to(bf)
    positions = torch.randint(0, 40, shape, generator=gen).to(dev)
  out = B.embed_norm(ids, table, gamma, beta, 1e-6, scale=scale, positions=positions, pos_table=pos_table)
  n = lambda t: t.float().cpu().numpy()
  ref = torch.from_numpy(BO.embed_norm(ids.cpu().numpy(), n(table), n(gamma), n(beta), 1e-6, scale,
                                       positions.cpu().numpy() if with_pos else None, n(pos_table) if with_pos else None))
  assert out.shape == (*shape, width) and out.dtype == bf
  assert _rel(out.double().cpu(), ref) <= 8e-3
  # indices outside the table are clamped into it
  far = B.embed_norm(torch.full(shape, vocab + 5, device=dev), table, gamma, beta, 1e-6, scale=scale,
                     positions=positions, pos_table=pos_table)
  last = B.embed_norm(torch.full(shape, vocab - 1, device=dev), table, gamma, beta, 1e-6, scale=scale,
                      positions=positions, pos_table=pos_table)
  assert torch.equal(far, last)


@pytest.mark.gpu
def test_gemm_silu_takes_views_that_start_off_a_16_byte_boundary(gpu):
  # dense tensors whose first element sits 2 bytes into an allocation: the wrapper copies them for the library
  from recml_amd import hstu_block_ops as B
  gen = torch.Generator().manual_seed(3)
  dev, bf = "cuda:0", torch.bfloat16
  M, K, N = 130, 256, 512
  x = (torch.randn((M, K), generator=gen) * 0.5).to(dev).to(bf)
  w = (torch.randn((K, N), generator=gen) * 0.05).to(dev).to(bf)
  res = (torch.randn((M, N), generator=gen) * 0.5).to(dev).to(bf)

  def shifted(t):
    flat = torch.empty(t.numel() + 1, device=dev, dtype=bf)
    view = flat[1:].view(t.shape)
    view.copy_(t)
    assert view.is_contiguous() and view.data_ptr() % 16 != 0
    return view

  ref = B.gemm_silu(x, w, None, True, residual=res)
  assert torch.equal(B.gemm_silu(shifted(x), w, None, True, residual=res), ref)
  assert torch.equal(B.gemm_silu(x, shifted(w), None, True, residual=res), ref)
  assert torch.equal(B.gemm_silu(x, w, None, True, residual=shifted(res)), ref)


@pytest.mark.gpu
def test_layer_norm_gradient_width_is_checked_up_front(gpu):
  from recml_amd import hstu_block_ops as B
  dev, bf = "cuda:0", torch.bfloat16
  W = 4096
  x = torch.randn((3, W), device=dev).to(bf)
  g, b = torch.ones(W, device=dev, dtype=bf), torch.zeros(W, device=dev, dtype=bf)
  assert B.layer_norm(x, g, b).shape == (3, W)          # the forward alone takes this width
  with pytest.raises(ValueError, match="gradient of the layer norm"):
    B.layer_norm(x.requires_grad_(), g, b)
  with pytest.raises(ValueError, match="gradient of the layer norm"):
    B.norm_gate(x, x.detach(), g, b)
  with torch.no_grad():
    assert B.norm_gate(x, x, g, b).shape == (3, W)


@pytest.mark.gpu
def test_block_ops_argument_errors(gpu):
  from recml_amd import hstu_block_ops as B
  z = torch.zeros((4, 64), device="cuda:0", dtype=torch.bfloat16)
  with pytest.raises(ValueError, match="bfloat16"):
    B.norm_gate(z.float(), z, z[0], z[0])
  with pytest.raises(ValueError, match="differ in shape"):
    B.norm_gate(z, z[:2], z[0], z[0])
  with pytest.raises(ValueError, match="x \\[M, K\\]"):
    B.gemm_silu(z, z)
  with pytest.raises(ValueError, match="GPU tensor"):
    B.gemm_silu(z.cpu(), z.cpu().t())
