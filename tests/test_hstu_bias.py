"""Bias producer modules: dense form against the oracle (CPU), fused form and table gradients on the GPU."""

import numpy as np
import pytest
import torch

from oracle import hstu_oracle as O
from dense_torch import dense_attention_torch
from recml_amd import hstu_bias


def test_dense_forms_match_the_oracle():
  g = torch.Generator().manual_seed(0)
  n = 9
  pos = hstu_bias.RelativePositionalBias(16, generator=g)
  ts = torch.tensor([[100, 160, 400, 4000, 4001, 9000, 9000, 20000, 10 ** 9 + 5]])
  dense = pos(ts).detach().numpy()
  w = pos._pos_biases.detach().numpy()
  assert dense.shape == (1, n, n)
  assert np.array_equal(dense, O.rel_pos_bias_recipe(w, n).astype(np.float32))      # the reference's own recipe
  both = hstu_bias.RelativeBucketedTimeAndPositionBasedBias(16, generator=g)
  want = O.rel_pos_bias(both._positional_bias._pos_biases.detach().numpy(), n) + \
      O.time_bias(ts.numpy(), both._ts_w.detach().numpy())
  assert np.allclose(both(ts).detach().numpy(), want, atol=0, rtol=0)
  assert np.array_equal(hstu_bias.default_bucketization(torch.tensor([0, 1, 2, 3, 10, 3600, 86400, 10 ** 9, -7])).numpy(),
                        O.default_bucketization(np.array([0, 1, 2, 3, 10, 3600, 86400, 10 ** 9, -7])))
  # a custom bucketization cannot be fused: the dense bias is handed over instead
  sq = hstu_bias.RelativeBucketedTimeAndPositionBasedBias(16, bucketization_fn=lambda x: x.abs().float().sqrt().long(), generator=g)
  assert set(sq.attention_kwargs(ts)) == {"bias"} and set(both.attention_kwargs(ts)) == {"pos_bias", "timestamps", "ts_bias"}


@pytest.mark.gpu
def test_fused_bias_and_table_gradients(gpu):
  import recml_amd
  g = torch.Generator().manual_seed(1)
  B, L, H, d = 2, 48, 2, 32
  mod = hstu_bias.RelativeBucketedTimeAndPositionBasedBias(L, stddev=0.3, device="cuda:0", generator=g)
  rnd = lambda *s: (torch.randn(s, generator=g) * 0.4).to("cuda:0")
  q, k, v, dout = rnd(B, L, H, d), rnd(B, L, H, d), rnd(B, L, H, d), rnd(B, L, H, d)
  ts = (1_600_000_000 + torch.cumsum(torch.randint(1, 20000, (B, L), generator=g), dim=1)).to("cuda:0")
  lens = torch.tensor([48, 30], device="cuda:0")
  out = recml_amd.hstu_attention_autograd(q, k, v, seq_lens=lens, **mod.attention_kwargs(ts))
  (out * dout).sum().backward()
  # the same through the dense bias tensor and torch autograd on the reference formulation
  ref_mod = hstu_bias.RelativeBucketedTimeAndPositionBasedBias(L, device="cuda:0", generator=g)
  ref_mod.load_state_dict(mod.state_dict())
  s = torch.einsum("bthd,bshd->bhts", q, k) + ref_mod(ts)[:, None]
  keep = torch.tril(torch.ones(L, L, device="cuda:0", dtype=torch.bool))[None] & \
      (torch.arange(L, device="cuda:0")[None, :, None] < lens[:, None, None]) & (torch.arange(L, device="cuda:0")[None, None, :] < lens[:, None, None])
  p = torch.where(keep[:, None], torch.nn.functional.silu(s) / L, torch.zeros_like(s))
  ref = torch.einsum("bhts,bshd->bthd", p, v)
  assert float((out - ref).detach().abs().max() / ref.detach().abs().max()) <= 1e-5
  (ref * dout).sum().backward()
  for name in ("_ts_w", "_positional_bias._pos_biases"):
    a = dict(mod.named_parameters())[name].grad
    b = dict(ref_mod.named_parameters())[name].grad
    assert float((a - b).abs().max() / b.abs().max()) <= 2e-5, name


@pytest.mark.gpu
def test_custom_bucketization_keeps_the_table_gradient(gpu):
  """A custom bucketization function cannot be fused as a table: the module hands the block a dense bias, and
  the bias weights still receive their gradient -- through the attention's backward kernels, which return the
  gradient of a dense bias -- with frozen block weights too; against the same block with the op in plain torch."""
  import torch
  from recml_amd import hstu_bias, hstu_ops
  from recml_amd.hstu_layer import HSTUBlock
  dev = torch.device("cuda:0")
  gen = torch.Generator().manual_seed(0)
  B, L, D, H = 2, 140, 32, 2
  sqrt_buckets = lambda x: torch.sqrt(x.abs().clamp(1, int(1e9)).double() / 3600.0).to(torch.int64)
  mod = hstu_bias.RelativeBucketedTimeAndPositionBasedBias(L, num_buckets=16, bucketization_fn=sqrt_buckets, device=dev,
                                                           generator=gen)
  ts = torch.cumsum(torch.randint(1, 20000, (B, L), generator=gen), dim=1).to(dev)
  blk = HSTUBlock(D, H, device=dev, generator=gen)
  for p in blk.parameters():
    p.requires_grad_(False)
  x = torch.randn((B, L, D), generator=gen).to(dev)
  lens = torch.tensor([L, 77], device=dev)

  def grads(fused):
    saved = hstu_ops.hstu_attention_autograd
    if not fused:
      hstu_ops.hstu_attention_autograd = lambda q, k, v, **kw: dense_attention_torch(q, k, v, **kw)
    try:
      for p in mod.parameters():
        p.grad = None
      kw = mod.attention_kwargs(ts)
      assert set(kw) == {"bias"} and kw["bias"].requires_grad
      out = blk(x, seq_lens=lens, attention_bias=kw["bias"])
      out.square().sum().backward()
      return mod._ts_w.grad.clone(), mod._positional_bias._pos_biases.grad.clone()
    finally:
      hstu_ops.hstu_attention_autograd = saved

  got, want = grads(True), grads(False)
  for g, w in zip(got, want):
    assert float(w.abs().max()) > 0
    assert float((g - w).abs().max() / w.abs().max()) <= 2e-4


def test_dense_attention_in_plain_torch_equals_the_oracle():
  import torch
  from recml_amd import hstu_bias, hstu_ops
  B, L, H = 2, 12, 2
  torch.manual_seed(0)
  mod = hstu_bias.RelativeBucketedTimeAndPositionBasedBias(L, num_buckets=16)
  ts = torch.cumsum(torch.randint(1, 20000, (B, L)), dim=1)
  from oracle import hstu_oracle as O
  q, k, v = (torch.randn(B, L, H, 8) for _ in range(3))
  lens = np.array([L, 7])
  tsw, dense = torch.randn(17), torch.randn(B, L, L) * 0.1
  pos = mod._positional_bias.table(L).detach()
  got = dense_attention_torch(q, k, v, seq_lens=torch.from_numpy(lens), pos_bias=pos, timestamps=ts, ts_bias=tsw,
                                       bias=dense).numpy()
  want = O.hstu_attention_ref(q.numpy(), k.numpy(), v.numpy(), seq_lens=lens, pos_tab=pos.numpy(), timestamps=ts.numpy(),
                              ts_tab=tsw.numpy(), bias=dense.numpy())
  assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max()
  assert (got[1, 7:] == 0).all()
