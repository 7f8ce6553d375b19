"""HSTU block / model harness: the oracle's pieces pinned on the CPU, the torch
harness (with the HIP attention inside) against the oracle on the GPU."""

import numpy as np
import pytest
import torch

from oracle import hstu_block_oracle as BO
from oracle import hstu_oracle as O
from dense_torch import dense_attention_torch


def test_layer_norm_definition_and_torch():
  # hand case: x = [1, 2, 3, 4]: mean 2.5, biased var 1.25
  x = np.array([[1.0, 2.0, 3.0, 4.0]])
  got = BO.layer_norm(x, np.ones(4), np.zeros(4), 0.0)
  assert np.allclose(got, (x - 2.5) / np.sqrt(1.25), rtol=0, atol=1e-15)
  got = BO.layer_norm(x, np.array([2.0, 2, 2, 2]), np.array([1.0, 1, 1, 1]), 1e-6)
  assert np.allclose(got, 2 * (x - 2.5) / np.sqrt(1.25 + 1e-6) + 1, atol=1e-15)
  # joint normalisation over two axes == normalisation of the flattened vector
  rng = np.random.default_rng(0)
  y = rng.standard_normal((3, 5, 4, 8))
  g, b = rng.standard_normal((4, 8)), rng.standard_normal((4, 8))
  two = BO.layer_norm(y, g, b, 1e-6, axes=(-2, -1))
  flat = BO.layer_norm(y.reshape(3, 5, 32), g.reshape(32), b.reshape(32), 1e-6).reshape(y.shape)
  assert np.allclose(two, flat, atol=1e-14)
  # an independent implementation
  t = torch.nn.functional.layer_norm(torch.from_numpy(y.reshape(3, 5, 32)), (32,), torch.from_numpy(g.reshape(32)),
                                     torch.from_numpy(b.reshape(32)), 1e-6).numpy().reshape(y.shape)
  assert np.allclose(two, t, atol=1e-12)


def test_param_count_matches_reference_literal():
  # recml/layers/keras/hstu_test.py:38-48 with vocab 500, positions 20, dim 32, 3 layers
  want = (500 * 32) + (20 * 32) + 3 * ((32 * 32 * 4 + 32 * 32) + (2 * 32) * 2) + (2 * 32) + (500 * 32)
  assert BO.hstu_param_count(500, 20, 32, 3) == want
  from recml_amd.hstu_layer import HSTU
  m = HSTU(vocab_size=500, max_positions=20, model_dim=32, num_heads=4, num_layers=3, dropout=0.1)
  assert m.count_params() == want
  with pytest.raises(ValueError, match="padding_mask"):
    m(torch.zeros((2, 3), dtype=torch.long))
  with pytest.raises(NotImplementedError):
    from recml_amd.hstu_layer import HSTUBlock
    HSTUBlock(32, 4, softmax_attention=True)


def test_block_oracle_padded_rows_and_independence():
  # padded rows: attention output 0 -> LN gives beta -> out = W(u * beta) + x; sequences independent
  rng = np.random.default_rng(1)
  B, L, D, H = 2, 6, 16, 2
  w = _rand_block(rng, D, H)
  x = rng.standard_normal((B, L, D))
  lens = np.array([6, 3])
  out = BO.hstu_block(x, w, num_heads=H, seq_lens=lens)
  normed = BO.layer_norm(x, w["input_ln_gamma"], w["input_ln_beta"], 1e-6)
  u = O.silu(np.einsum("btd,dnh->btnh", normed, w["u_kernel"]))
  pad = np.einsum("btnh,nhd->btd", u * w["attn_ln_beta"], w["output_kernel"]) + x
  assert np.allclose(out[1, 3:], pad[1, 3:], atol=1e-12)
  x2 = x.copy()
  x2[0] += 1.0
  out2 = BO.hstu_block(x2, w, num_heads=H, seq_lens=lens)
  assert np.array_equal(out2[1], out[1])
  # causality: changing a later token leaves earlier rows alone
  x3 = x.copy()
  x3[0, 4] += 1.0
  out3 = BO.hstu_block(x3, w, num_heads=H, seq_lens=lens)
  assert np.allclose(out3[0, :4], out[0, :4], atol=1e-13) and not np.allclose(out3[0, 4:], out[0, 4:])


def _rand_block(rng, D, H, bias=False):
  hd = D // H
  w = {f"{n}_kernel": rng.standard_normal((D, H, hd)) / np.sqrt(D) for n in "uqkv"}
  w["output_kernel"] = rng.standard_normal((H, hd, D)) / np.sqrt(D)
  w["input_ln_gamma"] = 1 + 0.1 * rng.standard_normal(D)
  w["input_ln_beta"] = 0.1 * rng.standard_normal(D)
  w["attn_ln_gamma"] = 1 + 0.1 * rng.standard_normal((H, hd))
  w["attn_ln_beta"] = 0.1 * rng.standard_normal((H, hd))
  if bias:
    for n in "uqkv":
      w[f"{n}_bias"] = 0.1 * rng.standard_normal((H, hd))
    w["output_bias"] = 0.1 * rng.standard_normal(D)
  return w


def _load_block(block, w, dtype):
  name_map = {"output_kernel": "output_kernel", "output_bias": "output_bias"}
  for k, val in w.items():
    getattr(block, name_map.get(k, k)).data = torch.from_numpy(np.asarray(val)).to(device="cuda:0", dtype=dtype)


def test_block_dropout_arguments_follow_the_mode():
  # recml/layers/keras/hstu.py:386-387 drops attention weights when training and only then
  from recml_amd.hstu_layer import HSTUBlock
  with pytest.raises(ValueError, match="dropout"):
    HSTUBlock(32, 2, dropout=1.0)
  blk = HSTUBlock(32, 2, dropout=0.1)
  assert blk.training
  assert blk._dropout_kw(5) == dict(dropout_p=0.1, dropout_seed=5)
  torch.manual_seed(3)
  a, b = blk._dropout_kw(), blk._dropout_kw()
  torch.manual_seed(3)
  assert blk._dropout_kw() == a and a != b and a["dropout_p"] == 0.1 and 0 <= a["dropout_seed"] < 2 ** 62
  blk.eval()
  assert blk._dropout_kw() == {} and blk._dropout_kw(5) == {}
  assert HSTUBlock(32, 2)._dropout_kw(5) == {}


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 3e-2)])
def test_block_in_training_mode_drops_attention_weights(gpu, dtype, tol):
  """A block with a dropout rate: in training mode its output is the oracle's block with the same rate and seed
  (padded and packed); the seed it draws follows torch's generator; in eval mode, where the reference applies no
  dropout either, the output is that of a block without a rate.  The model adds dropout on the embeddings."""
  import recml_amd
  from recml_amd.hstu_layer import HSTUBlock
  dev = "cuda:0"
  rng = np.random.default_rng(12)
  B, L, D, H = 3, 150, 128, 2
  lens = np.array([150, 40, 97], dtype=np.int32)
  w = _rand_block(rng, D, H)
  blk = HSTUBlock(D, H, dropout=0.3, dtype=dtype, device=dev)
  plain = HSTUBlock(D, H, dtype=dtype, device=dev)
  _load_block(blk, w, dtype)
  _load_block(plain, w, dtype)
  rd = lambda a: torch.from_numpy(np.asarray(a)).to(device=dev, dtype=dtype).double().cpu().numpy()
  wq = {k: rd(v) for k, v in w.items()}
  xq = rd(rng.standard_normal((B, L, D)))
  pos = 0.1 * rng.standard_normal(2 * L - 1)
  x, lt, pt = torch.from_numpy(xq).to(device=dev, dtype=dtype), torch.from_numpy(lens).to(dev), torch.from_numpy(pos).float().to(dev)
  assert blk.training
  ref = BO.hstu_block(xq, wq, num_heads=H, seq_lens=lens, pos_tab=pos, dropout_p=0.3, dropout_seed=77)
  base = BO.hstu_block(xq, wq, num_heads=H, seq_lens=lens, pos_tab=pos)
  assert np.abs(ref - base).max() > 0.05 * np.abs(base).max()          # the case tells the two apart
  out = blk(x, seq_lens=lt, pos_bias=pt, dropout_seed=77).double().cpu().numpy()
  for b in range(B):
    assert np.abs(out[b, :lens[b]] - ref[b, :lens[b]]).max() <= tol * np.abs(ref).max(), b
  # packed tokens: the same pattern (it is a function of the sequence's index and the positions within it)
  off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
  xj = torch.cat([x[b, :lens[b]] for b in range(B)])
  outj = blk.forward_jagged(xj, torch.from_numpy(off).to(dev), L, pos_bias=pt, dropout_seed=77).double().cpu().numpy()
  for b in range(B):
    assert np.abs(outj[off[b]:off[b + 1]] - ref[b, :lens[b]]).max() <= tol * np.abs(ref).max(), b
  # seeds drawn from torch's generator: repeatable under manual_seed, different from call to call
  torch.manual_seed(5)
  o1, o2 = blk(x, seq_lens=lt, pos_bias=pt), blk(x, seq_lens=lt, pos_bias=pt)
  torch.manual_seed(5)
  assert torch.equal(blk(x, seq_lens=lt, pos_bias=pt), o1) and not torch.equal(o1, o2)
  blk.eval()
  assert torch.equal(blk(x, seq_lens=lt, pos_bias=pt), plain(x, seq_lens=lt, pos_bias=pt))
  assert torch.equal(blk(x, seq_lens=lt, pos_bias=pt, dropout_seed=77), plain(x, seq_lens=lt, pos_bias=pt))
  if dtype == torch.bfloat16:
    model = recml_amd.HSTU(vocab_size=50, max_positions=L, model_dim=D, num_heads=H, num_layers=2, dropout=0.2,
                           dtype=dtype, device=dev, add_head=False)
    ids = torch.randint(0, 50, (B, L), device=dev)
    torch.manual_seed(1)                # (seeds torch's CPU generator, where the blocks draw, and the GPU's, where F.dropout does)
    t1 = model(ids, seq_lens=lt)
    t2 = model(ids, seq_lens=lt)
    torch.manual_seed(1)
    t3 = model(ids, seq_lens=lt)
    assert t1.shape == (B, L, D) and torch.equal(t1, t3) and not torch.equal(t1, t2) and bool(torch.isfinite(t1.float()).all())
    model.eval()
    with torch.no_grad():
      e1, e2 = model(ids, seq_lens=lt), model(ids, seq_lens=lt)
    assert torch.equal(e1, e2) and not torch.equal(e1, t1)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 3e-2)])
def test_block_on_gpu_against_oracle(gpu, dtype, tol):
  from recml_amd.hstu_layer import HSTUBlock
  rng = np.random.default_rng(2)
  B, L, D, H = 3, 70, 128, 2
  lens = np.array([70, 33, 1], dtype=np.int32)
  for use_bias, scaled in ((False, False), (True, True)):
    w = _rand_block(rng, D, H, bias=use_bias)
    x = rng.standard_normal((B, L, D))
    pos = 0.1 * rng.standard_normal(2 * L - 1)
    blk = HSTUBlock(D, H, use_bias=use_bias, scaled_pointwise_attn=scaled, dtype=dtype, device="cuda:0")
    _load_block(blk, w, dtype)
    rd = lambda a: torch.from_numpy(np.asarray(a)).to(device="cuda:0", dtype=dtype).double().cpu().numpy()
    wq = {k: rd(v) for k, v in w.items()}          # the oracle sees the weights as stored
    xq = rd(x)
    ref = BO.hstu_block(xq, wq, num_heads=H, seq_lens=lens, scaled_pointwise_attn=scaled, pos_tab=pos)
    out = blk(torch.from_numpy(xq).to(device="cuda:0", dtype=dtype), seq_lens=torch.from_numpy(lens).cuda(),
              pos_bias=torch.from_numpy(pos).float().cuda()).double().cpu().numpy()
    assert np.abs(out - ref).max() / np.abs(ref).max() <= tol
    # the reference's calling convention: dense mask + dense bias
    mask = O.make_causal_mask((np.arange(L)[None] < lens[:, None]).astype(np.float32))
    out2 = blk(torch.from_numpy(xq).to(device="cuda:0", dtype=dtype), attention_mask=torch.from_numpy(mask).cuda(),
               attention_bias=torch.from_numpy(O.rel_pos_bias(pos, L)).float().cuda()).double().cpu().numpy()
    assert np.abs(out2 - ref).max() / np.abs(ref).max() <= tol


@pytest.mark.gpu
def test_model_on_gpu_against_oracle(gpu):
  from recml_amd.hstu_layer import HSTU
  m = HSTU(vocab_size=500, max_positions=20, model_dim=32, num_heads=4, num_layers=3, device="cuda:0", seed=3)
  ids = torch.tensor([[1, 2, 3], [4, 5, 0]], device="cuda:0")
  pm = torch.tensor([[1, 1, 1], [1, 1, 0]], device="cuda:0")
  out = m(ids, pm)
  assert tuple(out.shape) == (2, 3, 500) and out.dtype == torch.float32   # hstu_test.py:52-60
  g = lambda p: p.detach().double().cpu().numpy()
  w = {"item_embedding": g(m.item_embedding), "position_embedding": g(m.position_embedding),
       "final_norm_gamma": g(m.final_norm_gamma), "final_norm_beta": g(m.final_norm_beta),
       "reverse_embedding": g(m.reverse_embedding),
       "blocks": [{n: g(p) for n, p in b.named_parameters()} for b in m.decoder_blocks]}
  ref = BO.hstu_model(ids.cpu().numpy(), w, num_heads=4, seq_lens=np.array([3, 2]))
  assert np.abs(out.double().cpu().numpy() - ref).max() / np.abs(ref).max() <= 2e-5
  # packed tokens: the same values on the valid positions, zeros elsewhere
  outj = m(ids, pm, jagged=True).double().cpu().numpy()
  assert np.abs(outj[0] - ref[0]).max() / np.abs(ref).max() <= 2e-5
  assert np.abs(outj[1, :2] - ref[1, :2]).max() / np.abs(ref).max() <= 2e-5 and (outj[1, 2] == 0).all()
  # the reference's other way in (hstu.py:604-615): the dense mask itself, here the one it would build
  import recml_amd
  outm = m(ids, attention_mask=recml_amd.make_causal_mask(pm.float())).double().cpu().numpy()
  assert np.abs(outm - ref).max() / np.abs(ref).max() <= 2e-5
  with pytest.raises(ValueError, match="attention_mask"):
    m(ids, attention_mask=recml_amd.make_causal_mask(pm.float()), seq_lens=torch.tensor([3, 2], device="cuda:0"))


@pytest.mark.gpu
def test_block_config4_shape_bf16(gpu):
  # B=128, L=1024, D=512, H=8 (hd=64), lens U{128..1024}, pos bias: one layer at full size,
  # checked on three sequences (the block treats sequences independently)
  from recml_amd.hstu_layer import HSTUBlock
  rng = np.random.default_rng(4)
  B, L, D, H = 128, 1024, 512, 8
  lens = rng.integers(128, L + 1, B).astype(np.int32)
  lens[:3] = [1024, 128, 517]
  blk = HSTUBlock(D, H, dtype=torch.bfloat16, device="cuda:0", generator=torch.Generator().manual_seed(4))
  x = (torch.randn((B, L, D), generator=torch.Generator().manual_seed(5)) * 1.0).to(device="cuda:0", dtype=torch.bfloat16)
  pos = (torch.randn((2 * L - 1,), generator=torch.Generator().manual_seed(6)) * 0.02).cuda()
  out = blk(x, seq_lens=torch.from_numpy(lens).cuda(), pos_bias=pos)
  assert tuple(out.shape) == (B, L, D) and torch.isfinite(out.float()).all()
  w = {n: p.detach().double().cpu().numpy() for n, p in blk.named_parameters()}
  ref = BO.hstu_block(x[:3].double().cpu().numpy(), w, num_heads=H, seq_lens=lens[:3], pos_tab=pos.double().cpu().numpy())
  got = out[:3].double().cpu().numpy()
  assert np.abs(got - ref).max() / np.abs(ref).max() <= 3e-2


@pytest.mark.gpu
def test_model_config4_full_size_bf16(gpu):
  """Benchmark configuration 4 as a whole: 10 M x 512 bf16 embedding table (10.24 GB), Zipf(1.05) item ids,
  4 blocks, D = 512, H = 8 (head dim 64), B = 128, L = 1024, lengths U{128..1024}, position bias; padded and
  packed forward (recml/layers/keras/hstu.py:585-621), checked against the fp64 oracle on the longest, the
  shortest and a median sequence, which also carry ids at the very end of the table (rows past 2^31 bytes /
  row size would expose 32-bit addressing)."""
  from recml_amd.hstu_layer import HSTU
  free, _ = torch.cuda.mem_get_info()
  if free < 16 << 30:
    pytest.skip("needs 16 GB of free device memory")
  rng = np.random.Generator(np.random.PCG64(4))
  B, L, D, H, layers, vocab = 128, 1024, 512, 8, 4, 10_000_000
  lens = rng.integers(128, L + 1, B).astype(np.int32)
  lens[:2] = [L, 128]                                      # the longest and the shortest possible
  ids = np.minimum(rng.zipf(1.05, (B, L)), vocab - 1).astype(np.int64)
  order = np.argsort(lens, kind="stable")
  pick = [int(order[-1]), int(order[0]), int(order[B // 2])]
  for b in pick:                                           # ids near the end of the table in every checked sequence
    ids[b, 5:9] = [vocab - 1, vocab - 2, vocab - 1000, 4_200_000]      # 4.2 M x 1 KB rows lies beyond 2^32 bytes
  ids[np.arange(L)[None, :] >= lens[:, None]] = 0
  dev = torch.device("cuda:0")
  model = HSTU(vocab_size=8, max_positions=L, model_dim=D, num_heads=H, num_layers=layers, add_head=False,
               dtype=torch.bfloat16, device=dev, seed=4)
  table = torch.empty((vocab, D), dtype=torch.bfloat16, device=dev)
  table.normal_(0.0, 0.01, generator=torch.Generator(device=dev).manual_seed(4))
  model.item_embedding = torch.nn.Parameter(table, requires_grad=False)
  pos = (torch.randn((2 * L - 1,), generator=torch.Generator().manual_seed(5)) * 0.02).to(dev)
  ids_d, lens_d = torch.from_numpy(ids).to(dev), torch.from_numpy(lens).to(dev)
  with torch.no_grad():
    out = model(ids_d, seq_lens=lens_d, pos_bias=pos)
    outj = model(ids_d, seq_lens=lens_d, pos_bias=pos, jagged=True)
  torch.cuda.synchronize()
  assert tuple(out.shape) == (B, L, D) and bool(torch.isfinite(out.float()).all())
  # packed == padded on every valid position of the whole batch (the padded form carries the padding's own
  # embeddings through the blocks, the packed form returns zeros there)
  keep = (torch.arange(L, device=dev)[None, :] < lens_d[:, None])[:, :, None]
  scale = float(out.float().abs().max())
  assert float(((outj.float() - out.float()) * keep).abs().max()) / scale <= 2e-2
  assert bool((outj.float() * ~keep == 0).all())
  # the oracle on the three sequences: weights as stored (bf16 -> fp64), the table reduced to the rows they use
  g = lambda t: t.detach().double().cpu().numpy()
  sub = ids[pick]
  uniq, inv = np.unique(sub, return_inverse=True)
  w = {"item_embedding": g(table[torch.from_numpy(uniq).to(dev)]), "position_embedding": g(model.position_embedding),
       "final_norm_gamma": g(model.final_norm_gamma), "final_norm_beta": g(model.final_norm_beta),
       "blocks": [{n: g(p) for n, p in blk.named_parameters()} for blk in model.decoder_blocks]}
  ref = BO.hstu_model(inv.reshape(sub.shape), w, num_heads=H, seq_lens=lens[pick], pos_tab=g(pos))
  rs = np.abs(ref).max()
  for row, b in enumerate(pick):
    n = int(lens[b])
    # bf16 activations between every step of four blocks: 3e-2 of the largest output (one block alone is held to 3e-2 too)
    for name, got in (("padded", out), ("packed", outj)):
      err = np.abs(got[b, :n].double().cpu().numpy() - ref[row, :n]).max() / rs
      assert err <= 3e-2, (name, b, n, err)


def _dense_attention(q, k, v, *, seq_lens=None, seq_offsets=None, max_len=None, n=None, alpha=1.0, pos_bias=None,
                     dropout_p=0.0, dropout_seed=0, **_):
  """Differentiable dense torch form of the op (padded layout, causal, lengths, position table, dropout by the
  oracle's keep pattern)."""
  B, L, H, d = q.shape
  s = alpha * torch.einsum("bihd,bjhd->bhij", q.float(), k.float())
  i = torch.arange(L, device=q.device)
  if pos_bias is not None:
    s = s + pos_bias.float()[:, (L - 1) + i[None, :] - i[:, None]][None]
  keep = (i[None, :] <= i[:, None])[None] & (i[None, None, :] < seq_lens[:, None, None]) & (i[None, :, None] < seq_lens[:, None, None])
  p = torch.nn.functional.silu(s) / n * keep[:, None]
  if dropout_p > 0:
    p = p * torch.from_numpy(O.dropout_keep_mask(dropout_seed, dropout_p, B, H, L, L)).to(q.device) / (1.0 - dropout_p)
  return torch.einsum("bhij,bjhd->bihd", p, v.float()).to(q.dtype)


@pytest.mark.gpu
@pytest.mark.parametrize("drop", [0.0, 0.25])
@pytest.mark.parametrize("dtype,hd,tol", [(torch.float32, 16, 2e-4), (torch.bfloat16, 64, 6e-2)])
def test_block_gradients_through_the_hip_backward(gpu, dtype, hd, tol, drop):
  """A trainable block: gradients with the HIP attention (forward and backward kernels, q / k / v being
  strided slices of the fused projection) against the same block with a dense torch attention; with a
  dropout rate too (training mode, the seed given: the backward kernels regenerate the forward's pattern)."""
  from recml_amd import hstu_layer
  from recml_amd.hstu_layer import HSTUBlock
  dev = torch.device("cuda:0")
  B, L, H = 3, 160, 2
  D = H * hd
  gen = torch.Generator().manual_seed(5)
  blk = HSTUBlock(D, H, dropout=drop, dtype=dtype, device=dev, generator=gen)
  blk.requires_grad_(True)
  x = (torch.randn((B, L, D), generator=gen) * 0.5).to(dev).to(dtype).requires_grad_(True)
  lens = torch.tensor([160, 77, 1], dtype=torch.int32, device=dev)
  pos = (torch.randn((H, 2 * L - 1), generator=gen) * 0.3).to(dev).requires_grad_(True)
  dout = torch.randn((B, L, D), generator=gen).to(dev).to(dtype)

  def grads(attention, fused_training):
    saved = hstu_layer._attention
    hstu_layer._attention = attention
    if not fused_training:
      blk._fused_training = lambda *a: False          # torch's layer norms and gate, the attention as a function of its own
    try:
      for t in [x, pos, *blk.parameters()]:
        t.grad = None
      out = blk(x, seq_lens=lens, pos_bias=pos, dropout_seed=4242)
      (out.float() * dout.float()).sum().backward()
      return {"x": x.grad.float().clone(), "pos": pos.grad.float().clone(),
              **{n: p.grad.float().clone() for n, p in blk.named_parameters() if p.grad is not None}}
    finally:
      hstu_layer._attention = saved
      blk.__dict__.pop("_fused_training", None)

  # the block as it trains (in bf16: norms, gate and attention through the kernels, the projection's
  # gradient written in place) against plain torch everywhere with a dense torch attention
  got = grads(hstu_layer._attention, True)
  want = grads(_dense_attention, False)
  assert set(got) == set(want) and "q_kernel" in got and "output_kernel" in got and "attn_ln_gamma" in got
  for name in want:
    err = float((got[name] - want[name]).abs().max() / want[name].abs().max().clamp_min(1e-30))
    assert err <= tol, (name, err)


@pytest.mark.gpu
@pytest.mark.parametrize("use_bias", [False, True])
def test_packed_block_trains_through_the_fused_steps(gpu, use_bias):
  """forward_jagged in bf16 with gradients: the fused training steps (kernel layer norms, attention + norm
  + gate as one function) against the same block with torch's norms and gate around the attention
  function, on packed tokens with timestamps and both tables; and the fused path is the one taken."""
  from recml_amd import hstu_layer, hstu_block_ops
  from recml_amd.hstu_layer import HSTUBlock
  dev, bf = torch.device("cuda:0"), torch.bfloat16
  H, hd = 4, 64
  D = H * hd
  gen = torch.Generator().manual_seed(9)
  lens = [200, 1, 77, 130]
  T, L = sum(lens), 256
  offsets = torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int32, device=dev)
  blk = HSTUBlock(D, H, use_bias=use_bias, dtype=bf, device=dev, generator=gen)
  if use_bias:
    with torch.no_grad():
      for name, prm in blk.named_parameters():
        if name.endswith("_bias"):
          prm.copy_((torch.randn(prm.shape, generator=gen) * 0.1).to(dev).to(bf))
  blk.requires_grad_(True)
  x = (torch.randn((T, D), generator=gen) * 0.5).to(dev).to(bf).requires_grad_(True)
  pos = (torch.randn((H, 2 * L - 1), generator=gen) * 0.3).to(dev).requires_grad_(True)
  tsb = (torch.randn((H, 33), generator=gen) * 0.3).to(dev).requires_grad_(True)
  stamps = torch.cat([torch.cumsum(torch.randint(1, 5000, (n,), generator=gen), 0) for n in lens]).to(dev)
  dout = torch.randn((T, D), generator=gen).to(dev).to(bf)
  calls = []
  real = hstu_block_ops.norm_gate_bwd

  def counted(*a, **k):
    calls.append(k.get("du_out") is not None)
    return real(*a, **k)

  def grads(fused_training):
    if not fused_training:
      blk._fused_training = lambda *a: False
    try:
      for t in [x, pos, tsb, *blk.parameters()]:
        t.grad = None
      out = blk.forward_jagged(x, offsets, L, pos_bias=pos, timestamps=stamps, ts_bias=tsb)
      (out.float() * dout.float()).sum().backward()
      return out.detach().float(), {"x": x.grad.float().clone(), "pos": pos.grad.float().clone(), "ts": tsb.grad.float().clone(),
                                   **{n: p.grad.float().clone() for n, p in blk.named_parameters() if p.grad is not None}}
    finally:
      blk.__dict__.pop("_fused_training", None)

  hstu_block_ops.norm_gate_bwd = counted
  try:
    out_f, got = grads(True)
  finally:
    hstu_block_ops.norm_gate_bwd = real
  assert calls == [True, False]                       # the gate's backward writing in place, then the input norm's
  out_t, want = grads(False)
  assert float((out_f - out_t).abs().max() / out_t.abs().max()) <= 2e-2
  assert set(got) == set(want) and {"u_kernel", "attn_ln_beta", "input_ln_gamma"} <= set(got)
  assert ("output_bias" in got and "q_bias" in got) == use_bias
  for name in want:
    err = float((got[name] - want[name]).abs().max() / want[name].abs().max().clamp_min(1e-30))
    assert err <= 4e-2, (name, err)                   # bf16 activations on both sides, rounded at different points


@pytest.mark.gpu
@pytest.mark.parametrize("drop", [0.0, 0.2])
@pytest.mark.parametrize("dtype,hd,tol", [(torch.float32, 16, 2e-4), (torch.bfloat16, 64, 6e-2)])
def test_block_gradients_with_the_reference_mask_convention(gpu, dtype, hd, tol, drop):
  """Training a block the way the reference calls it -- a dense [B, L, L] mask and a constant dense bias:
  the attention's forward and backward kernels take the mask and the bias as they are (no gradient is asked
  for the bias); against the same block with the attention in plain torch."""
  from recml_amd import hstu_ops
  from recml_amd.hstu_layer import HSTUBlock
  dev = torch.device("cuda:0")
  B, L, H = 2, 144, 2
  D = H * hd
  gen = torch.Generator().manual_seed(6)
  blk = HSTUBlock(D, H, dropout=drop, dtype=dtype, device=dev, generator=gen)
  blk.requires_grad_(True)
  x = (torch.randn((B, L, D), generator=gen) * 0.5).to(dev).to(dtype).requires_grad_(True)
  lens = torch.tensor([144, 50], device=dev)
  i = torch.arange(L, device=dev)
  mask = ((i[None, :] <= i[:, None])[None] & (i[None, None, :] < lens[:, None, None]) & (i[None, :, None] < lens[:, None, None]))
  bias = (torch.randn((B, L, L), generator=gen) * 0.3).to(dev)
  dout = torch.randn((B, L, D), generator=gen).to(dev).to(dtype)

  def grads(fused):
    saved = hstu_ops.hstu_attention_autograd
    if not fused:
      hstu_ops.hstu_attention_autograd = lambda q, k, v, **kw: dense_attention_torch(q, k, v, **kw)
    try:
      for t in [x, *blk.parameters()]:
        t.grad = None
      out = blk(x, attention_mask=mask, attention_bias=bias, dropout_seed=9)
      (out.float() * dout.float()).sum().backward()
      return {"x": x.grad.float().clone(), **{n: p.grad.float().clone() for n, p in blk.named_parameters() if p.grad is not None}}
    finally:
      hstu_ops.hstu_attention_autograd = saved

  got, want = grads(True), grads(False)
  assert set(got) == set(want) and "q_kernel" in got and "output_kernel" in got
  for name in want:
    err = float((got[name] - want[name]).abs().max() / want[name].abs().max().clamp_min(1e-30))
    assert err <= tol, (name, err)


@pytest.mark.gpu
def test_model_trains_the_same_from_a_dense_mask_and_from_lengths(gpu):
  """The reference's model hands every block make_causal_mask's dense [B, L, L] mask (hstu.py:604-615); here the
  same model trains from the lengths.  Both ways in, bf16, gradients of every parameter: the same up to the
  rounding of two different kernel paths (the dense mask goes through the matrix-core kernels tile by tile)."""
  import recml_amd
  from recml_amd import hstu_ops
  dev, bf = "cuda:0", torch.bfloat16
  B, L, D, H = 3, 160, 128, 2
  model = recml_amd.HSTU(vocab_size=60, max_positions=L, model_dim=D, num_heads=H, num_layers=2, dtype=bf, device=dev,
                         add_head=False, seed=2)
  model.requires_grad_(True)
  ids = torch.randint(1, 60, (B, L), device=dev)
  pm = (torch.arange(L, device=dev)[None, :] < torch.tensor([160, 77, 9], device=dev)[:, None]).float()
  dout = torch.randn((B, L, D), device=dev).to(bf)
  seen = []
  real = hstu_ops.hstu_attention_bwd

  def spy(*a, **k):
    k["_variant_out"] = seen
    return real(*a, **k)

  def grads(**kw):
    for prm in model.parameters():
      prm.grad = None
    out = model(ids, **kw)
    (out.float() * dout.float() * pm[:, :, None]).sum().backward()      # (padded rows carry their embeddings: not compared)
    return {n: prm.grad.float().clone() for n, prm in model.named_parameters() if prm.grad is not None}

  hstu_ops.hstu_attention_bwd = spy
  try:
    got = grads(attention_mask=recml_amd.make_causal_mask(pm))
  finally:
    hstu_ops.hstu_attention_bwd = real
  assert seen == ["hstu_bwd_mfma_bf16"] * 2
  want = grads(padding_mask=pm)
  assert set(got) == set(want) and "item_embedding" in got
  for name in want:
    err = float((got[name] - want[name]).abs().max() / want[name].abs().max().clamp_min(1e-30))
    assert err <= 6e-2, (name, err)
