"""AttentionBatch: the preparation of a batch (work list, 32-bit timestamps, scaled tables) shared by
several calls.  A call that reuses it must give the bits of a call that prepares for itself, and
anything the preparation was built from that changes must be noticed."""

import numpy as np
import pytest
import torch

import recml_amd
from recml_amd import hstu_ops
from oracle import hstu_oracle as O

pytestmark = pytest.mark.gpu
bf = torch.bfloat16


def _dev(x, dtype=None):
  t = torch.from_numpy(np.ascontiguousarray(x)).to("cuda:0")
  return t if dtype is None else t.to(dtype)


def _jagged_case(rng, lens, H=8, d=128, L=640):
  off = np.zeros(len(lens) + 1, dtype=np.int32)
  off[1:] = np.cumsum(lens)
  T = int(off[-1])
  qkv = [O.round_bf16(rng.standard_normal((T, H, d)).astype(np.float32) * 0.3) for _ in range(3)]
  pos = (rng.standard_normal((H, 2 * L - 1)) * 0.2).astype(np.float32)
  tab = (rng.standard_normal((H, 129)) * 0.2).astype(np.float32)
  ts = np.concatenate([1_600_000_000 + np.cumsum(np.ceil(rng.exponential(3600.0, n)).astype(np.int64)) for n in lens])
  return qkv, off, pos, tab, ts


def test_layers_share_one_preparation(gpu):
  rng = np.random.default_rng(1500)
  lens = np.array([640, 600, 333, 17, 0, 129, 512], dtype=np.int32)
  L = 640
  (q0, k0, v0), off, pos, tab, ts = _jagged_case(rng, lens, L=L)
  kw = dict(seq_offsets=_dev(off), max_len=L, pos_bias=_dev(pos), ts_bias=_dev(tab), timestamps=_dev(ts))
  batch = hstu_ops.AttentionBatch()
  for layer in range(4):
    q, k, v = (_dev(O.round_bf16(x * (1.0 + 0.1 * layer)), bf) for x in (q0, k0, v0))
    alone = recml_amd.hstu_attention(q, k, v, **kw)
    shared = recml_amd.hstu_attention(q, k, v, batch=batch, **kw)
    assert torch.equal(alone, shared), layer
  assert batch.prepared_calls == 3
  ref = O.hstu_attention_jagged_ref(O.round_bf16(q0 * 1.3), O.round_bf16(k0 * 1.3), O.round_bf16(v0 * 1.3), off, L,
                                    pos_tab=pos, ts_tab=tab, timestamps=ts)
  err = np.abs(shared.float().cpu().numpy() - ref).max() / np.abs(ref).max()
  assert err <= 2e-2


def test_changed_inputs_are_prepared_again(gpu):
  rng = np.random.default_rng(1501)
  B, L, H, d = 4, 384, 8, 128
  q, k, v = (_dev(O.round_bf16(rng.standard_normal((B, L, H, d)).astype(np.float32) * 0.3), bf) for _ in range(3))
  lens = _dev(np.array([384, 200, 77, 300], dtype=np.int32))
  pos = _dev((rng.standard_normal((H, 2 * L - 1)) * 0.2).astype(np.float32))
  batch = hstu_ops.AttentionBatch()
  a = recml_amd.hstu_attention(q, k, v, seq_lens=lens, pos_bias=pos, batch=batch)
  b = recml_amd.hstu_attention(q, k, v, seq_lens=lens, pos_bias=pos, batch=batch)
  assert batch.prepared_calls == 1 and torch.equal(a, b)
  # lengths changed in place: same tensor, new contents
  lens[1] = 384
  c = recml_amd.hstu_attention(q, k, v, seq_lens=lens, pos_bias=pos, batch=batch)
  assert batch.prepared_calls == 1
  assert torch.equal(c, recml_amd.hstu_attention(q, k, v, seq_lens=lens, pos_bias=pos))
  assert not torch.equal(c, a)
  # the table changed in place
  pos.mul_(2.0)
  e = recml_amd.hstu_attention(q, k, v, seq_lens=lens, pos_bias=pos, batch=batch)
  assert batch.prepared_calls == 1
  assert torch.equal(e, recml_amd.hstu_attention(q, k, v, seq_lens=lens, pos_bias=pos))
  # another option (no causal mask), then another shape
  f = recml_amd.hstu_attention(q, k, v, seq_lens=lens, pos_bias=pos, causal=False, batch=batch)
  assert batch.prepared_calls == 1
  assert torch.equal(f, recml_amd.hstu_attention(q, k, v, seq_lens=lens, pos_bias=pos, causal=False))
  g = recml_amd.hstu_attention(q[:2], k[:2], v[:2], seq_lens=lens[:2], pos_bias=pos, batch=batch)
  assert torch.equal(g, recml_amd.hstu_attention(q[:2], k[:2], v[:2], seq_lens=lens[:2], pos_bias=pos))
  # and reuse works again afterwards
  h2 = recml_amd.hstu_attention(q[:2], k[:2], v[:2], seq_lens=lens[:2], pos_bias=pos, batch=batch)
  assert batch.prepared_calls == 2 and torch.equal(g, h2)


def test_model_prepares_once_for_its_blocks(gpu, monkeypatch):
  made = []
  real = hstu_ops.AttentionBatch

  class Counting(real):
    def __init__(self):
      super().__init__()
      made.append(self)

  monkeypatch.setattr(hstu_ops, "AttentionBatch", Counting)
  torch.manual_seed(0)
  B, L = 6, 256
  model = recml_amd.HSTU(vocab_size=1000, max_positions=L, model_dim=256, num_heads=2, num_layers=3,
                         dtype=bf, device="cuda:0", add_head=False)
  ids = torch.randint(0, 1000, (B, L), device="cuda:0")
  lens = torch.tensor([256, 200, 31, 128, 1, 77], device="cuda:0", dtype=torch.int32)
  pos = torch.randn(2, 2 * L - 1, device="cuda:0") * 0.1
  with torch.no_grad():
    for jagged in (False, True):
      made.clear()
      out = model(ids, seq_lens=lens, pos_bias=pos, jagged=jagged)
      assert len(made) == 1 and made[0].prepared_calls == 2, (jagged, [m.prepared_calls for m in made])
      # the same blocks, each call preparing for itself
      monkeypatch.setattr(hstu_ops, "AttentionBatch", lambda: None)
      ref = model(ids, seq_lens=lens, pos_bias=pos, jagged=jagged)
      monkeypatch.setattr(hstu_ops, "AttentionBatch", Counting)
      assert torch.equal(out, ref), jagged


def test_model_forward_under_inference_mode(gpu):
  """torch.inference_mode(): the tensors the model builds for its layers (lengths, offsets, packed timestamps)
  are inference tensors; the shared preparation takes them, and the output is that of torch.no_grad()."""
  torch.manual_seed(1)
  B, L = 5, 256
  model = recml_amd.HSTU(vocab_size=500, max_positions=L, model_dim=256, num_heads=2, num_layers=2,
                         dtype=bf, device="cuda:0", add_head=False)
  ids = torch.randint(0, 500, (B, L), device="cuda:0")
  lens = torch.tensor([256, 200, 31, 128, 1], device="cuda:0", dtype=torch.int32)
  pos = torch.randn(2, 2 * L - 1, device="cuda:0") * 0.1
  for jagged in (False, True):
    with torch.no_grad():
      ref = model(ids, seq_lens=lens, pos_bias=pos, jagged=jagged)
    with torch.inference_mode():
      out = model(ids, seq_lens=lens, pos_bias=pos, jagged=jagged)
      again = model(ids.clone(), seq_lens=lens.clone(), pos_bias=pos.clone(), jagged=jagged)    # inference tensors as inputs
    assert torch.equal(out, ref) and torch.equal(again, ref), jagged


def test_layers_share_the_scan_of_a_dense_mask(gpu):
  """The layer-side call with a [B, L, L] mask: the preparation reads the mask for each query tile's range of
  key steps; calls on the same batch reuse it, and a mask edited in place is read again."""
  rng = np.random.default_rng(1503)
  B, L, H, d = 3, 400, 2, 128
  q, k, v = (O.round_bf16(rng.standard_normal((B, L, H, d)).astype(np.float32) * 0.3) for _ in range(3))
  lens = np.array([400, 150, 31])
  pad = (np.arange(L)[None] < lens[:, None]).astype(np.float32)
  mask_np = O.make_causal_mask(pad).astype(bool)
  bias_np = (rng.standard_normal((B, L, L)) * 0.5).astype(np.float32)
  mask, bias = _dev(mask_np), _dev(bias_np)
  qd, kd, vd = (_dev(t, bf) for t in (q, k, v))
  batch = hstu_ops.AttentionBatch()
  outs = [recml_amd.pointwise_attention(qd, kd, vd, mask, bias, batch=batch) for _ in range(3)]
  assert batch.prepared_calls == 2
  alone = recml_amd.pointwise_attention(qd, kd, vd, mask, bias)
  for o in outs:
    assert torch.equal(o, alone)
  ref = O.pointwise_attention_dense(q, k, v, mask_np, bias_np)
  assert np.abs(alone.float().cpu().numpy() - ref).max() <= 2e-2 * np.abs(ref).max()
  # the mask opened up in place (every pair kept): ranges found for the causal mask would drop most of it
  mask.fill_(True)
  again = recml_amd.pointwise_attention(qd, kd, vd, mask, bias, batch=batch)
  assert batch.prepared_calls == 2
  ref = O.pointwise_attention_dense(q, k, v, np.ones((B, L, L)), bias_np)
  assert np.abs(again.float().cpu().numpy() - ref).max() <= 2e-2 * np.abs(ref).max()
