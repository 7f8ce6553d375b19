"""Backward of the attention op on the GPU against the numpy oracle (itself pinned by finite differences)."""

import numpy as np
import pytest
import torch

import recml_amd
from oracle import hstu_oracle as O

pytestmark = pytest.mark.gpu


def _dev(x, dtype=None):
  t = torch.from_numpy(np.ascontiguousarray(x)).to("cuda:0")
  return t if dtype is None else t.to(dtype)


def _rel(a, b):
  return float(np.abs(a - b).max() / max(np.abs(b).max(), 1e-30))


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 2e-2)])
def test_backward_lengths_and_tables(gpu, dtype, tol):
  rng = np.random.default_rng(21)
  B, L, H, d = 3, 70, 2, 32
  lens = np.array([70, 33, 1], dtype=np.int32)
  rd = O.round_bf16 if dtype == torch.bfloat16 else (lambda x: x)
  q, k, v, dout = (rd(rng.standard_normal((B, L, H, d)).astype(np.float32) * 0.5) for _ in range(4))
  pos = (rng.standard_normal((H, 2 * L - 1)) * 0.3).astype(np.float32)
  tab = (rng.standard_normal((129,)) * 0.3).astype(np.float32)
  ts = 1_600_000_000 + np.cumsum(np.ceil(rng.exponential(3600.0, (B, L))), axis=1).astype(np.int64)
  kw = dict(seq_lens=lens, pos_tab=pos, timestamps=ts, ts_tab=tab)
  want = O.hstu_attention_bwd_ref(q, k, v, dout, **kw)
  got = recml_amd.hstu_attention_bwd(_dev(q, dtype), _dev(k, dtype), _dev(v, dtype), _dev(dout, dtype),
                                     seq_lens=_dev(lens), pos_bias=_dev(pos), timestamps=_dev(ts), ts_bias=_dev(tab))
  for name, g, w in zip(("dq", "dk", "dv", "dpos", "dts"), got, want):
    assert tuple(g.shape) == w.shape, name
    assert _rel(g.float().cpu().numpy(), w) <= tol, name
  dq, dk, dv = (g.float().cpu().numpy() for g in got[:3])
  for b in range(B):
    assert (dq[b, lens[b]:] == 0).all() and (dk[b, lens[b]:] == 0).all() and (dv[b, lens[b]:] == 0).all()


def test_backward_jagged_equals_padded(gpu):
  rng = np.random.default_rng(22)
  B, L, H, d = 4, 90, 2, 64
  lens = np.array([90, 17, 64, 33], dtype=np.int32)
  q, k, v, dout = (rng.standard_normal((B, L, H, d)).astype(np.float32) * 0.4 for _ in range(4))
  pos = (rng.standard_normal((2 * L - 1,)) * 0.3).astype(np.float32)
  want = O.hstu_attention_bwd_ref(q, k, v, dout, seq_lens=lens, pos_tab=pos)
  pack = lambda x: O.padded_to_jagged(x, lens)
  (qj, off), (kj, _), (vj, _), (dj, _) = pack(q), pack(k), pack(v), pack(dout)
  got = recml_amd.hstu_attention_bwd(_dev(qj), _dev(kj), _dev(vj), _dev(dj), seq_offsets=_dev(off.astype(np.int32)),
                                     max_len=L, pos_bias=_dev(pos))
  for name, g, w in zip(("dq", "dk", "dv"), got[:3], want[:3]):
    assert _rel(O.jagged_to_padded(g.cpu().numpy(), off, L), w) <= 2e-5, name
  assert _rel(got[3].cpu().numpy(), want[3]) <= 2e-5 and got[4] is None


def test_backward_options(gpu):
  # segment ids + window (the reference's test recipe, hstu_ops_test.py:36-83), then full mask + dense bias + cross length
  rng = np.random.default_rng(23)
  B, L, H, d = 2, 40, 2, 16
  q, k, v, dout = (rng.standard_normal((B, L, H, d)).astype(np.float32) for _ in range(4))
  seg = np.ones((B, L), np.int32)
  seg[0, 25:] = 0
  seg[1, 10:30] = 2
  kw = dict(alpha=1 / np.sqrt(d), q_segment_ids=seg, kv_segment_ids=seg, sliding_window_size=7)
  want = O.hstu_attention_bwd_ref(q, k, v, dout, **kw)
  got = recml_amd.hstu_attention_bwd(_dev(q), _dev(k), _dev(v), _dev(dout), alpha=kw["alpha"], q_segment_ids=_dev(seg),
                                     kv_segment_ids=_dev(seg), sliding_window_size=7)
  for name, g, w in zip(("dq", "dk", "dv"), got[:3], want[:3]):
    assert _rel(g.cpu().numpy(), w) <= 2e-5, name     # the reference accepts 5e-3 here
  Lk = 55
  k2, v2 = (rng.standard_normal((B, Lk, H, d)).astype(np.float32) for _ in range(2))
  m = rng.random((B, L, Lk)) > 0.3
  bias = rng.standard_normal((B, L, Lk)).astype(np.float32)
  want = O.hstu_attention_bwd_ref(q, k2, v2, dout, causal=False, mask=m, bias=bias, n=7.0)
  got = recml_amd.hstu_attention_bwd(_dev(q), _dev(k2), _dev(v2), _dev(dout), causal=False, mask=_dev(m), bias=_dev(bias), n=7.0)
  for name, g, w in zip(("dq", "dk", "dv"), got[:3], want[:3]):
    assert _rel(g.cpu().numpy(), w) <= 2e-5, name


def test_autograd_function(gpu):
  rng = np.random.default_rng(24)
  B, L, H, d = 2, 64, 2, 64
  lens = np.array([64, 20], dtype=np.int32)
  mk = lambda *s: torch.from_numpy(rng.standard_normal(s).astype(np.float32) * 0.4).to("cuda:0").requires_grad_(True)
  q, k, v = mk(B, L, H, d), mk(B, L, H, d), mk(B, L, H, d)
  pos = mk(H, 2 * L - 1)
  dout = torch.from_numpy(rng.standard_normal((B, L, H, d)).astype(np.float32)).to("cuda:0")
  out = recml_amd.hstu_attention_autograd(q, k, v, pos_bias=pos, seq_lens=_dev(lens))
  (out * dout).sum().backward()
  n = lambda t: t.detach().cpu().numpy()
  want = O.hstu_attention_bwd_ref(n(q), n(k), n(v), n(dout), seq_lens=lens, pos_tab=n(pos))
  for name, g, w in zip(("dq", "dk", "dv", "dpos"), (q.grad, k.grad, v.grad, pos.grad), want):
    assert _rel(n(g), w) <= 2e-5, name


@pytest.mark.parametrize("name,d,B,L,H,lens,pos,ts,causal,jagged", [
    ("full-length", 128, 2, 256, 2, None, False, False, True, False),
    ("lengths", 128, 3, 300, 2, [300, 129, 1], False, False, True, False),
    ("non-causal", 128, 2, 200, 1, [200, 77], False, False, False, False),
    ("pos", 128, 3, 300, 2, [300, 129, 33], True, False, True, False),
    ("ts", 128, 3, 300, 2, [300, 129, 33], False, True, True, False),
    ("pos+ts jagged", 128, 4, 420, 2, [420, 129, 33, 256], True, True, True, True),
    ("pos+ts non-causal", 128, 2, 200, 2, [200, 100], True, True, False, False),
    ("d64 lengths", 64, 3, 300, 2, [300, 129, 1], False, False, True, False),
    ("d64 pos+ts jagged", 64, 4, 420, 2, [420, 129, 33, 256], True, True, True, True),
    ("d64 pos non-causal", 64, 2, 200, 4, [200, 100], True, False, False, False),
    ("d32 lengths", 32, 3, 300, 2, [300, 129, 1], False, False, True, False),
    ("d32 pos+ts jagged", 32, 4, 420, 2, [420, 129, 33, 256], True, True, True, True),
    ("d32 ts non-causal", 32, 2, 200, 1, [200, 100], False, True, False, False),
    # work-list mappings: H < 8, H = 16, and the two cases without a list (H = 3; more sequences than the builder takes)
    ("H=4", 64, 5, 200, 4, [200, 1, 77, 129, 128], True, False, True, True),
    ("H=16", 32, 2, 150, 16, [150, 31], True, False, True, False),
    ("H=3 static grid", 64, 3, 140, 3, [140, 5, 129], True, False, True, True),
])
def test_backward_matrix_core_kernels(gpu, name, d, B, L, H, lens, pos, ts, causal, jagged):
  """bf16, d in {32, 64, 128}: the matrix-core pair of kernels, checked against the oracle (table gradients too)."""
  rng = np.random.default_rng(31)
  bf = torch.bfloat16
  q, k, v, dout = (O.round_bf16(rng.standard_normal((B, L, H, d)).astype(np.float32) * 0.5) for _ in range(4))
  full = np.full((B,), L, np.int32)
  ln = full if lens is None else np.array(lens, np.int32)
  kw, gk = {}, dict(causal=causal)
  if lens is not None:
    kw["seq_lens"] = ln
  if pos:
    kw["pos_tab"] = (rng.standard_normal((H, 2 * L - 1)) * 0.3).astype(np.float32)
    gk["pos_bias"] = _dev(kw["pos_tab"])
  if ts:
    kw["ts_tab"] = (rng.standard_normal((129,)) * 0.3).astype(np.float32)
    t = 1_600_000_000 + np.cumsum(np.ceil(rng.exponential(3600.0, (B, L))), axis=1).astype(np.int64)
    for b in range(B):
      t[b, ln[b]:] = t[b, ln[b] - 1]     # what the jagged layout's clamp to the last row sees
    kw["timestamps"] = t
    gk["ts_bias"] = _dev(kw["ts_tab"])
  want = O.hstu_attention_bwd_ref(q, k, v, dout, causal=causal, **kw)
  variant = []
  gk["_variant_out"] = variant
  if jagged:
    pack = lambda x: O.padded_to_jagged(x, ln)
    (qj, off), (kj, _), (vj, _), (dj, _) = pack(q), pack(k), pack(v), pack(dout)
    if ts:
      gk["timestamps"] = _dev(np.concatenate([kw["timestamps"][b, :ln[b]] for b in range(B)]))
    got = recml_amd.hstu_attention_bwd(_dev(qj, bf), _dev(kj, bf), _dev(vj, bf), _dev(dj, bf),
                                       seq_offsets=_dev(off.astype(np.int32)), max_len=L, **gk)
    tabs = got[3:]
    got = [O.jagged_to_padded(g.float().cpu().numpy(), off, L) for g in got[:3]]
  else:
    if ts:
      gk["timestamps"] = _dev(kw["timestamps"])
    if lens is not None:
      gk["seq_lens"] = _dev(ln)
    got = recml_amd.hstu_attention_bwd(_dev(q, bf), _dev(k, bf), _dev(v, bf), _dev(dout, bf), **gk)
    tabs = got[3:]
    got = [g.float().cpu().numpy() for g in got[:3]]
  assert variant == ["hstu_bwd_mfma_bf16"]
  # table gradients: fp32 sums of the same dS (every pair in the bucket the law gives it)
  for nm, g, w in (("dpos", tabs[0], want[3]), ("dts", tabs[1], want[4])):
    assert (g is None) == (w is None), nm
    if g is not None:
      assert _rel(g.cpu().numpy().reshape(w.shape), w) <= 2e-2, nm
  for nm, g, w in zip(("dq", "dk", "dv"), got, want[:3]):
    err = np.abs(g - w).max(axis=(2, 3)) / np.abs(w).max()
    assert err.max() <= 2e-2, (nm, err.max())
    for b in range(B):
      assert (g[b, ln[b]:] == 0).all(), nm


@pytest.mark.parametrize("d,L,window,causal,pos", [
    (128, 400, 37, True, True),
    (128, 400, 150, False, True),
    (64, 300, 0, True, False),
    (32, 520, 260, False, True),
])
def test_backward_sliding_window_on_the_matrix_cores(gpu, d, L, window, causal, pos):
  rng = np.random.default_rng(200 + window)
  B, H = 3, 2
  bf = torch.bfloat16
  lens = np.array([L, L // 2 + 3, 1], dtype=np.int32)
  q, k, v, dout = (O.round_bf16(rng.standard_normal((B, L, H, d)).astype(np.float32) * 0.5) for _ in range(4))
  kw, gk = dict(seq_lens=lens), dict(seq_lens=_dev(lens))
  if pos:
    kw["pos_tab"] = (rng.standard_normal((H, 2 * L - 1)) * 0.3).astype(np.float32)
    gk["pos_bias"] = _dev(kw["pos_tab"])
  want = O.hstu_attention_bwd_ref(q, k, v, dout, causal=causal, sliding_window_size=window, **kw)
  variant = []
  got = recml_amd.hstu_attention_bwd(_dev(q, bf), _dev(k, bf), _dev(v, bf), _dev(dout, bf), causal=causal,
                                     sliding_window_size=window, _variant_out=variant, **gk)
  assert variant == ["hstu_bwd_mfma_bf16"]
  for nm, g, w in zip(("dq", "dk", "dv", "dpos"), got[:4], want[:4]):
    assert (g is None) == (w is None), nm
    if g is not None:
      assert _rel(g.float().cpu().numpy().reshape(w.shape), w) <= 2e-2, nm
  for b in range(B):
    for g in got[:3]:
      assert (g[b, lens[b]:] == 0).all()


@pytest.mark.parametrize("d,L,causal,window,pos", [
    (128, 400, True, None, True),
    (64, 260, False, 40, False),
    (32, 132, True, None, False),
])
def test_backward_segment_ids_on_the_matrix_cores(gpu, d, L, causal, window, pos):
  """Packed rows (several segments per row and a padding segment) through the matrix-core backward."""
  rng = np.random.default_rng(400 + L)
  B, H = 3, 2
  bf = torch.bfloat16
  q, k, v, dout = (O.round_bf16(rng.standard_normal((B, L, H, d)).astype(np.float32) * 0.5) for _ in range(4))
  seg = np.zeros((B, L), np.int32)
  seg[0, :L // 3], seg[0, L // 3: L - 7] = 1, 2
  seg[1, :] = 5
  cuts = np.sort(rng.choice(np.arange(1, L), 9, replace=False))
  seg[2] = np.searchsorted(cuts, np.arange(L), side="right") + 1
  kw, gk = {}, {}
  if pos:
    kw["pos_tab"] = (rng.standard_normal((H, 2 * L - 1)) * 0.3).astype(np.float32)
    gk["pos_bias"] = _dev(kw["pos_tab"])
  want = O.hstu_attention_bwd_ref(q, k, v, dout, causal=causal, q_segment_ids=seg, kv_segment_ids=seg,
                                  sliding_window_size=window, **kw)
  variant = []
  got = recml_amd.hstu_attention_bwd(_dev(q, bf), _dev(k, bf), _dev(v, bf), _dev(dout, bf), causal=causal,
                                     q_segment_ids=_dev(seg), kv_segment_ids=_dev(seg), sliding_window_size=window,
                                     _variant_out=variant, **gk)
  assert variant == ["hstu_bwd_mfma_bf16"]
  for nm, g, w in zip(("dq", "dk", "dv", "dpos"), got[:4], want[:4]):
    assert (g is None) == (w is None), nm
    if g is not None:
      assert _rel(g.float().cpu().numpy().reshape(w.shape), w) <= 2e-2, nm


def test_backward_many_short_sequences_static_grid(gpu):
  """More sequences than the work-list builder takes (8192): the kernels enumerate (sequence, head, tile) themselves."""
  rng = np.random.default_rng(33)
  B, L, H, d = 8200, 33, 1, 32
  bf = torch.bfloat16
  lens = rng.integers(1, L + 1, B).astype(np.int32)
  q, k, v, dout = (O.round_bf16(rng.standard_normal((B, L, H, d)).astype(np.float32) * 0.5) for _ in range(4))
  want = O.hstu_attention_bwd_ref(q, k, v, dout, seq_lens=lens)
  variant = []
  got = recml_amd.hstu_attention_bwd(_dev(q, bf), _dev(k, bf), _dev(v, bf), _dev(dout, bf), seq_lens=_dev(lens), _variant_out=variant)
  assert variant == ["hstu_bwd_mfma_bf16"]
  for nm, g, w in zip(("dq", "dk", "dv"), got[:3], want[:3]):
    assert _rel(g.float().cpu().numpy(), w) <= 2e-2, nm


@pytest.mark.parametrize("seed", list(range(2000, 2014)))
def test_matrix_core_backward_on_random_option_mixes(gpu, seed):
  """bf16 backward against the oracle over random mixes of head dim, heads, layout, causal / full,
  window, segment ids and the two biases with their table gradients (fixed seeds)."""
  rng = np.random.default_rng(seed)
  d = int(rng.choice([32, 64, 128]))
  H = int(rng.choice([1, 2, 4, 8]))
  L = int(rng.choice([36, 100, 128, 132, 260]))
  B = int(rng.integers(1, 4))
  causal = bool(rng.integers(0, 2))
  window = None if rng.random() < 0.6 else int(rng.integers(0, L))
  seg = L % 4 == 0 and rng.random() < 0.3
  jagged = (not seg) and rng.random() < 0.5
  bf = torch.bfloat16
  lens = rng.integers(1, L + 1, B).astype(np.int32)
  lens[rng.integers(0, B)] = L
  q, k, v, dout = (O.round_bf16(rng.standard_normal((B, L, H, d)).astype(np.float32) * 0.5) for _ in range(4))
  kw, gk = dict(causal=causal), dict(causal=causal)
  if window is not None:
    kw["sliding_window_size"] = gk["sliding_window_size"] = window
  if rng.random() < 0.5:
    kw["pos_tab"] = (rng.standard_normal((H if rng.random() < 0.5 else 1, 2 * L - 1)) * 0.3).astype(np.float32)
    gk["pos_bias"] = _dev(kw["pos_tab"])
  t = None
  if rng.random() < 0.5:
    kw["ts_tab"] = (rng.standard_normal((H if rng.random() < 0.5 else 1, 65)) * 0.3).astype(np.float32)
    t = 1_700_000_000 + np.cumsum(np.ceil(rng.exponential(5000.0, (B, L))), axis=1).astype(np.int64)
    for b in range(B):
      t[b, lens[b]:] = t[b, lens[b] - 1]
    kw["timestamps"] = t
    gk["ts_bias"] = _dev(kw["ts_tab"])
  if seg:
    cuts = np.sort(rng.choice(np.arange(1, L), 3, replace=False))
    sid = np.tile(np.searchsorted(cuts, np.arange(L), side="right").astype(np.int32), (B, 1))
    kw["q_segment_ids"] = kw["kv_segment_ids"] = sid
    gk["q_segment_ids"] = gk["kv_segment_ids"] = _dev(sid)
    lens = np.full((B,), L, np.int32)
  else:
    kw["seq_lens"] = lens
  want = O.hstu_attention_bwd_ref(q, k, v, dout, **kw)
  variant = []
  gk["_variant_out"] = variant
  if jagged:
    pack = lambda x: O.padded_to_jagged(x, lens)
    (qj, off), (kj, _), (vj, _), (dj, _) = pack(q), pack(k), pack(v), pack(dout)
    if t is not None:
      gk["timestamps"] = _dev(np.concatenate([t[b, :lens[b]] for b in range(B)]))
    got = recml_amd.hstu_attention_bwd(_dev(qj, bf), _dev(kj, bf), _dev(vj, bf), _dev(dj, bf),
                                       seq_offsets=_dev(off.astype(np.int32)), max_len=L, **gk)
    grads = [O.jagged_to_padded(g.float().cpu().numpy(), off, L) for g in got[:3]]
  else:
    if t is not None:
      gk["timestamps"] = _dev(t)
    if not seg:
      gk["seq_lens"] = _dev(lens)
    got = recml_amd.hstu_attention_bwd(_dev(q, bf), _dev(k, bf), _dev(v, bf), _dev(dout, bf), **gk)
    grads = [g.float().cpu().numpy() for g in got[:3]]
  assert variant == ["hstu_bwd_mfma_bf16"]
  for nm, g, w in zip(("dq", "dk", "dv"), grads, want[:3]):
    err = np.abs(g - w).max(axis=(2, 3)) / max(np.abs(w).max(), 1e-30)
    assert err.max() <= 2e-2, (nm, seed, err.max())
  for nm, g, w in (("dpos", got[3], want[3]), ("dts", got[4], want[4])):
    assert (g is None) == (w is None), nm
    if g is not None:
      assert _rel(g.cpu().numpy().reshape(w.shape), w) <= 2e-2, (nm, seed)


@pytest.mark.parametrize("seed", list(range(5000, 5014)))
def test_general_backward_on_random_option_mixes(gpu, seed):
  """fp32 storage (the general backward) against the oracle over random mixes of the options the
  matrix-core pair does not take: explicit mask, dense bias, keys and queries of different lengths,
  odd head dims, together with lengths or segment ids, window and the table biases (fixed seeds)."""
  rng = np.random.default_rng(seed)
  B = int(rng.integers(1, 4))
  H = int(rng.integers(1, 4))
  d = int(rng.choice([8, 24, 32, 48]))
  dv = d if rng.random() < 0.7 else int(rng.choice([8, 40]))
  Lq = int(rng.integers(1, 70))
  cross = rng.random() < 0.3
  Lk = int(rng.integers(1, 70)) if cross else Lq
  causal = bool(rng.random() < 0.5)
  q = rng.standard_normal((B, Lq, H, d)).astype(np.float32) * 0.5
  k = rng.standard_normal((B, Lk, H, d)).astype(np.float32) * 0.5
  v = rng.standard_normal((B, Lk, H, dv)).astype(np.float32) * 0.5
  dout = rng.standard_normal((B, Lq, H, dv)).astype(np.float32) * 0.5
  kw, gk = dict(causal=causal, n=7.0, alpha=0.3), dict(causal=causal, n=7.0, alpha=0.3)
  if rng.random() < 0.4:
    kw["sliding_window_size"] = gk["sliding_window_size"] = int(rng.integers(0, 40))
  if rng.random() < 0.5:
    m = rng.random((B, Lq, Lk) if rng.random() < 0.5 else (Lq, Lk)) < 0.6
    kw["mask"], gk["mask"] = m, _dev(m)
  if rng.random() < 0.5:
    bias = (rng.standard_normal((B if rng.random() < 0.5 else 1, Lq, Lk)) * 0.5).astype(np.float32)
    kw["bias"], gk["bias"] = bias, _dev(bias)
  lens = None
  if rng.random() < 0.35:
    cq, ck = np.sort(rng.integers(0, Lq + 1, 2)), np.sort(rng.integers(0, Lk + 1, 2))
    qs = np.tile(np.searchsorted(cq, np.arange(Lq), side="right").astype(np.int32), (B, 1))
    ks = np.tile(np.searchsorted(ck, np.arange(Lk), side="right").astype(np.int32), (B, 1))
    kw["q_segment_ids"], kw["kv_segment_ids"] = qs, ks
    gk["q_segment_ids"], gk["kv_segment_ids"] = _dev(qs), _dev(ks)
  elif not cross and rng.random() < 0.6:
    lens = rng.integers(0, Lq + 1, B).astype(np.int32)
    kw["seq_lens"], gk["seq_lens"] = lens, _dev(lens)
  if not cross and rng.random() < 0.5:
    kw["pos_tab"] = (rng.standard_normal((H if rng.random() < 0.5 else 1, 2 * Lq - 1)) * 0.3).astype(np.float32)
    gk["pos_bias"] = _dev(kw["pos_tab"])
  t = None
  if not cross and rng.random() < 0.5:
    nb = int(rng.choice([16, 64, 128]))
    kw["ts_tab"] = (rng.standard_normal((H if rng.random() < 0.5 else 1, nb + 1)) * 0.3).astype(np.float32)
    t = 1_700_000_000 + np.cumsum(np.ceil(rng.exponential(3000.0, (B, Lq))), axis=1).astype(np.int64)
    kw["timestamps"] = t
    gk["ts_bias"], gk["timestamps"] = _dev(kw["ts_tab"]), _dev(t)
  want = O.hstu_attention_bwd_ref(q, k, v, dout, **kw)
  variant = []
  got = recml_amd.hstu_attention_bwd(_dev(q), _dev(k), _dev(v), _dev(dout), _variant_out=variant, **gk)
  torch.cuda.synchronize()
  case = dict(seed=seed, B=B, H=H, d=d, dv=dv, Lq=Lq, Lk=Lk, causal=causal, keys=sorted(kw), variant=variant)
  for nm, g, w in zip(("dq", "dk", "dv"), got[:3], want[:3]):
    g = g.cpu().numpy()
    assert g.shape == w.shape and np.isfinite(g).all(), (nm, case)
    err = np.abs(g - w).max(axis=(2, 3)) / max(np.abs(w).max(), 1e-30)
    assert err.max(initial=0.0) <= 2e-5, (nm, case, err.max(initial=0.0))
    if lens is not None:
      for b in range(B):
        assert (g[b, lens[b]:] == 0).all(), (nm, case)
  for nm, g, w in (("dpos", got[3], want[3]), ("dts", got[4], want[4])):
    assert (g is None) == (w is None), (nm, case)
    if g is not None:
      assert _rel(g.cpu().numpy().reshape(w.shape), w) <= 2e-5, (nm, case)


def test_gradients_of_fused_projection_slices_share_one_buffer(gpu):
  """q, k, v cut out of one [T, 4, H, d] projection (as the block does): the gradients come back as
  slices of one buffer laid out like the projection, not three buffers that each span it, and equal
  those of separate tensors."""
  rng = np.random.default_rng(77)
  T, H, d = 300, 2, 128
  off = np.array([0, 130, 300], dtype=np.int32)
  uqkv = torch.from_numpy(O.round_bf16(rng.standard_normal((T, 4, H, d)).astype(np.float32) * 0.4)).to("cuda:0", torch.bfloat16)
  dout = torch.from_numpy(O.round_bf16(rng.standard_normal((T, H, d)).astype(np.float32) * 0.4)).to("cuda:0", torch.bfloat16)
  _, q, k, v = uqkv.unbind(dim=1)
  kw = dict(seq_offsets=torch.from_numpy(off).to("cuda:0"), max_len=170)
  variant = []
  dq, dk, dv, _, _ = recml_amd.hstu_attention_bwd(q, k, v, dout, _variant_out=variant, **kw)
  assert variant == ["hstu_bwd_mfma_bf16"]
  assert dq.stride() == q.stride() and dk.stride() == k.stride() and dv.stride() == v.stride()
  store = {t.untyped_storage().data_ptr() for t in (dq, dk, dv)}
  assert len(store) == 1
  assert dq.untyped_storage().nbytes() <= 1.4 * 3 * q.numel() * 2
  want = recml_amd.hstu_attention_bwd(q.contiguous(), k.contiguous(), v.contiguous(), dout, **kw)
  for g, w_ in zip((dq, dk, dv), want[:3]):
    assert torch.equal(g.contiguous(), w_)


def test_backward_work_list_over_two_segments_of_sequences(gpu):
  """1500 sequences: the work list (built without key-range splits for the backward) takes them 1024 at a time."""
  rng = np.random.default_rng(34)
  B, L, H, d = 1500, 40, 8, 32
  bf = torch.bfloat16
  lens = rng.integers(0, L + 1, B).astype(np.int32)
  q, k, v, dout = (O.round_bf16(rng.standard_normal((B, L, H, d)).astype(np.float32) * 0.5) for _ in range(4))
  want = O.hstu_attention_bwd_ref(q, k, v, dout, seq_lens=lens)
  variant = []
  got = recml_amd.hstu_attention_bwd(_dev(q, bf), _dev(k, bf), _dev(v, bf), _dev(dout, bf), seq_lens=_dev(lens), _variant_out=variant)
  assert variant == ["hstu_bwd_mfma_bf16"]
  for nm, g, w in zip(("dq", "dk", "dv"), got[:3], want[:3]):
    assert _rel(g.float().cpu().numpy(), w) <= 2e-2, nm


@pytest.mark.parametrize("d,dv", [(3, 5), (20, 20), (36, 100), (128, 128), (129, 64), (160, 160)])
@pytest.mark.parametrize("storage", ["fp32", "fp32 views"])
def test_general_backward_head_dims_and_storage(gpu, d, dv, storage):
  """The general backward over head dims that are no multiple of 4 or 16, differ between q/k and v, or go beyond
  128 (those stay on the FMA kernels), with rows that allow 16-byte loads and rows that do not; three tiles of 128
  rows with a partial last one, lengths, causal, both table biases with their gradients."""
  rng = np.random.default_rng(5700 + 7 * d + dv)
  B, L, H = 2, 300, 2
  lens = np.array([300, 77], dtype=np.int32)
  mk = lambda dd: rng.standard_normal((B, L, H, dd)).astype(np.float32) * 0.4
  q, k, v, dout = mk(d), mk(d), mk(dv), mk(dv)
  pos = (rng.standard_normal((H, 2 * L - 1)) * 0.3).astype(np.float32)
  tab = (rng.standard_normal((1, 65)) * 0.3).astype(np.float32)
  t = 1_700_000_000 + np.cumsum(np.ceil(rng.exponential(3000.0, (B, L))), axis=1).astype(np.int64)
  def place(x):
    xd = _dev(x)
    if storage != "fp32 views":
      return xd
    buf = torch.zeros((B, L, H, x.shape[-1] + 3), dtype=torch.float32, device="cuda:0")
    buf[..., 1:1 + x.shape[-1]] = xd
    return buf[..., 1:1 + x.shape[-1]]
  kw = dict(n=float(L), alpha=0.25, causal=True, seq_lens=lens, pos_tab=pos, ts_tab=tab, timestamps=t)
  want = O.hstu_attention_bwd_ref(q, k, v, dout, **kw)
  variant = []
  got = recml_amd.hstu_attention_bwd(place(q), place(k), place(v), place(dout), _variant_out=variant, n=float(L), alpha=0.25,
                                     causal=True, seq_lens=_dev(lens), pos_bias=_dev(pos), ts_bias=_dev(tab), timestamps=_dev(t))
  torch.cuda.synchronize()
  assert variant[-1].startswith("hstu_bwd_general"), variant
  for nm, g, w in zip(("dq", "dk", "dv"), got[:3], want[:3]):
    g = g.cpu().numpy()
    assert g.shape == w.shape and np.isfinite(g).all(), nm
    assert np.abs(g - w).max() <= 2e-5 * np.abs(w).max(), (nm, np.abs(g - w).max() / np.abs(w).max())
    assert (g[1, 77:] == 0).all(), nm
  for nm, g, w in (("dpos", got[3], want[3]), ("dts", got[4], want[4])):
    assert _rel(g.cpu().numpy().reshape(w.shape), w) <= 2e-5, nm


def test_general_kernels_on_a_jagged_batch(gpu):
  """fp32 storage in the jagged layout (forward and backward on the fp32 matrix cores): sequences of 0, 1, 129 and
  300 tokens (empty, one row, one row past a tile, two tiles and a partial one), both table biases and gradients."""
  rng = np.random.default_rng(5900)
  H, d, L = 2, 64, 320
  lens = np.array([300, 0, 1, 129, 64], dtype=np.int32)
  off = np.zeros(len(lens) + 1, dtype=np.int32)
  off[1:] = np.cumsum(lens)
  T = int(off[-1])
  q, k, v, dout = (rng.standard_normal((T, H, d)).astype(np.float32) * 0.4 for _ in range(4))
  pos = (rng.standard_normal((H, 2 * L - 1)) * 0.3).astype(np.float32)
  tab = (rng.standard_normal((H, 129)) * 0.3).astype(np.float32)
  ts = np.concatenate([1_600_000_000 + np.cumsum(np.ceil(rng.exponential(3600.0, n)).astype(np.int64)) for n in lens])
  gk = dict(seq_offsets=_dev(off), max_len=L, n=float(L), alpha=0.3, pos_bias=_dev(pos), ts_bias=_dev(tab), timestamps=_dev(ts))
  out = recml_amd.hstu_attention(_dev(q), _dev(k), _dev(v), **gk).cpu().numpy()
  variant = []
  got = recml_amd.hstu_attention_bwd(_dev(q), _dev(k), _dev(v), _dev(dout), _variant_out=variant, **gk)
  torch.cuda.synchronize()
  assert variant[-1] == "hstu_bwd_general<float>"
  dpos = np.zeros_like(pos, dtype=np.float64)
  dts = np.zeros_like(tab, dtype=np.float64)
  for b, n in enumerate(lens):
    if n == 0:
      continue
    sl = slice(int(off[b]), int(off[b + 1]))
    kw = dict(n=float(L), alpha=0.3, pos_tab=pos[:, L - n: L + n - 1], ts_tab=tab, timestamps=ts[sl][None])
    ref = O.hstu_attention_ref(q[sl][None], k[sl][None], v[sl][None], **kw)
    assert np.abs(out[sl] - ref[0]).max() <= 1e-5 * max(np.abs(ref).max(), 1e-30), b
    want = O.hstu_attention_bwd_ref(q[sl][None], k[sl][None], v[sl][None], dout[sl][None], **kw)
    for nm, g, w in zip(("dq", "dk", "dv"), got[:3], want[:3]):
      assert np.abs(g[sl].cpu().numpy() - w[0]).max() <= 2e-5 * max(np.abs(w).max(), 1e-30), (nm, b)
    dpos[:, L - n: L + n - 1] += want[3]
    dts += want[4]
  assert _rel(got[3].cpu().numpy().reshape(dpos.shape), dpos) <= 2e-5
  assert _rel(got[4].cpu().numpy().reshape(dts.shape), dts) <= 2e-5


@pytest.mark.parametrize("d", [32, 160])
@pytest.mark.parametrize("shared", [False, True])
@pytest.mark.parametrize("storage", ["fp32", "bf16"])
def test_dense_bias_gradient(gpu, d, shared, storage):
  """The gradient of a dense [B | 1, L, Lkv] bias (dS summed over the heads, and over the batch when shared)
  from the general backward -- matrix-core kernels at d = 32, FMA kernels at d = 160 -- with an explicit
  mask, lengths and keys of another length than the queries; dq, dk, dv alongside."""
  rng = np.random.default_rng(6100 + d + shared)
  B, L, Lk, H = 3, 150, 170, 2
  q = rng.standard_normal((B, L, H, d)).astype(np.float32) * 0.4
  k, v = (rng.standard_normal((B, Lk, H, d)).astype(np.float32) * 0.4 for _ in range(2))
  dout = rng.standard_normal((B, L, H, d)).astype(np.float32) * 0.4
  mask = rng.random((B, L, Lk)) < 0.7
  bias = (rng.standard_normal((1 if shared else B, L, Lk)) * 0.4).astype(np.float32)
  tol = 2e-5
  dt = torch.float32
  if storage == "bf16":
    q, k, v, dout = (O.round_bf16(t) for t in (q, k, v, dout))
    dt = torch.bfloat16
  want = O.hstu_attention_bwd_ref(q, k, v, dout, n=9.0, alpha=0.3, causal=False, mask=mask, bias=bias, bias_grad=True)
  variant = []
  got = recml_amd.hstu_attention_bwd(_dev(q, dt), _dev(k, dt), _dev(v, dt), _dev(dout, dt), n=9.0, alpha=0.3, causal=False,
                                     mask=_dev(mask), bias=_dev(bias), bias_grad=True, _variant_out=variant)
  torch.cuda.synchronize()
  assert variant[-1].startswith("hstu_bwd_general")
  assert got[5].shape == bias.shape and got[5].dtype == torch.float32
  assert _rel(got[5].cpu().numpy(), want[5]) <= (tol if storage == "fp32" else 2e-2)
  for nm, g, w in zip(("dq", "dk", "dv"), got[:3], want[:3]):
    assert _rel(g.float().cpu().numpy(), w) <= (tol if storage == "fp32" else 2e-2), nm
  # through autograd: the same gradient reaches a bias that requires it
  bt = _dev(bias).requires_grad_(True)
  out = recml_amd.hstu_attention_autograd(_dev(q, dt), _dev(k, dt), _dev(v, dt), n=9.0, alpha=0.3, causal=False,
                                          mask=_dev(mask), bias=bt)
  (out.float() * _dev(dout)).sum().backward()
  assert _rel(bt.grad.cpu().numpy(), want[5]) <= (tol if storage == "fp32" else 2e-2)


@pytest.mark.parametrize("shape", ["band", "blocks", "ragged16", "offset_view", "empty_tile"])
def test_general_kernels_leave_out_the_steps_a_mask_empties(gpu, shape):
  """The general kernels find, per tile, the first and last step an explicit mask keeps anything in and run
  only those.  Masks whose live range is cut on both sides, per row tile and per key tile: a band, diagonal
  blocks, a tile the mask empties altogether; and the two layouts that switch the search off (a key length
  that is no multiple of 16, a mask view that starts off a 16-byte boundary).  Forward and backward in fp32
  against the oracle, the dense bias's gradient included."""
  rng = np.random.default_rng(7300 + len(shape))
  B, L, H, d = 2, 400, 2, 32
  Lk = 400 if shape != "ragged16" else 390
  i, j = np.arange(L)[:, None], np.arange(Lk)[None, :]
  if shape in ("band", "ragged16", "offset_view"):
    mask = (j <= i) & (j >= i - 70)                      # a band: live keys start late and end early for most tiles
  elif shape == "blocks":
    mask = (i // 96) == (j // 96)                        # diagonal blocks that straddle the 128-row tiles
  else:
    mask = (j <= i) & ~((i >= 128) & (i < 256))          # rows 128..255 keep nothing: one whole row tile is empty
    mask &= ~((j >= 256) & (j < 384))                    # and so is one whole key tile
  mask = np.broadcast_to(mask, (B, L, Lk)) & (rng.random((B, L, Lk)) < 0.9)
  q = rng.standard_normal((B, L, H, d)).astype(np.float32) * 0.4
  k, v = (rng.standard_normal((B, Lk, H, d)).astype(np.float32) * 0.4 for _ in range(2))
  dout = rng.standard_normal((B, L, H, d)).astype(np.float32) * 0.4
  bias = (rng.standard_normal((B, L, Lk)) * 0.4).astype(np.float32)
  want_out = O.hstu_attention_ref(q, k, v, n=7.0, alpha=0.3, causal=False, mask=mask, bias=bias)
  want = O.hstu_attention_bwd_ref(q, k, v, dout, n=7.0, alpha=0.3, causal=False, mask=mask, bias=bias, bias_grad=True)
  md = _dev(mask.astype(np.uint8))
  if shape == "offset_view":
    flat = torch.zeros(B * L * Lk + 16, dtype=torch.uint8, device=md.device)
    flat[5: 5 + B * L * Lk] = md.reshape(-1)
    md = flat[5: 5 + B * L * Lk].view(B, L, Lk)
    assert md.data_ptr() % 16 != 0
  args = [_dev(t) for t in (q, k, v)]
  out = recml_amd.hstu_attention(*args, n=7.0, alpha=0.3, causal=False, mask=md, bias=_dev(bias))
  variant = []
  got = recml_amd.hstu_attention_bwd(*args, _dev(dout), n=7.0, alpha=0.3, causal=False, mask=md, bias=_dev(bias),
                                     bias_grad=True, _variant_out=variant)
  torch.cuda.synchronize()
  assert variant[-1].startswith("hstu_bwd_general")
  assert _rel(out.cpu().numpy(), want_out) <= 2e-5
  for nm, g, w in zip(("dq", "dk", "dv"), got[:3], want[:3]):
    assert _rel(g.cpu().numpy(), w) <= 2e-5, nm
  assert _rel(got[5].cpu().numpy(), want[5]) <= 2e-5
  if shape == "empty_tile":
    assert float(out[:, 128:256].abs().max()) == 0 and float(got[0][:, 128:256].abs().max()) == 0
    assert float(got[1][:, 256:384].abs().max()) == 0 and float(got[2][:, 256:384].abs().max()) == 0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_gradients_written_into_given_slices(gpu, dtype):
  """grads_out: dq, dk, dv land in the slices of one tensor laid out like a fused projection (what the block's
  backward hands over), bit for bit what the call returns on its own, and nothing else of that tensor is
  touched; buffers of another layout are refused."""
  rng = np.random.default_rng(8100)
  B, L, H, d = 2, 200, 2, 64
  fused = _dev(rng.standard_normal((B, L, 4, H, d)).astype(np.float32) * 0.4, dtype)
  q, k, v = fused[:, :, 1], fused[:, :, 2], fused[:, :, 3]
  dout = _dev(rng.standard_normal((B, L, H, d)).astype(np.float32) * 0.4, dtype)
  lens = _dev(np.array([200, 77], np.int32))
  pos = _dev((rng.standard_normal((H, 2 * L - 1)) * 0.3).astype(np.float32))
  want = recml_amd.hstu_attention_bwd(q, k, v, dout, seq_lens=lens, pos_bias=pos)
  grad = torch.full_like(fused, 7.0)
  got = recml_amd.hstu_attention_bwd(q, k, v, dout, seq_lens=lens, pos_bias=pos,
                                     grads_out=(grad[:, :, 1], grad[:, :, 2], grad[:, :, 3]))
  torch.cuda.synchronize()
  for i in range(3):
    assert got[i].data_ptr() == grad[:, :, 1 + i].data_ptr()
    assert torch.equal(grad[:, :, 1 + i], want[i])
  assert bool((grad[:, :, 0] == 7.0).all())
  # the position table's gradient is summed by atomic adds in an order that varies: equal to rounding
  assert _rel(got[3].cpu().numpy(), want[3].cpu().numpy()) <= 1e-5
  with pytest.raises(ValueError, match="grads_out"):
    recml_amd.hstu_attention_bwd(q, k, v, dout, seq_lens=lens, pos_bias=pos,
                                 grads_out=(torch.empty_like(q), grad[:, :, 2], grad[:, :, 3]))


@pytest.mark.parametrize("d,dv,view,products,layout", [
    (16, 16, False, True, "padded"), (48, 80, False, True, "padded"), (48, 80, False, True, "jagged"), (64, 32, False, True, "padded"),
    (128, 128, False, True, "padded + zero bias"),          # (a dense bias keeps d = 128 off the hand-scheduled pair)
    (40, 40, False, False, "padded"), (40, 40, False, False, "jagged"), (64, 64, True, False, "padded"), (160, 160, False, False, "padded")])
def test_general_backward_in_bf16_storage(gpu, d, dv, view, products, layout):
  """bf16 tensors on the general backward: head dims in multiples of 16 with rows on 16-byte boundaries take the
  bf16 products, everything else -- other head dims, rows that start off a boundary, head dims beyond 128 -- the
  fp32 ones; both against the oracle on the same bf16 inputs, table gradients included."""
  rng = np.random.default_rng(8300 + 3 * d + dv + view)
  bf = torch.bfloat16
  B, L, Lk, H = 3, 200, 200, 2
  lens = np.array([200, 77, 130], dtype=np.int32)
  mk = lambda dd: O.round_bf16(rng.standard_normal((B, L, H, dd)).astype(np.float32) * 0.4)
  q, k, v, dout = mk(d), mk(d), mk(dv), mk(dv)
  pos = (rng.standard_normal((H, 2 * L - 1)) * 0.3).astype(np.float32)
  tab = (rng.standard_normal((1, 33)) * 0.3).astype(np.float32)
  t = 1_700_000_000 + np.cumsum(np.ceil(rng.exponential(3000.0, (B, L))), axis=1).astype(np.int64)
  for b in range(B):
    t[b, lens[b]:] = t[b, lens[b] - 1]
  kw = dict(n=float(L), alpha=0.25, causal=True, seq_lens=lens, pos_tab=pos, ts_tab=tab, timestamps=t, sliding_window_size=150)
  zero_bias = np.zeros((1, L, L), np.float32) if layout.endswith("zero bias") else None
  want = O.hstu_attention_bwd_ref(q, k, v, dout, bias=zero_bias, **kw)

  def place(x):
    if layout == "jagged":
      x = O.padded_to_jagged(x, lens)[0]
    xd = _dev(x, bf)
    if not view:
      return xd
    buf = torch.zeros(xd.shape[:-1] + (x.shape[-1] + 8,), dtype=bf, device="cuda:0")
    buf[..., 1:1 + x.shape[-1]] = xd
    return buf[..., 1:1 + x.shape[-1]]                # rows start two bytes off a 16-byte boundary
  gk = dict(n=float(L), alpha=0.25, causal=True, pos_bias=_dev(pos), ts_bias=_dev(tab), sliding_window_size=150)
  if layout == "jagged":
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    gk.update(seq_offsets=_dev(off), max_len=L, timestamps=_dev(O.padded_to_jagged(t[..., None, None], lens)[0].reshape(-1)))
  else:
    gk.update(seq_lens=_dev(lens), timestamps=_dev(t))
  if zero_bias is not None:
    gk.update(bias=_dev(zero_bias))
  variant = []
  got = recml_amd.hstu_attention_bwd(place(q), place(k), place(v), place(dout), _variant_out=variant, **gk)
  torch.cuda.synchronize()
  assert variant[-1] == ("hstu_bwd_general<bf16, bf16 products>" if products else "hstu_bwd_general<bf16>"), variant
  for nm, g, w in zip(("dq", "dk", "dv"), got[:3], want[:3]):
    g = g.float().cpu().numpy()
    if layout == "jagged":
      g = O.jagged_to_padded(g, off, L)
    assert np.isfinite(g).all() and _rel(g, w) <= 2e-2, (nm, _rel(g, w))
  for nm, g, w in (("dpos", got[3], want[3]), ("dts", got[4], want[4])):
    assert _rel(g.cpu().numpy().reshape(w.shape), w) <= 2e-2, nm


def test_reference_named_entry_points_are_differentiable(gpu):
  """The reference's own test of the op (recml/core/ops/hstu_ops_test.py:25-96): value_and_grad of
  sum((attn - targets)^2) through pointwise_splash_attention with segment ids, against the dense form.  Here through
  torch autograd, against the oracle's pw_attn_ref and its backward; the layer-side call the same way."""
  rng = np.random.default_rng(50)
  B, L, H, d = 2, 64, 2, 32
  q, k, v, targets = (rng.standard_normal((B, L, H, d)).astype(np.float32) for _ in range(4))
  seg = np.zeros((B, L), np.int32)
  seg[0, :40] = 1
  seg[1, :13] = 1
  qt, kt, vt = (_dev(x).requires_grad_(True) for x in (q, k, v))
  attn = recml_amd.pointwise_splash_attention(recml_amd.MaskType.CAUSAL, qt, kt, vt, q_segment_ids=_dev(seg),
                                              kv_segment_ids=_dev(seg))
  ((attn - _dev(targets)) ** 2).sum().backward()
  ref = O.pw_attn_ref(q, k, v, seg)
  got = attn.detach().cpu().numpy()
  np.testing.assert_allclose(got, ref, atol=1e-5, rtol=1e-5)           # the reference accepts 5e-3
  dq, dk, dv, _, _ = O.hstu_attention_bwd_ref(q, k, v, 2.0 * (ref - targets), alpha=1 / np.sqrt(d), n=L,
                                              q_segment_ids=seg, kv_segment_ids=seg)
  for nm, g, w in (("dq", qt.grad, dq), ("dk", kt.grad, dk), ("dv", vt.grad, dv)):
    assert _rel(g.cpu().numpy(), w) <= 2e-5, nm
  # without a gradient asked for, the same values from the forward alone
  with torch.no_grad():
    again = recml_amd.pointwise_splash_attention(recml_amd.MaskType.CAUSAL, qt, kt, vt, q_segment_ids=_dev(seg),
                                                 kv_segment_ids=_dev(seg))
  assert torch.equal(again, attn.detach())
  # the layer-side call with a dense mask and a bias that is trained
  mask = O.make_causal_mask((np.arange(L)[None] < np.array([[40], [13]])).astype(np.float32))
  bias = (rng.standard_normal((B, L, L)) * 0.3).astype(np.float32)
  for t in (qt, kt, vt):
    t.grad = None
  bt = _dev(bias).requires_grad_(True)
  out = recml_amd.pointwise_attention(qt, kt, vt, _dev(mask), bt)
  ((out - _dev(targets)) ** 2).sum().backward()
  ref = O.pointwise_attention_dense(q, k, v, mask, bias)
  np.testing.assert_allclose(out.detach().cpu().numpy(), ref, atol=1e-5, rtol=1e-5)
  want = O.hstu_attention_bwd_ref(q, k, v, 2.0 * (ref - targets), causal=False, mask=mask, bias=bias, bias_grad=True)
  for nm, g, w in (("dq", qt.grad, want[0]), ("dk", kt.grad, want[1]), ("dv", vt.grad, want[2]), ("dbias", bt.grad, want[5])):
    assert _rel(g.cpu().numpy(), w) <= 2e-5, nm


MASK_CASES = [
    # name, d, B, L, H, mask kind, batched, causal flag, dropout
    ("d128 causal + lengths as a mask", 128, 2, 300 - 300 % 16, 2, "causal_lens", True, False, 0.0),
    ("d128 random mask, shared", 128, 2, 272, 2, "random", False, False, 0.0),
    ("d128 random mask with the causal flag", 128, 3, 400, 1, "random", True, True, 0.0),
    ("d128 band", 128, 2, 512, 2, "band", False, False, 0.0),
    ("d128 causal + lengths, dropout", 128, 2, 256, 2, "causal_lens", True, False, 0.3),
    ("d64 causal + lengths as a mask", 64, 3, 208, 4, "causal_lens", True, False, 0.0),
    ("d64 random mask", 64, 2, 160, 2, "random", True, False, 0.0),
    ("d32 random mask, shared", 32, 2, 144, 2, "random", False, False, 0.0),
    ("d128 empty rows and columns", 128, 2, 256, 2, "holes", True, False, 0.0),
]


@pytest.mark.parametrize("name,d,B,L,H,kind,batched,causal,drop", MASK_CASES, ids=[c[0] for c in MASK_CASES])
def test_backward_with_a_dense_mask_on_the_matrix_cores(gpu, name, d, B, L, H, kind, batched, causal, drop):
  """The layer-side calling convention without a dense bias (recml/layers/keras/hstu.py:380-384 with
  make_causal_mask's [B, L, L] mask): bf16, d in {32, 64, 128} take the matrix-core pair, the mask tile by tile."""
  rng = np.random.default_rng(60)
  bf = torch.bfloat16
  q, k, v, dout = (O.round_bf16(rng.standard_normal((B, L, H, d)).astype(np.float32) * 0.5) for _ in range(4))
  i = np.arange(L)
  if kind == "causal_lens":
    lens = np.array([L, L // 2 + 5, 1][:B])
    m = (i[None, None, :] <= i[None, :, None]) & (i[None, :, None] < lens[:, None, None]) & (i[None, None, :] < lens[:, None, None])
  elif kind == "random":
    m = rng.random((B if batched else 1, L, L)) > 0.4
  elif kind == "band":
    m = (np.abs(i[None, :, None] - i[None, None, :]) <= 70) & (i[None, None, :] <= i[None, :, None] + 3)
  else:
    # whole 128-row tiles, whole 32-key steps and whole 128-key tiles without a kept pair, and single kept pairs
    m = np.zeros((B, L, L), bool)
    m[0, 130:140, 0:20] = True
    m[0, 255, 255] = True
    m[1, 0, 0] = True
    m[1, 200:256, 64:96] = rng.random((56, 32)) > 0.5
  if not batched:
    m = m[0] if m.ndim == 3 else m
  kw = dict(causal=causal, mask=m, n=float(L) / 3, dropout_p=drop, dropout_seed=77)
  want = O.hstu_attention_bwd_ref(q, k, v, dout, **kw)
  variant = []
  got = recml_amd.hstu_attention_bwd(_dev(q, bf), _dev(k, bf), _dev(v, bf), _dev(dout, bf), _variant_out=variant,
                                     **{**kw, "mask": _dev(m)})
  assert variant == ["hstu_bwd_mfma_bf16"]
  for nm, g, w in zip(("dq", "dk", "dv"), got[:3], want[:3]):
    g = g.float().cpu().numpy()
    assert np.abs(w).max() > 0, nm
    assert _rel(g, w) <= 2e-2, nm
    assert ((w == 0) <= (g == 0)).all(), nm          # rows and keys that keep nothing: exactly 0
  assert got[3] is None and got[4] is None
  # keys and queries of different lengths: the general pair
  variant = []
  m2 = np.ones((L, L + 16), bool)
  recml_amd.hstu_attention_bwd(_dev(q, bf), _dev(np.concatenate([k, k[:, :16]], 1), bf), _dev(np.concatenate([v, v[:, :16]], 1), bf),
                               _dev(dout, bf), _variant_out=variant, causal=False, mask=_dev(m2))
  assert variant[0].startswith("hstu_bwd_general")


def test_backward_with_a_dense_mask_and_lengths_on_the_matrix_cores(gpu):
  """The mask as one more factor next to the lengths and the causal flag (the C ABI's meaning of `mask`)."""
  rng = np.random.default_rng(61)
  B, L, H, d = 3, 336, 2, 128
  bf = torch.bfloat16
  q, k, v, dout = (O.round_bf16(rng.standard_normal((B, L, H, d)).astype(np.float32) * 0.5) for _ in range(4))
  lens = np.array([336, 129, 40], np.int32)
  m = rng.random((L, L)) > 0.5
  want = O.hstu_attention_bwd_ref(q, k, v, dout, seq_lens=lens, mask=m, alpha=0.5)
  variant = []
  got = recml_amd.hstu_attention_bwd(_dev(q, bf), _dev(k, bf), _dev(v, bf), _dev(dout, bf), seq_lens=_dev(lens), mask=_dev(m),
                                     alpha=0.5, _variant_out=variant)
  assert variant == ["hstu_bwd_mfma_bf16"]
  for nm, g, w in zip(("dq", "dk", "dv"), got[:3], want[:3]):
    g = g.float().cpu().numpy()
    assert _rel(g, w) <= 2e-2, nm
    for b in range(B):
      assert (g[b, lens[b]:] == 0).all(), nm


@pytest.mark.parametrize("seed", range(6))
def test_backward_with_a_dense_mask_random_shapes(gpu, seed):
  rng = np.random.default_rng(700 + seed)
  bf = torch.bfloat16
  d = int(rng.choice([32, 64, 128]))
  B, H = int(rng.integers(1, 4)), int(rng.integers(1, 4))
  L = 16 * int(rng.integers(1, 30))
  q, k, v, dout = (O.round_bf16(rng.standard_normal((B, L, H, d)).astype(np.float32) * 0.5) for _ in range(4))
  batched = bool(rng.integers(0, 2))
  density = float(rng.choice([0.02, 0.3, 0.9]))
  m = rng.random((B, L, L) if batched else (L, L)) < density
  kw = dict(causal=bool(rng.integers(0, 2)), mask=m, n=float(rng.integers(1, L + 1)), alpha=float(rng.uniform(0.2, 1.0)))
  if rng.integers(0, 2):
    kw["seq_lens"] = rng.integers(0, L + 1, B).astype(np.int32)
  if rng.integers(0, 2):
    kw.update(dropout_p=0.25, dropout_seed=int(rng.integers(0, 2 ** 40)))
  case = dict(seed=seed, d=d, B=B, H=H, L=L, batched=batched, density=density, keys=sorted(kw))
  want = O.hstu_attention_bwd_ref(q, k, v, dout, **kw)
  gk = {**kw, "mask": _dev(m)}
  if "seq_lens" in kw:
    gk["seq_lens"] = _dev(kw["seq_lens"])
  variant = []
  got = recml_amd.hstu_attention_bwd(_dev(q, bf), _dev(k, bf), _dev(v, bf), _dev(dout, bf), _variant_out=variant, **gk)
  assert variant == ["hstu_bwd_mfma_bf16"], case
  scale = max(np.abs(w).max() for w in want[:3])
  for nm, g, w in zip(("dq", "dk", "dv"), got[:3], want[:3]):
    g = g.float().cpu().numpy()
    assert np.abs(g - w).max() <= 2e-2 * max(np.abs(w).max(), 0.05 * scale), (nm, case)
    assert ((w == 0) <= (g == 0)).all(), (nm, case)


BIAS_CASES = [
    # name, d, B, L, H, bias batched, with a mask, the bias gradient, dropout
    ("d128 bias per sequence + mask, gradient", 128, 2, 272, 2, True, True, True, 0.0),
    ("d128 shared bias, lengths, gradient", 128, 3, 400, 2, False, False, True, 0.0),
    ("d128 bias + mask, no gradient", 128, 2, 256, 1, True, True, False, 0.0),
    ("d128 shared bias + shared mask, gradient, dropout", 128, 2, 208, 2, False, True, True, 0.3),
    ("d64 bias per sequence + mask, gradient", 64, 3, 176, 4, True, True, True, 0.0),
    ("d32 shared bias, gradient", 32, 2, 144, 2, False, False, True, 0.0),
]


@pytest.mark.parametrize("name,d,B,L,H,batched,with_mask,grad,drop", BIAS_CASES, ids=[c[0] for c in BIAS_CASES])
def test_backward_with_a_dense_bias_on_the_matrix_cores(gpu, name, d, B, L, H, batched, with_mask, grad, drop):
  """The layer-side calling convention in full (recml/layers/keras/hstu.py:371-384: a dense bias shared by the heads,
  a dense mask): the matrix-core pair takes both operands tile by tile and returns the bias's gradient (dS summed
  over the heads, and over the sequences for a shared bias)."""
  rng = np.random.default_rng(62)
  bf = torch.bfloat16
  q, k, v, dout = (O.round_bf16(rng.standard_normal((B, L, H, d)).astype(np.float32) * 0.5) for _ in range(4))
  bias = (rng.standard_normal((B if batched else 1, L, L)) * 0.5).astype(np.float32)
  lens = np.array([L, L // 2 + 5, 1][:B], np.int32)
  kw = dict(n=float(L) / 3, bias=bias, dropout_p=drop, dropout_seed=5)
  gk = dict(n=float(L) / 3, bias=_dev(bias), dropout_p=drop, dropout_seed=5)
  if with_mask:
    i = np.arange(L)
    m = (rng.random((B, L, L) if batched else (L, L)) > 0.3) & (i[None, :] <= i[:, None] + 2)
    kw.update(causal=False, mask=m)
    gk.update(causal=False, mask=_dev(m))
  else:
    kw.update(seq_lens=lens)
    gk.update(seq_lens=_dev(lens))
  want = O.hstu_attention_bwd_ref(q, k, v, dout, bias_grad=grad, **kw)
  variant = []
  got = recml_amd.hstu_attention_bwd(_dev(q, bf), _dev(k, bf), _dev(v, bf), _dev(dout, bf), bias_grad=grad,
                                     _variant_out=variant, **gk)
  assert variant == ["hstu_bwd_mfma_bf16"]
  for nm, g, w in zip(("dq", "dk", "dv"), got[:3], want[:3]):
    g = g.float().cpu().numpy()
    assert np.abs(w).max() > 0 and _rel(g, w) <= 2e-2, nm
    assert ((w == 0) <= (g == 0)).all(), nm
  if grad:
    g, w = got[5].cpu().numpy(), want[5]
    assert g.shape == w.shape == bias.shape
    assert np.abs(w).max() > 0 and _rel(g, w) <= 2e-2
    assert ((w == 0) <= (g == 0)).all()                # pairs nobody keeps get no gradient
  else:
    assert len(got) == 5


@pytest.mark.parametrize("batched", [False, True])
def test_backward_with_dense_operands_in_the_jagged_layout(gpu, batched):
  """Packed tokens with a dense mask and bias ([L, L]-shaped per sequence position): forward and backward on the matrix
  cores, the bias gradient included."""
  rng = np.random.default_rng(63)
  B, L, H, d = 3, 272, 2, 128
  lens = np.array([272, 100, 33], np.int32)
  bf = torch.bfloat16
  q, k, v, dout = (O.round_bf16(rng.standard_normal((B, L, H, d)).astype(np.float32) * 0.5) for _ in range(4))
  m = rng.random((B, L, L) if batched else (L, L)) > 0.4
  bias = (rng.standard_normal((B if batched else 1, L, L)) * 0.5).astype(np.float32)
  want = O.hstu_attention_bwd_ref(q, k, v, dout, seq_lens=lens, mask=m, bias=bias, bias_grad=True)
  want_out = O.hstu_attention_ref(q, k, v, seq_lens=lens, mask=m, bias=bias)
  pack = lambda x: O.padded_to_jagged(x, lens)
  (qj, off), (kj, _), (vj, _), (dj, _) = pack(q), pack(k), pack(v), pack(dout)
  kw = dict(seq_offsets=_dev(off.astype(np.int32)), max_len=L, mask=_dev(m), bias=_dev(bias))
  out = recml_amd.hstu_attention(_dev(qj, bf), _dev(kj, bf), _dev(vj, bf), **kw)
  assert _rel(O.jagged_to_padded(out.float().cpu().numpy(), off, L), want_out) <= 2e-2
  variant = []
  got = recml_amd.hstu_attention_bwd(_dev(qj, bf), _dev(kj, bf), _dev(vj, bf), _dev(dj, bf), bias_grad=True, _variant_out=variant, **kw)
  assert variant == ["hstu_bwd_mfma_bf16"]
  for nm, g, w in zip(("dq", "dk", "dv"), got[:3], want[:3]):
    assert _rel(O.jagged_to_padded(g.float().cpu().numpy(), off, L), w) <= 2e-2, nm
  assert _rel(got[5].cpu().numpy(), want[5]) <= 2e-2
