"""The matrix-core forward takes the entries of its work list in one of two ways (bf16, d = 128): one
workgroup per entry, or resident workgroups that draw entry after entry.  Both do the same arithmetic
in the same order: every case here runs both (forced by the flag bits of the C ABI) and asks for the
same bits, and checks one of them against the oracle."""

import numpy as np
import pytest
import torch

from recml_amd import _lib, hstu_ops, workloads
from oracle import hstu_oracle as O

pytestmark = pytest.mark.gpu

BF16_TOL = 2e-2
bf = torch.bfloat16


def _dev(x, dtype=None):
  t = torch.from_numpy(np.ascontiguousarray(x)).to("cuda:0")
  return t if dtype is None else t.to(dtype)


def _rel(a, b):
  return np.abs(np.asarray(a, np.float64) - b).max() / max(np.abs(b).max(), 1e-30)


def _both(q, k, v, **kw):
  """Runs the call once per way, three times over (the draw counters and arrival counters must be left
  ready for the next call); returns the two outputs."""
  outs = {}
  for name, flag in (("one", _lib.FWD_ONE_ITEM_PER_WORKGROUP), ("resident", _lib.FWD_RESIDENT_WORKGROUPS)):
    out = torch.empty_like(v)
    a, keep = hstu_ops.build_args(q, k, v, out, **kw)
    assert hstu_ops.kernel_variant(a) == "hstu_fwd_mfma_bf16"
    a.flags |= flag
    first = None
    for rep in range(3):
      out.fill_(float("nan"))
      hstu_ops._run(a, keep)
      got = out.float().cpu().numpy()
      if first is None:
        first = got
      else:
        assert np.array_equal(first, got), (name, rep)
    outs[name] = first
  return outs["one"], outs["resident"]


# lengths whose last tile ends after 1 .. 9 steps of 32 keys, an empty sequence, one of two full tiles
LENS = np.array([1, 32, 33, 64, 0, 65, 96, 97, 128, 129, 160, 161, 192, 223, 256, 257, 288], dtype=np.int32)


@pytest.mark.parametrize("H", [1, 2, 8, 16])
@pytest.mark.parametrize("bias", [False, True])
def test_every_step_count_jagged(gpu, H, bias):
  rng = np.random.default_rng(1200 + H + bias)
  L, d = 288, 128
  off = np.zeros(len(LENS) + 1, dtype=np.int32)
  off[1:] = np.cumsum(LENS)
  T = int(off[-1])
  q, k, v = (O.round_bf16(rng.standard_normal((T, H, d)).astype(np.float32) * 0.3) for _ in range(3))
  kw, gk = {}, {}
  if bias:
    kw["pos_tab"] = (rng.standard_normal((H, 2 * L - 1)) * 0.2).astype(np.float32)
    kw["ts_tab"] = (rng.standard_normal((H, 129)) * 0.2).astype(np.float32)
    ts = np.concatenate([1_600_000_000 + np.cumsum(np.ceil(rng.exponential(3600.0, n)).astype(np.int64)) for n in LENS])
    kw["timestamps"] = ts
    gk = dict(pos_bias=_dev(kw["pos_tab"]), ts_bias=_dev(kw["ts_tab"]), timestamps=_dev(ts))
  one, res = _both(_dev(q, bf), _dev(k, bf), _dev(v, bf), seq_offsets=_dev(off), max_len=L, **gk)
  assert np.array_equal(one, res)
  ref = O.hstu_attention_jagged_ref(q, k, v, off, L, **kw)
  assert _rel(res, ref) <= BF16_TOL


@pytest.mark.parametrize("causal,window", [(True, None), (False, None), (True, 70), (False, 40)])
def test_padded_layout_with_lengths_and_windows(gpu, causal, window):
  rng = np.random.default_rng(1300 + causal + (window or 0))
  B, L, H, d = 5, 420, 8, 128
  lens = np.array([420, 383, 131, 0, 1], dtype=np.int32)
  q, k, v = (O.round_bf16(rng.standard_normal((B, L, H, d)).astype(np.float32) * 0.4) for _ in range(3))
  pos = (rng.standard_normal((H, 2 * L - 1)) * 0.3).astype(np.float32)
  one, res = _both(_dev(q, bf), _dev(k, bf), _dev(v, bf), seq_lens=_dev(lens), causal=causal,
                   sliding_window_size=window, pos_bias=_dev(pos))
  assert np.array_equal(one, res)
  ref = O.hstu_attention_ref(q, k, v, seq_lens=lens, causal=causal, sliding_window_size=window, pos_tab=pos)
  assert _rel(res, ref) <= BF16_TOL


def test_split_tiles_and_many_items_per_workgroup(gpu):
  """A few long sequences among many short ones: the long tiles are split over their keys (their parts
  meet at the arrival counters), and there are more entries than resident workgroups."""
  rng = np.random.default_rng(1400)
  H, d, L = 8, 128, 2048
  lens = np.concatenate([[2048, 1999, 1500], rng.integers(1, 400, 120)]).astype(np.int32)
  off = np.zeros(len(lens) + 1, dtype=np.int32)
  off[1:] = np.cumsum(lens)
  T = int(off[-1])
  q, k, v = (O.round_bf16(rng.standard_normal((T, H, d)).astype(np.float32) * 0.3) for _ in range(3))
  pos = (rng.standard_normal((H, 2 * L - 1)) * 0.2).astype(np.float32)
  tab = (rng.standard_normal((H, 129)) * 0.2).astype(np.float32)
  ts = np.concatenate([1_600_000_000 + np.cumsum(np.ceil(rng.exponential(3600.0, n)).astype(np.int64)) for n in lens])
  one, res = _both(_dev(q, bf), _dev(k, bf), _dev(v, bf), seq_offsets=_dev(off), max_len=L,
                   pos_bias=_dev(pos), ts_bias=_dev(tab), timestamps=_dev(ts))
  assert np.array_equal(one, res)
  # the oracle on the three long sequences (split) and ten of the short ones
  for b in list(range(3)) + list(range(3, 123, 12)):
    sl = slice(int(off[b]), int(off[b + 1]))
    o1 = np.array([0, lens[b]], dtype=np.int32)
    ref = O.hstu_attention_jagged_ref(q[sl], k[sl], v[sl], o1, L, pos_tab=pos, ts_tab=tab, timestamps=ts[sl])
    assert _rel(res[sl], ref) <= BF16_TOL, b


def test_headline_shape(gpu):
  w = workloads.config3()
  t = lambda x: None if x is None else _dev(x)
  one, res = _both(t(w.q).to(bf), t(w.k).to(bf), t(w.v).to(bf), seq_offsets=t(w.seq_offsets), max_len=w.L,
                   n=w.n, alpha=w.alpha, pos_bias=t(w.pos_tab), ts_bias=t(w.ts_tab), timestamps=t(w.timestamps))
  assert np.array_equal(one, res)


@pytest.mark.parametrize("d", [128, 64])
def test_more_sequences_than_one_list_segment(gpu, d):
  """2600 sequences: the list builder takes them 1024 at a time, in batch order (no sorting), with the
  item and chunk-slot counts carried from one segment to the next; one long sequence in the third segment
  has tiles that are split."""
  rng = np.random.default_rng(1600 + d)
  H, L, B = 8, 1024, 2600
  lens = rng.integers(0, 150, B).astype(np.int32)
  lens[2100] = 1024
  lens[7] = 700
  off = np.zeros(B + 1, dtype=np.int32)
  off[1:] = np.cumsum(lens)
  T = int(off[-1])
  q, k, v = (O.round_bf16(rng.standard_normal((T, H, d)).astype(np.float32) * 0.3) for _ in range(3))
  pos = (rng.standard_normal((H, 2 * L - 1)) * 0.2).astype(np.float32)
  if d == 128:
    one, res = _both(_dev(q, bf), _dev(k, bf), _dev(v, bf), seq_offsets=_dev(off), max_len=L, pos_bias=_dev(pos))
    assert np.array_equal(one, res)
  else:
    import recml_amd
    res = recml_amd.hstu_attention(_dev(q, bf), _dev(k, bf), _dev(v, bf), seq_offsets=_dev(off), max_len=L,
                                   pos_bias=_dev(pos)).float().cpu().numpy()
  for b in [0, 7, 1023, 1024, 1025, 2047, 2048, 2100, 2599] + list(rng.integers(0, B, 12)):
    sl = slice(int(off[b]), int(off[b + 1]))
    if lens[b] == 0:
      continue
    o1 = np.array([0, lens[b]], dtype=np.int32)
    ref = O.hstu_attention_jagged_ref(q[sl], k[sl], v[sl], o1, L, pos_tab=pos)
    assert _rel(res[sl], ref) <= BF16_TOL, b
  # every row was written by someone: nothing is left of the fill
  assert np.isfinite(res).all()
