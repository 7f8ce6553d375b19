"""Attention dropout without a GPU: the oracle's keep rule against known answers and against the library's host
function, its statistics, and the oracle's forward and backward with dropout.

The reference applies keras' Dropout to the masked attention weights in training
(recml/layers/keras/hstu.py:386-387): a weight is dropped with probability `rate`, a survivor is scaled by
1 / (1 - rate).  Which weights are drawn comes from keras' seed generator there and cannot be reproduced; here it
is a fixed 32-bit hash of (seed, sequence, head, i, j), which the host library, every kernel and the oracle share.
"""

import ctypes as C

import numpy as np
import pytest

from oracle import hstu_oracle as O
from recml_amd import _lib

M = 0xFFFFFFFF


def _scalar_hash(seed, b, h, H, i, j):
  """The hash with Python's unbounded integers, one pair at a time."""
  z = (seed & M) ^ 0x9E3779B9
  z = ((z ^ (z >> 16)) * 0x85EBCA6B) & M
  z ^= (seed >> 32) & M
  z = ((z ^ (z >> 13)) * 0xC2B2AE35) & M
  key = z ^ (z >> 16)
  z = (key + (b * H + h) * 0x9E3779B1) & M
  z = ((z ^ (z >> 15)) * 0x2C1B3C6D) & M
  kbh = z ^ (z >> 13)
  ij = (kbh + i * 0x85EBCA77 + j * 0xC2B2AE3D) & M
  z = (ij * 0x2C1B3C6D) & M
  return ((z ^ (z >> 16)) * 0x297A2D39) & M


# (seed, b, h, H, i, j) -> seed key, hash: worked once and kept as literals
KNOWN = [
    ((0, 0, 0, 1, 0, 0), 0x92CA2F0E, 0xE5E1963A),
    ((1, 0, 0, 1, 0, 0), 0x36DEB503, 0x87169A29),
    ((0x123456789ABCDEF0, 3, 5, 8, 2047, 1023), 0x6546363E, 0xA8933E67),
    ((42, 1, 1, 2, 7, 3), 0xE5D9EED0, 0xA3B70A2A),
    ((2 ** 64 - 1, 63, 7, 8, 8191, 8190), 0x786EF1A2, 0xB3570E92),
]


@pytest.mark.parametrize("args,key,want", KNOWN)
def test_hash_known_answers(args, key, want):
  seed, b, h, H, i, j = args
  assert O.dropout_seed_key(seed) == key
  assert _scalar_hash(*args) == want
  # the vectorised oracle: the pair sits at [0, h, i, j] of the block that starts at sequence b
  got = O.dropout_hash(seed, 1, H, i + 1, j + 1, b0=b, rows=[0, i], cols=[j])
  assert got.dtype == np.uint32 and got.shape == (1, H, 2, 1) and int(got[0, h, 1, 0]) == want


def test_threshold():
  assert O.dropout_threshold(0.0) == 0 and O.dropout_threshold(-1.0) == 0
  assert O.dropout_threshold(0.5) == 1 << 31
  assert O.dropout_threshold(0.25) == 1 << 30
  assert O.dropout_threshold(0.3) == 1288490240            # float32(0.3) * 2^32, exactly representable
  assert O.dropout_threshold(np.nextafter(np.float32(1), np.float32(0))) == 0xFFFFFF00
  assert O.dropout_keep_mask(7, 0.0, 2, 3, 5, 4).all()


def test_vectorised_hash_matches_scalar_everywhere_on_a_small_grid():
  B, H, L, Lkv, b0, seed = 3, 4, 17, 13, 5, 0xDEADBEEFCAFE
  got = O.dropout_hash(seed, B, H, L, Lkv, b0=b0)
  for b in range(B):
    for h in range(H):
      for i in range(L):
        for j in range(Lkv):
          assert int(got[b, h, i, j]) == _scalar_hash(seed, b0 + b, h, H, i, j)


def test_host_function_matches_oracle():
  lib = _lib.load()
  rng = np.random.default_rng(3)
  for seed, p in ((0, 0.1), (42, 0.3), (2 ** 63 + 12345, 0.5), (2 ** 64 - 1, 0.97)):
    B, H, L, Lkv = 3, 5, 40, 37
    want = O.dropout_keep_mask(seed, p, B, H, L, Lkv)
    for _ in range(400):
      b, h, i, j = (int(rng.integers(n)) for n in (B, H, L, Lkv))
      got = lib.hstu_attn_dropout_keep(C.c_uint64(seed), C.c_float(p), b, h, H, i, j)
      assert got == int(want[b, h, i, j]), (seed, p, b, h, i, j)
  assert lib.hstu_attn_dropout_keep(C.c_uint64(9), C.c_float(0.0), 0, 0, 1, 0, 0) == 1
  # a large position and sequence index: the arithmetic wraps the same way on both sides
  big = O.dropout_keep_mask(11, 0.5, 1, 8, 1, 9000, b0=100000)
  for j in (0, 4095, 8999):
    assert lib.hstu_attn_dropout_keep(C.c_uint64(11), C.c_float(0.5), 100000, 7, 8, 0, j) == int(big[0, 7, 0, j])


@pytest.mark.parametrize("p", [0.05, 0.3, 0.5, 0.9])
def test_keep_share_and_independence(p):
  B, H, L = 2, 4, 256
  keep = O.dropout_keep_mask(1234, p, B, H, L, L)
  n = keep.size
  sd = (p * (1 - p) / n) ** 0.5
  assert abs(keep.mean() - (1 - p)) < 5 * sd
  # per row and per column too (a hash that favoured an axis would show here)
  row_sd = (p * (1 - p) / L) ** 0.5
  assert np.abs(keep.mean(axis=3) - (1 - p)).max() < 5.5 * row_sd
  assert np.abs(keep.mean(axis=2) - (1 - p)).max() < 5.5 * row_sd
  x = keep.astype(np.float64) - keep.mean()
  var = (x * x).mean()
  corr = lambda a, b: float((a * b).mean() / var)
  lim = 5.0 / (n / 2) ** 0.5
  assert abs(corr(x[..., 1:], x[..., :-1])) < lim            # neighbouring keys
  assert abs(corr(x[..., 1:, :], x[..., :-1, :])) < lim      # neighbouring rows
  assert abs(corr(x[..., 1:, 1:], x[..., :-1, :-1])) < lim   # along the diagonal
  assert abs(corr(x[:, 1:], x[:, :-1])) < lim                # neighbouring heads
  assert abs(corr(x[1:], x[:-1])) < 2 * lim                  # neighbouring sequences
  other = O.dropout_keep_mask(1235, p, B, H, L, L).astype(np.float64)
  assert abs(corr(x, other - other.mean())) < lim            # neighbouring seeds
  # the same pair under a smaller rate survives whenever it survives under a larger one (one hash, two thresholds)
  assert (O.dropout_keep_mask(1234, p / 2, B, H, L, L) | ~keep).all()


@pytest.mark.parametrize("p", [0.1, 0.5, 0.9])
def test_keep_pattern_has_no_structure_along_the_index_lattice(p):
  """The pair's part of the hash sees a lattice (a constant step per row and per key): lag correlations along rows,
  keys and both diagonals up to 128 apart, and the variance of the survivors' count in square patches, rows and
  columns, against what independent draws give."""
  L = 512
  keep = O.dropout_keep_mask(77, p, 2, 2, L, L).astype(np.float64)
  x = keep - (1 - p)
  var = p * (1 - p)
  worst = 0.0
  for lag in (1, 2, 3, 4, 7, 8, 16, 31, 32, 33, 64, 127, 128):
    for a, b in ((x[..., lag:], x[..., :-lag]), (x[..., lag:, :], x[..., :-lag, :]),
                 (x[..., lag:, lag:], x[..., :-lag, :-lag]), (x[..., lag:, :-lag], x[..., :-lag, lag:])):
      worst = max(worst, abs(float((a * b).mean()) / var * a.size ** 0.5))
  assert worst < 5.0                                    # 52 z-scores of about a million products each
  for ps in (2, 4, 8, 32):
    counts = keep.reshape(2, 2, L // ps, ps, L // ps, ps).sum(axis=(3, 5))
    assert 0.9 < counts.var() / (ps * ps * var) < 1.1, ps
  assert 0.8 < keep.sum(axis=3).var() / (L * var) < 1.2 and 0.8 < keep.sum(axis=2).var() / (L * var) < 1.2


def _tiny(rng, B=2, L=7, H=2, d=4, dv=3):
  return (rng.standard_normal((B, L, H, d)), rng.standard_normal((B, L, H, d)), rng.standard_normal((B, L, H, dv)))


def test_forward_with_dropout_is_the_masked_weights_times_the_keep_factor():
  """Brute force, pair by pair, over the oracle's own undropped weights: out = sum_j keep ? P / (1 - p) : 0."""
  rng = np.random.default_rng(5)
  q, k, v = _tiny(rng)
  B, L, H, _ = q.shape
  p, seed, lens = 0.4, 99, np.array([7, 5])
  pos = rng.standard_normal((H, 2 * L - 1))
  got = O.hstu_attention_ref(q, k, v, seq_lens=lens, alpha=0.6, n=4.0, pos_tab=pos, dropout_p=p, dropout_seed=seed)
  want = np.zeros_like(got)
  thr = O.dropout_threshold(p)
  scale = float(np.float32(1) / (np.float32(1) - np.float32(p)))
  for b in range(B):
    for h in range(H):
      for i in range(int(lens[b])):
        for j in range(i + 1):
          if _scalar_hash(seed, b, h, H, i, j) < thr:
            continue
          s = 0.6 * float(q[b, i, h] @ k[b, j, h]) + pos[h, (L - 1) + j - i]
          want[b, i, h] += s / (1 + np.exp(-s)) / 4.0 * scale * v[b, j, h]
  np.testing.assert_allclose(got, want, rtol=1e-12, atol=1e-12)
  # p = 0 is the op without dropout, bit for bit
  base = O.hstu_attention_ref(q, k, v, seq_lens=lens, alpha=0.6, n=4.0, pos_tab=pos)
  assert np.array_equal(O.hstu_attention_ref(q, k, v, seq_lens=lens, alpha=0.6, n=4.0, pos_tab=pos, dropout_p=0.0,
                                             dropout_seed=5), base)
  # the layer-side form takes the same pattern
  mask = O.make_causal_mask((np.arange(L)[None] < lens[:, None]).astype(np.float64))
  bias = np.stack([O.rel_pos_bias(pos[0], L)[0]])
  a = O.pointwise_attention_dense(q, k, v, mask, bias, dropout_p=p, dropout_seed=seed)
  bb = O.hstu_attention_ref(q, k, v, seq_lens=lens, pos_tab=pos[0], dropout_p=p, dropout_seed=seed)
  np.testing.assert_allclose(a, bb, rtol=1e-12, atol=1e-12)


def test_forward_with_dropout_is_unbiased():
  """Inverted dropout: the mean over seeds is the undropped output (hstu.py:386-387 with keras' scaling)."""
  rng = np.random.default_rng(6)
  q, k, v = _tiny(rng, B=1, L=6, H=2)
  base = O.hstu_attention_ref(q, k, v, n=3.0)
  p, n_seeds = 0.3, 4000
  acc = np.zeros_like(base)
  sq = np.zeros_like(base)
  for seed in range(n_seeds):
    o = O.hstu_attention_ref(q, k, v, n=3.0, dropout_p=p, dropout_seed=seed)
    acc += o
    sq += o * o
  mean = acc / n_seeds
  sem = np.sqrt(np.maximum(sq / n_seeds - mean ** 2, 0) / n_seeds)
  assert (np.abs(mean - base) <= 5 * sem + 1e-12).all()
  assert sem.max() > 0


def test_jagged_reference_uses_the_sequence_index():
  rng = np.random.default_rng(7)
  lens = np.array([5, 0, 7])
  L, H = 7, 2
  q, k, v = _tiny(rng, B=3, L=L, H=H)
  qj, off = O.padded_to_jagged(q, lens)
  kj, _ = O.padded_to_jagged(k, lens)
  vj, _ = O.padded_to_jagged(v, lens)
  pad = O.hstu_attention_ref(q, k, v, seq_lens=lens, dropout_p=0.5, dropout_seed=8)
  jag = O.hstu_attention_jagged_ref(qj, kj, vj, off, L, dropout_p=0.5, dropout_seed=8)
  np.testing.assert_allclose(O.jagged_to_padded(jag, off, L), pad, rtol=1e-12, atol=1e-12)


def _fd_grad(f, x, eps=1e-6):
  g = np.zeros_like(x, dtype=np.float64)
  it = np.nditer(x, flags=["multi_index"])
  for _ in it:
    idx = it.multi_index
    old = x[idx]
    x[idx] = old + eps
    fp = f()
    x[idx] = old - eps
    fm = f()
    x[idx] = old
    g[idx] = (fp - fm) / (2 * eps)
  return g


def test_backward_with_dropout_against_finite_differences():
  """With the seed fixed the forward is a smooth function of its inputs: its central differences pin the
  backward reference (the factor must sit on P for dV and on dS for dQ, dK and the tables)."""
  rng = np.random.default_rng(8)
  q, k, v = _tiny(rng, B=2, L=6)
  B, L, H, _ = q.shape
  dout = rng.standard_normal(v.shape)
  pos = rng.standard_normal((H, 2 * L - 1))
  tst = rng.standard_normal((1, 130))
  ts = 1000 + np.cumsum(rng.integers(1, 5000, (B, L)), axis=1)
  kw = dict(alpha=0.7, n=5.0, seq_lens=np.array([6, 4]), pos_tab=pos, timestamps=ts, ts_tab=tst, dropout_p=0.35,
            dropout_seed=2024)
  loss = lambda: float((O.hstu_attention_ref(q, k, v, **kw) * dout).sum())
  dq, dk, dv, dpos, dts = O.hstu_attention_bwd_ref(q, k, v, dout, **kw)
  for name, x, g in (("q", q, dq), ("k", k, dk), ("v", v, dv), ("pos", pos, dpos), ("ts", tst, dts)):
    fd = _fd_grad(loss, x)
    assert np.abs(fd - g).max() <= 1e-7 * max(1.0, np.abs(fd).max()), name
    assert np.abs(g).max() > 0
  # and it differs from the gradient without dropout
  dq0 = O.hstu_attention_bwd_ref(q, k, v, dout, **{**kw, "dropout_p": 0.0})[0]
  assert np.abs(dq0 - dq).max() > 1e-3
