"""Pins the CPU oracle: reference-held literals, closed forms, brute force.

Every check here is chosen so that a plausible mistake in oracle/hstu_oracle.py
(a dropped term, a transposed operand, an off-by-one in the bias index, the
wrong timestamp for the query row) fails at least one of them.
"""

import math

import numpy as np
import pytest

from oracle import hstu_oracle as O


# ---- masks: the reference's own literals (recml/layers/keras/utils_test.py:38-76)

PADDING = np.array([[1, 1, 1], [1, 0, 0], [1, 1, 0]], dtype=np.float32)
ATTN_EXPECTED = np.array(
    [
        [[1, 1, 1], [1, 1, 1], [1, 1, 1]],
        [[1, 0, 0], [0, 0, 0], [0, 0, 0]],
        [[1, 1, 0], [1, 1, 0], [0, 0, 0]],
    ],
    dtype=np.float32,
)
CAUSAL_EXPECTED = np.array(
    [
        [[1, 0, 0], [1, 1, 0], [1, 1, 1]],
        [[1, 0, 0], [0, 0, 0], [0, 0, 0]],
        [[1, 0, 0], [1, 1, 0], [0, 0, 0]],
    ],
    dtype=np.float32,
)


def test_make_attention_mask_reference_literals():
  np.testing.assert_array_equal(O.make_attention_mask(PADDING), ATTN_EXPECTED)


def test_make_causal_mask_reference_literals():
  np.testing.assert_array_equal(O.make_causal_mask(PADDING), CAUSAL_EXPECTED)


def test_length_mask_equals_causal_mask_of_end_padded_batch():
  # seq_lens form of the op == dense form with make_causal_mask(padding)
  rng = np.random.default_rng(0)
  B, L, H, d = 3, 7, 2, 4
  q, k, v = (rng.standard_normal((B, L, H, d)) for _ in range(3))
  lens = np.array([7, 1, 4])
  pad = (np.arange(L)[None] < lens[:, None]).astype(np.float32)
  a = O.pointwise_attention_dense(q, k, v, O.make_causal_mask(pad))
  b = O.hstu_attention_ref(q, k, v, seq_lens=lens)
  np.testing.assert_allclose(a, b, rtol=0, atol=1e-15)


# ---- relative position bias


@pytest.mark.parametrize("n", range(2, 10))
def test_rel_pos_closed_form_matches_recipe(n):
  w = np.arange(1, 2 * n + 3, dtype=np.float64)  # longer than needed, like max_len
  rec = O.rel_pos_bias_recipe(w, n)
  assert rec.shape == (1, n, n)
  np.testing.assert_array_equal(rec, O.rel_pos_bias(w, n))
  # corners and Toeplitz structure
  assert rec[0, 0, n - 1] == w[2 * n - 2]
  assert rec[0, n - 1, 0] == w[0]
  assert rec[0, 0, 0] == w[n - 1]
  assert (np.diff(np.diagonal(rec[0])) == 0).all()


# ---- timestamp buckets


def test_bucketization_hand_cases():
  delta = np.array([0, 1, 2, 3, 10, 3600, 86400, 10**9, 3 * 10**9, -5, -3600])
  #                ln/0.301: 0  0  2.30 3.65 7.65 27.2  37.8   68.8   clip    5.35  27.2
  want = np.array([0, 0, 2, 3, 7, 27, 37, 68, 68, 5, 27])
  np.testing.assert_array_equal(O.default_bucketization(delta), want)
  np.testing.assert_array_equal(O.bucketize_law(delta), want)


def test_bucket_thresholds_are_the_law():
  th = O.bucket_thresholds()
  assert len(th) == 69 and th[0] == 1 and th[-1] <= 10**9
  # the textbook values ceil(e^(0.301 k)) where nothing is close: e^0.301 = 1.351, 1.826, 2.467, 3.333, 4.504,
  # 6.086, 8.224, 11.11, 15.01, 20.29, 27.41, 37.04
  assert list(th[:13]) == [1, 2, 2, 3, 4, 5, 7, 9, 12, 16, 21, 28, 38]
  # by construction: T_k is where the law first reaches k
  for kk, t in enumerate(th):
    assert O.bucketize_law(np.array([t]))[0] >= kk
    if t > 1:
      assert O.bucketize_law(np.array([t - 1]))[0] < kk
  # an independent evaluation of the same expression (python floats instead of numpy arrays)
  size = float(np.float32(0.301))
  for t in th[1:]:
    for x in (int(t) - 1, int(t), int(t) + 1):
      assert O.bucketize_law(np.array([x]))[0] == math.floor(math.log(float(np.float32(x))) / size)
  # number of thresholds at or below x == the bucket of x
  rng = np.random.default_rng(1)
  x = np.concatenate([np.arange(1, 5000), rng.integers(1, 10**9, 200000)])
  np.testing.assert_array_equal(np.searchsorted(th, x, side="right") - 1, O.bucketize_law(x))
  # the literal float32 recipe agrees with the law away from the enumerated boundary set
  far = ~O.near_bucket_boundary(x)
  np.testing.assert_array_equal(O.default_bucketization(x)[far], O.bucketize_law(x)[far])
  assert far.mean() > 0.999


def test_bucket_law_other_sizes_and_clip():
  for size in (0.25, 0.301, 0.5, 1.0):
    th = O.bucket_thresholds(size)
    x = np.concatenate([th, th - 1, th + 1])
    x = x[x >= 1]
    np.testing.assert_array_equal(np.searchsorted(th, x, side="right") - 1, O.bucketize_law(x, size))
  # beyond 1e9 the clip holds the bucket; the sign does not matter
  assert O.bucketize_law(np.array([10**9, 10**9 + 5, 2 * 10**9, 5 * 10**12, -5 * 10**12])).tolist() == [68] * 5


def test_time_delta_worked_example():
  # row i uses ts[i+1]; the last row reuses its own timestamp, so the last
  # two rows coincide and the causal diagonal is ts[i+1]-ts[i], not 0
  ts = np.array([[100, 160, 400, 4000]])
  want = np.array([[[60, 0, -240, -3840],
                    [300, 240, 0, -3600],
                    [3900, 3840, 3600, 0],
                    [3900, 3840, 3600, 0]]])
  np.testing.assert_array_equal(O.time_delta(ts), want)
  w = np.arange(129, dtype=np.float64) * 10
  tb = O.time_bias(ts, w)
  assert tb.shape == (1, 4, 4)
  assert tb[0, 0, 0] == w[int(math.log(60) / 0.301)]
  assert tb[0, 1, 3] == w[int(math.log(3600) / 0.301)]
  assert tb[0, 0, 1] == w[0]
  # clip to the table: tiny table
  tb2 = O.time_bias(ts, np.arange(5.0), num_buckets=4)
  assert tb2.max() == 4.0


# ---- attention


def test_silu_special_values():
  assert O.silu(0.0) == 0.0
  assert abs(O.silu(40.0) - 40.0) < 1e-12
  assert abs(O.silu(-40.0)) < 1e-12 and O.silu(-40.0) <= 0
  x = np.linspace(-6, 6, 101)
  np.testing.assert_allclose(O.silu(x) - O.silu(-x), x, atol=1e-14)
  xm = -1.2784645427610738
  assert abs(O.silu(xm) - (-0.27846454276107)) < 1e-12
  assert O.silu(xm - 1e-3) > O.silu(xm) < O.silu(xm + 1e-3)


def _tiny(seed=0, B=2, L=6, H=2, d=3, dv=3):
  rng = np.random.default_rng(seed)
  q = rng.standard_normal((B, L, H, d))
  k = rng.standard_normal((B, L, H, d))
  v = rng.standard_normal((B, L, H, dv))
  return q, k, v


def test_dense_matches_bruteforce_plain():
  q, k, v = _tiny()
  a = O.hstu_attention_ref(q, k, v)
  b = O.hstu_attention_bruteforce(q, k, v)
  np.testing.assert_allclose(a, b, rtol=1e-12, atol=1e-14)


def test_dense_matches_bruteforce_all_options():
  q, k, v = _tiny(1, B=3, L=7, H=2, d=4, dv=5)
  rng = np.random.default_rng(2)
  lens = np.array([7, 3, 1])
  pos = rng.standard_normal((2, 13))
  tst = rng.standard_normal((2, 129))
  ts = np.cumsum(rng.integers(1, 100000, (3, 7)), axis=1) + 1_600_000_000
  a = O.hstu_attention_ref(q, k, v, seq_lens=lens, n=11, alpha=0.5, pos_tab=pos,
                           timestamps=ts, ts_tab=tst, sliding_window_size=3)
  b = O.hstu_attention_bruteforce(q, k, v, seq_lens=lens, n=11, alpha=0.5, pos_tab=pos,
                                  timestamps=ts, ts_tab=tst, sliding_window_size=3)
  np.testing.assert_allclose(a, b, rtol=1e-12, atol=1e-14)
  assert (a[1, 3:] == 0).all() and (a[2, 1:] == 0).all()
  # shared (one-head) tables
  a1 = O.hstu_attention_ref(q, k, v, pos_tab=pos[0], timestamps=ts, ts_tab=tst[1])
  b1 = O.hstu_attention_bruteforce(q, k, v, pos_tab=pos[0], timestamps=ts, ts_tab=tst[1])
  np.testing.assert_allclose(a1, b1, rtol=1e-12, atol=1e-14)


def test_full_mask_and_segments_match_bruteforce():
  q, k, v = _tiny(3)
  seg = np.array([[1, 1, 1, 1, 0, 0], [1, 1, 2, 2, 2, 0]])
  a = O.hstu_attention_ref(q, k, v, causal=False, q_segment_ids=seg, kv_segment_ids=seg)
  b = O.hstu_attention_bruteforce(q, k, v, causal=False, q_segment_ids=seg, kv_segment_ids=seg)
  np.testing.assert_allclose(a, b, rtol=1e-12, atol=1e-14)


def test_pw_attn_ref_is_scaled_segment_form():
  # hstu_ops_test.py:44-58 == canonical op with alpha=1/sqrt(d), n=L, segment mask
  q, k, v = _tiny(4, B=2, L=6, H=2, d=4, dv=4)
  seg = np.array([[1, 1, 1, 1, 0, 0], [1, 1, 1, 1, 1, 1]])
  a = O.pw_attn_ref(q, k, v, seg)
  b = O.hstu_attention_bruteforce(q, k, v, alpha=1 / math.sqrt(4), causal=True,
                                  q_segment_ids=seg, kv_segment_ids=seg)
  np.testing.assert_allclose(a, b, rtol=1e-12, atol=1e-14)
  # padded rows attend to earlier padded keys: not zero, unlike the length form
  assert np.abs(a[0, 5]).max() > 0
  c = O.hstu_attention_ref(q, k, v, alpha=0.5, seq_lens=np.array([4, 6]))
  np.testing.assert_allclose(a[0, :4], c[0, :4], rtol=1e-12, atol=1e-14)
  assert (c[0, 4:] == 0).all()


def test_layer_dense_form_scaled_and_unscaled():
  # hstu.py:365-378: scaled divides q by sqrt(d) and skips 1/L
  q, k, v = _tiny(5)
  mask = O.make_causal_mask(np.ones((2, 6)))
  bias = np.random.default_rng(6).standard_normal((2, 6, 6))
  a = O.pointwise_attention_dense(q, k, v, mask, bias)
  b = O.hstu_attention_ref(q, k, v, bias=bias)
  np.testing.assert_allclose(a, b, rtol=1e-13, atol=1e-15)
  a2 = O.pointwise_attention_dense(q, k, v, mask, bias, scaled=True)
  b2 = O.hstu_attention_ref(q, k, v, bias=bias, alpha=1 / math.sqrt(3), n=1)
  np.testing.assert_allclose(a2, b2, rtol=1e-13, atol=1e-15)


def test_single_key_closed_form():
  rng = np.random.default_rng(7)
  q, k, v = (rng.standard_normal((1, 1, 1, 5)) for _ in range(3))
  w = np.array([0.3])
  out = O.hstu_attention_ref(q, k, v, alpha=0.7, n=4, pos_tab=w)
  s = 0.7 * float(q.ravel() @ k.ravel()) + 0.3
  want = s / (1 + math.exp(-s)) / 4 * v.ravel()
  np.testing.assert_allclose(out.ravel(), want, rtol=1e-13)


def test_zero_q_gives_toeplitz_of_table():
  # S = bias only  =>  out = tril(Toeplitz(silu(w))) @ v / n : pins where the bias is added
  L, d = 5, 3
  rng = np.random.default_rng(8)
  k = rng.standard_normal((1, L, 1, d))
  v = rng.standard_normal((1, L, 1, d))
  w = rng.standard_normal(2 * L - 1)
  out = O.hstu_attention_ref(np.zeros((1, L, 1, d)), k, v, pos_tab=w)
  T = np.zeros((L, L))
  for i in range(L):
    for j in range(i + 1):
      T[i, j] = O.silu(w[(L - 1) + j - i])
  want = (T @ v[0, :, 0]) / L
  np.testing.assert_allclose(out[0, :, 0], want, rtol=1e-13)


def test_causality_padding_and_linearity_invariants():
  q, k, v = _tiny(9, B=2, L=8, H=2, d=4, dv=4)
  lens = np.array([5, 8])
  base = O.hstu_attention_ref(q, k, v, seq_lens=lens)
  # future keys/values do not matter
  k2, v2 = k.copy(), v.copy()
  k2[:, 6:] += 100.0
  v2[:, 6:] -= 50.0
  pert = O.hstu_attention_ref(q, k2, v2, seq_lens=lens)
  np.testing.assert_array_equal(base[:, :6], pert[:, :6])
  # content of padded positions does not matter, padded rows are exactly 0
  q3, k3, v3 = q.copy(), k.copy(), v.copy()
  q3[0, 5:], k3[0, 5:], v3[0, 5:] = 7.0, -3.0, 1e6
  np.testing.assert_array_equal(base[0], O.hstu_attention_ref(q3, k3, v3, seq_lens=lens)[0])
  assert (base[0, 5:] == 0).all()
  # linear in 1/n, alpha equivalent to scaling q
  np.testing.assert_allclose(O.hstu_attention_ref(q, k, v, n=4) * 0.5,
                             O.hstu_attention_ref(q, k, v, n=8), rtol=1e-14)
  np.testing.assert_allclose(O.hstu_attention_ref(q, k, v, alpha=0.25),
                             O.hstu_attention_ref(q * 0.25, k, v), rtol=1e-13)
  # full mask, all valid = plain silu(QK^T)V/N
  s = np.einsum("bthd,bshd->bhts", q, k)
  want = np.einsum("bhts,bshd->bthd", O.silu(s) / 8, v)
  np.testing.assert_allclose(O.hstu_attention_ref(q, k, v, causal=False), want, rtol=1e-13)


def test_explicit_mask_and_window():
  q, k, v = _tiny(10, B=1, L=6, H=1, d=3, dv=3)
  m = np.tril(np.ones((6, 6), dtype=bool))
  np.testing.assert_array_equal(O.hstu_attention_ref(q, k, v, causal=False, mask=m),
                                O.hstu_attention_ref(q, k, v, causal=True))
  # an explicit mask is one more factor of M, whatever its rank: with the causal flag on top, a mask that keeps
  # exactly the pairs above the diagonal leaves nothing, one that keeps everything leaves the causal result
  upper = np.triu(np.ones((6, 6), dtype=bool), 1)
  assert not O.hstu_attention_ref(q, k, v, causal=True, mask=upper).any()
  assert not O.hstu_attention_ref(q, k, v, causal=True, mask=upper[None]).any()
  np.testing.assert_array_equal(O.hstu_attention_ref(q, k, v, causal=True, mask=np.ones((6, 6), dtype=bool)),
                                O.hstu_attention_ref(q, k, v, causal=True))
  dq, dk, dv, _, _ = O.hstu_attention_bwd_ref(q, k, v, np.ones_like(v), causal=True, mask=upper)
  assert not dq.any() and not dk.any() and not dv.any()
  w = O.hstu_attention_ref(q, k, v, sliding_window_size=0)
  s = np.einsum("bthd,bthd->bth", q, k)
  np.testing.assert_allclose(w, (O.silu(s) / 6)[..., None] * v, rtol=1e-13)
  with pytest.raises(ValueError):
    O.splash_mask(6, 6, explicit=np.ones((5, 6), dtype=bool))
  with pytest.raises(ValueError):
    O.splash_mask(6, 6, q_segment_ids=np.ones((1, 6)))


def test_jagged_equals_padded():
  rng = np.random.default_rng(11)
  B, L, H, d = 3, 9, 2, 4
  lens = np.array([9, 1, 4])
  q, k, v = (rng.standard_normal((B, L, H, d)) for _ in range(3))
  pos = rng.standard_normal((H, 2 * L - 1))
  tst = rng.standard_normal((H, 129))
  ts = np.cumsum(rng.integers(1, 10**6, (B, L)), axis=1)
  for b in range(B):  # padding repeats the last valid timestamp
    ts[b, lens[b]:] = ts[b, lens[b] - 1]
  padded = O.hstu_attention_ref(q, k, v, seq_lens=lens, pos_tab=pos, timestamps=ts, ts_tab=tst)
  qj, off = O.padded_to_jagged(q, lens)
  kj, _ = O.padded_to_jagged(k, lens)
  vj, _ = O.padded_to_jagged(v, lens)
  tj, _ = O.padded_to_jagged(ts, lens)
  jag = O.hstu_attention_jagged_ref(qj, kj, vj, off, L, pos_tab=pos, timestamps=tj, ts_tab=tst)
  np.testing.assert_allclose(O.jagged_to_padded(jag, off, L), padded, rtol=1e-13, atol=1e-15)


def test_round_bf16():
  x = np.array([1.0, 1.00390625, 1.005859375, -2.5, 0.0, 3.1415926], dtype=np.float32)
  r = O.round_bf16(x)
  assert r[0] == 1.0 and r[3] == -2.5 and r[4] == 0.0
  assert r[1] == 1.0            # tie to even (1 + 2^-8 -> 1)
  assert r[2] == 1.0078125      # above the tie rounds up
  assert abs(r[5] - 3.140625) < 1e-6
  import torch
  t = torch.from_numpy(np.random.default_rng(0).standard_normal(1000).astype(np.float32))
  np.testing.assert_array_equal(O.round_bf16(t.numpy()), t.bfloat16().float().numpy())


def test_e4m3fn_rounding_against_torch_cast():
  import torch
  codes = np.arange(256, dtype=np.uint8)
  vals = torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy()
  finite = np.isfinite(vals)
  assert finite.sum() == 254 and np.abs(vals[finite]).max() == 448.0
  v = vals[finite]
  # every representable value is a fixed point and encodes to its own bit pattern
  assert (O.round_e4m3fn(v) == v).all()
  assert (O.encode_e4m3fn(v) == codes[finite]).all()
  # midpoints between neighbours (ties to even) and points either side of them
  pos = np.sort(np.unique(v[v >= 0]))
  mids = (pos[:-1] + pos[1:]) / 2
  probe = np.concatenate([mids, mids * (1 + 1e-6), mids * (1 - 1e-6)]).astype(np.float32)
  probe = np.concatenate([probe, -probe])
  rng = np.random.default_rng(0)
  probe = np.concatenate([probe, rng.uniform(-448, 448, 20000).astype(np.float32),
                          (rng.standard_normal(20000) * 0.05).astype(np.float32)])
  want = torch.from_numpy(probe).to(torch.float8_e4m3fn).float().numpy()
  got = O.round_e4m3fn(probe)
  assert (got == want).all()
  q, scale = O.quantize_e4m3fn_per_head(rng.standard_normal((5, 7, 3, 16)).astype(np.float32))
  assert scale.shape == (3,) and np.abs(q).max() == 448.0 and (O.round_e4m3fn(q) == q).all()


def test_rows_near_bucket_boundary():
  # ln(15245) / 0.301 = 32.0000004: a boundary case of the law in fp32; 15000 is not
  assert O.near_bucket_boundary(np.array([15245]))[0] and not O.near_bucket_boundary(np.array([15000]))[0]
  # sequence 0: row 0's next timestamp is 15245 after key 0; sequence 1: nowhere near a boundary
  ts = np.array([1000, 1000 + 15245, 1000 + 15245 + 7, 5000, 5003, 5010], dtype=np.int64)
  off = np.array([0, 3, 6])
  flag = O.rows_near_bucket_boundary(ts, off)
  assert flag.tolist()[0] is True and not flag[3:].any()


def _fd_grad(f, x, eps=1e-6):
  """Central finite differences of the scalar f with respect to every entry of x (fp64)."""
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


@pytest.mark.parametrize("case", ["lengths_bias", "segments_window", "full_mask_dense_bias", "shared_dense_bias"])
def test_backward_oracle_against_finite_differences(case):
  rng = np.random.default_rng(11)
  B, L, H, d, dv = 2, 6, 2, 4, 3
  q, k = rng.standard_normal((B, L, H, d)), rng.standard_normal((B, L, H, d))
  v, dout = rng.standard_normal((B, L, H, dv)), rng.standard_normal((B, L, H, dv))
  kw = dict(alpha=0.7, n=5.0)
  pos = ts_tab = None
  if case == "lengths_bias":
    pos = rng.standard_normal((H, 2 * L - 1))
    ts_tab = rng.standard_normal((1, 130))             # one row shared by the heads
    ts = 1000 + np.cumsum(rng.integers(1, 5000, (B, L)), axis=1)
    kw.update(seq_lens=np.array([6, 4]), pos_tab=pos, timestamps=ts, ts_tab=ts_tab)
  elif case == "segments_window":
    seg = np.array([[1, 1, 1, 2, 2, 0], [1, 1, 1, 1, 1, 1]])
    pos = rng.standard_normal((2 * L - 1,))            # one row shared by the heads
    kw.update(q_segment_ids=seg, kv_segment_ids=seg, sliding_window_size=2, pos_tab=pos)
  else:
    m = rng.random((B, L, L)) > 0.3
    kw.update(causal=case == "shared_dense_bias", mask=m,
              bias=rng.standard_normal((B, L, L) if case == "full_mask_dense_bias" else (1, L, L)))
  loss = lambda: float((O.hstu_attention_ref(q, k, v, **kw) * dout).sum())
  if "bias" in kw:
    dq, dk, dvv, dpos, dts, dbias = O.hstu_attention_bwd_ref(q, k, v, dout, bias_grad=True, **kw)
    fd = _fd_grad(loss, kw["bias"])
    assert dbias.shape == kw["bias"].shape and np.abs(fd - dbias).max() <= 1e-7 * max(1.0, np.abs(fd).max())
    assert np.abs(dbias).max() > 0
  else:
    dq, dk, dvv, dpos, dts = O.hstu_attention_bwd_ref(q, k, v, dout, **kw)
  for name, x, g in (("q", q, dq), ("k", k, dk), ("v", v, dvv)):
    fd = _fd_grad(loss, x)
    assert np.abs(fd - g).max() <= 1e-7 * max(1.0, np.abs(fd).max()), name
  if pos is not None:
    fd = _fd_grad(loss, pos)
    assert dpos.shape == pos.shape and np.abs(fd - dpos).max() <= 1e-7 * max(1.0, np.abs(fd).max())
  else:
    assert dpos is None
  if ts_tab is not None:
    fd = _fd_grad(loss, ts_tab)
    assert dts.shape == ts_tab.shape and np.abs(fd - dts).max() <= 1e-7 * max(1.0, np.abs(fd).max())
    assert np.abs(dts).max() > 0
