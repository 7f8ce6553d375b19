"""CPU oracle for the HSTU pointwise-SiLU attention forward.

TEST INFRASTRUCTURE ONLY.  This module restates, in numpy, the dense
formulation that RecML runs for HSTU attention and the helpers that feed it.
Nothing in the shipped package imports it; only tests, the smoke check and the
benchmark's CPU-baseline leg do, and only as the checker.

Each function cites the reference lines it follows (paths relative to the
reference checkout):

  default_bucketization         recml/layers/keras/hstu.py:33-55
  rel_pos_bias_recipe           recml/layers/keras/hstu.py:91-113
  rel_pos_bias                  closed form of the above, w[(n-1)+j-i]
  time_bias                     recml/layers/keras/hstu.py:190-221
  make_attention_mask           recml/layers/keras/utils.py:29-36
  make_causal_mask              recml/layers/keras/utils.py:39-41
  pointwise_attention_dense     recml/layers/keras/hstu.py:356-390
  pw_attn_ref                   recml/core/ops/hstu_ops_test.py:44-58
  splash_mask                   recml/core/ops/hstu_ops.py:926-945, 107-194
  hstu_attention_ref            the union of the above behind one signature
  hstu_attention_bwd_ref        its gradients; math of recml/core/ops/hstu_ops.py:461-517
  dropout_keep_mask             which weights survive attention dropout
                                (recml/layers/keras/hstu.py:386-387 applies keras'
                                Dropout to the masked weights: survivors are
                                scaled by 1/(1-rate)); the draw itself is this
                                library's counter-based hash, not keras' generator

How each function is pinned (tests/test_oracle.py):

  make_attention_mask / make_causal_mask  the reference's own 3x3 literals
                                (recml/layers/keras/utils_test.py:38-76).
  rel_pos_bias                  the pad/tile/reshape/slice recipe re-run at
                                n = 2..9 plus both corner values.
  default_bucketization / time_bias  hand-worked integer cases and the
                                worked example ts=[100,160,400,4000].
  pointwise_attention_dense / pw_attn_ref / hstu_attention_ref
                                fp64 brute-force loops on tiny inputs, the
                                single-key closed form, the zero-Q Toeplitz
                                case, SiLU special values, causality and
                                padding invariants, linearity in 1/N.
  hstu_attention_bwd_ref        central finite differences of the pinned forward
                                in fp64 (every input and both tables), on tiny
                                inputs with every option.
  round_e4m3fn / encode_e4m3fn  torch's CPU float8_e4m3fn cast on every code
                                point, every midpoint and random values (fp8
                                is not in the reference at all).
  dropout_keep_mask             the integer hash against known answers worked
                                with Python's unbounded integers, rate 0 and the
                                survivors' share; hstu_attention_ref with dropout
                                by its mean over many seeds (the undropped
                                output) and by brute force over the keep mask.
                                The random stream itself is parity unpinned by
                                nature: the reference draws from keras' seed
                                generator and holds no dropout outputs.
  splash_mask with sliding_window_size  parity unpinned: the window rule
                                (|i-j| <= w) comes from jax's splash-attention
                                LocalMask, which is not vendored in the
                                reference and cannot be run here.
  default_bucketization at bucket boundaries  parity unpinned against the
                                reference: it computes log and the divide in
                                fp32 inside XLA, and integers next to
                                e^(0.301 k) can land on either side there.
                                `bucketize_law` (the same expression with log
                                and divide in fp64) is the definition every
                                kernel and every reference output here follows
                                exactly; `bucket_thresholds` are its integer
                                thresholds, `bucket_boundary_set` lists where
                                the literal fp32 recipe may differ from it.
"""

from __future__ import annotations

import math

import numpy as np

# ---------------------------------------------------------------------------
# Bias producers
# ---------------------------------------------------------------------------


def default_bucketization(delta, bucket_size: float = 0.301):
  """fp32 restatement of recml/layers/keras/hstu.py:33-55.

  clip(|x|, 1, 1e9) -> log (fp32) -> / bucket_size (fp32) -> trunc to int.
  """
  x = np.abs(np.asarray(delta).astype(np.int64))
  x = np.clip(x, 1, int(1e9))
  logv = np.log(x.astype(np.float32))
  b = (logv / np.float32(bucket_size)).astype(np.float32)
  return b.astype(np.int64)  # C-style truncation; values are >= 0


def _law_size(bucket_size) -> float:
  """The bucket size as the float32 the reference's fp32 divide sees, widened to double."""
  return float(np.float32(bucket_size))


def bucketize_law(delta, bucket_size: float = 0.301):
  """THE bucket law: recml/layers/keras/hstu.py:48-55 with log and divide taken in fp64.

    floor(ln(fl32(clip(|x|, 1, 1e9))) / fl32(bucket_size))

  The reference casts the clipped integer to float32, takes a float32 log and
  divides by the float32 bucket size; only the last two roundings are replaced
  by fp64 here, which turns the law into a set of integer thresholds
  (`bucket_thresholds`).  Every kernel and every reference output in this
  repository follows it exactly, bucket boundaries included.
  """
  x = np.abs(np.asarray(delta).astype(np.int64))
  x = np.clip(x, 1, int(1e9)).astype(np.float32).astype(np.float64)
  return np.floor(np.log(x) / _law_size(bucket_size)).astype(np.int64)


def bucket_thresholds(bucket_size: float = 0.301, x_max: int = 10 ** 9):
  """T_k = smallest integer x in [1, x_max] with bucketize_law(x) >= k, k = 0..bucketize_law(x_max).

  Found by bisection on the law itself (it is monotone in x), so that
  bucketize_law(x) == number of k >= 1 with T_k <= x by construction.
  """
  law = lambda x: int(bucketize_law(np.asarray([x]), bucket_size)[0])
  kmax = law(x_max)
  out = []
  for k in range(kmax + 1):
    lo, hi = 1, int(x_max)
    while lo < hi:
      mid = (lo + hi) // 2
      if law(mid) >= k:
        hi = mid
      else:
        lo = mid + 1
    out.append(lo)
  return np.asarray(out, dtype=np.int64)


def bucket_boundary_set(bucket_size: float = 0.301, ulps: float = 8.0):
  """|delta| values where an fp32 evaluation may legitimately differ by one.

  A value x is in the set when ln(x)/bucket_size lies within `ulps` fp32 ulps
  of an integer; there the fp32 log/divide of any given library can round to
  either side.  Returned as a sorted int64 array of integers in [1, 1e9]
  (one representative per fp32-rounding class is enough for the tests, the
  membership test `near_bucket_boundary` is what the parity tests use).
  """
  th = bucket_thresholds(bucket_size)
  cand = []
  for t in th[1:]:
    for d in range(-2, 3):
      x = int(t) + d
      if x >= 1 and near_bucket_boundary(np.asarray([x]), bucket_size, ulps)[0]:
        cand.append(x)
  return np.asarray(sorted(set(cand)), dtype=np.int64)


def near_bucket_boundary(delta, bucket_size: float = 0.301, ulps: float = 8.0):
  """True where ln(fl32(clip|delta|))/bucket_size is within `ulps` fp32 ulps of an integer."""
  x = np.abs(np.asarray(delta).astype(np.int64))
  x = np.clip(x, 1, int(1e9)).astype(np.float32).astype(np.float64)
  y = np.log(x) / _law_size(bucket_size)
  dist = np.abs(y - np.rint(y))
  tol = ulps * np.spacing(np.maximum(y, 1.0).astype(np.float32)).astype(np.float64)
  return (dist <= tol) & (np.rint(y) >= 1)


def rows_near_bucket_boundary(timestamps, seq_offsets, causal: bool = True, bucket_size: float = 0.301):
  """Jagged timestamps [T] -> bool [T]: rows whose time delta to one of their (causal) keys is
  a boundary case of the bucket law (near_bucket_boundary).  On such a row an fp32 evaluation
  of the law may land in the neighbouring bucket (parity unpinned there), so checkers compare
  those rows with a looser bound."""
  ts = np.asarray(timestamps).astype(np.int64)
  off = np.asarray(seq_offsets).astype(np.int64)
  flag = np.zeros(ts.shape[0], dtype=bool)
  for b in range(len(off) - 1):
    t = ts[off[b]:off[b + 1]]
    if t.size == 0:
      continue
    d = time_delta(t[None])[0]
    near = near_bucket_boundary(d, bucket_size)
    if causal:
      near &= np.tril(np.ones_like(near, dtype=bool))
    flag[off[b]:off[b + 1]] = near.any(axis=1)
  return flag


def rel_pos_bias_recipe(w, n: int):
  """The pad/tile/reshape/slice recipe of recml/layers/keras/hstu.py:105-113.

  w has at least 2n-1 entries.  Returns [1, n, n].  Degenerate for n == 1 in
  the reference (empty slice); callers use n >= 2.
  """
  w = np.asarray(w)
  padded = np.pad(w[: 2 * n - 1], (0, n))          # length 3n-1
  tiled = np.tile(padded, n)                       # length n(3n-1)
  full = tiled[:-n].reshape(1, n, 3 * n - 2)
  excess = (2 * n - 1) // 2
  return full[:, :, excess:-excess]


def rel_pos_bias(w, n: int):
  """Closed form of the recipe: bias[i, j] = w[(n-1) + j - i]."""
  w = np.asarray(w)
  i = np.arange(n)[:, None]
  j = np.arange(n)[None, :]
  return w[(n - 1) + j - i][None]


def time_delta(ts):
  """delta[b,i,j] = ext[b,i+1] - ext[b,j], ext = concat(ts, ts[:, -1:]).

  recml/layers/keras/hstu.py:194-202: the query row uses the NEXT item's
  timestamp; the last row reuses its own.
  """
  ts = np.asarray(ts).astype(np.int64)
  ext = np.concatenate([ts, ts[:, -1:]], axis=1)
  return ext[:, 1:, None] - ext[:, None, :-1]


def time_bias(ts, ts_w, num_buckets: int = 128, bucket_size: float = 0.301,
              law: bool = True):
  """recml/layers/keras/hstu.py:190-221.  ts [B,n] ints, ts_w [num_buckets+1].

  The reference's one-hot matmul with ts_w is a gather ts_w[bucket].
  law=True (the default) buckets by `bucketize_law`, law=False by the literal
  float32 recipe `default_bucketization`; the two differ only on the
  enumerated boundary set.
  """
  d = time_delta(ts)
  fn = bucketize_law if law else default_bucketization
  bucket = np.clip(fn(d, bucket_size), 0, num_buckets)
  return np.asarray(ts_w)[bucket]


# ---------------------------------------------------------------------------
# Masks
# ---------------------------------------------------------------------------


def make_attention_mask(mask, dtype=np.float32):
  """recml/layers/keras/utils.py:29-36: outer product of the padding mask."""
  m = np.asarray(mask)
  return (m[..., :, None] * m[..., None, :]).astype(dtype)


def make_causal_mask(mask, dtype=np.float32):
  """recml/layers/keras/utils.py:39-41: tril of the above."""
  return np.tril(make_attention_mask(mask, dtype=dtype))


def splash_mask(q_len, kv_len, *, causal=True, explicit=None,
                sliding_window_size=None, q_segment_ids=None,
                kv_segment_ids=None):
  """Boolean mask the Pallas op applies (recml/core/ops/hstu_ops.py:926-979,
  107-194): CausalMask (j <= i) / FullMask / explicit [q_len,kv_len] array,
  AND LocalMask(window=(w,w), offset=0) i.e. |i-j| <= w, AND equality of
  segment ids.  Returns [B or 1, q_len, kv_len] bool.
  """
  i = np.arange(q_len)[:, None]
  j = np.arange(kv_len)[None, :]
  if explicit is not None:
    m = np.asarray(explicit).astype(bool)
    if m.shape != (q_len, kv_len):
      raise ValueError(
          f"Mask shape {m.shape} does not match query and key length"
          f" ({q_len}, {kv_len}).")
  elif causal:
    m = j <= i
  else:
    m = np.ones((q_len, kv_len), dtype=bool)
  if sliding_window_size is not None:
    m = m & (np.abs(i - j) <= sliding_window_size)
  m = m[None]
  if (q_segment_ids is None) != (kv_segment_ids is None):
    raise ValueError(
        "Both or neither of `q_segment_ids` and `kv_segment_ids` must be"
        " provided.")
  if q_segment_ids is not None:
    qs = np.asarray(q_segment_ids)
    ks = np.asarray(kv_segment_ids)
    m = m & (qs[:, :, None] == ks[:, None, :])
  return m


# ---------------------------------------------------------------------------
# Attention
# ---------------------------------------------------------------------------


def silu(x):
  x = np.asarray(x)
  # x * sigmoid(x), written to be safe for large |x|
  return x / (1.0 + np.exp(-x))


def pointwise_attention_dense(q, k, v, attention_mask, attention_bias=None,
                              scaled: bool = False, dtype=np.float64,
                              dropout_p: float = 0.0, dropout_seed: int = 0):
  """recml/layers/keras/hstu.py:356-390; dropout_p > 0 is its training form
  (:386-387): the masked weights times dropout_keep_mask / (1 - dropout_p).

  q,k,v [B,L,H,d]; attention_mask [B,L,Lkv] (non-zero = keep);
  attention_bias [B or 1,L,Lkv] broadcast over heads.
  """
  q = np.asarray(q, dtype=dtype)
  k = np.asarray(k, dtype=dtype)
  v = np.asarray(v, dtype=dtype)
  if scaled:
    q = q / np.asarray(q.shape[-1] ** 0.5, dtype=dtype)
  s = np.einsum("bthd,bshd->bhts", q, k)
  if attention_bias is not None:
    s = s + np.asarray(attention_bias, dtype=dtype)[:, None]
  p = silu(s)
  if not scaled:
    p = p / q.shape[1]
  keep = np.asarray(attention_mask).astype(bool)[:, None]
  p = np.where(keep, p, np.zeros_like(p))
  if dropout_p > 0:
    B, H, L, Lkv = p.shape
    p = p * _dropout_factor(dropout_p, dropout_seed, B, H, L, Lkv, 0, dtype)
  return np.einsum("bhts,bshd->bthd", p, v)


def pw_attn_ref(q, k, v, segment_ids, dtype=np.float64):
  """recml/core/ops/hstu_ops_test.py:44-58 (forward value only).

  1/sqrt(d) on q, silu / L, tril(seg_q == seg_kv) mask.  Note that with
  prefix segment ids (1..1,0..0) padded rows attend to earlier padded keys.
  """
  q = np.asarray(q, dtype=dtype)
  k = np.asarray(k, dtype=dtype)
  v = np.asarray(v, dtype=dtype)
  seg = np.asarray(segment_ids)
  q = q * 1.0 / (q.shape[-1] ** 0.5)
  logits = np.einsum("btnh,bsnh->bnts", q, k)
  s = silu(logits) / q.shape[1]
  mask = np.tril(seg[..., :, None] == seg[..., None, :])[:, None]
  s = np.where(mask, s, np.zeros_like(s))
  return np.einsum("bnts,bsnh->btnh", s, v)


def _bias_term(L, Lkv, H, pos_tab, timestamps, ts_tab, ts_bucket_size, law):
  """[B or 1, H or 1, L, Lkv] fp64 bias from the tables, or None."""
  bias = None
  if pos_tab is not None:
    pt = np.asarray(pos_tab, dtype=np.float64)
    if pt.ndim == 1:
      pt = pt[None]
    if Lkv != L:
      raise ValueError("relative-position bias needs q_len == kv_len")
    pb = np.stack([rel_pos_bias(pt[h], L)[0] for h in range(pt.shape[0])])
    bias = pb[None]                                     # [1,Hp,L,L]
  if ts_tab is not None:
    tt = np.asarray(ts_tab, dtype=np.float64)
    if tt.ndim == 1:
      tt = tt[None]
    nb = tt.shape[1] - 1
    tb = np.stack(
        [time_bias(timestamps, tt[h], nb, ts_bucket_size, law=law)
         for h in range(tt.shape[0])], axis=1)          # [B,Ht,L,L]
    bias = tb if bias is None else bias + tb
  return bias


# ---------------------------------------------------------------------------
# Attention dropout: which (b, h, i, j) survive
# ---------------------------------------------------------------------------

_U32 = np.uint64(0xFFFFFFFF)
DROP_CI = 0x85EBCA77
DROP_CJ = 0xC2B2AE3D


def _u32(x):
  return np.asarray(x, dtype=np.uint64) & _U32


def dropout_threshold(p: float) -> int:
  """round(p * 2^32), 0 for p <= 0, capped at 2^32 - 1: a pair is dropped when its hash is below it."""
  t = float(np.float32(p)) * 4294967296.0
  if t <= 0.0:
    return 0
  return 0xFFFFFFFF if t >= 4294967295.0 else int(t + 0.5)


def dropout_seed_key(seed: int) -> int:
  """Folds a 64-bit seed into 32 bits (two rounds of xor-shift and multiply)."""
  seed = int(seed) & 0xFFFFFFFFFFFFFFFF
  z = (seed & 0xFFFFFFFF) ^ 0x9E3779B9
  z = ((z ^ (z >> 16)) * 0x85EBCA6B) & 0xFFFFFFFF
  z ^= seed >> 32
  z = ((z ^ (z >> 13)) * 0xC2B2AE35) & 0xFFFFFFFF
  return z ^ (z >> 16)


def dropout_hash(seed: int, B: int, H: int, L: int, Lkv: int, b0: int = 0, rows=None, cols=None):
  """uint32 [B, H, L, Lkv]: hash(b, h, i, j) = mix(bhkey(seedkey, (b0 + b) * H + h) + i * CI + j * CJ), all in
  wrapping 32-bit arithmetic (bhkey: one multiply-add and one xor-shift-multiply round; mix(x): y = x * M1, then
  (y ^ (y >> 16)) * M2).
  `rows` / `cols`: the query / key indices to evaluate instead of all of range(L) / range(Lkv)."""
  key = np.uint64(dropout_seed_key(seed))
  bh = _u32((np.arange(b0, b0 + B, dtype=np.uint64)[:, None] * np.uint64(H)
             + np.arange(H, dtype=np.uint64)[None, :]))
  z = _u32(key + _u32(bh * np.uint64(0x9E3779B1)))
  z = _u32((z ^ (z >> np.uint64(15))) * np.uint64(0x2C1B3C6D))
  kbh = z ^ (z >> np.uint64(13))                                             # [B, H]
  i = _u32(np.asarray(range(L) if rows is None else rows, dtype=np.uint64) * np.uint64(DROP_CI))
  j = _u32(np.asarray(range(Lkv) if cols is None else cols, dtype=np.uint64) * np.uint64(DROP_CJ))
  ij = _u32(kbh[:, :, None, None] + i[None, None, :, None] + j[None, None, None, :])
  z = _u32(ij * np.uint64(0x2C1B3C6D))
  z = _u32((z ^ (z >> np.uint64(16))) * np.uint64(0x297A2D39))
  return z.astype(np.uint32)


def dropout_keep_mask(seed: int, p: float, B: int, H: int, L: int, Lkv: int, b0: int = 0):
  """bool [B, H, L, Lkv]: True where the weight of (sequence b0 + b, head h, query i, key j) survives:
  dropout_hash >= dropout_threshold(p).  With p == 0 everything survives."""
  thr = dropout_threshold(p)
  if thr == 0:
    return np.ones((B, H, L, Lkv), dtype=bool)
  return dropout_hash(seed, B, H, L, Lkv, b0) >= np.uint32(thr)


def _dropout_factor(p, seed, B, H, L, Lkv, b0, dtype):
  """[B, H, L, Lkv] factor on the masked weights: 0 for a dropped pair, 1 / (1 - p) for a survivor (the
  scale in fp32, as the library's host code forms it)."""
  keep = dropout_keep_mask(seed, p, B, H, L, Lkv, b0)
  scale = float(np.float32(1.0) / (np.float32(1.0) - np.float32(p)))
  return np.where(keep, scale, 0.0).astype(dtype)


def hstu_attention_ref(q, k, v, *, seq_lens=None, n=None, alpha=1.0,
                       causal=True, pos_tab=None, timestamps=None,
                       ts_tab=None, ts_bucket_size=0.301, bucket_law=True,
                       q_segment_ids=None, kv_segment_ids=None,
                       sliding_window_size=None, mask=None, bias=None,
                       dropout_p=0.0, dropout_seed=0, dropout_b0=0,
                       dtype=np.float64):
  """Dense restatement of the whole op on padded [B,L,H,d] inputs.

    S = alpha * q.k (+ pos_tab[h, (L-1)+j-i]) (+ ts_tab[h, bucket]) (+ bias)
    P = silu(S) / n            (n defaults to L, recml/layers/keras/hstu.py:377-378)
    M = causal & (lengths | segments) & window & explicit mask
    out = (M ? P : 0) @ v      rows >= seq_lens[b] are exactly 0

  `seq_lens` reproduces make_causal_mask on an end-padded batch
  (recml/layers/keras/utils.py:29-41 as used at hstu.py:609); segment ids
  reproduce recml/core/ops/hstu_ops_test.py:44-58.
  `mask` is an explicit [L,Lkv] or [B,L,Lkv] keep-mask, `bias` a dense
  [B or 1,L,Lkv] additive term shared by all heads (hstu.py:373-374).
  `dropout_p` > 0 is the training form (hstu.py:386-387): the masked weights
  times dropout_keep_mask(dropout_seed, ...) / (1 - dropout_p); `dropout_b0` is
  the index of the batch's first sequence in that mask.
  """
  q = np.asarray(q, dtype=dtype)
  k = np.asarray(k, dtype=dtype)
  v = np.asarray(v, dtype=dtype)
  B, L, H, _ = q.shape
  Lkv = k.shape[1]
  n = L if n is None else n
  s = alpha * np.einsum("bthd,bshd->bhts", q, k)
  tb = _bias_term(L, Lkv, H, pos_tab, timestamps, ts_tab, ts_bucket_size,
                  bucket_law)
  if tb is not None:
    s = s + tb.astype(dtype)
  if bias is not None:
    s = s + np.asarray(bias, dtype=dtype)[:, None]
  p = silu(s) / n
  # The explicit mask is one more factor of M here (the C ABI's meaning), for [L,Lkv] and [B,L,Lkv]
  # alike; splash_mask's own `explicit` argument is the reference's mask_type array, which stands
  # in place of the causal / full choice, and callers that mean that pass causal=False.
  m = splash_mask(L, Lkv, causal=causal, explicit=None,
                  sliding_window_size=sliding_window_size,
                  q_segment_ids=q_segment_ids, kv_segment_ids=kv_segment_ids)
  if mask is not None:
    mk = np.asarray(mask).astype(bool)
    if mk.shape[-2:] != (L, Lkv):
      raise ValueError(
          f"Mask shape {mk.shape} does not match query and key length"
          f" ({L}, {Lkv}).")
    m = m & (mk if mk.ndim == 3 else mk[None])
  if seq_lens is not None:
    lens = np.asarray(seq_lens)
    vq = np.arange(L)[None, :] < lens[:, None]
    vk = np.arange(Lkv)[None, :] < lens[:, None]
    m = m & (vq[:, :, None] & vk[:, None, :])
  p = np.where(m[:, None], p, np.zeros_like(p))
  if dropout_p > 0:
    p = p * _dropout_factor(dropout_p, dropout_seed, B, H, L, Lkv, dropout_b0, dtype)
  # Keys beyond the sequence never contribute, whatever the padding holds.
  return np.einsum("bhts,bshd->bthd", p, v)


def hstu_attention_bwd_ref(q, k, v, dout, *, seq_lens=None, n=None, alpha=1.0,
                           causal=True, pos_tab=None, timestamps=None,
                           ts_tab=None, ts_bucket_size=0.301, bucket_law=True,
                           q_segment_ids=None, kv_segment_ids=None,
                           sliding_window_size=None, mask=None, bias=None,
                           bias_grad=False, dropout_p=0.0, dropout_seed=0,
                           dropout_b0=0, dtype=np.float64):
  """Gradients of sum(out * dout) for hstu_attention_ref, dense, on padded inputs.

  The math of the reference's backward kernel (recml/core/ops/hstu_ops.py:461-517):
    dV = P^T dO;  dP = dO V^T;  dS = dP * sigma(S) (1 + S (1 - sigma(S))) / n  (masked);
    dQ = alpha dS K;  dK = alpha dS^T Q
  extended by the bias terms of the forward: every (i, j) adds dS to the table entry it
  read (position entry (L-1)+j-i, timestamp entry bucket(i, j)), summed over heads when
  the table has one row for all heads.  Returns dq, dk, dv, dpos_tab (or None),
  dts_tab (or None) with the shapes of the inputs; with bias_grad=True also the gradient
  of the dense `bias` (dS summed over the heads, and over the batch when the bias is
  shared by it: jax's derivative of recml/layers/keras/hstu.py:373-374), shaped like it.
  With dropout the factor of the forward (0, or 1 / (1 - dropout_p)) multiplies P and dS alike.
  """
  q = np.asarray(q, dtype=dtype)
  k = np.asarray(k, dtype=dtype)
  v = np.asarray(v, dtype=dtype)
  dout = np.asarray(dout, dtype=dtype)
  B, L, H, _ = q.shape
  Lkv = k.shape[1]
  n = L if n is None else n
  s = alpha * np.einsum("bthd,bshd->bhts", q, k)
  tb = _bias_term(L, Lkv, H, pos_tab, timestamps, ts_tab, ts_bucket_size, bucket_law)
  if tb is not None:
    s = s + tb.astype(dtype)
  if bias is not None:
    s = s + np.asarray(bias, dtype=dtype)[:, None]
  # The explicit mask is one more factor of M here (the C ABI's meaning), for [L,Lkv] and [B,L,Lkv]
  # alike; splash_mask's own `explicit` argument is the reference's mask_type array, which stands
  # in place of the causal / full choice, and callers that mean that pass causal=False.
  m = splash_mask(L, Lkv, causal=causal, explicit=None,
                  sliding_window_size=sliding_window_size,
                  q_segment_ids=q_segment_ids, kv_segment_ids=kv_segment_ids)
  if mask is not None:
    mk = np.asarray(mask).astype(bool)
    if mk.shape[-2:] != (L, Lkv):
      raise ValueError(
          f"Mask shape {mk.shape} does not match query and key length"
          f" ({L}, {Lkv}).")
    m = m & (mk if mk.ndim == 3 else mk[None])
  if seq_lens is not None:
    lens = np.asarray(seq_lens)
    vq = np.arange(L)[None, :] < lens[:, None]
    vk = np.arange(Lkv)[None, :] < lens[:, None]
    m = m & (vq[:, :, None] & vk[:, None, :])
  m = np.broadcast_to(m, (B, L, Lkv))[:, None]
  sg = 1.0 / (1.0 + np.exp(-s))
  p = np.where(m, s * sg / n, 0.0)
  if dropout_p > 0:
    fac = _dropout_factor(dropout_p, dropout_seed, B, H, L, Lkv, dropout_b0, dtype)
    p = p * fac
  dv = np.einsum("bhts,bthd->bshd", p, dout)
  dp = np.einsum("bthd,bshd->bhts", dout, v)
  ds = np.where(m, dp * sg * (1.0 + s * (1.0 - sg)) / n, 0.0)
  if dropout_p > 0:
    ds = ds * fac
  dq = alpha * np.einsum("bhts,bshd->bthd", ds, k)
  dk = alpha * np.einsum("bhts,bthd->bshd", ds, q)
  dpos = dts = None
  if pos_tab is not None:
    pt = np.atleast_2d(np.asarray(pos_tab))
    dpos = np.zeros(pt.shape, dtype=dtype)
    idx = (L - 1) + np.arange(Lkv)[None, :] - np.arange(L)[:, None]          # [L, Lkv]
    per_head = ds.sum(axis=0)                                                  # [H, L, Lkv]
    for h in range(H):
      np.add.at(dpos[h if pt.shape[0] > 1 else 0], idx, per_head[h])
    dpos = dpos.reshape(np.asarray(pos_tab).shape)
  if ts_tab is not None:
    tt = np.atleast_2d(np.asarray(ts_tab))
    nb = tt.shape[1] - 1
    dts = np.zeros(tt.shape, dtype=dtype)
    fn = bucketize_law if bucket_law else default_bucketization
    bucket = np.clip(fn(time_delta(timestamps), ts_bucket_size), 0, nb)
    for h in range(H):
      np.add.at(dts[h if tt.shape[0] > 1 else 0], bucket, ds[:, h])
    dts = dts.reshape(np.asarray(ts_tab).shape)
  if bias_grad:
    bshape = np.asarray(bias).shape
    dbias = ds.sum(axis=1)                                                     # [B, L, Lkv]
    if len(bshape) == 2 or bshape[0] == 1:
      dbias = dbias.sum(axis=0, keepdims=len(bshape) == 3)
    return dq, dk, dv, dpos, dts, dbias.reshape(bshape)
  return dq, dk, dv, dpos, dts


def hstu_attention_bruteforce(q, k, v, *, seq_lens=None, n=None, alpha=1.0,
                              causal=True, pos_tab=None, timestamps=None,
                              ts_tab=None, ts_bucket_size=0.301,
                              q_segment_ids=None, kv_segment_ids=None,
                              sliding_window_size=None):
  """Pure-Python fp64 loops, written independently of the vectorised path.

  Small inputs only.  Timestamp rule spelled out per pair: row i uses
  ts[min(i+1, L-1)], bucket = trunc(ln(clip(|dt|,1,1e9))/size) clipped to the
  table (recml/layers/keras/hstu.py:194-212, 48-55).
  """
  q = np.asarray(q, dtype=np.float64)
  k = np.asarray(k, dtype=np.float64)
  v = np.asarray(v, dtype=np.float64)
  B, L, H, d = q.shape
  Lkv = k.shape[1]
  dv = v.shape[-1]
  n = L if n is None else n
  out = np.zeros((B, L, H, dv))
  for b in range(B):
    nb = L if seq_lens is None else int(seq_lens[b])
    nbk = Lkv if seq_lens is None else int(seq_lens[b])
    for h in range(H):
      for i in range(L):
        if i >= nb:
          continue
        for j in range(Lkv):
          if j >= nbk:
            continue
          if causal and j > i:
            continue
          if sliding_window_size is not None and abs(i - j) > sliding_window_size:
            continue
          if q_segment_ids is not None and (
              int(q_segment_ids[b][i]) != int(kv_segment_ids[b][j])):
            continue
          s = alpha * float(np.dot(q[b, i, h], k[b, j, h]))
          if pos_tab is not None:
            pt = np.asarray(pos_tab)
            row = pt if pt.ndim == 1 else pt[h if pt.shape[0] > 1 else 0]
            s += float(row[(L - 1) + j - i])
          if ts_tab is not None:
            tt = np.asarray(ts_tab)
            row = tt if tt.ndim == 1 else tt[h if tt.shape[0] > 1 else 0]
            dt = int(timestamps[b][min(i + 1, L - 1)]) - int(timestamps[b][j])
            x = min(max(abs(dt), 1), 10**9)
            bk = int(math.log(float(np.float32(x))) / ts_bucket_size)
            bk = min(max(bk, 0), len(row) - 1)
            s += float(row[bk])
          p = s / (1.0 + math.exp(-s)) / n
          out[b, i, h] += p * v[b, j, h]
  return out


# ---------------------------------------------------------------------------
# Layout helpers and storage rounding used by parity tests
# ---------------------------------------------------------------------------


def round_bf16(x):
  """Round fp32 -> bf16 (nearest even) and return as fp32."""
  a = np.ascontiguousarray(np.asarray(x, dtype=np.float32))
  u = a.view(np.uint32).astype(np.uint64)
  r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
  return r.astype(np.uint32).view(np.float32).reshape(a.shape)


E4M3FN_MAX = 448.0


def round_e4m3fn(x):
  """Round to the nearest float8 e4m3fn value (ties to even, saturating at
  +-448) and return it as fp32.

  The format (OCP 8-bit floating point, "fn" = finite + NaN, no infinities):
  1 sign, 4 exponent bits with bias 7, 3 mantissa bits; normal values
  2^e * (1 + m/8) for e in -6..8 (e = 8 only up to m = 6, i.e. 448),
  subnormals m * 2^-9.  Not part of the reference (its README lists fp8 as
  roadmap only); pinned against torch's CPU float8_e4m3fn cast.
  """
  a = np.asarray(x, dtype=np.float64)
  mag = np.minimum(np.abs(a), E4M3FN_MAX)
  # exponent of the value, clamped to the subnormal range
  e = np.floor(np.log2(np.maximum(mag, 2.0 ** -20)))
  e = np.clip(e, -6, 8)
  step = 2.0 ** (e - 3)                       # spacing of representable values in [2^e, 2^(e+1))
  r = np.round(mag / step) * step             # np.round is ties-to-even
  r = np.minimum(r, E4M3FN_MAX)
  return (np.sign(a) * r).astype(np.float32)


def encode_e4m3fn(x):
  """uint8 bit patterns of values that are already exactly representable."""
  a = np.asarray(x, dtype=np.float64)
  sign = (np.signbit(a)).astype(np.uint8) << 7
  mag = np.abs(a)
  e = np.floor(np.log2(np.maximum(mag, 2.0 ** -20)))
  normal = mag >= 2.0 ** -6
  e = np.clip(e, -6, 8)
  m_norm = np.round((mag / 2.0 ** e - 1.0) * 8).astype(np.int64)
  m_sub = np.round(mag / 2.0 ** -9).astype(np.int64)
  code = np.where(normal, ((e + 7).astype(np.int64) << 3) | m_norm, m_sub)
  return (sign | code.astype(np.uint8)).astype(np.uint8)


def quantize_e4m3fn_per_head(x):
  """Per-head symmetric quantisation of [..., H, d]: scale[h] = amax_h / 448,
  returns (x / scale rounded to e4m3fn, as fp32; scale [H] fp32)."""
  a = np.asarray(x, dtype=np.float32)
  H = a.shape[-2]
  amax = np.abs(a).reshape(-1, H, a.shape[-1]).max(axis=(0, 2))
  scale = (np.maximum(amax, 1e-30) / E4M3FN_MAX).astype(np.float32)
  q = round_e4m3fn(a / scale[:, None])
  return q, scale


def padded_to_jagged(x, seq_lens):
  """[B,L,...] -> [sum(len),...] plus offsets[B+1]."""
  lens = np.asarray(seq_lens).astype(np.int64)
  off = np.zeros(len(lens) + 1, dtype=np.int64)
  off[1:] = np.cumsum(lens)
  parts = [np.asarray(x)[b, : lens[b]] for b in range(len(lens))]
  return np.concatenate(parts, axis=0), off


def jagged_to_padded(x, offsets, L):
  off = np.asarray(offsets)
  B = len(off) - 1
  x = np.asarray(x)
  out = np.zeros((B, L) + x.shape[1:], dtype=x.dtype)
  for b in range(B):
    out[b, : off[b + 1] - off[b]] = x[off[b]: off[b + 1]]
  return out


def attention_flops(seq_lens, H, d_qk, d_v):
  """Unmasked causal work: sum_b H * n(n+1)/2 * (2 d_qk + 2 d_v)."""
  nn = np.asarray(seq_lens).astype(np.int64)
  return int((H * (nn * (nn + 1) // 2) * (2 * d_qk + 2 * d_v)).sum())


def hstu_attention_jagged_ref(q, k, v, seq_offsets, max_len, *, n=None,
                              alpha=1.0, causal=True, pos_tab=None,
                              timestamps=None, ts_tab=None,
                              ts_bucket_size=0.301, bucket_law=True,
                              dropout_p=0.0, dropout_seed=0,
                              dtype=np.float64, sequences=None):
  """The op on jagged [T,H,d] inputs, one sequence at a time.

  Sequence b of length m is the padded op at L = max_len restricted to its
  first m rows: the position table is indexed (max_len-1)+j-i, so the slice
  pos_tab[:, max_len-m : max_len+m-1] is the 2m-1 table of an m-long
  sequence; jagged timestamps [T] make the last row reuse its own timestamp
  (the padded form does the same when padding repeats the last timestamp).
  `sequences` optionally restricts the work to some sequence indices; other
  rows of the result are left at zero.
  """
  off = np.asarray(seq_offsets).astype(np.int64)
  B = len(off) - 1
  L = int(max_len)
  n = L if n is None else n
  q = np.asarray(q)
  out = np.zeros(q.shape[:-1] + (np.asarray(v).shape[-1],), dtype=dtype)
  pt = None if pos_tab is None else np.atleast_2d(np.asarray(pos_tab))
  for b in (range(B) if sequences is None else sequences):
    s, e = int(off[b]), int(off[b + 1])
    m = e - s
    if m <= 0:
      continue
    sub_pos = None if pt is None else pt[:, L - m: L + m - 1]
    ts = None if timestamps is None else np.asarray(timestamps)[s:e][None]
    if m == 1 and sub_pos is not None:
      # a one-entry table; rel_pos_bias handles n == 1 (the recipe does not)
      sub_pos = pt[:, L - 1: L]
    out[s:e] = hstu_attention_ref(
        q[s:e][None], np.asarray(k)[s:e][None], np.asarray(v)[s:e][None],
        n=n, alpha=alpha, causal=causal, pos_tab=sub_pos, timestamps=ts,
        ts_tab=ts_tab, ts_bucket_size=ts_bucket_size, bucket_law=bucket_law,
        dropout_p=dropout_p, dropout_seed=dropout_seed, dropout_b0=b,
        dtype=dtype)[0]
  return out
