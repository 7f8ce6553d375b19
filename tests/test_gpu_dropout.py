"""Attention dropout on the GPU: every kernel drops exactly the pairs the oracle's keep rule names (read back pair
by pair through one-hot operands), and forward and backward match the oracle with the same rate and seed.

The reference drops attention weights in training (recml/layers/keras/hstu.py:386-387, keras' Dropout on the
masked weights).  Its random stream is keras' own; what is checked here is the law (a dropped weight is 0, a
survivor is scaled by 1 / (1 - rate)) with this library's keep rule, the same in all kernels.
"""

import numpy as np
import pytest
import torch

import recml_amd
from recml_amd import hstu_ops
from oracle import hstu_oracle as O

pytestmark = pytest.mark.gpu

BF = torch.bfloat16


def _dev(x, dtype=None):
  t = torch.from_numpy(np.ascontiguousarray(x)).to("cuda:0")
  return t if dtype is None else t.to(dtype)


def _rel(a, b):
  return float(np.abs(a - b).max() / max(np.abs(b).max(), 1e-30))


def _variant(q, k, v, **kw):
  out = torch.empty(tuple(q.shape[:-1]) + (v.shape[-1],), dtype=v.dtype, device=q.device)
  args, keep = hstu_ops.build_args(q, k, v, out, **kw)
  return hstu_ops.kernel_variant(args)


def _one_hot_rows(B, L, H, d, base=1.0, lo=0, n=None):
  """x[b, t, h, (t - lo) % d] = base * 2^((t - lo) // d) for the positions t in [lo, lo + n), 0 elsewhere: a product
  with it files every such position under its own column, the positions that share a column under different binary
  digits."""
  x = np.zeros((B, L, H, d), np.float32)
  t = np.arange(lo, L if n is None else min(L, lo + n))
  x[:, t, :, (t - lo) % d] = (base * 2.0 ** ((t - lo) // d))[:, None, None]
  return x


def _digits(keep, axis_len, d, axis):
  """sum over the positions t = c + d m along `axis` of keep * 2^m, per column c: what a product with
  _one_hot_rows leaves, up to the constant weight of a pair."""
  w = 2.0 ** (np.arange(axis_len) // d)
  folded = np.zeros(keep.shape[:axis] + (d,) + keep.shape[axis + 1:], np.float64)
  kw = keep * w.reshape((-1,) + (1,) * (keep.ndim - 1 - axis))
  for c0 in range(0, axis_len, d):
    n = min(d, axis_len - c0)
    sl_src = [slice(None)] * keep.ndim
    sl_dst = [slice(None)] * keep.ndim
    sl_src[axis] = slice(c0, c0 + n)
    sl_dst[axis] = slice(0, n)
    folded[tuple(sl_dst)] += kw[tuple(sl_src)]
  return folded


def _check_pattern(got, want, what):
  """got = const * want with one constant for all entries (rounding of bf16 aside), and exactly 0 where want is."""
  assert got.shape == want.shape, what
  assert ((got == 0) == (want == 0)).all(), (what, int(((got == 0) != (want == 0)).sum()))
  nz = want != 0
  assert nz.any(), what
  ratio = got[nz] / want[nz]
  # a wrong pair moves an entry by at least 1 part in 15 (four binary digits); bf16 rounding by 1 in 256
  assert ratio.min() > 0 and ratio.max() / ratio.min() < 1.03, (what, float(ratio.min()), float(ratio.max()))


def _valid(lens, L, causal=True):
  i = np.arange(L)
  m = (i[None, :, None] < lens[:, None, None]) & (i[None, None, :] < lens[:, None, None])
  if causal:
    m = m & (i[None, None, :] <= i[None, :, None])
  return m                                                      # [B, L, L]


FWD_PATTERN_CASES = [
    # name, d, B, H, L, lens, extras, jagged, expected variant
    ("d128 no bias", 128, 2, 2, 512, [512, 300], (), False, "hstu_fwd_mfma_bf16"),
    ("d128 pos+ts jagged", 128, 3, 2, 512, [512, 300, 77], ("pos", "ts"), True, "hstu_fwd_mfma_bf16"),
    ("d128 work list", 128, 40, 4, 512, None, ("pos",), True, "hstu_fwd_mfma_bf16"),
    ("d128 segments", 128, 2, 2, 384, [384, 384], ("seg",), False, "hstu_fwd_mfma_bf16"),
    ("d128 dense mask", 128, 2, 2, 384, [384, 200], ("mask",), False, "hstu_fwd_mfma_bf16"),
    ("d128 fp8", 128, 2, 2, 512, [512, 129], ("fp8",), False, "hstu_fwd_mfma_fp8"),
    ("d64 ts", 64, 2, 4, 256, [256, 100], ("ts",), False, "hstu_fwd_mfma_bf16"),
    ("d32 pos", 32, 2, 2, 128, [128, 33], ("pos",), True, "hstu_fwd_mfma_bf16"),
    # one long sequence among short ones: its tiles' key ranges are split between workgroups; read back through the
    # first and through the last 512 keys
    ("d128 split tiles, first keys", 128, 3, 2, 2048, [2048, 64, 64], ("pos", "ts", "lo=0"), True, "hstu_fwd_mfma_bf16"),
    ("d128 split tiles, last keys", 128, 3, 2, 2048, [2048, 64, 64], ("lo=1536",), True, "hstu_fwd_mfma_bf16"),
    ("d128 not causal", 128, 2, 2, 384, [384, 130], ("full",), False, "hstu_fwd_mfma_bf16"),
    ("fp32 general", 48, 2, 3, 192, [192, 50], ("pos", "fp32"), False, "hstu_fwd_general<float>"),
    ("bf16 general d48", 48, 2, 2, 192, [192, 101], ("pos",), False, "hstu_fwd_general<bf16>"),
]


@pytest.mark.parametrize("name,d,B,H,L,lens,extras,jagged,variant", FWD_PATTERN_CASES, ids=[c[0] for c in FWD_PATTERN_CASES])
def test_forward_drops_exactly_the_oracles_pairs(gpu, name, d, B, H, L, lens, extras, jagged, variant):
  """Constant logits (q = k = 1/8 in every channel, bias tables of zeros) make every weight the same number; V with
  one 1 per row files each key under its own output channel (keys d apart share one, as binary digits).  The
  output then spells the keep pattern of every (row, key) pair."""
  rng = np.random.default_rng(5)
  p, seed = 0.3, 0xABCDEF0123
  ln = np.array(lens, np.int32) if lens is not None else rng.integers(1, L + 1, B).astype(np.int32)
  ln[0] = L
  dt = torch.float32 if "fp32" in extras else BF
  lo = next((int(e[3:]) for e in extras if e.startswith("lo=")), 0)
  causal = "full" not in extras
  q = np.full((B, L, H, d), 0.125, np.float32)
  v = _one_hot_rows(B, L, H, d, lo=lo, n=4 * d)
  kw = dict(n=1.0, alpha=8.0 / d, dropout_p=p, dropout_seed=seed, causal=causal)
  if "pos" in extras:
    kw["pos_bias"] = _dev(np.zeros((H, 2 * L - 1), np.float32))
  if "ts" in extras:
    kw["ts_bias"] = _dev(np.zeros((H, 65), np.float32))
    stamps = 1_600_000_000 + np.cumsum(rng.integers(1, 100_000, (B, L)), axis=1).astype(np.int64)
  valid = _valid(ln, L, causal)
  if "seg" in extras:
    seg = np.ones((B, L), np.int32)
    seg[1, 200:] = 2
    kw["q_segment_ids"] = kw["kv_segment_ids"] = _dev(seg)
    valid = _valid(np.full(B, L), L) & (seg[:, :, None] == seg[:, None, :])
  elif "mask" in extras:
    kw["mask"] = _dev(valid)
    kw["causal"] = False
  qt, kt, vt = _dev(q, dt), _dev(q, dt), _dev(v, dt)
  if "fp8" in extras:
    qt, kt = qt.to(torch.float8_e4m3fn), kt.to(torch.float8_e4m3fn)
  if jagged:
    pack = lambda t: torch.cat([t[b, :ln[b]] for b in range(B)])
    off = np.concatenate([[0], np.cumsum(ln)]).astype(np.int32)
    qt, kt, vt = pack(qt), pack(kt), pack(vt)
    kw.update(seq_offsets=_dev(off), max_len=L)
    if "ts" in extras:
      kw["timestamps"] = _dev(np.concatenate([stamps[b, :ln[b]] for b in range(B)]))
  else:
    if "seg" not in extras and "mask" not in extras:
      kw["seq_lens"] = _dev(ln)
    if "ts" in extras:
      kw["timestamps"] = _dev(stamps)
  assert _variant(qt, kt, vt, **kw) == variant
  out = recml_amd.hstu_attention(qt, kt, vt, **kw).float().cpu().numpy()
  if jagged:
    out = O.jagged_to_padded(out, off, L)
  keep = O.dropout_keep_mask(seed, p, B, H, L, L) & valid[:, None]            # [B, H, L, L]
  seen = keep[..., lo:lo + 4 * d].astype(np.float64)                           # the keys V files
  want = _digits(seen, seen.shape[3], d, axis=3).transpose(0, 2, 1, 3)         # [B, L, H, d]
  _check_pattern(out.astype(np.float64), want, name)
  # and about the rate's share of the valid pairs was dropped
  share = keep.sum() / (valid.sum() * H)
  assert abs(share - (1 - p)) < 0.02


BWD_PATTERN_CASES = [
    ("d128", 128, 2, 2, 512, [512, 300], False, False),
    ("d128 pos+ts jagged", 128, 3, 2, 512, [512, 300, 77], True, True),
    ("d128 work list", 128, 40, 4, 512, None, True, False),
    ("d64", 64, 2, 4, 256, [256, 100], False, False),
    ("d32 jagged", 32, 2, 2, 128, [128, 33], True, True),
]


@pytest.mark.parametrize("name,d,B,H,L,lens,jagged,tables", BWD_PATTERN_CASES, ids=[c[0] for c in BWD_PATTERN_CASES])
def test_matrix_core_backward_drops_exactly_the_oracles_pairs(gpu, name, d, B, H, L, lens, jagged, tables):
  """The same reading for the two matrix-core backward kernels.  With q = 0 every logit is the (constant) position
  bias, so P and dS / dP are constants.  Call 1: K with one entry per row and a constant dP spell the pattern
  into dQ (the dQ kernel); dO with one entry per row spells it into dV (the dK/dV kernel's P side).  Call 2: k = 0,
  Q with one entry per row spells it into dK (that kernel's dS side)."""
  rng = np.random.default_rng(6)
  p, seed = 0.4, 77
  ln = np.array(lens, np.int32) if lens is not None else rng.integers(1, L + 1, B).astype(np.int32)
  ln[0] = L
  valid = _valid(ln, L)
  keep = (O.dropout_keep_mask(seed, p, B, H, L, L) & valid[:, None]).astype(np.float64)     # [B, H, i, j]
  kw = dict(n=1.0, alpha=1.0, dropout_p=p, dropout_seed=seed, pos_bias=_dev(np.ones((H, 2 * L - 1), np.float32)))
  if tables:
    kw["ts_bias"] = _dev(np.zeros((H, 65), np.float32))
    stamps = 1_600_000_000 + np.cumsum(rng.integers(1, 100_000, (B, L)), axis=1).astype(np.int64)
  off = np.concatenate([[0], np.cumsum(ln)]).astype(np.int32)
  pack = lambda t: torch.cat([t[b, :ln[b]] for b in range(B)])

  def run(q, k, v, dout):
    ts = [_dev(x, BF) for x in (q, k, v, dout)]
    k2 = dict(kw)
    if jagged:
      ts = [pack(t) for t in ts]
      k2.update(seq_offsets=_dev(off), max_len=L)
      if tables:
        k2["timestamps"] = _dev(np.concatenate([stamps[b, :ln[b]] for b in range(B)]))
    else:
      k2["seq_lens"] = _dev(ln)
      if tables:
        k2["timestamps"] = _dev(stamps)
    variant = []
    got = recml_amd.hstu_attention_bwd(*ts, _variant_out=variant, **k2)
    assert variant == ["hstu_bwd_mfma_bf16"]
    g = [x.float().cpu().numpy().astype(np.float64) for x in got[:3]]
    return [O.jagged_to_padded(x, off, L) for x in g] if jagged else g

  zeros = np.zeros((B, L, H, d), np.float32)
  hot = _one_hot_rows(B, L, H, d)
  const = np.full((B, L, H, d), 0.25, np.float32)
  # call 1: dP[i, j] = dO[i] . v[j] = 2^(i // d) / 4 (a row factor, divided out below)
  dq, dk, dv = run(zeros, hot, const, hot)
  rowf = (2.0 ** (np.arange(L) // d))[None, :, None, None]
  _check_pattern(dq / rowf, _digits(keep, L, d, axis=3).transpose(0, 2, 1, 3), name + " dq")
  _check_pattern(dv, _digits(keep, L, d, axis=2).transpose(0, 3, 1, 2), name + " dv")
  assert (dk == 0).all()                                          # q = 0
  # call 2: dP = dO . v constant; dk[j, c] = sum over rows i = c mod d of keep * dS * 2^(i // d)
  dq, dk, dv = run(hot, zeros, const, const)
  _check_pattern(dk, _digits(keep, L, d, axis=2).transpose(0, 3, 1, 2), name + " dk")


def _random_case(rng, B, L, Lk, H, d, dv, scale=0.5, bf16=False):
  rd = O.round_bf16 if bf16 else (lambda x: x)
  q = rd(rng.standard_normal((B, L, H, d)).astype(np.float32) * scale)
  k = rd(rng.standard_normal((B, Lk, H, d)).astype(np.float32) * scale)
  v = rd(rng.standard_normal((B, Lk, H, dv)).astype(np.float32) * scale)
  dout = rd(rng.standard_normal((B, L, H, dv)).astype(np.float32) * scale)
  return q, k, v, dout


GENERAL_CASES = [
    # name, dtype, d, dv, L, Lk, options, forward variant, backward variant
    ("fp32 segments+window", torch.float32, 16, 16, 70, 70, "seg", "hstu_fwd_general<float>", "hstu_bwd_general<float>"),
    ("fp32 tables", torch.float32, 32, 24, 90, 90, "tables", "hstu_fwd_general<float>", "hstu_bwd_general<float>"),
    ("fp32 d160", torch.float32, 160, 136, 50, 50, "tables", "hstu_fwd_general<float>", "hstu_bwd_general<float>"),
    ("fp32 mask+bias cross", torch.float32, 16, 16, 40, 56, "dense", "hstu_fwd_general<float>", "hstu_bwd_general<float>"),
    ("bf16 d48 tables", BF, 48, 48, 150, 150, "tables", "hstu_fwd_general<bf16>", "hstu_bwd_general<bf16, bf16 products>"),
    ("bf16 d64 mask+bias cross", BF, 64, 64, 100, 132, "dense", None, "hstu_bwd_general<bf16, bf16 products>"),
    ("bf16 d40", BF, 40, 40, 80, 80, "tables", "hstu_fwd_general<bf16>", "hstu_bwd_general<bf16>"),
]


@pytest.mark.parametrize("name,dtype,d,dv,L,Lk,opt,fwd_variant,bwd_variant", GENERAL_CASES, ids=[c[0] for c in GENERAL_CASES])
def test_general_kernels_with_dropout_against_oracle(gpu, name, dtype, d, dv, L, Lk, opt, fwd_variant, bwd_variant):
  """Forward and backward of the kernels that take every option, on random data, against the oracle with the same
  rate and seed.  In fp32 the tolerance is far below one pair's contribution, so a pair dropped or kept
  differently from the oracle fails it."""
  rng = np.random.default_rng(40)
  B, H = 3, 2
  bf = dtype == BF
  q, k, v, dout = _random_case(rng, B, L, Lk, H, d, dv, bf16=bf)
  p, seed = 0.35, 2 ** 40 + 17
  ok, gk = dict(dropout_p=p, dropout_seed=seed), dict(dropout_p=p, dropout_seed=seed)
  if opt == "seg":
    seg = np.ones((B, L), np.int32)
    seg[0, 25:] = 0
    seg[1, 10:30] = 2
    ok.update(alpha=0.25, q_segment_ids=seg, kv_segment_ids=seg, sliding_window_size=21)
    gk.update(alpha=0.25, q_segment_ids=_dev(seg), kv_segment_ids=_dev(seg), sliding_window_size=21)
  elif opt == "tables":
    lens = np.array([L, L // 2 + 1, 1], np.int32)
    pos = (rng.standard_normal((H, 2 * L - 1)) * 0.3).astype(np.float32)
    tab = (rng.standard_normal((33,)) * 0.3).astype(np.float32)
    ts = 1_600_000_000 + np.cumsum(np.ceil(rng.exponential(3600.0, (B, L))), axis=1).astype(np.int64)
    ok.update(seq_lens=lens, pos_tab=pos, timestamps=ts, ts_tab=tab)
    gk.update(seq_lens=_dev(lens), pos_bias=_dev(pos), timestamps=_dev(ts), ts_bias=_dev(tab))
  else:
    m = rng.random((B, L, Lk)) > 0.3
    bias = rng.standard_normal((B, L, Lk)).astype(np.float32)
    ok.update(causal=False, mask=m, bias=bias, n=9.0)
    gk.update(causal=False, mask=_dev(m), bias=_dev(bias), n=9.0)
  tol = 2e-2 if bf else 2e-5
  qt, kt, vt, dt_ = (_dev(x, dtype) for x in (q, k, v, dout))
  if fwd_variant is not None:
    assert _variant(qt, kt, vt, **gk) == fwd_variant
  out = recml_amd.hstu_attention(qt, kt, vt, **gk).float().cpu().numpy()
  want = O.hstu_attention_ref(q, k, v, **ok)
  assert _rel(out, want) <= tol
  assert _rel(O.hstu_attention_ref(q, k, v, **{**ok, "dropout_p": 0.0}), want) > 0.05      # the case tells them apart
  variant = []
  got = recml_amd.hstu_attention_bwd(qt, kt, vt, dt_, _variant_out=variant, **gk)
  assert variant == [bwd_variant]
  wants = O.hstu_attention_bwd_ref(q, k, v, dout, **ok)
  for nm, g, w in zip(("dq", "dk", "dv", "dpos", "dts"), got, wants):
    assert (g is None) == (w is None), nm
    if g is not None:
      assert _rel(g.float().cpu().numpy().reshape(w.shape), w) <= tol, nm


MFMA_CASES = [
    ("d128 pos+ts jagged", 128, 4, 420, 2, [420, 129, 33, 256], True, True, True, None),
    ("d128 lengths", 128, 3, 300, 2, [300, 129, 1], False, False, False, None),
    ("d128 window", 128, 2, 400, 2, [400, 203], True, False, False, 37),
    ("d64 pos+ts jagged", 64, 4, 420, 2, [420, 129, 33, 256], True, True, True, None),
    ("d32 ts", 32, 2, 200, 4, [200, 100], False, True, False, None),
]


@pytest.mark.parametrize("name,d,B,L,H,lens,pos,ts,jagged,window", MFMA_CASES, ids=[c[0] for c in MFMA_CASES])
def test_matrix_core_kernels_with_dropout_against_oracle(gpu, name, d, B, L, H, lens, pos, ts, jagged, window):
  rng = np.random.default_rng(41)
  q, k, v, dout = _random_case(rng, B, L, L, H, d, d, bf16=True)
  ln = np.array(lens, np.int32)
  p, seed = 0.2, 31337
  ok = dict(seq_lens=ln, dropout_p=p, dropout_seed=seed)
  gk = dict(dropout_p=p, dropout_seed=seed)
  if window is not None:
    ok["sliding_window_size"] = gk["sliding_window_size"] = window
  if pos:
    ok["pos_tab"] = (rng.standard_normal((H, 2 * L - 1)) * 0.3).astype(np.float32)
    gk["pos_bias"] = _dev(ok["pos_tab"])
  if ts:
    ok["ts_tab"] = (rng.standard_normal((129,)) * 0.3).astype(np.float32)
    t = 1_600_000_000 + np.cumsum(np.ceil(rng.exponential(3600.0, (B, L))), axis=1).astype(np.int64)
    for b in range(B):
      t[b, ln[b]:] = t[b, ln[b] - 1]
    ok["timestamps"] = t
    gk["ts_bias"] = _dev(ok["ts_tab"])
  ts_ = [_dev(x, BF) for x in (q, k, v, dout)]
  off = np.concatenate([[0], np.cumsum(ln)]).astype(np.int32)
  if jagged:
    ts_ = [torch.cat([t_[b, :ln[b]] for b in range(B)]) for t_ in ts_]
    gk.update(seq_offsets=_dev(off), max_len=L)
    if ts:
      gk["timestamps"] = _dev(np.concatenate([ok["timestamps"][b, :ln[b]] for b in range(B)]))
  else:
    gk["seq_lens"] = _dev(ln)
    if ts:
      gk["timestamps"] = _dev(ok["timestamps"])
  unpack = (lambda x: O.jagged_to_padded(x, off, L)) if jagged else (lambda x: x)
  assert _variant(*ts_[:3], **gk) == "hstu_fwd_mfma_bf16"
  out = unpack(recml_amd.hstu_attention(*ts_[:3], **gk).float().cpu().numpy())
  want = O.hstu_attention_ref(q, k, v, **ok)
  assert _rel(out, want) <= 2e-2
  assert _rel(O.hstu_attention_ref(q, k, v, **{**ok, "dropout_p": 0.0}), want) > 0.05
  variant = []
  got = recml_amd.hstu_attention_bwd(*ts_, _variant_out=variant, **gk)
  assert variant == ["hstu_bwd_mfma_bf16"]
  wants = O.hstu_attention_bwd_ref(q, k, v, dout, **ok)
  for nm, g, w in zip(("dq", "dk", "dv"), got[:3], wants[:3]):
    assert _rel(unpack(g.float().cpu().numpy()), w) <= 2e-2, nm
  for nm, g, w in (("dpos", got[3], wants[3]), ("dts", got[4], wants[4])):
    assert (g is None) == (w is None), nm
    if g is not None:
      assert _rel(g.cpu().numpy().reshape(w.shape), w) <= 2e-2, nm


def test_dropout_arguments_and_determinism(gpu):
  rng = np.random.default_rng(42)
  B, L, H, d = 2, 256, 2, 128
  q, k, v, _ = _random_case(rng, B, L, L, H, d, d, bf16=True)
  qt, kt, vt = (_dev(x, BF) for x in (q, k, v))
  base = recml_amd.hstu_attention(qt, kt, vt)
  # rate 0 is the op without dropout, bit for bit, whatever the seed; the stream of interior steps included
  assert torch.equal(recml_amd.hstu_attention(qt, kt, vt, dropout_p=0.0, dropout_seed=123), base)
  a = recml_amd.hstu_attention(qt, kt, vt, dropout_p=0.5, dropout_seed=1)
  assert torch.equal(recml_amd.hstu_attention(qt, kt, vt, dropout_p=0.5, dropout_seed=1), a)
  assert not torch.equal(recml_amd.hstu_attention(qt, kt, vt, dropout_p=0.5, dropout_seed=2), a)
  assert not torch.equal(a, base)
  for bad in (1.0, -0.1, 1.5, float("nan")):
    with pytest.raises(ValueError, match="dropout_p"):
      recml_amd.hstu_attention(qt, kt, vt, dropout_p=bad)
  # the host's rule is the kernels' rule
  assert hstu_ops.dropout_keep(1, 0.5, 1, 1, H, 200, 100) == bool(O.dropout_keep_mask(1, 0.5, B, H, L, L)[1, 1, 200, 100])
  # the mean over seeds approaches the output without dropout (inverted dropout is unbiased)
  acc = torch.zeros_like(base, dtype=torch.float32)
  n = 64
  for s in range(n):
    acc += recml_amd.hstu_attention(qt, kt, vt, dropout_p=0.25, dropout_seed=1000 + s).float()
  # (relative L2 distance: about 0.07 from the noise of 64 draws; 0.25 if the survivors were not scaled)
  err = (acc / n - base.float()).norm() / base.float().norm()
  assert float(err) < 0.12


def test_autograd_function_with_dropout(gpu):
  rng = np.random.default_rng(43)
  B, L, H, d = 2, 64, 2, 64
  lens = np.array([64, 20], dtype=np.int32)
  mk = lambda *s: torch.from_numpy(rng.standard_normal(s).astype(np.float32) * 0.4).to("cuda:0").requires_grad_(True)
  q, k, v = mk(B, L, H, d), mk(B, L, H, d), mk(B, L, H, d)
  pos = mk(H, 2 * L - 1)
  dout = torch.from_numpy(rng.standard_normal((B, L, H, d)).astype(np.float32)).to("cuda:0")
  out = recml_amd.hstu_attention_autograd(q, k, v, pos_bias=pos, seq_lens=_dev(lens), dropout_p=0.3, dropout_seed=5)
  (out * dout).sum().backward()
  n = lambda t: t.detach().cpu().numpy()
  kw = dict(seq_lens=lens, pos_tab=n(pos), dropout_p=0.3, dropout_seed=5)
  assert _rel(n(out), O.hstu_attention_ref(n(q), n(k), n(v), **kw)) <= 2e-5
  want = O.hstu_attention_bwd_ref(n(q), n(k), n(v), n(dout), **kw)
  for name, g, w in zip(("dq", "dk", "dv", "dpos"), (q.grad, k.grad, v.grad, pos.grad), want):
    assert _rel(n(g), w) <= 2e-5, name


def test_matrix_core_forward_with_keys_and_queries_of_different_lengths(gpu):
  """Lq != Lkv (padded, not causal): i counts queries and j keys in the keep rule, also where the two axes differ."""
  rng = np.random.default_rng(44)
  B, Lq, Lk, H, d = 2, 200, 330, 2, 128
  q, k, v, _ = _random_case(rng, B, Lq, Lk, H, d, d, bf16=True)
  qt, kt, vt = (_dev(x, BF) for x in (q, k, v))
  kw = dict(causal=False, n=50.0, dropout_p=0.5, dropout_seed=99)
  assert _variant(qt, kt, vt, **kw) == "hstu_fwd_mfma_bf16"
  out = recml_amd.hstu_attention(qt, kt, vt, **kw).float().cpu().numpy()
  want = O.hstu_attention_ref(q, k, v, **kw)
  assert _rel(out, want) <= 2e-2
  # with i and j swapped in the rule the result is another one altogether
  keep_t = O.dropout_keep_mask(99, 0.5, B, H, Lk, Lq).transpose(0, 1, 3, 2)
  s = np.einsum("bthd,bshd->bhts", q.astype(np.float64), k.astype(np.float64))
  wrong = np.einsum("bhts,bshd->bthd", O.silu(s) / 50.0 * keep_t * 2.0, v.astype(np.float64))
  assert _rel(wrong, want) > 0.2
