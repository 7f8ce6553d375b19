"""GPU parity: the HIP path (through the C ABI) against the CPU oracle.

Tolerances (stated once, used everywhere below):
  fp32   max|out-ref| <= 1e-5 * max|ref|
  bf16   max|out-ref| <= 2e-2 * max|ref|   (inputs rounded to bf16 for both)
  masked / padded output positions are exactly 0.
"""

import math

import numpy as np
import pytest
import torch

import recml_amd
from recml_amd import hstu_ops, workloads
from oracle import hstu_oracle as O

pytestmark = pytest.mark.gpu

FP32_TOL = 1e-5
BF16_TOL = 2e-2


def _dev(x, dtype=None, dev="cuda:0"):
  if x is None:
    return None
  t = torch.from_numpy(np.ascontiguousarray(x)).to(dev)
  return t if dtype is None else t.to(dtype)


def _err(out, ref):
  ref = np.asarray(ref, dtype=np.float64)
  out = np.asarray(out, dtype=np.float64)
  return np.abs(out - ref).max() / max(np.abs(ref).max(), 1e-30)


def _store(x, dtype):
  """fp32 master -> what the kernel and the oracle both see."""
  return O.round_bf16(x) if dtype == torch.bfloat16 else np.asarray(x, np.float32)


def run_workload(w, dtype, **over):
  q, k, v = (_store(t, dtype) for t in (w.q, w.k, w.v))
  kw = dict(n=w.n, alpha=w.alpha, pos_bias=_dev(w.pos_tab),
            ts_bias=_dev(w.ts_tab), timestamps=_dev(w.timestamps))
  if w.layout == "jagged":
    kw.update(seq_offsets=_dev(w.seq_offsets), max_len=w.L)
  else:
    kw.update(seq_lens=_dev(w.seq_lens))
  kw.update(over)
  out = recml_amd.hstu_attention(_dev(q, dtype), _dev(k, dtype), _dev(v, dtype), **kw)
  torch.cuda.synchronize()
  return q, k, v, out.float().cpu().numpy()


def oracle_workload(w, q, k, v, dtype=np.float64, sequences=None):
  if w.layout == "jagged":
    return O.hstu_attention_jagged_ref(
        q, k, v, w.seq_offsets, w.L, n=w.n, alpha=w.alpha, pos_tab=w.pos_tab,
        timestamps=w.timestamps, ts_tab=w.ts_tab, dtype=dtype, sequences=sequences)
  return O.hstu_attention_ref(
      q, k, v, seq_lens=w.seq_lens, n=w.n, alpha=w.alpha, pos_tab=w.pos_tab,
      timestamps=w.timestamps, ts_tab=w.ts_tab, dtype=dtype)


# ---- configuration 1: fp32, the reference's CPU-runnable case


def test_config1_fp32(gpu):
  w = workloads.config1()
  q, k, v, out = run_workload(w, torch.float32)
  ref = oracle_workload(w, q, k, v)
  assert _err(out, ref) <= FP32_TOL
  # same inputs through the bf16 MFMA kernel
  qb, kb, vb, outb = run_workload(w, torch.bfloat16)
  assert _err(outb, oracle_workload(w, qb, kb, vb)) <= BF16_TOL


def test_golden_config1(gpu):
  g = np.load("tests/golden/config1_fp64.npz")
  w = workloads.config1()
  _, _, _, out = run_workload(w, torch.float32)
  assert _err(out, g["out"]) <= FP32_TOL


def test_golden_small_jagged(gpu):
  g = np.load("tests/golden/small_jagged_fp64.npz")
  w = workloads.small_jagged()
  _, _, _, out = run_workload(w, torch.float32)
  assert _err(out, g["out"]) <= FP32_TOL
  _, _, _, outb = run_workload(w, torch.bfloat16)
  assert _err(outb, g["out_bf16_inputs"]) <= BF16_TOL


# ---- configuration 2: bf16 padded + per-head position bias


def test_config2_bf16_padded_pos_bias(gpu):
  w = workloads.config2()
  q, k, v, out = run_workload(w, torch.bfloat16)
  ref = oracle_workload(w, q, k, v, dtype=np.float32)
  assert _err(out, ref) <= BF16_TOL
  for b in range(w.B):
    assert (out[b, w.seq_lens[b]:] == 0).all(), "padded rows must be exact zeros"
  # padding content is ignored: poison it
  q2, k2, v2 = (t.copy() for t in (w.q, w.k, w.v))
  for b in range(w.B):
    q2[b, w.seq_lens[b]:] = np.nan
    k2[b, w.seq_lens[b]:] = np.inf
    v2[b, w.seq_lens[b]:] = np.nan
  w2 = workloads.Workload(**{**w.__dict__, "q": q2, "k": k2, "v": v2})
  _, _, _, out2 = run_workload(w2, torch.bfloat16)
  np.testing.assert_array_equal(out, out2)


def test_config2_general_kernel_agrees(gpu):
  # same workload in fp32 storage goes through the general kernel
  w = workloads.config2()
  q, k, v, out = run_workload(w, torch.float32)
  ref = oracle_workload(w, q, k, v, dtype=np.float64)
  assert _err(out, ref) <= FP32_TOL


# ---- configuration 3: jagged, power-law lengths, position + timestamp bias


def test_config3_reduced_fp32_and_bf16(gpu):
  w = workloads.config3(B=8, L=512, H=2, d=128)
  q, k, v, out = run_workload(w, torch.float32)
  ref = oracle_workload(w, q, k, v)
  assert _err(out, ref) <= FP32_TOL
  qb, kb, vb, outb = run_workload(w, torch.bfloat16)
  assert _err(outb, oracle_workload(w, qb, kb, vb)) <= BF16_TOL


def _check_all_sequences_c(w, q, k, v, out, tol):
  """Every sequence of a jagged workload against the C oracle (double accumulation), plus the numpy
  oracle on the shortest sequence so that the two restatements are seen to agree at this size."""
  from oracle import c_oracle
  ref = c_oracle.hstu_attention_c(q, k, v, seq_offsets=w.seq_offsets, max_len=w.L, n=w.n, alpha=w.alpha,
                                  pos_tab=w.pos_tab, timestamps=w.timestamps, ts_tab=w.ts_tab, acc="f64")
  scale = np.abs(ref).max()
  assert np.isfinite(out).all()
  per_seq = [np.abs(out[w.seq_offsets[b]:w.seq_offsets[b + 1]] - ref[w.seq_offsets[b]:w.seq_offsets[b + 1]]).max(initial=0.0) / scale
             for b in range(w.B)]
  worst = int(np.argmax(per_seq))
  assert per_seq[worst] <= tol, f"sequence {worst} (length {w.seq_lens[worst]}): {per_seq[worst]}"
  b = int(np.argmin(w.seq_lens))
  ref_np = oracle_workload(w, q, k, v, dtype=np.float64, sequences=[b])
  sl = slice(w.seq_offsets[b], w.seq_offsets[b + 1])
  assert np.abs(ref_np[sl] - ref[sl]).max() / scale <= 1e-6


def test_config3_full_size_bf16(gpu):
  # the headline batch, all 64 sequences
  w = workloads.config3()
  q, k, v, out = run_workload(w, torch.bfloat16)
  _check_all_sequences_c(w, q, k, v, out, BF16_TOL)


def test_config4_attention_full_size_bf16(gpu):
  # the attention call of the model configuration (B=128, L=1024, H=8, d=64, position bias only)
  w = workloads.config4_attention()
  q, k, v, out = run_workload(w, torch.bfloat16)
  _check_all_sequences_c(w, q, k, v, out, BF16_TOL)


def test_config5_full_size_bf16_and_fp8(gpu):
  # the long-sequence configuration (B=32, L=4096, H=8, d=128): bf16, then fp8 q / k against the oracle on
  # exactly the dequantised values; all 32 sequences, C oracle
  w = workloads.config5()
  q, k, v, out = run_workload(w, torch.bfloat16)
  _check_all_sequences_c(w, q, k, v, out, BF16_TOL)
  q8, qs, qd = _quant(w.q)
  k8, ks, kd = _quant(w.k)
  out8 = recml_amd.hstu_attention(q8, k8, _dev(v, torch.bfloat16), q_scale=qs, k_scale=ks, seq_offsets=_dev(w.seq_offsets),
                                  max_len=w.L, n=w.n, alpha=w.alpha, pos_bias=_dev(w.pos_tab))
  torch.cuda.synchronize()
  _check_all_sequences_c(w, qd.astype(np.float32), kd.astype(np.float32), v, out8.float().cpu().numpy(), BF16_TOL)


@pytest.mark.parametrize("d", [32, 64, 128])
@pytest.mark.parametrize("causal", [True, False])
def test_mfma_head_dims_and_full_mask(gpu, d, causal):
  rng = np.random.default_rng(100 + d)
  B, L, H = 3, 200, 2
  lens = np.array([200, 77, 1], dtype=np.int32)
  q, k, v = (O.round_bf16(rng.standard_normal((B, L, H, d)).astype(np.float32) * 0.3) for _ in range(3))
  out = recml_amd.hstu_attention(_dev(q, torch.bfloat16), _dev(k, torch.bfloat16), _dev(v, torch.bfloat16),
                                 seq_lens=_dev(lens), causal=causal, n=50)
  ref = O.hstu_attention_ref(q, k, v, seq_lens=lens, causal=causal, n=50)
  assert _err(out.float().cpu().numpy(), ref) <= BF16_TOL


@pytest.mark.parametrize("layout", ["padded", "jagged"])
def test_few_long_sequences(gpu, layout):
  # few sequences of very different lengths, length not a multiple of any tile size,
  # called twice on the same buffers (a call must not depend on what the previous one left)
  rng = np.random.default_rng(77)
  B, L, H, d = 3, 1100, 2, 64
  lens = np.array([1100, 513, 40], dtype=np.int32)
  q, k, v = (O.round_bf16(rng.standard_normal((B, L, H, d)).astype(np.float32) * 0.2) for _ in range(3))
  pos = rng.standard_normal((H, 2 * L - 1)).astype(np.float32) * 0.1
  ts = 1_600_000_000 + np.cumsum(np.ceil(rng.exponential(3600.0, (B, L))), axis=1).astype(np.int64)
  tab = (rng.standard_normal((H, 129)) * 0.1).astype(np.float32)
  ref = O.hstu_attention_ref(q, k, v, seq_lens=lens, pos_tab=pos, timestamps=ts, ts_tab=tab, dtype=np.float32)
  for rep in range(2):
    if layout == "padded":
      out = recml_amd.hstu_attention(_dev(q, torch.bfloat16), _dev(k, torch.bfloat16), _dev(v, torch.bfloat16),
                                     seq_lens=_dev(lens), pos_bias=_dev(pos), timestamps=_dev(ts),
                                     ts_bias=_dev(tab)).float().cpu().numpy()
      for b in range(B):
        assert (out[b, lens[b]:] == 0).all()
    else:
      qj, off = O.padded_to_jagged(q, lens)
      kj, _ = O.padded_to_jagged(k, lens)
      vj, _ = O.padded_to_jagged(v, lens)
      outj = recml_amd.hstu_attention(_dev(qj, torch.bfloat16), _dev(kj, torch.bfloat16), _dev(vj, torch.bfloat16),
                                      seq_offsets=_dev(off.astype(np.int32)), max_len=L, pos_bias=_dev(pos),
                                      timestamps=_dev(ts), ts_bias=_dev(tab))
      out = O.jagged_to_padded(outj.float().cpu().numpy(), off, L)
    assert _err(out, ref) <= BF16_TOL
  # full (non-causal) mask through the same path
  out = recml_amd.hstu_attention(_dev(q, torch.bfloat16), _dev(k, torch.bfloat16), _dev(v, torch.bfloat16),
                                 seq_lens=_dev(lens), causal=False).float().cpu().numpy()
  assert _err(out, O.hstu_attention_ref(q, k, v, seq_lens=lens, causal=False, dtype=np.float32)) <= BF16_TOL


@pytest.mark.parametrize("B,L,H,d,layout", [
    (5, 200, 1, 64, "jagged"),      # one head: eight work items share a round of XCDs
    (2, 700, 3, 64, "padded"),      # 3 heads: no work list (static enumeration), key ranges split
    (2, 700, 3, 64, "jagged"),
    (3, 300, 12, 32, "jagged"),     # 12 heads: static enumeration, no split
    (4, 260, 16, 32, "padded"),     # 16 heads: two rounds of XCDs per item
    (1100, 40, 2, 32, "jagged"),    # more sequences than the list builder sorts
    (8200, 33, 1, 32, "padded"),    # more sequences than the list builder takes: static enumeration
])
def test_block_mappings(gpu, B, L, H, d, layout):
  rng = np.random.default_rng(B * 7 + H)
  lens = rng.integers(1, L + 1, B).astype(np.int32)
  lens[0] = L
  q, k, v = (O.round_bf16(rng.standard_normal((B, L, H, d)).astype(np.float32) * 0.3) for _ in range(3))
  pos = (rng.standard_normal((H, 2 * L - 1)) * 0.1).astype(np.float32)
  ref = O.hstu_attention_ref(q, k, v, seq_lens=lens, pos_tab=pos, dtype=np.float32)
  if layout == "padded":
    out = recml_amd.hstu_attention(_dev(q, torch.bfloat16), _dev(k, torch.bfloat16), _dev(v, torch.bfloat16),
                                   seq_lens=_dev(lens), pos_bias=_dev(pos)).float().cpu().numpy()
  else:
    qj, off = O.padded_to_jagged(q, lens)
    kj, _ = O.padded_to_jagged(k, lens)
    vj, _ = O.padded_to_jagged(v, lens)
    a, keep = hstu_ops.build_args(_dev(qj, torch.bfloat16), _dev(kj, torch.bfloat16), _dev(vj, torch.bfloat16),
                                  torch.empty((qj.shape[0], H, d), dtype=torch.bfloat16, device="cuda:0"),
                                  seq_offsets=_dev(off.astype(np.int32)), max_len=L, pos_bias=_dev(pos))
    assert hstu_ops.kernel_variant(a) == "hstu_fwd_mfma_bf16"
    hstu_ops._run(a, keep)
    out = O.jagged_to_padded(keep[3].float().cpu().numpy(), off, L)
  assert _err(out, ref) <= BF16_TOL
  for b in range(min(B, 50)):
    assert (out[b, lens[b]:] == 0).all()


def test_ragged_and_empty(gpu):
  rng = np.random.default_rng(5)
  H, d, L = 2, 64, 300
  lens = np.array([0, 1, 300, 0, 129, 64], dtype=np.int32)
  off = np.zeros(len(lens) + 1, dtype=np.int32)
  off[1:] = np.cumsum(lens)
  T = int(off[-1])
  q, k, v = (O.round_bf16(rng.standard_normal((T, H, d)).astype(np.float32) * 0.2) for _ in range(3))
  pos = rng.standard_normal((H, 2 * L - 1)).astype(np.float32) * 0.1
  for dt in (torch.bfloat16, torch.float32):
    out = recml_amd.hstu_attention(_dev(q, dt), _dev(k, dt), _dev(v, dt), seq_offsets=_dev(off),
                                   max_len=L, pos_bias=_dev(pos))
    ref = O.hstu_attention_jagged_ref(q, k, v, off, L, pos_tab=pos)
    assert _err(out.float().cpu().numpy(), ref) <= (BF16_TOL if dt == torch.bfloat16 else FP32_TOL)
  # an empty batch and an all-empty batch are no-ops
  e = torch.empty((0, H, d), dtype=torch.bfloat16, device="cuda:0")
  o = recml_amd.hstu_attention(e, e, e, seq_offsets=_dev(np.zeros(3, np.int32)), max_len=L)
  assert o.shape == (0, H, d)


def test_jagged_equals_padded_on_gpu(gpu):
  w = workloads.config3(B=6, L=384, H=2, d=64)
  q, k, v, outj = run_workload(w, torch.bfloat16)
  L = w.L
  qp, kp, vp = (O.jagged_to_padded(t, w.seq_offsets, L) for t in (q, k, v))
  tsp = O.jagged_to_padded(w.timestamps, w.seq_offsets, L)
  for b in range(w.B):
    tsp[b, w.seq_lens[b]:] = tsp[b, w.seq_lens[b] - 1]
  outp = recml_amd.hstu_attention(
      _dev(qp, torch.bfloat16), _dev(kp, torch.bfloat16), _dev(vp, torch.bfloat16),
      seq_lens=_dev(w.seq_lens), n=w.n, pos_bias=_dev(w.pos_tab), ts_bias=_dev(w.ts_tab),
      timestamps=_dev(tsp)).float().cpu().numpy()
  np.testing.assert_array_equal(O.jagged_to_padded(outj, w.seq_offsets, L), outp)


# ---- operator options (general kernel)


def test_splash_signature_segment_ids(gpu):
  # the reference's own test recipe (hstu_ops_test.py:29-58) at a smaller shape
  rng = np.random.default_rng(42)
  B, L, H, d = 8, 256, 2, 128
  q, k, v = (rng.standard_normal((B, L, H, d)).astype(np.float32) for _ in range(3))
  lens = (rng.random(B) * L).astype(np.int64)
  seg = (np.arange(L)[None] < lens[:, None]).astype(np.int32)
  out = recml_amd.pointwise_splash_attention(
      recml_amd.MaskType.CAUSAL, _dev(q), _dev(k), _dev(v),
      q_segment_ids=_dev(seg), kv_segment_ids=_dev(seg))
  ref = O.pw_attn_ref(q, k, v, seg)
  o = out.cpu().numpy()
  # the reference accepts atol=rtol=5e-3 here (hstu_ops_test.py:80-83); we hold 1e-5
  assert _err(o, ref) <= FP32_TOL
  np.testing.assert_allclose(o, ref, atol=5e-3, rtol=5e-3)
  # bf16 storage goes through the same kernel
  qb, kb, vb = (O.round_bf16(t) for t in (q, k, v))
  outb = recml_amd.pointwise_splash_attention(
      "causal", _dev(qb, torch.bfloat16), _dev(kb, torch.bfloat16), _dev(vb, torch.bfloat16),
      q_segment_ids=_dev(seg), kv_segment_ids=_dev(seg))
  assert _err(outb.float().cpu().numpy(), O.pw_attn_ref(qb, kb, vb, seg)) <= BF16_TOL


def test_splash_full_explicit_window_cross_length(gpu):
  rng = np.random.default_rng(43)
  B, Lq, Lk, H, d = 2, 70, 95, 3, 48
  q = rng.standard_normal((B, Lq, H, d)).astype(np.float32)
  k = rng.standard_normal((B, Lk, H, d)).astype(np.float32)
  v = rng.standard_normal((B, Lk, H, d)).astype(np.float32)
  alpha = 1 / math.sqrt(d)
  out = recml_amd.pointwise_splash_attention(recml_amd.MaskType.FULL, _dev(q), _dev(k), _dev(v))
  ref = O.hstu_attention_ref(q, k, v, causal=False, alpha=alpha, n=Lq)
  assert _err(out.cpu().numpy(), ref) <= FP32_TOL
  m = rng.random((Lq, Lk)) < 0.4
  out = recml_amd.pointwise_splash_attention(m, _dev(q), _dev(k), _dev(v), scale=0.2)
  ref = O.hstu_attention_ref(q, k, v, causal=False, mask=m, alpha=0.2, n=Lq)
  assert _err(out.cpu().numpy(), ref) <= FP32_TOL
  for wdw in (0, 5, 64):
    out = recml_amd.pointwise_splash_attention("causal", _dev(q), _dev(k), _dev(v), sliding_window_size=wdw)
    ref = O.hstu_attention_ref(q, k, v, causal=True, sliding_window_size=wdw, alpha=alpha, n=Lq)
    assert _err(out.cpu().numpy(), ref) <= FP32_TOL
    out = recml_amd.pointwise_splash_attention("full", _dev(q), _dev(k), _dev(v), sliding_window_size=wdw)
    ref = O.hstu_attention_ref(q, k, v, causal=False, sliding_window_size=wdw, alpha=alpha, n=Lq)
    assert _err(out.cpu().numpy(), ref) <= FP32_TOL


@pytest.mark.parametrize("Lq,Lk", [(200, 336), (336, 208), (100, 2080)])
def test_cross_length_on_matrix_cores(gpu, Lq, Lk):
  # keys and queries of different lengths in bf16: FULL, causal, sliding window, an explicit [Lq, Lk] mask, segment ids
  rng = np.random.default_rng(46)
  B, H, d = 2, 3, 64
  q = O.round_bf16(rng.standard_normal((B, Lq, H, d)).astype(np.float32) * 0.3)
  k = O.round_bf16(rng.standard_normal((B, Lk, H, d)).astype(np.float32) * 0.3)
  v = O.round_bf16(rng.standard_normal((B, Lk, H, d)).astype(np.float32) * 0.3)
  qd, kd, vd = (_dev(t, torch.bfloat16) for t in (q, k, v))
  m = rng.random((Lq, Lk)) < 0.4
  cases = [dict(causal=False), dict(causal=True), dict(causal=True, sliding_window_size=40),
           dict(causal=False, sliding_window_size=7), dict(causal=False, mask=m)]
  for kw in cases:
    out = torch.full((B, Lq, H, d), float("nan"), dtype=torch.bfloat16, device=qd.device)
    dkw = dict(kw)
    if "mask" in dkw:
      dkw["mask"] = _dev(m.astype(np.uint8))
    args, keep = hstu_ops.build_args(qd, kd, vd, out, n=Lq, alpha=0.125, **dkw)
    assert hstu_ops.kernel_variant(args) == "hstu_fwd_mfma_bf16", kw
    hstu_ops._run(args, keep)
    torch.cuda.synchronize()
    ref = O.hstu_attention_ref(q, k, v, alpha=0.125, n=Lq, **kw)
    assert _err(out.float().cpu().numpy(), ref) <= BF16_TOL, kw


def test_layer_call_dense_mask_and_bias(gpu):
  # HSTUBlock._pointwise_attention (hstu.py:356-390): dense [B,L,L] mask + bias
  rng = np.random.default_rng(44)
  B, L, H, d = 3, 50, 2, 32
  q, k, v = (rng.standard_normal((B, L, H, d)).astype(np.float32) for _ in range(3))
  lens = np.array([50, 20, 1])
  pad = (np.arange(L)[None] < lens[:, None]).astype(np.float32)
  mask = recml_amd.make_causal_mask(_dev(pad))
  np.testing.assert_array_equal(mask.cpu().numpy(), O.make_causal_mask(pad))
  bias = rng.standard_normal((B, L, L)).astype(np.float32)
  for scaled in (False, True):
    out = recml_amd.pointwise_attention(_dev(q), _dev(k), _dev(v), mask, _dev(bias),
                                        scaled_pointwise_attn=scaled)
    ref = O.pointwise_attention_dense(q, k, v, O.make_causal_mask(pad), bias, scaled=scaled)
    assert _err(out.cpu().numpy(), ref) <= FP32_TOL
    for b in range(B):
      assert (out[b, lens[b]:] == 0).all()
  # same result from lengths, never building the mask
  out2 = recml_amd.pointwise_attention(_dev(q), _dev(k), _dev(v), None, _dev(bias), seq_lens=_dev(lens))
  ref = O.pointwise_attention_dense(q, k, v, O.make_causal_mask(pad), bias)
  assert _err(out2.cpu().numpy(), ref) <= FP32_TOL


@pytest.mark.parametrize("d", [32, 64, 128])
@pytest.mark.parametrize("what", ["mask+bias", "mask", "bias", "shared"])
def test_layer_call_dense_on_matrix_cores(gpu, d, what):
  # the same dense call in bf16: the matrix-core kernel takes the [B, L, L] mask and bias tiles through its ring.
  # L = 176: whole 16-byte mask pieces, a partial last key tile and a partial last query tile.
  rng = np.random.default_rng(440 + d)
  B, L, H = 3, 176, 2
  q, k, v = (O.round_bf16(rng.standard_normal((B, L, H, d)).astype(np.float32) * 0.3) for _ in range(3))
  lens = np.array([176, 77, 1])
  pad = (np.arange(L)[None] < lens[:, None]).astype(np.float32)
  causal = O.make_causal_mask(pad)
  mask = bias = None
  if what in ("mask+bias", "mask"):
    mask = causal
  if what == "shared":
    mask = (rng.random((L, L)) < 0.5)          # one [L, L] mask and bias for the whole batch
    bias = rng.standard_normal((L, L)).astype(np.float32) * 0.5
  elif what in ("mask+bias", "bias"):
    bias = rng.standard_normal((B, L, L)).astype(np.float32) * 0.5
  qd, kd, vd = (_dev(t, torch.bfloat16) for t in (q, k, v))
  out = torch.full_like(vd, float("nan"))
  args, keep = hstu_ops.build_args(qd, kd, vd, out, n=L, alpha=1.0, causal=False,
                                   mask=None if mask is None else _dev(np.asarray(mask, np.uint8)),
                                   bias=_dev(bias))
  assert hstu_ops.kernel_variant(args) == "hstu_fwd_mfma_bf16"
  hstu_ops._run(args, keep)
  torch.cuda.synchronize()
  got = out.float().cpu().numpy()
  ref_mask = np.ones((B, L, L)) if mask is None else np.broadcast_to(np.asarray(mask, np.float64), (B, L, L))
  ref_bias = None if bias is None else (bias[None] if bias.ndim == 2 else bias)
  ref = O.pointwise_attention_dense(q, k, v, ref_mask, ref_bias)
  assert _err(got, ref) <= BF16_TOL
  if what in ("mask+bias", "mask"):
    for b in range(B):
      assert (got[b, lens[b]:] == 0).all()     # fully masked rows: exact zeros


def test_dense_bias_with_lengths_on_matrix_cores(gpu):
  # the dense bias on top of the causal flag and a length mask (padded), and in the jagged layout
  rng = np.random.default_rng(447)
  B, L, H, d = 3, 208, 2, 64
  lens = np.array([208, 97, 33], dtype=np.int32)
  q, k, v = (O.round_bf16(rng.standard_normal((B, L, H, d)).astype(np.float32) * 0.3) for _ in range(3))
  bias = rng.standard_normal((B, L, L)).astype(np.float32) * 0.5
  pad = (np.arange(L)[None] < lens[:, None]).astype(np.float32)
  ref = O.pointwise_attention_dense(q, k, v, O.make_causal_mask(pad), bias)
  qd, kd, vd = (_dev(t, torch.bfloat16) for t in (q, k, v))
  out = torch.full_like(vd, float("nan"))
  args, keep = hstu_ops.build_args(qd, kd, vd, out, n=L, alpha=1.0, causal=True, seq_lens=_dev(lens), bias=_dev(bias))
  assert hstu_ops.kernel_variant(args) == "hstu_fwd_mfma_bf16"
  hstu_ops._run(args, keep)
  torch.cuda.synchronize()
  got = out.float().cpu().numpy()
  assert _err(got, ref) <= BF16_TOL
  for b in range(B):
    assert (got[b, lens[b]:] == 0).all()
  # jagged: the same sequences packed; bias rows and columns are the positions within a sequence
  off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
  pack = lambda t: np.concatenate([t[b, :lens[b]] for b in range(B)])
  qj, kj, vj = (_dev(pack(t), torch.bfloat16) for t in (q, k, v))
  outj = torch.full_like(vj, float("nan"))
  args, keep = hstu_ops.build_args(qj, kj, vj, outj, n=L, alpha=1.0, causal=True, seq_offsets=_dev(off), max_len=L, bias=_dev(bias))
  assert hstu_ops.kernel_variant(args) == "hstu_fwd_mfma_bf16"
  hstu_ops._run(args, keep)
  torch.cuda.synchronize()
  assert _err(outj.float().cpu().numpy(), pack(ref)) <= BF16_TOL


def test_dense_bias_large_on_matrix_cores(gpu):
  # a longer case (several query tiles, the key range split over workgroups) against the numpy oracle's
  # dense layer form on the same bf16-rounded inputs; the general kernel (fp32 call) against it as well
  rng = np.random.default_rng(450)
  B, L, H, d = 2, 1040, 2, 64
  q, k, v = (O.round_bf16(rng.standard_normal((B, L, H, d)).astype(np.float32) * 0.3) for _ in range(3))
  lens = np.array([1040, 333])
  pad = (np.arange(L)[None] < lens[:, None]).astype(np.float32)
  mask_np = O.make_causal_mask(pad)
  bias_np = rng.standard_normal((B, L, L)).astype(np.float32) * 0.5
  mask, bias = _dev(mask_np.astype(np.uint8)), _dev(bias_np)
  got = recml_amd.pointwise_attention(_dev(q, torch.bfloat16), _dev(k, torch.bfloat16), _dev(v, torch.bfloat16), mask, bias)
  gen = recml_amd.pointwise_attention(_dev(q), _dev(k), _dev(v), mask, bias)
  torch.cuda.synchronize()
  ref = O.pointwise_attention_dense(q, k, v, mask_np, bias_np)
  assert _err(got.float().cpu().numpy(), ref) <= BF16_TOL
  assert _err(gen.cpu().numpy(), ref) <= FP32_TOL
  assert (got[1, 333:] == 0).all()


@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("shape", ["band", "blocks", "lower-left", "nothing", "one pair"])
@pytest.mark.parametrize("batched", [True, False])
def test_dense_mask_step_ranges(gpu, d, shape, batched):
  # The preparation kernel finds, per tile of 128 query rows, the range of 32-key steps in which the mask keeps
  # anything, and the main kernel runs only those.  Masks whose kept pairs start late, end early, leave whole
  # tiles or whole sequences empty, or keep one single pair; 3 query tiles (the last one partial), keys of
  # another length than the queries, with and without a bias.
  rng = np.random.default_rng(460 + d + len(shape))
  B, L, Lkv, H = 3, 300, 464, 2
  q = O.round_bf16(rng.standard_normal((B, L, H, d)).astype(np.float32) * 0.3)
  k, v = (O.round_bf16(rng.standard_normal((B, Lkv, H, d)).astype(np.float32) * 0.3) for _ in range(2))
  nb = B if batched else 1
  mask = np.zeros((nb, L, Lkv), dtype=np.uint8)
  i, j = np.arange(L)[:, None], np.arange(Lkv)[None, :]
  if shape == "band":
    for b in range(nb):
      mask[b] = (np.abs(j - i - 40 * b) <= 45) & (rng.random((L, Lkv)) < 0.8)
  elif shape == "blocks":
    for b in range(nb):
      mask[b, 128:256, 64 + 32 * b:96 + 32 * b] = 1      # one step of the second tile; the other tiles keep nothing
      mask[b, 290:, 400:] = rng.random((10, 64)) < 0.5   # the partial last tile: its last two steps
  elif shape == "lower-left":
    mask[:, 200:, :33] = 1
  elif shape == "one pair":
    mask[nb - 1, 129, 463] = 1
  bias = rng.standard_normal((B, L, Lkv)).astype(np.float32) * 0.5 if d == 128 else None
  qd, kd, vd = (_dev(t, torch.bfloat16) for t in (q, k, v))
  out = torch.full((B, L, H, d), float("nan"), dtype=torch.bfloat16, device="cuda:0")
  args, keep = hstu_ops.build_args(qd, kd, vd, out, n=L, alpha=1.0, causal=False,
                                   mask=_dev(mask if batched else mask[0]), bias=_dev(bias))
  assert hstu_ops.kernel_variant(args) == "hstu_fwd_mfma_bf16"
  hstu_ops._run(args, keep)
  torch.cuda.synchronize()
  got = out.float().cpu().numpy()
  full = np.broadcast_to(mask.astype(np.float64), (B, L, Lkv))
  ref = O.pointwise_attention_dense(q, k, v, full, bias)      # (divides by the query length, like n = L)
  assert np.isfinite(got).all()
  assert np.abs(got - ref).max() <= BF16_TOL * max(np.abs(ref).max(), 1e-3)
  # rows that keep no key: exact zeros
  empty = full.sum(axis=2) == 0
  assert (got[empty] == 0).all()


def test_shared_tables_and_strided_inputs(gpu):
  rng = np.random.default_rng(45)
  B, L, H, d = 2, 130, 4, 64
  lens = np.array([130, 61], dtype=np.int32)
  qkv = O.round_bf16(rng.standard_normal((B, L, 3, H, d)).astype(np.float32) * 0.3)
  pos = rng.standard_normal(2 * L - 1).astype(np.float32) * 0.1
  tst = rng.standard_normal(129).astype(np.float32) * 0.1
  ts = np.cumsum(rng.integers(1, 10**5, (B, L)), axis=1).astype(np.int64)
  t = _dev(qkv, torch.bfloat16)
  out = recml_amd.hstu_attention(t[:, :, 0], t[:, :, 1], t[:, :, 2], seq_lens=_dev(lens),
                                 pos_bias=_dev(pos), ts_bias=_dev(tst), timestamps=_dev(ts))
  ref = O.hstu_attention_ref(qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2], seq_lens=lens,
                             pos_tab=pos, ts_tab=tst, timestamps=ts)
  assert _err(out.float().cpu().numpy(), ref) <= BF16_TOL


def test_timestamp_buckets_on_gpu(gpu):
  # one key, zero q: out = silu(ts_tab[bucket]) * v / n  reveals the bucket per delta.  Every |delta| within
  # +-2 of every threshold of the law, both signs, both kernels: the bucket must be the law's, exactly.
  th = O.bucket_thresholds()
  near = np.concatenate([th[1:] + o for o in (-2, -1, 0, 1, 2)])
  deltas = np.concatenate([[0, 1, 2, 3, 10, 3600, 86400, 10**9 - 1, 10**9, 10**9 + 1, 2 * 10**9, 5 * 10**12],
                           near[near >= 0]]).astype(np.int64)
  table = (np.arange(129) + 1).astype(np.float32) / 64.0      # adjacent buckets differ by >= 0.8 % in silu(table)
  want_bucket = np.clip(O.bucketize_law(deltas), 0, 128)
  want = O.silu(table[want_bucket].astype(np.float64))
  for dt_ in (torch.float32, torch.bfloat16):
    for sign in (1, -1):
      B = len(deltas)
      ts = np.zeros((B, 2), dtype=np.int64)
      ts[:, 0] = 1_600_000_000
      ts[:, 1] = ts[:, 0] + sign * deltas      # row 0 sees ts[1] - ts[0]
      q = np.zeros((B, 2, 1, 32), np.float32)
      v = np.ones((B, 2, 1, 32), np.float32)
      out = recml_amd.hstu_attention(_dev(q, dt_), _dev(q, dt_), _dev(v, dt_), ts_bias=_dev(table),
                                     timestamps=_dev(ts), n=1).float().cpu().numpy()[:, 0, 0, 0]
      if dt_ == torch.float32:
        assert (np.abs(out - want) <= 1e-5 * want).all()
      # the bucket itself, read back from the output: the table entry whose silu is nearest (bf16 rounds P
      # and the output, 2 x 2^-9 relative, well inside half the 0.8 % between neighbours)
      all_vals = O.silu(table.astype(np.float64))
      got_bucket = np.abs(out[:, None] - all_vals[None, :]).argmin(axis=1)
      bad = np.nonzero(got_bucket != want_bucket)[0]
      assert bad.size == 0, (str(dt_), sign, deltas[bad][:8], got_bucket[bad][:8], want_bucket[bad][:8])


def test_timestamp_spans_sorted_unsorted_and_huge(gpu):
  # sequences whose time span fits 31 bits (sorted and shuffled) next to ones whose span does not:
  # each goes down a different timestamp path of the bf16 kernel, all must match the oracle
  rng = np.random.default_rng(41)
  B, L, H, d = 6, 300, 2, 64
  lens = np.array([300, 257, 96, 300, 33, 180], dtype=np.int32)
  q, k, v = (O.round_bf16(rng.standard_normal((B, L, H, d)).astype(np.float32) * 0.2) for _ in range(3))
  ts = 1_600_000_000 + np.cumsum(np.ceil(rng.exponential(3600.0, (B, L))), axis=1).astype(np.int64)
  ts[1] = rng.permutation(ts[1])                       # unsorted: keys later than the query exist
  ts[2] = -5_000_000_000 + ts[2] * 40                  # span of 96 * 3600 * 40 < 2^31, negative origin
  ts[3, 150:] += 3_000_000_000                         # span > 2^31
  ts[4] = rng.integers(-2**40, 2**40, L)               # huge, unsorted
  ts[5] = ts[5, 0]                                     # all equal
  tab = (rng.standard_normal((H, 129)) * 0.5).astype(np.float32)
  pos = (rng.standard_normal((2 * L - 1,)) * 0.1).astype(np.float32)
  ref = O.hstu_attention_ref(q, k, v, seq_lens=lens, pos_tab=pos, timestamps=ts, ts_tab=tab, dtype=np.float32)
  out = recml_amd.hstu_attention(_dev(q, torch.bfloat16), _dev(k, torch.bfloat16), _dev(v, torch.bfloat16),
                                 seq_lens=_dev(lens), pos_bias=_dev(pos), timestamps=_dev(ts), ts_bias=_dev(tab))
  assert _err(out.float().cpu().numpy(), ref) <= BF16_TOL
  qj, off = O.padded_to_jagged(q, lens)
  kj, _ = O.padded_to_jagged(k, lens)
  vj, _ = O.padded_to_jagged(v, lens)
  tsj = np.concatenate([ts[b, :lens[b]] for b in range(B)])
  # jagged timestamps end at the sequence: the last row's "next" timestamp is its own
  refj = O.hstu_attention_jagged_ref(qj, kj, vj, off, L, pos_tab=pos, timestamps=tsj, ts_tab=tab, dtype=np.float32)
  outj = recml_amd.hstu_attention(_dev(qj, torch.bfloat16), _dev(kj, torch.bfloat16), _dev(vj, torch.bfloat16),
                                  seq_offsets=_dev(off.astype(np.int32)), max_len=L, pos_bias=_dev(pos),
                                  timestamps=_dev(tsj), ts_bias=_dev(tab))
  assert _err(outj.float().cpu().numpy(), refj) <= BF16_TOL


def _quant(x):
  """Per-head float8_e4m3fn quantisation on the host: (fp8 tensor on the GPU, scales, dequantised fp32)."""
  xq, scale = O.quantize_e4m3fn_per_head(x)
  dev8 = torch.from_numpy(xq).to("cuda:0").to(torch.float8_e4m3fn)   # exact: xq is representable
  return dev8, _dev(scale), xq * scale[:, None]


@pytest.mark.parametrize("d", [32, 64, 128])
def test_fp8_qk_against_dequantised_oracle(gpu, d):
  rng = np.random.default_rng(50 + d)
  B, L, H = 3, 200, 2
  lens = np.array([200, 77, 129], dtype=np.int32)
  q, k = (rng.standard_normal((B, L, H, d)).astype(np.float32) * 0.3 for _ in range(2))
  v = O.round_bf16(rng.standard_normal((B, L, H, d)).astype(np.float32) * 0.3)
  pos = (rng.standard_normal((H, 2 * L - 1)) * 0.1).astype(np.float32)
  ts = 1_600_000_000 + np.cumsum(np.ceil(rng.exponential(3600.0, (B, L))), axis=1).astype(np.int64)
  tab = (rng.standard_normal((H, 129)) * 0.2).astype(np.float32)
  q8, qs, qd = _quant(q)
  k8, ks, kd = _quant(k)
  # the kernel's error alone: oracle on exactly the values the kernel multiplies
  ref = O.hstu_attention_ref(qd, kd, v, seq_lens=lens, pos_tab=pos, timestamps=ts, ts_tab=tab, dtype=np.float32)
  out = recml_amd.hstu_attention(q8, k8, _dev(v, torch.bfloat16), q_scale=qs, k_scale=ks, seq_lens=_dev(lens),
                                 pos_bias=_dev(pos), timestamps=_dev(ts), ts_bias=_dev(tab))
  assert out.dtype == torch.bfloat16
  out = out.float().cpu().numpy()
  assert _err(out, ref) <= BF16_TOL
  for b in range(B):
    assert (out[b, lens[b]:] == 0).all()
  # against the unquantised inputs: the quantisation error itself (reported, loosely bounded)
  full = O.hstu_attention_ref(q, k, v, seq_lens=lens, pos_tab=pos, timestamps=ts, ts_tab=tab, dtype=np.float32)
  assert _err(out, full) <= 0.15
  # jagged, no bias, non-causal
  qj8 = torch.cat([q8[b, :lens[b]] for b in range(B)])
  kj8 = torch.cat([k8[b, :lens[b]] for b in range(B)])
  vj, off = O.padded_to_jagged(v, lens)
  outj = recml_amd.hstu_attention(qj8, kj8, _dev(vj, torch.bfloat16), q_scale=qs, k_scale=ks,
                                  seq_offsets=_dev(off.astype(np.int32)), max_len=L, causal=False)
  refj = O.hstu_attention_ref(qd, kd, v, seq_lens=lens, causal=False, dtype=np.float32)
  assert _err(O.jagged_to_padded(outj.float().cpu().numpy(), off, L), refj) <= BF16_TOL


def test_fp8_argument_errors(gpu):
  z8 = torch.zeros((2, 8, 2, 32), device="cuda:0").to(torch.float8_e4m3fn)
  zb = torch.zeros((2, 8, 2, 32), device="cuda:0", dtype=torch.bfloat16)
  with pytest.raises(ValueError, match="bfloat16 v"):
    recml_amd.hstu_attention(z8, z8, z8)
  with pytest.raises(ValueError, match="matrix-core"):
    recml_amd.hstu_attention(z8, z8, zb, bias=torch.zeros((2, 8, 8), device="cuda:0"))
  with pytest.raises(ValueError, match="q_scale"):
    recml_amd.hstu_attention(zb, zb, zb, q_scale=torch.ones(2, device="cuda:0"))
  assert recml_amd.hstu_attention(z8, z8, zb).abs().max().item() == 0.0
  assert recml_amd.hstu_attention(z8, z8, zb, sliding_window_size=2).abs().max().item() == 0.0


def test_argument_errors(gpu):
  z = torch.zeros((2, 8, 2, 32), device="cuda:0")
  seg = torch.ones((2, 8), dtype=torch.int32, device="cuda:0")
  with pytest.raises(ValueError, match="Both or neither"):
    recml_amd.pointwise_splash_attention("causal", z, z, z, q_segment_ids=seg)
  with pytest.raises(ValueError, match="Mask shape"):
    recml_amd.pointwise_splash_attention(np.ones((7, 8), bool), z, z, z)
  with pytest.raises(ValueError, match="Unsupported mask type"):
    recml_amd.pointwise_splash_attention("banded", z, z, z)
  with pytest.raises(ValueError):
    recml_amd.hstu_attention(z, z[:, :, :1], z)
  with pytest.raises(ValueError):
    recml_amd.hstu_attention(z.cpu(), z, z)
  with pytest.raises(ValueError):
    recml_amd.hstu_attention(z.double(), z.double(), z.double())


@pytest.mark.parametrize("d,L,window,causal,pos", [
    (128, 400, 0, True, False),       # the diagonal only
    (128, 400, 37, True, True),
    (128, 400, 150, False, True),     # the band reaches over several tiles on both sides
    (64, 300, 31, False, False),
    (32, 520, 260, True, True),
])
def test_sliding_window_on_the_matrix_core_kernel(gpu, d, L, window, causal, pos):
  """|i - j| <= window under the bf16 matrix-core kernel: steps outside the band are skipped,
  blocks on its edges masked (the window rule itself is the oracle's reading of jax's LocalMask)."""
  rng = np.random.default_rng(100 + window)
  B, H = 3, 2
  lens = np.array([L, L // 2 + 3, 1], dtype=np.int32)
  q, k, v = (O.round_bf16(rng.standard_normal((B, L, H, d)).astype(np.float32) * 0.3) for _ in range(3))
  kw, gk = {}, {}
  if pos:
    kw["pos_tab"] = (rng.standard_normal((H, 2 * L - 1)) * 0.1).astype(np.float32)
    gk["pos_bias"] = _dev(kw["pos_tab"])
  ref = O.hstu_attention_ref(q, k, v, seq_lens=lens, causal=causal, sliding_window_size=window, dtype=np.float32, **kw)
  bf = torch.bfloat16
  a, keep = hstu_ops.build_args(_dev(q, bf), _dev(k, bf), _dev(v, bf), torch.empty((B, L, H, d), dtype=bf, device="cuda:0"),
                                seq_lens=_dev(lens), causal=causal, sliding_window_size=window, **gk)
  assert hstu_ops.kernel_variant(a) == "hstu_fwd_mfma_bf16"
  hstu_ops._run(a, keep)
  out = keep[3].float().cpu().numpy()
  assert _err(out, ref) <= BF16_TOL
  for b in range(B):
    assert (out[b, lens[b]:] == 0).all()
  # jagged layout, same values
  (qj, off), (kj, _), (vj, _) = (O.padded_to_jagged(x, lens) for x in (q, k, v))
  outj = recml_amd.hstu_attention(_dev(qj, bf), _dev(kj, bf), _dev(vj, bf), seq_offsets=_dev(off.astype(np.int32)), max_len=L,
                                  causal=causal, sliding_window_size=window, **gk)
  assert _err(O.jagged_to_padded(outj.float().cpu().numpy(), off, L), ref) <= BF16_TOL


@pytest.mark.parametrize("window", [399, 400, 5000, 2 ** 31 - 1, 2 ** 40])
def test_sliding_window_that_covers_everything(gpu, window):
  """A window that reaches across the whole sequence restricts nothing (the reference's LocalMask
  treats it so): same output as without a window, in both kernels, up to the largest values."""
  rng = np.random.default_rng(7)
  B, L, H, d = 2, 400, 2, 64
  lens = np.array([L, 123], dtype=np.int32)
  q, k, v = (O.round_bf16(rng.standard_normal((B, L, H, d)).astype(np.float32) * 0.3) for _ in range(3))
  for dt_ in (torch.bfloat16, torch.float32):
    for causal in (True, False):
      run = lambda **kw: recml_amd.hstu_attention(_dev(q, dt_), _dev(k, dt_), _dev(v, dt_), seq_lens=_dev(lens), causal=causal, **kw)
      plain, win = run(), run(sliding_window_size=window)
      assert float(plain.float().abs().max()) > 0
      if window >= L:
        assert torch.equal(plain, win), (str(dt_), causal)        # passed on as "no window": the very same launch
      else:
        # the widest real window keeps every pair too; the window path sums a long tile in one piece
        # where the plain path may split its keys: equal up to the rounding of the output
        tol = 2.0 ** -7 if dt_ == torch.bfloat16 else 1e-6
        assert float((plain.float() - win.float()).abs().max()) <= tol * float(plain.float().abs().max()), (str(dt_), causal)


@pytest.mark.parametrize("d,L,causal,window,pos", [
    (128, 400, True, None, False),
    (128, 400, True, 50, True),
    (64, 260, False, None, True),
    (32, 132, True, None, False),
])
def test_segment_ids_on_the_matrix_core_kernel(gpu, d, L, causal, window, pos):
  """Packed rows: several segments per row plus a padding segment (the reference's test recipe,
  hstu_ops_test.py:36-41, has two), bf16 on the matrix-core kernel."""
  rng = np.random.default_rng(300 + L)
  B, H = 3, 2
  bf = torch.bfloat16
  q, k, v = (O.round_bf16(rng.standard_normal((B, L, H, d)).astype(np.float32) * 0.3) for _ in range(3))
  seg = np.zeros((B, L), np.int32)
  seg[0, :L // 3], seg[0, L // 3: L - 7] = 1, 2            # two sequences and a short padding tail
  seg[1, :] = 5                                             # one sequence over the whole row
  cuts = np.sort(rng.choice(np.arange(1, L), 9, replace=False))
  seg[2] = np.searchsorted(cuts, np.arange(L), side="right") + 1   # ten short ones
  kw, gk = {}, {}
  if pos:
    kw["pos_tab"] = (rng.standard_normal((H, 2 * L - 1)) * 0.1).astype(np.float32)
    gk["pos_bias"] = _dev(kw["pos_tab"])
  ref = O.hstu_attention_ref(q, k, v, causal=causal, q_segment_ids=seg, kv_segment_ids=seg,
                             sliding_window_size=window, dtype=np.float32, **kw)
  a, keep = hstu_ops.build_args(_dev(q, bf), _dev(k, bf), _dev(v, bf), torch.empty((B, L, H, d), dtype=bf, device="cuda:0"),
                                causal=causal, q_segment_ids=_dev(seg), kv_segment_ids=_dev(seg),
                                sliding_window_size=window, **gk)
  assert hstu_ops.kernel_variant(a) == "hstu_fwd_mfma_bf16"
  hstu_ops._run(a, keep)
  assert _err(keep[3].float().cpu().numpy(), ref) <= BF16_TOL


def _random_case(seed):
  rng = np.random.default_rng(seed)
  d = int(rng.choice([32, 64, 128]))
  H = int(rng.choice([1, 2, 4, 8, 16]))
  L = int(rng.choice([36, 100, 128, 132, 260, 300]))
  B = int(rng.integers(1, 5))
  causal = bool(rng.integers(0, 2))
  window = None if rng.random() < 0.6 else int(rng.integers(0, L))
  seg = L % 4 == 0 and rng.random() < 0.3
  jagged = (not seg) and rng.random() < 0.5
  pos = rng.random() < 0.5
  ts = rng.random() < 0.5
  lens = rng.integers(1, L + 1, B).astype(np.int32)
  lens[rng.integers(0, B)] = L
  return dict(d=d, H=H, L=L, B=B, causal=causal, window=window, seg=seg, jagged=jagged, pos=pos, ts=ts, lens=lens, rng=rng)


@pytest.mark.parametrize("seed", list(range(1000, 1024)))
def test_matrix_core_forward_on_random_option_mixes(gpu, seed):
  """bf16 forward against the oracle over random mixes of head dim, heads, layout, causal / full,
  window, segment ids and the two biases (fixed seeds; every mix stays on the matrix-core kernel)."""
  c = _random_case(seed)
  rng, B, L, H, d, lens = c["rng"], c["B"], c["L"], c["H"], c["d"], c["lens"]
  bf = torch.bfloat16
  q, k, v = (O.round_bf16(rng.standard_normal((B, L, H, d)).astype(np.float32) * 0.3) for _ in range(3))
  kw, gk = dict(causal=c["causal"]), dict(causal=c["causal"])
  if c["window"] is not None:
    kw["sliding_window_size"] = gk["sliding_window_size"] = c["window"]
  if c["pos"]:
    heads = H if rng.random() < 0.5 else 1
    kw["pos_tab"] = (rng.standard_normal((heads, 2 * L - 1)) * 0.2).astype(np.float32)
    gk["pos_bias"] = _dev(kw["pos_tab"])
  t = None
  if c["ts"]:
    heads = H if rng.random() < 0.5 else 1
    kw["ts_tab"] = (rng.standard_normal((heads, 65)) * 0.2).astype(np.float32)
    t = 1_700_000_000 + np.cumsum(np.ceil(rng.exponential(5000.0, (B, L))), axis=1).astype(np.int64)
    for b in range(B):
      t[b, lens[b]:] = t[b, lens[b] - 1]
    kw["timestamps"] = t
    gk["ts_bias"] = _dev(kw["ts_tab"])
  if c["seg"]:
    cuts = np.sort(rng.choice(np.arange(1, L), 3, replace=False))
    seg = np.tile(np.searchsorted(cuts, np.arange(L), side="right").astype(np.int32), (B, 1))
    kw["q_segment_ids"] = kw["kv_segment_ids"] = seg
    gk["q_segment_ids"] = gk["kv_segment_ids"] = _dev(seg)
    lens = np.full((B,), L, np.int32)
  else:
    kw["seq_lens"] = lens
  ref = O.hstu_attention_ref(q, k, v, dtype=np.float32, **kw)
  if c["jagged"]:
    (qj, off), (kj, _), (vj, _) = (O.padded_to_jagged(x, lens) for x in (q, k, v))
    if t is not None:
      gk["timestamps"] = _dev(np.concatenate([t[b, :lens[b]] for b in range(B)]))
    a, keep = hstu_ops.build_args(_dev(qj, bf), _dev(kj, bf), _dev(vj, bf), torch.empty((qj.shape[0], H, d), dtype=bf, device="cuda:0"),
                                  seq_offsets=_dev(off.astype(np.int32)), max_len=L, **gk)
  else:
    if t is not None:
      gk["timestamps"] = _dev(t)
    if not c["seg"]:
      gk["seq_lens"] = _dev(lens)
    a, keep = hstu_ops.build_args(_dev(q, bf), _dev(k, bf), _dev(v, bf), torch.empty((B, L, H, d), dtype=bf, device="cuda:0"), **gk)
  assert hstu_ops.kernel_variant(a) == "hstu_fwd_mfma_bf16", c
  hstu_ops._run(a, keep)
  out = keep[3].float().cpu().numpy()
  if c["jagged"]:
    out = O.jagged_to_padded(out, off, L)
  err = np.abs(out - ref).max(axis=(2, 3)) / max(np.abs(ref).max(), 1e-30)
  assert err.max() <= BF16_TOL, (c, err.max())
  for b in range(B):
    assert (out[b, lens[b]:] == 0).all()


@pytest.mark.parametrize("seed", list(range(3000, 3016)))
def test_matrix_core_forward_on_random_dense_and_cross_length_mixes(gpu, seed):
  """bf16 forward against the oracle over random mixes of dense mask / dense bias (shared or per
  sequence), different key and query lengths, causal / full, window, lengths, head dim and heads
  (fixed seeds; every mix stays on the matrix-core kernel)."""
  rng = np.random.default_rng(seed)
  B = int(rng.integers(1, 5))
  H = int(rng.choice([1, 2, 3, 4, 8]))
  d = int(rng.choice([32, 64, 128]))
  Lq = 16 * int(rng.integers(1, 40))
  cross = rng.random() < 0.4
  Lk = 16 * int(rng.integers(1, 40)) if cross else Lq
  use_mask = rng.random() < 0.6
  use_bias = rng.random() < 0.6
  if not (use_mask or use_bias or cross):
    use_bias = True
  causal = bool(rng.random() < 0.5)
  window = int(rng.integers(0, 200)) if rng.random() < 0.3 else None
  q = O.round_bf16(rng.standard_normal((B, Lq, H, d)).astype(np.float32) * 0.3)
  k = O.round_bf16(rng.standard_normal((B, Lk, H, d)).astype(np.float32) * 0.3)
  v = O.round_bf16(rng.standard_normal((B, Lk, H, d)).astype(np.float32) * 0.3)
  kw, gk = dict(causal=causal), dict(causal=causal)
  if window is not None:
    kw["sliding_window_size"] = gk["sliding_window_size"] = window
  if use_mask:
    batched = rng.random() < 0.5
    m = rng.random((B, Lq, Lk) if batched else (Lq, Lk)) < rng.choice([0.1, 0.5, 0.9])
    if rng.random() < 0.3:
      m[..., : Lq // 2, :] = False          # whole tiles masked out: the kernel skips their blocks
    kw["mask"] = m
    gk["mask"] = _dev(m.astype(np.uint8))
  if use_bias:
    batched = rng.random() < 0.5 and B > 1
    bias = (rng.standard_normal((B, Lq, Lk) if batched else (1, Lq, Lk)) * 0.5).astype(np.float32)
    kw["bias"] = bias
    gk["bias"] = _dev(bias)
  lens = None
  if not cross and rng.random() < 0.5:
    lens = rng.integers(1, Lq + 1, B).astype(np.int32)
    kw["seq_lens"] = lens
    gk["seq_lens"] = _dev(lens)
  case = dict(seed=seed, B=B, H=H, d=d, Lq=Lq, Lk=Lk, mask=use_mask, bias=use_bias, causal=causal, window=window, lens=lens)
  bf = torch.bfloat16
  out = torch.full((B, Lq, H, d), float("nan"), dtype=bf, device="cuda:0")
  a, keep = hstu_ops.build_args(_dev(q, bf), _dev(k, bf), _dev(v, bf), out, n=Lq, alpha=0.2, **gk)
  assert hstu_ops.kernel_variant(a) == "hstu_fwd_mfma_bf16", case
  hstu_ops._run(a, keep)
  torch.cuda.synchronize()
  ref = O.hstu_attention_ref(q, k, v, n=Lq, alpha=0.2, dtype=np.float32, **kw)
  got = out.float().cpu().numpy()
  assert np.isfinite(got).all(), case
  assert _err(got, ref) <= BF16_TOL, (case, _err(got, ref))
  if lens is not None:
    for b in range(B):
      assert (got[b, lens[b]:] == 0).all(), case


@pytest.mark.parametrize("seed", list(range(4000, 4016)))
def test_general_kernel_on_random_option_mixes(gpu, seed):
  """fp32 storage (the general kernel) against the oracle over random mixes of every option at once: lengths or
  segment ids, explicit mask, dense bias, both table biases, window, causal / full, different key and query
  lengths, odd head dims (fixed seeds)."""
  rng = np.random.default_rng(seed)
  B = int(rng.integers(1, 4))
  H = int(rng.integers(1, 4))
  d = int(rng.choice([8, 24, 32, 48, 72]))
  dv = d if rng.random() < 0.7 else int(rng.choice([8, 40]))
  Lq = int(rng.integers(1, 90))
  cross = rng.random() < 0.3
  Lk = int(rng.integers(1, 90)) if cross else Lq
  causal = bool(rng.random() < 0.5)
  q = rng.standard_normal((B, Lq, H, d)).astype(np.float32) * 0.5
  k = rng.standard_normal((B, Lk, H, d)).astype(np.float32) * 0.5
  v = rng.standard_normal((B, Lk, H, dv)).astype(np.float32) * 0.5
  kw, gk = dict(causal=causal), dict(causal=causal)
  if rng.random() < 0.4:
    kw["sliding_window_size"] = gk["sliding_window_size"] = int(rng.integers(0, 40))
  if rng.random() < 0.5:
    batched = rng.random() < 0.5
    m = rng.random((B, Lq, Lk) if batched else (Lq, Lk)) < 0.6
    kw["mask"], gk["mask"] = m, _dev(m.astype(np.uint8))
  if rng.random() < 0.5:
    batched = rng.random() < 0.5 and B > 1
    bias = (rng.standard_normal((B, Lq, Lk) if batched else (1, Lq, Lk)) * 0.5).astype(np.float32)
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
    heads = H if rng.random() < 0.5 else 1
    kw["pos_tab"] = (rng.standard_normal((heads, 2 * Lq - 1)) * 0.3).astype(np.float32)
    gk["pos_bias"] = _dev(kw["pos_tab"])
  t = None
  if not cross and rng.random() < 0.5:
    heads = H if rng.random() < 0.5 else 1
    nb = int(rng.choice([16, 64, 128]))
    kw["ts_tab"] = (rng.standard_normal((heads, nb + 1)) * 0.3).astype(np.float32)
    t = 1_700_000_000 + np.cumsum(np.ceil(rng.exponential(3000.0, (B, Lq))), axis=1).astype(np.int64)
    kw["timestamps"] = t
    gk["ts_bias"], gk["timestamps"] = _dev(kw["ts_tab"]), _dev(t)
  out = torch.full((B, Lq, H, dv), float("nan"), dtype=torch.float32, device="cuda:0")
  a, keep = hstu_ops.build_args(_dev(q), _dev(k), _dev(v), out, n=7.0, alpha=0.3, **gk)
  assert hstu_ops.kernel_variant(a) == "hstu_fwd_general<float>"
  hstu_ops._run(a, keep)
  torch.cuda.synchronize()
  ref = O.hstu_attention_ref(q, k, v, n=7.0, alpha=0.3, **kw)
  got = out.cpu().numpy()
  case = dict(seed=seed, B=B, H=H, d=d, dv=dv, Lq=Lq, Lk=Lk, causal=causal, keys=sorted(kw))
  assert np.isfinite(got).all(), case
  err = np.abs(got - ref).max(axis=(2, 3)) / max(np.abs(ref).max(), 1e-30)
  assert err.max(initial=0.0) <= FP32_TOL, (case, err.max(initial=0.0))
  if lens is not None:
    for b in range(B):
      assert (got[b, lens[b]:] == 0).all(), case


@pytest.mark.parametrize("d,dv", [(1, 1), (3, 5), (20, 20), (36, 100), (100, 36), (128, 128), (129, 64), (160, 160),
                                  (200, 256), (256, 256)])
@pytest.mark.parametrize("storage", ["fp32", "fp32 views", "bf16"])
def test_general_kernel_head_dims_and_storage(gpu, d, dv, storage):
  """The general kernel over head dims that are no multiple of 4 or 16, differ between q/k and v, or go beyond 128
  (its Q rows then sit in LDS and a workgroup takes fewer rows), with rows that allow 16-byte loads, rows that do
  not (views with an odd offset and stride), and bf16 storage; several 128-row tiles, a partial last key tile,
  lengths, causal, a position table."""
  rng = np.random.default_rng(4700 + 7 * d + dv)
  B, L, H = 2, 300, 2
  lens = np.array([300, 77], dtype=np.int32)
  mk = lambda dd: rng.standard_normal((B, L, H, dd)).astype(np.float32) * 0.4
  q, k, v = mk(d), mk(d), mk(dv)
  pos = (rng.standard_normal((H, 2 * L - 1)) * 0.3).astype(np.float32)
  if storage == "bf16":
    q, k, v = (O.round_bf16(t) for t in (q, k, v))
    dt = torch.bfloat16
  else:
    dt = torch.float32
  def place(t):
    x = _dev(t, dt)
    if storage != "fp32 views":
      return x
    # the same values inside a larger buffer: every row starts at an odd element offset
    buf = torch.zeros((B, L, H, t.shape[-1] + 3), dtype=dt, device="cuda:0")
    buf[..., 1:1 + t.shape[-1]] = x
    return buf[..., 1:1 + t.shape[-1]]
  qd, kd, vd = place(q), place(k), place(v)
  out = torch.full((B, L, H, dv), float("nan"), dtype=dt, device="cuda:0")
  a, keep = hstu_ops.build_args(qd, kd, vd, out, n=float(L), alpha=0.25, causal=True, seq_lens=_dev(lens), pos_bias=_dev(pos))
  variant = hstu_ops.kernel_variant(a)
  if storage == "bf16" and d == dv and d == 128:
    assert variant == "hstu_fwd_mfma_bf16"       # (the one case here that the bf16 matrix-core kernel takes)
  else:
    assert variant.startswith("hstu_fwd_general")
  hstu_ops._run(a, keep)
  torch.cuda.synchronize()
  got = out.float().cpu().numpy()
  ref = O.hstu_attention_ref(q, k, v, n=float(L), alpha=0.25, causal=True, seq_lens=lens, pos_tab=pos)
  tol = FP32_TOL if storage != "bf16" else BF16_TOL
  assert np.isfinite(got).all()
  assert np.abs(got - ref).max() <= tol * np.abs(ref).max()
  assert (got[1, 77:] == 0).all()
