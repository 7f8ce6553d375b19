"""Benchmark of the HSTU attention forward on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c3|c3full|c2|c4|c5|c4-model|c4-block-steps] [--backward]

A step is one pass of the attention forward over one synthetic batch whose
inputs already sit in HBM.  The default workload is the one the headline
metric is quoted on: B=64, max_len=2048, H=8, d=128 bf16, jagged power-law
lengths, relative-position + timestamp bias, N=2048.  Prints ONE JSON line.

FLOPs counted: sum_b H * n_b(n_b+1)/2 * (2 d_qk + 2 d_v) (unmasked causal
pairs only; bias, SiLU and mask are not counted).

`value` and `ms_per_step` are the whole call (preparation kernel + attention
kernel) over K back-to-back steps.  `roofline.achieved` is the attention
kernel alone: the same K launches timed one by one with HIP events with the
preparation kernel skipped (its results are still in the workspace).
`roofline.step_ms_cold_avg` is the whole call after a 1 GiB fill has pushed
the inputs out of the caches.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
  sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_FP8_TFLOPS = 5000.0    # MI355X dense fp8 MFMA
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E


def make_workload(name):
  from recml_amd import workloads
  if name == "c3":
    return workloads.config3()
  if name == "c3full":
    return workloads.config3(full=True)
  if name == "c3full-nobias":
    return workloads.config3(full=True, bias=False)
  if name == "c3-nobias":
    return workloads.config3(bias=False)
  if name in ("c3full-ts", "c3full-pos", "c3-ts", "c3-pos"):
    # one bias only (profiling aid)
    w = workloads.config3(full=name.startswith("c3full"))
    if name.endswith("-ts"):
      w.pos_tab = None
    else:
      w.ts_tab = None
      w.timestamps = None
    return w
  if name == "c2":
    return workloads.config2()
  if name == "c4":
    return workloads.config4_attention()
  if name == "c5":
    return workloads.config5()
  if name == "c5-bf16":
    return workloads.config5(fp8=False)
  raise SystemExit(f"unknown workload {name}")


def to_device(w, dev):
  import torch
  t = lambda x: None if x is None else torch.from_numpy(np.ascontiguousarray(x)).to(dev)
  q, k, v = (t(x) for x in (w.q, w.k, w.v))
  kw = dict(n=w.n, alpha=w.alpha, pos_bias=t(w.pos_tab), ts_bias=t(w.ts_tab),
            timestamps=t(w.timestamps))
  if w.dtype == "fp8":
    # per-head symmetric quantisation of q and k: scale = amax / 448
    def quant(x):
      scale = x.abs().amax(dim=tuple(i for i in range(x.dim()) if i != x.dim() - 2)).clamp_min(1e-30) / 448.0
      return (x / scale[:, None]).to(torch.float8_e4m3fn), scale
    (q, qs), (k, ks) = quant(q), quant(k)
    kw.update(q_scale=qs, k_scale=ks)
    v = v.to(torch.bfloat16)
  else:
    q, k, v = (x.to(torch.bfloat16) for x in (q, k, v))
  if w.layout == "jagged":
    kw.update(seq_offsets=t(w.seq_offsets), max_len=w.L)
  else:
    kw.update(seq_lens=t(w.seq_lens))
  return q, k, v, kw


def cpu_baseline(w, q, k, v, out_gpu, dev_kw):
  """The C restatement of the op (oracle/hstu_oracle.c, float accumulation,
  OpenMP over sequence x head) timed on this host, and used as the checker."""
  from oracle import c_oracle
  threads = c_oracle.max_threads()
  qf, kf, vf = (x.float().cpu().numpy() for x in (q, k, v))
  if w.dtype == "fp8":   # the checker works on the dequantised inputs the kernel sees
    qf = qf * dev_kw["q_scale"].cpu().numpy()[:, None]
    kf = kf * dev_kw["k_scale"].cpu().numpy()[:, None]
  kw = dict(n=w.n, alpha=w.alpha, pos_tab=w.pos_tab, timestamps=w.timestamps,
            ts_tab=w.ts_tab, acc="f32")
  if w.layout == "jagged":
    kw.update(seq_offsets=w.seq_offsets, max_len=w.L)
  else:
    kw.update(seq_lens=w.seq_lens)
  # bounded sample: whole batches until ~10 s or 3 repetitions
  times = []
  ref = None
  t_all = time.perf_counter()
  while len(times) < 3 and time.perf_counter() - t_all < 10.0:
    t0 = time.perf_counter()
    ref = c_oracle.hstu_attention_c(qf, kf, vf, **kw)
    times.append(time.perf_counter() - t0)
  best = min(times)
  err = float(np.abs(out_gpu - ref).max() / max(np.abs(ref).max(), 1e-30))
  return {
      "value": w.flops / best / 1e12, "unit": "TFLOP/s", "cores": threads,
      "kind": "port",
      "port_of": "sparse C restatement of the op (oracle/hstu_oracle.c): per-row loops over the kept keys only, "
                 "no dense L x L tensors; faster than what the reference's CPU path does (see dense_einsum)",
      "sample": f"{len(times)} full batches of the same workload ({w.flops / 1e9:.1f} GFLOP each), "
                f"best of {len(times)}, {best * 1e3:.0f} ms; C restatement with float accumulation, "
                "masked work skipped",
      "seqs_per_s": w.B / best,
      "dense_einsum": dense_einsum_cpu(w, qf, kf, vf),
  }, err


def dense_einsum_cpu(w, qf, kf, vf):
  """What the reference's CPU path computes (recml/layers/keras/hstu.py:371-389): dense [L, L] logits
  by einsum, the bias tensors added, SiLU, / N, times the dense mask, einsum with V -- here in torch
  fp32 on the host cores for one (sequence, head) chunk padded to max_len, the longest sequence of
  the batch.  TFLOP/s counts the chunk's unmasked flops like `value` does."""
  import torch
  b = int(np.argmax(w.seq_lens))
  n_b, L, d = int(w.seq_lens[b]), w.L, w.d
  if w.layout == "jagged":
    o0 = int(w.seq_offsets[b])
    rows = slice(o0, o0 + n_b)
    pad = lambda x: np.concatenate([x[rows, 0], np.zeros((L - n_b, x.shape[-1]), np.float32)])
    ts_b = None if w.timestamps is None else np.concatenate([w.timestamps[rows], np.full(L - n_b, w.timestamps[o0 + n_b - 1])])
  else:
    pad = lambda x: x[b, :, 0]
    ts_b = None if w.timestamps is None else w.timestamps[b]
  q, k, v = (torch.from_numpy(np.ascontiguousarray(pad(x))) for x in (qf, kf, vf))
  pos = None if w.pos_tab is None else torch.from_numpy(w.pos_tab[0].astype(np.float32))
  tab = None if w.ts_tab is None else torch.from_numpy(w.ts_tab[0].astype(np.float32))
  ts = None if ts_b is None else torch.from_numpy(np.ascontiguousarray(ts_b))
  idx = torch.arange(L)
  keep = ((idx[None, :] <= idx[:, None]) & (idx[None, :] < n_b) & (idx[:, None] < n_b)).float()

  def once():
    s = torch.einsum("qd,kd->qk", q, k) * w.alpha
    if pos is not None:
      s = s + pos[(L - 1) + idx[None, :] - idx[:, None]]
    if tab is not None:
      nxt = torch.cat([ts[1:], ts[-1:]])
      dt = (nxt[:, None] - ts[None, :]).abs().clamp(1, 10**9).float()
      bucket = (torch.log(dt) / 0.301).to(torch.int64).clamp(0, tab.numel() - 1)
      s = s + tab[bucket]
    p = torch.nn.functional.silu(s) / w.n * keep
    return torch.einsum("qk,kd->qd", p, v)

  once()
  times = []
  t_all = time.perf_counter()
  while len(times) < 5 and time.perf_counter() - t_all < 5.0:
    t0 = time.perf_counter()
    once()
    times.append(time.perf_counter() - t0)
  best = min(times)
  unmasked = 4.0 * d * (n_b * (n_b + 1) / 2)
  return {"value": unmasked / best / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(),
          "sample": f"one (sequence, head) chunk of the workload padded to {L} x {L} (sequence {b}, {n_b} tokens), "
                    f"torch fp32 on the host, best of {len(times)}: {best * 1e3:.1f} ms; dense flops {4.0 * d * L * L / 1e9:.2f} G, "
                    f"unmasked {unmasked / 1e9:.2f} G",
          "chunk_ms": best * 1e3, "chunks_in_batch": int(w.B * w.H)}


def measured_traffic(workload):
  """HBM bytes per launch from the rocprofv3 counter runs recorded in profiles/traffic.json
  (FETCH_SIZE + WRITE_SIZE of the attention kernel, scaled by a copy kernel of known size)."""
  path = os.path.join(ROOT, "profiles", "traffic.json")
  if not os.path.exists(path):
    return None
  rec = json.load(open(path)).get(workload)
  return None if rec is None else rec["hbm_bytes_per_launch"]


PEAK_FP32_TFLOPS = 157.3    # MI355X dense fp32


def bench_model(args, dev):
  """Config 4 end to end: embedding gather (10 M x 512 bf16 table, Zipf ids) -> 4 HSTU blocks
  (D=512, H=8, head dim 64, position bias) -> final norm, padded [128, 1024] batch with
  lengths U{128..1024}.  torch for everything but the attention.  One JSON line."""
  import torch
  import recml_amd
  rng = np.random.Generator(np.random.PCG64(4))
  B, L, D, H, layers, vocab = 128, 1024, 512, 8, 4, 10_000_000
  lens = rng.integers(128, L + 1, B).astype(np.int32)
  ids = np.minimum(rng.zipf(1.05, (B, L)), vocab - 1).astype(np.int64)
  ids[np.arange(L)[None, :] >= lens[:, None]] = 0
  model = recml_amd.HSTU(vocab_size=8, max_positions=L, model_dim=D, num_heads=H, num_layers=layers, add_head=False,
                         dtype=torch.bfloat16, device=dev, seed=4)
  table = torch.empty((vocab, D), dtype=torch.bfloat16, device=dev)
  table.normal_(0.0, 0.01, generator=torch.Generator(device=dev).manual_seed(4))
  model.item_embedding = torch.nn.Parameter(table, requires_grad=False)
  ids_d = torch.from_numpy(ids).to(dev)
  lens_d = torch.from_numpy(lens).to(dev)
  pos = (torch.randn((2 * L - 1,), generator=torch.Generator().manual_seed(5)) * 0.02).to(dev)
  steps, warm = max(1, args.steps // 10), max(2, args.warmup // 10)
  with torch.no_grad():
    def timed(fn):
      for _ in range(warm):
        o = fn()
      torch.cuda.synchronize()
      t0 = time.perf_counter()
      for _ in range(steps):
        o = fn()
      torch.cuda.synchronize()
      return (time.perf_counter() - t0) * 1e3 / steps, o
    ms, out = timed(lambda: model(ids_d, seq_lens=lens_d, pos_bias=pos))
    ms_jagged, outj = timed(lambda: model(ids_d, seq_lens=lens_d, pos_bias=pos, jagged=True))
    keep = (torch.arange(L, device=dev)[None, :] < lens_d[:, None])[:, :, None]
    jag_err = float(((outj.float() - out.float()) * keep).abs().max() / out.float().abs().max())
    # the attention alone on the same shapes (padded layout with lengths, as the block calls it)
    q = torch.randn((B, L, 4, H, D // H), device=dev, dtype=torch.bfloat16)
    att = lambda: recml_amd.hstu_attention(q[:, :, 1], q[:, :, 2], q[:, :, 3], seq_lens=lens_d, pos_bias=pos)
    for _ in range(warm):
      att()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
      att()
    torch.cuda.synchronize()
    att_ms = (time.perf_counter() - t0) * 1e3 / steps
  assert tuple(out.shape) == (B, L, D) and bool(torch.isfinite(out.float()).all())
  # one training step's forward + backward on packed tokens: the blocks and the position table
  # take gradients (attention through the HIP backward kernels), the embedding table stays frozen
  for blk in model.decoder_blocks:
    blk.requires_grad_(True)
  pos_t = pos.clone().requires_grad_(True)
  dout = torch.randn((B, L, D), generator=torch.Generator().manual_seed(6)).to(dev).to(torch.bfloat16)
  def train_step():
    for prm in model.parameters():
      prm.grad = None
    pos_t.grad = None
    o = model(ids_d, seq_lens=lens_d, pos_bias=pos_t, jagged=True)
    (o * dout).sum().backward()
    return o
  for _ in range(warm):
    train_step()
  torch.cuda.synchronize()
  t0 = time.perf_counter()
  for _ in range(steps):
    train_step()
  torch.cuda.synchronize()
  train_ms = (time.perf_counter() - t0) * 1e3 / steps
  assert bool(torch.isfinite(pos_t.grad).all()) and float(pos_t.grad.abs().max()) > 0
  # the same step with torch left to pick each matrix product's kernel by timing the candidates once
  # (torch.cuda.tunable: the products are torch's, and the library's first choice for the weight
  # gradients' shapes -- a small output, 70 k rows to sum over -- leaves most of the chip idle)
  train_tuned_ms = None
  try:
    if not args.tuned:
      raise RuntimeError("switched off (--no-tuned-products)")
    import torch.cuda.tunable as tunable
    import tempfile
    tunable.enable(True)
    tunable.set_filename(os.path.join(tempfile.gettempdir(), "recml_amd_bench_tuned_products.csv"))   # (it writes its choices at exit)
    tunable.set_max_tuning_duration(15)
    tunable.set_max_tuning_iterations(10)
    for _ in range(warm):
      train_step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
      train_step()
    torch.cuda.synchronize()
    train_tuned_ms = (time.perf_counter() - t0) * 1e3 / steps
    tunable.enable(False)
  except Exception as e:   # an older torch without the module, or a tuning failure: the plain figure stands
    print(f"tunable products not measured: {e}", file=sys.stderr)
  nn = lens.astype(np.int64)
  attn_flops = int((H * (nn * (nn + 1) // 2) * 4 * (D // H)).sum()) * layers
  proj_flops = B * L * (2 * D * 4 * D + 2 * D * D) * layers
  print(json.dumps({
      "metric": "HSTU 4-layer forward (config 4), sequences/s", "value": B / (ms * 1e-3), "unit": "seqs/s", "n_gpus": 1,
      "steps": steps, "warmup": warm, "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
      "dtype": "bf16", "data": "synthetic",
      "config": {"workload": f"C4 model: B={B} L={L} D={D} H={H} layers={layers} vocab={vocab} lens U{{128..1024}}, padded, pos bias, no head"},
      "ms_per_step_packed_tokens": ms_jagged, "seqs_per_s_packed_tokens": B / (ms_jagged * 1e-3),
      "packed_vs_padded_max_abs_over_max": jag_err,
      "train_fwd_bwd_ms_packed_tokens": train_ms,
      "train_fwd_bwd_ms_packed_tokens_tuned_products": train_tuned_ms,
      "attention_ms_per_layer": att_ms, "attention_share": layers * att_ms / ms,
      "attention_gflop_unmasked": attn_flops / 1e9, "projection_gflop_padded": proj_flops / 1e9,
      "model_tflops": (attn_flops + proj_flops) / (ms * 1e-3) / 1e12}))


def bench_block_steps(args, dev):
  """The two fused block steps at the config-4 size (T = 73 728 packed tokens, D = 512): one JSON line.

  value / roofline: the norm + gate step, which is bound by HBM (3 x T x D x 2 bytes: the attention
  output and the U slice read once, the result written once); the projection product with the SiLU
  epilogue is reported beside it in TFLOP/s."""
  import torch
  import recml_amd
  from oracle import hstu_block_oracle as BO
  T, D = 73728, 512
  bf = torch.bfloat16
  gen = torch.Generator(device=dev).manual_seed(7)
  fused = torch.randn((T, 4, D), device=dev, dtype=bf, generator=gen)
  u = fused[:, 0]
  attn = (torch.randn((T, D), device=dev, generator=gen) * 1e-3).to(bf)
  gamma = (1 + 0.1 * torch.randn(D, device=dev, generator=gen)).to(bf)
  beta = (0.1 * torch.randn(D, device=dev, generator=gen)).to(bf)
  x = (torch.randn((T, D), device=dev, generator=gen) * 0.5).to(bf)
  w = (torch.randn((D, 4 * D), device=dev, generator=gen) * 0.05).to(bf)

  def timed(fn):
    for _ in range(args.warmup):
      fn()
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for a, b in ev:
      a.record()
      fn()
      b.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / args.steps
    return wall, float(np.mean([a.elapsed_time(b) for a, b in ev]))

  ng = lambda: recml_amd.norm_gate(attn, u, gamma, beta, 1e-6)
  wall_ng, ker_ng = timed(ng)
  wall_t, _ = timed(lambda: u * torch.nn.functional.layer_norm(attn, (D,), gamma, beta, 1e-6))
  wall_g, ker_g = timed(lambda: recml_amd.gemm_silu(x, w, None, True))
  wall_gt, _ = timed(lambda: torch.nn.functional.silu(x @ w))
  # the same step's gradients (training): 5 x T x D x 2 bytes (row, gate and gradient in; d_attn and d_u out),
  # d_u into a slice of a projection-shaped tensor as the block's backward has it; and torch's autograd of the same
  from recml_amd import hstu_block_ops
  dout = torch.randn((T, D), device=dev, dtype=bf, generator=gen)
  dfused = torch.empty_like(fused)
  wall_nb, ker_nb = timed(lambda: hstu_block_ops.norm_gate_bwd(attn, u, gamma, beta, dout, 1e-6, du_out=dfused[:, 0]))
  leaves = [t.detach().clone().requires_grad_(True) for t in (attn, u.contiguous(), gamma, beta)]
  def torch_bwd():
    for t in leaves:
      t.grad = None
    (leaves[1] * torch.nn.functional.layer_norm(leaves[0], (D,), leaves[2], leaves[3], 1e-6)).backward(dout)
  wall_nbt, _ = timed(torch_bwd)
  # the front end: 10 M x 512 table, Zipf(1.05) ids as in the model workload, position table of 1024 rows
  vocab = 10_000_000
  table = torch.empty((vocab, D), dtype=bf, device=dev)
  table.normal_(0.0, 0.01, generator=gen)
  rng = np.random.Generator(np.random.PCG64(4))
  ids = torch.from_numpy(np.minimum(rng.zipf(1.05, T), vocab - 1).astype(np.int64)).to(dev)
  pos_table = (torch.randn((1024, D), device=dev, generator=gen) * 0.01).to(bf)
  positions = torch.from_numpy(rng.integers(0, 1024, T).astype(np.int64)).to(dev)
  wall_e, ker_e = timed(lambda: recml_amd.embed_norm(ids, table, gamma, beta, 1e-6, positions=positions, pos_table=pos_table))
  wall_et, _ = timed(lambda: torch.nn.functional.layer_norm(table[ids] + pos_table[positions], (D,), gamma, beta, 1e-6))
  uniq = int(torch.unique(ids).numel())
  nbytes = 3 * T * D * 2
  gflop = 2.0 * T * D * 4 * D / 1e9
  out = ng().float().cpu().numpy()
  rec = {
      "metric": "HSTU block norm + gate step, GB/s (config-4 size)", "value": nbytes / (wall_ng * 1e-3) / 1e9, "unit": "GB/s",
      "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": wall_ng, "higher_is_better": True,
      "scaling": "weak", "vs_baseline": None, "dtype": "bf16 storage, fp32 arithmetic", "data": "synthetic",
      "config": {"workload": f"C4 block steps: T={T} packed tokens, D={D}", "kernel": "hstu_norm_gate<1>"},
      "roofline": {"bound": "hbm", "achieved": nbytes / (ker_ng * 1e-3) / 1e9, "peak": 8000.0, "unit": "GB/s",
                   "frac": nbytes / (ker_ng * 1e-3) / 1e9 / 8000.0, "traffic": None, "kernel_ms_avg": ker_ng,
                   "algorithmic_bytes": nbytes},
      "torch_layer_norm_then_mul_ms": wall_t,
      "norm_gate_bwd": {"ms_per_call": wall_nb, "event_ms": ker_nb, "gb_per_s": 5 * T * D * 2 / (ker_nb * 1e-3) / 1e9,
                        "frac_of_hbm_peak": 5 * T * D * 2 / (ker_nb * 1e-3) / 1e9 / 8000.0, "algorithmic_bytes": 5 * T * D * 2,
                        "torch_forward_and_autograd_ms": wall_nbt},
      "embed_norm": {"ms_per_call": wall_e, "event_ms": ker_e, "torch_gather_add_layer_norm_ms": wall_et,
                     "unique_ids": uniq, "gb_per_s_rows_read_and_written": 2 * T * D * 2 / (ker_e * 1e-3) / 1e9},
      "gemm_silu": {"ms_per_call": wall_g, "event_ms": ker_g, "tflops": gflop / ker_g, "torch_mm_then_silu_ms": wall_gt,
                    "shape": [T, D, 4 * D]},
  }
  if not args.no_cpu:
    rows = 4096
    a_np, u_np = attn[:rows].float().cpu().numpy(), u[:rows].float().cpu().numpy()
    g_np, b_np = gamma.float().cpu().numpy(), beta.float().cpu().numpy()
    t0 = time.perf_counter()
    reps = 0
    while time.perf_counter() - t0 < 10.0:
      ref = BO.norm_gate(a_np, u_np, g_np, b_np, 1e-6)
      reps += 1
    dt = (time.perf_counter() - t0) / reps
    rec["cpu_baseline"] = {"value": 3 * rows * D * 2 / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                           "sample": f"numpy restatement on the first {rows} rows, {reps} repetitions in 10 s"}
    rec["parity_max_abs_over_max_ref"] = float(np.abs(out[:rows] - ref).max() / np.abs(ref).max())
    if not rec["parity_max_abs_over_max_ref"] <= 8e-3:
      raise SystemExit(f"norm + gate parity failed in the benchmark run: {rec['parity_max_abs_over_max_ref']}")
  print(json.dumps(rec))


def calib_copy(dev):
  """One 512 MiB device-to-device copy: a dispatch of known size to scale the HBM byte counters by."""
  import torch
  src = torch.empty(512 << 20, dtype=torch.uint8, device=dev)
  dst = torch.empty_like(src)
  dst.copy_(src)
  torch.cuda.synchronize()
  del src, dst


def bench_dense(args, dev):
  """The layer-side call (dense [B, L, L] causal mask + additive bias shared by heads) in bf16: one JSON line.

  B=16, L=2048, H=8, d=128.  FLOPs: the pairs the mask keeps.  Algorithmic bytes: Q, K, V, O once and the
  mask and the bias once (they are shared by the heads; the kernel re-reads them per head)."""
  import torch
  from recml_amd import hstu_ops
  from oracle import hstu_oracle as O
  B, L, H, d = 16, 2048, 8, 128
  gen = torch.Generator(device=dev).manual_seed(11)
  dt = torch.float32 if args.fp32 else torch.bfloat16
  q, k, v = (torch.randn((B, L, H, d), device=dev, generator=gen).mul_(0.3).to(dt) for _ in range(3))
  mask = torch.tril(torch.ones((L, L), device=dev, dtype=torch.uint8))[None].expand(B, L, L).contiguous()
  bias = torch.randn((B, L, L), device=dev, generator=gen).mul_(0.3)
  if args.backward:
    return bench_dense_backward(args, q, k, v, mask, bias)
  out = torch.empty_like(v)
  call_args, keep = hstu_ops.build_args(q, k, v, out, n=L, alpha=1.0, causal=False, mask=mask, bias=bias)
  variant = hstu_ops.kernel_variant(call_args)
  from recml_amd import _lib
  step = lambda: hstu_ops._run(call_args, keep)
  if args.calib_copy:
    calib_copy(dev)

  def timed(n):
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(n):
      step()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / n

  # a call that stands alone (its preparation kernel reads the whole mask once to find each query tile's range
  # of key steps), then calls on a prepared batch: what each layer of a model sees, the mask being the batch's
  for _ in range(args.warmup):
    step()
  with_prepare_ms = timed(args.steps)
  call_args.flags |= _lib.FWD_WORKSPACE_PREPARED
  for _ in range(args.warmup):
    step()
  ms = timed(args.steps)
  ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
  for a, b in ev:
    a.record()
    step()
    b.record()
  torch.cuda.synchronize()
  ker = float(np.mean([a.elapsed_time(b) for a, b in ev]))
  # 32-key steps the kernel runs for a tile of 128 rows of a causal mask: up to the tile's last row
  steps_run = sum(min((L + 31) // 32, (min(L, 128 * (qt + 1)) + 31) // 32) for qt in range((L + 127) // 128))
  flops = 4.0 * d * H * B * L * (L + 1) / 2
  nbytes = 4 * B * L * H * d * 2 + B * L * L * 5
  rec = {
      "metric": "HSTU attn fwd TFLOP/s (kept pairs), dense mask + bias, L=%d %s" % (L, "fp32" if args.fp32 else "bf16"),
      "value": flops / (with_prepare_ms * 1e-3) / 1e12,
      "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": with_prepare_ms,
      "timed_call": "hstu_attn_fwd, self-contained: every call runs the preparation kernel (which reads the mask once) and "
                    "the main kernel.  *_prepared_batch: the batch prepared once, as the layers of a model after the first call it",
      "ms_per_step_with_prepare": with_prepare_ms,
      "ms_per_step_prepared_batch": ms, "value_prepared_batch": flops / (ms * 1e-3) / 1e12,
      "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32" if args.fp32 else "bf16", "data": "synthetic",
      "config": {"workload": f"A1-dense: B={B} L={L} H={H} d={d} padded, [B,L,L] causal byte mask + fp32 bias, N={L}",
                 "kernel": variant},
      "roofline": {"bound": "hbm", "achieved": nbytes / (ker * 1e-3) / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                   "frac": nbytes / (ker * 1e-3) / 1e9 / PEAK_HBM_GBS, "traffic": measured_traffic("a1-dense"), "kernel_ms_avg": ker,
                   "algorithmic_bytes": nbytes, "algorithmic_flops": flops,
                   "dense_operand_bytes_as_read_by_all_heads": H * B * steps_run * 128 * 32 * 5,
                   "prepare_ms": with_prepare_ms - ms,
                   "mfma_frac": flops / (ker * 1e-3) / 1e12 / (PEAK_FP32_TFLOPS if args.fp32 else PEAK_BF16_TFLOPS)},
  }
  if not args.no_cpu:
    # the numpy restatement on the first sequence's first 256 rows and keys (the causal mask keeps earlier keys only)
    n = 256
    f = lambda t: t[:1, :n].float().cpu().numpy()
    t0 = time.perf_counter()
    ref = O.pointwise_attention_dense(f(q), f(k), f(v), mask[:1, :n, :n].cpu().numpy(), bias[:1, :n, :n].cpu().numpy())
    dt = time.perf_counter() - t0
    ref = ref * (n / L)     # the restatement divides by its own length
    got = out[:1, :n].float().cpu().numpy()
    err = float(np.abs(got - ref).max() / np.abs(ref).max())
    rec["cpu_baseline"] = {"value": 4.0 * d * H * n * (n + 1) / 2 / dt / 1e12, "unit": "TFLOP/s", "cores": 1, "kind": "port",
                           "sample": f"numpy restatement, first sequence, first {n} rows and keys, one evaluation"}
    rec["parity_max_abs_over_max_ref"] = err
    if not err <= 2e-2:
      raise SystemExit(f"parity failed in the benchmark run: {err}")
  print(json.dumps(rec))


def bench_dense_backward(args, q, k, v, mask, bias):
  """The backward of the layer-side call (dense mask + bias), without and with the gradient of the dense bias:
  one JSON line.  FLOPs: four products over the pairs the mask keeps."""
  import torch
  import recml_amd
  B, L, H, d = q.shape
  dout = torch.randn_like(q)
  variant = []
  steps, warm = max(1, args.steps // 10), max(1, args.warmup // 10)

  def timed(bias_grad, with_bias=True):
    run = lambda: recml_amd.hstu_attention_bwd(q, k, v, dout, n=L, alpha=1.0, causal=False, mask=mask,
                                               bias=bias if with_bias else None, bias_grad=bias_grad, _variant_out=variant)
    for _ in range(warm):
      run()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
      run()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps

  # the mask alone (what the reference's model hands its blocks): the matrix-core pair for bf16
  ms_mask = timed(False, with_bias=False)
  variant_mask = variant[-1]
  ms, ms_bias = timed(False), timed(True)
  flops = 8.0 * d * H * B * L * (L + 1) / 2
  fp32 = q.dtype == torch.float32
  mfma = variant[-1] == "hstu_bwd_mfma_bf16"
  bf16_products = mfma or "bf16 products" in variant[-1]
  peak = PEAK_BF16_TFLOPS if bf16_products else PEAK_FP32_TFLOPS
  print(json.dumps({
      "metric": "HSTU attn bwd TFLOP/s (kept pairs), dense mask + bias, L=%d %s" % (L, "fp32" if fp32 else "bf16"),
      "value": flops / (ms * 1e-3) / 1e12, "unit": "TFLOP/s", "n_gpus": 1, "steps": steps, "warmup": warm, "ms_per_step": ms,
      "ms_per_step_with_bias_gradient": ms_bias,
      "ms_per_step_mask_only": ms_mask, "kernel_mask_only": variant_mask,
      "value_mask_only": flops / (ms_mask * 1e-3) / 1e12,
      "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
      "dtype": "f32" if fp32 else ("bf16" if bf16_products else "bf16 storage, fp32 arithmetic"), "data": "synthetic",
      "config": {"workload": f"A1-dense backward: B={B} L={L} H={H} d={d} padded, [B,L,L] causal byte mask + fp32 bias, N={L}",
                 "kernel": variant[-1]},
      "roofline": {"bound": "mfma", "achieved": flops / (ms * 1e-3) / 1e12, "peak": peak, "unit": "TFLOP/s",
                   "frac": flops / (ms * 1e-3) / 1e12 / peak, "traffic": None,
                   "note": ("bf16 matrix-core kernels" if mfma else "general kernels, products on the %s matrix cores"
                            % ("bf16" if bf16_products else "fp32")) + "; time covers both kernels, the preparation, the memsets and the host call"},
  }))


def bench_backward(args, w, q, k, v, kw, dev):
  """The backward pass on the same workload, table gradients included: one JSON line.

  FLOPs counted: four products per unmasked pair (dV, dP, dQ, dK) = 2x the forward's; the
  recomputation of S (and of dP in the second kernel) is not counted."""
  import torch
  import recml_amd
  from oracle import hstu_oracle as O
  dout = torch.randn(v.shape, generator=torch.Generator().manual_seed(1)).to(dev).to(v.dtype)
  variant = []
  run = lambda: recml_amd.hstu_attention_bwd(q, k, v, dout, _variant_out=variant, **kw)
  steps, warm = max(1, args.steps // 10), max(1, args.warmup // 10)
  for _ in range(warm):
    got = run()
  torch.cuda.synchronize()
  t0 = time.perf_counter()
  for _ in range(steps):
    got = run()
  torch.cuda.synchronize()
  ms = (time.perf_counter() - t0) * 1e3 / steps
  flops = 2 * w.flops
  mfma = variant[-1] == "hstu_bwd_mfma_bf16"
  peak = PEAK_BF16_TFLOPS if mfma else PEAK_FP32_TFLOPS
  rec = {
      "metric": "HSTU attn bwd TFLOP/s (unmasked), L=%d %s" % (w.L, "fp32" if w.dtype == "fp32" else "bf16"), "value": flops / (ms * 1e-3) / 1e12,
      "unit": "TFLOP/s", "n_gpus": 1, "steps": steps, "warmup": warm, "ms_per_step": ms,
      "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
      "dtype": "bf16" if (mfma or "bf16 products" in variant[-1]) else ("f32" if w.dtype == "fp32" else "bf16 storage, fp32 arithmetic"),
      "data": "synthetic",
      "config": {"workload": w.name + " backward" + (f" dropout={args.dropout}" if args.dropout > 0 else ""),
                 "kernel": "hstu_bwd_dq_mfma + hstu_bwd_dkv_mfma" if mfma else
                           ("hstu_bwd_dq_mm + hstu_bwd_dkv_mm" if w.d <= 128 else "hstu_bwd_dq + hstu_bwd_dkv")},
      "roofline": {"bound": "mfma", "achieved": flops / (ms * 1e-3) / 1e12, "peak": peak, "unit": "TFLOP/s",
                   "frac": flops / (ms * 1e-3) / 1e12 / peak, "traffic": None,
                   "note": ("bf16 matrix-core kernels" if mfma else "general kernels, fp32 arithmetic" +
                            (" on the fp32 matrix cores" if w.d <= 128 else " by FMA loops")) +
                           "; time covers both kernels, the preparation kernel, the table memsets and the host call"},
  }
  if not args.no_cpu and w.layout == "jagged":
    # bounded sample: the numpy oracle on the shortest sequences that add up to ~5 % of the pairs
    off = w.seq_offsets
    order = np.argsort(w.seq_lens)
    take, pairs = [], 0
    total_pairs = int((w.seq_lens.astype(np.int64) ** 2).sum())
    for b in order:
      take.append(int(b))
      pairs += int(w.seq_lens[b]) ** 2
      if pairs > 0.05 * total_pairs:
        break
    qf, kf, vf, df = (x.float().cpu().numpy() for x in (q, k, v, dout))
    t0 = time.perf_counter()
    worst = 0.0
    fl = 0
    for b in take:
      sl = slice(int(off[b]), int(off[b + 1]))
      n = sl.stop - sl.start
      tsb = None if w.timestamps is None else w.timestamps[sl][None]
      ref = O.hstu_attention_bwd_ref(qf[sl][None], kf[sl][None], vf[sl][None], df[sl][None], n=w.n, alpha=w.alpha,
                                     pos_tab=None if w.pos_tab is None else w.pos_tab[:, w.L - n: w.L + n - 1],
                                     timestamps=tsb, ts_tab=w.ts_tab, dtype=np.float32)
      fl += 2 * w.H * (n * (n + 1) // 2) * 4 * w.d
      for g, r in zip(got[:3], ref[:3]):
        worst = max(worst, float(np.abs(g[sl].float().cpu().numpy() - r[0]).max() / max(np.abs(r).max(), 1e-30)))
    dt = time.perf_counter() - t0
    rec["cpu_baseline"] = {"value": fl / dt / 1e12, "unit": "TFLOP/s", "cores": os.cpu_count(), "kind": "port",
                           "sample": f"numpy fp32 dense backward on the {len(take)} shortest sequences "
                                     f"({fl / 1e9:.2f} GFLOP of unmasked work), {dt:.1f} s"}
    rec["parity_max_abs_over_max_ref"] = worst
    if not worst <= 2e-2:
      raise SystemExit(f"backward parity failed in the benchmark run: {worst}")
  print(json.dumps(rec))


def main():
  ap = argparse.ArgumentParser()
  ap.add_argument("--gpus", type=int, default=1)
  ap.add_argument("--steps", type=int, default=200)
  ap.add_argument("--warmup", type=int, default=20)
  ap.add_argument("--workload", default="c3")
  ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
  ap.add_argument("--no-cold", dest="cold", action="store_false",
                  help="skip the cold-cache variant (a 1 GiB fill between launches)")
  ap.add_argument("--backward", action="store_true", help="measure the backward pass instead of the forward")
  ap.add_argument("--fp32", action="store_true",
                  help="fp32 storage (Keras' default dtype): the general kernels on the fp32 matrix cores; a profiling aid, "
                       "not the contract's workload")
  ap.add_argument("--no-graph", dest="graph", action="store_false",
                  help="skip the variant that replays the timed calls as one HIP graph")
  ap.add_argument("--one-item-per-workgroup", action="store_true",
                  help="diagnostics: force one workgroup per work-list entry")
  ap.add_argument("--resident-workgroups", action="store_true",
                  help="diagnostics: force resident workgroups that loop over the work list")
  ap.add_argument("--compiler-scheduled-blocks", action="store_true",
                  help="diagnostics: interior steps through the compiler-scheduled block code instead of the hand-scheduled stream")
  ap.add_argument("--dropout", type=float, default=0.0,
                  help="diagnostics: the training form with this dropout rate on the attention weights (not the contract's "
                       "workload; the CPU leg is skipped, tests/test_gpu_dropout.py holds its parity)")
  ap.add_argument("--ramp-ms", type=float, default=300.0,
                  help="untimed calls for this long before anything is measured (clock ramp from idle)")
  ap.add_argument("--no-tuned-products", dest="tuned", action="store_false",
                  help="c4-model: skip the training step with torch's tuned matrix products (its search runs hundreds of "
                       "candidate kernels: leave it out under a profiler)")
  ap.add_argument("--calib-copy", action="store_true",
                  help="also run one 512 MiB device copy (reference point for HBM byte counters)")
  args = ap.parse_args()
  if args.gpus != 1:
    raise SystemExit("bench.py measures one GPU: this build has no multi-GPU path "
                     "(the forward shards over (sequence, head) with no exchange); run with --gpus 1")

  import torch
  import recml_amd
  from recml_amd import hstu_ops

  if not torch.cuda.is_available():
    raise SystemExit("bench.py needs a GPU")
  dev = torch.device("cuda:0")
  if args.workload == "c4-model":
    return bench_model(args, dev)
  if args.workload == "c4-block-steps":
    return bench_block_steps(args, dev)
  if args.workload == "a1-dense":
    return bench_dense(args, dev)
  w = make_workload(args.workload)
  q, k, v, kw = to_device(w, dev)
  if args.dropout > 0:
    kw.update(dropout_p=args.dropout, dropout_seed=1)
    args.no_cpu = True
  if args.fp32:
    if w.dtype == "fp8":
      raise SystemExit("--fp32 goes with the bf16 workloads")
    q, k, v = (torch.from_numpy(np.ascontiguousarray(x)).to(dev) for x in (w.q, w.k, w.v))
    w.dtype = "fp32"
  if args.backward:
    if w.dtype == "fp8":
      raise SystemExit("the backward takes fp32 or bf16 storage")
    return bench_backward(args, w, q, k, v, kw, dev)
  out = torch.empty_like(v)
  call_args, keep = hstu_ops.build_args(q, k, v, out, **kw)
  variant = hstu_ops.kernel_variant(call_args)
  from recml_amd import _lib
  if args.one_item_per_workgroup:
    call_args.flags |= _lib.FWD_ONE_ITEM_PER_WORKGROUP
  if args.resident_workgroups:
    call_args.flags |= _lib.FWD_RESIDENT_WORKGROUPS
  if args.compiler_scheduled_blocks:
    call_args.flags |= _lib.FWD_COMPILER_SCHEDULED_BLOCKS

  def step():
    hstu_ops._run(call_args, keep)

  if args.calib_copy:
    calib_copy(dev)

  def timed(fn, n):
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(n):
      fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / n

  starts = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps)]
  ends = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps)]

  def evented(fn):
    for i in range(args.steps):
      starts[i].record()
      fn()
      ends[i].record()
    torch.cuda.synchronize()
    return np.array([s.elapsed_time(e) for s, e in zip(starts, ends)])

  # The GPU's clocks take tens of milliseconds of work to come up from idle: untimed calls for a fixed
  # time first, so that a run with few steps measures the same machine state as one with many.
  t_ramp = time.perf_counter()
  while (time.perf_counter() - t_ramp) * 1e3 < args.ramp_ms:
    for _ in range(50):
      step()
    torch.cuda.synchronize()

  # The timed region: the call as the reference's op is called -- a function of its arguments that does all of
  # its work every time: the preparation kernel (work list, 32-bit timestamps, scaled tables, timestamp
  # descriptors) and the main kernel.  Exactly `steps` calls between two synchronisations, nothing else on
  # the stream.
  for _ in range(args.warmup):
    step()
  wall = timed(step, args.steps) * 1e-3 * args.steps
  # The preparation alone.
  call_args.flags |= _lib.FWD_PREPARE_ONLY
  prepare_ms = float(evented(step).mean())
  call_args.flags &= ~_lib.FWD_PREPARE_ONLY

  # The call as a layer of a model makes it: the batch was prepared once (above), every layer's call reuses
  # that (lengths, timestamps and tables are the same for all layers).  A secondary figure.
  call_args.flags |= _lib.FWD_WORKSPACE_PREPARED
  for _ in range(args.warmup):
    step()
  prepared_ms = timed(step, args.steps)

  # the same calls again with a pair of HIP events around each one, on the launch stream: the kernel
  # alone (the roofline figure)
  main_ms = evented(step)
  ev_ms = main_ms
  region_ms = starts[0].elapsed_time(ends[-1])

  # and recorded once into a HIP graph of `steps` calls (the entry point only enqueues and allocates
  # nothing): what a caller that replays its step as a graph sees per call
  graph_ms = None
  if args.graph:
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
      for i in range(args.steps):
        step()
    graph.replay()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    graph.replay()
    torch.cuda.synchronize()
    graph_ms = (time.perf_counter() - t1) * 1e3 / args.steps
    del graph
  call_args.flags &= ~_lib.FWD_WORKSPACE_PREPARED

  # The public entry point as a user calls it (arguments checked and the struct built on every call):
  # on its own (scratch allocated and prepared per call), and with one AttentionBatch for all calls.
  api_kw = dict(kw)
  for _ in range(max(3, args.warmup)):      # (the first calls pay torch's allocator for the scratch buffer)
    recml_amd.hstu_attention(q, k, v, out=out, **api_kw)
  api_ms = timed(lambda: recml_amd.hstu_attention(q, k, v, out=out, **api_kw), args.steps)
  shared = hstu_ops.AttentionBatch()
  recml_amd.hstu_attention(q, k, v, out=out, batch=shared, **api_kw)
  api_batch_ms = timed(lambda: recml_amd.hstu_attention(q, k, v, out=out, batch=shared, **api_kw), args.steps)
  assert shared.prepared_calls >= args.steps or not call_args.workspace_bytes     # (the general kernel prepares nothing)

  # Cold variant: a 1 GiB fill between launches pushes the inputs out of L2 and the memory-side cache.
  cold_ms = None
  if args.cold:
    junk = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
    cold = []
    for i in range(min(args.steps, 20)):
      junk.fill_(i & 0xff)
      starts[i].record()
      step()
      ends[i].record()
      torch.cuda.synchronize()
      cold.append(starts[i].elapsed_time(ends[i]))
    cold_ms = float(np.mean(cold))
    del junk

  ms_per_step = wall * 1e3 / args.steps
  step_ms = float(ev_ms.mean())
  kernel_ms = float(main_ms.mean())
  flops = w.flops
  tflops = flops / (ms_per_step * 1e-3) / 1e12
  achieved = flops / (kernel_ms * 1e-3) / 1e12
  bytes_alg = w.bytes_moved(4 if w.dtype == "fp32" else 2, 1 if w.dtype == "fp8" else None)
  ai = flops / bytes_alg
  # fp8 q/k: half of the flops (q k^T) run at the fp8 rate, half (P V) at the bf16 rate
  peak = PEAK_BF16_TFLOPS if w.dtype != "fp8" else 1.0 / (0.5 / PEAK_FP8_TFLOPS + 0.5 / PEAK_BF16_TFLOPS)
  if w.dtype == "fp32":
    peak = PEAK_FP32_TFLOPS
  capped_peak = min(peak, ai * PEAK_HBM_GBS / 1e3)

  rec = {
      "metric": "HSTU attn fwd TFLOP/s (unmasked), L=%d %s" % (w.L, {"fp8": "fp8", "fp32": "fp32"}.get(w.dtype, "bf16")),
      "value": tflops, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
      "warmup": args.warmup, "ms_per_step": ms_per_step,
      "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
      "dtype": {"fp8": "fp8 q/k, bf16 v/out", "fp32": "f32"}.get(w.dtype, "bf16"), "data": "synthetic",
      "config": {"workload": f"{w.name}: B={w.B} max_len={w.L} H={w.H} d={w.d} {w.layout} "
                             f"lens mean {w.seq_lens.mean():.0f} max {w.seq_lens.max()}, causal, "
                             f"pos_bias={'yes' if w.pos_tab is not None else 'no'} "
                             f"ts_bias={'yes' if w.ts_tab is not None else 'no'} N={w.n} alpha={w.alpha}"
                             + (f" dropout={args.dropout}" if args.dropout > 0 else ""),
                 "kernel": variant},
      "seqs_per_s": w.B / (ms_per_step * 1e-3),
      "timed_call": "hstu_attn_fwd, self-contained: every call runs the preparation kernel and the main kernel (value, "
                    "ms_per_step; the same as *_with_prepare).  *_prepared_batch: the batch prepared once "
                    "(HSTU_FWD_WORKSPACE_PREPARED), as the layers of a model after the first call it",
      "ms_per_step_with_prepare": ms_per_step,
      "value_with_prepare": tflops,
      "ms_per_step_prepared_batch": prepared_ms,
      "value_prepared_batch": flops / (prepared_ms * 1e-3) / 1e12,
      "api_ms_per_step": api_ms, "api_shared_batch_ms_per_step": api_batch_ms,
      "roofline": {
          "bound": "mfma", "achieved": achieved, "peak": peak,
          "unit": "TFLOP/s", "frac": achieved / peak, "traffic": measured_traffic(args.workload),
          "traffic_source": "profiles/traffic.json (rocprofv3 --pmc runs of this command, scaled by a copy of known size)"
                            if measured_traffic(args.workload) is not None else None,
          "kernel": variant, "kernel_ms_avg": kernel_ms, "kernel_ms_min": float(main_ms.min()),
          "kernel_ms_median": float(np.median(main_ms)),
          "step_ms_avg": step_ms, "step_ms_cold_avg": cold_ms,
          "prepare_ms": prepare_ms,
          "region_ms_per_step": region_ms / args.steps,
          "graph_replay_ms_per_step": graph_ms,
          "algorithmic_flops": flops, "algorithmic_bytes": bytes_alg,
          "arithmetic_intensity": ai,
          "hbm_GBps_algorithmic": bytes_alg / (kernel_ms * 1e-3) / 1e9,
          "roofline_capped_peak": capped_peak,
          "frac_of_capped_peak": achieved / capped_peak,
      },
  }
  if not args.no_cpu:
    base, err = cpu_baseline(w, q, k, v, out.float().cpu().numpy(), kw)
    rec["cpu_baseline"] = base
    rec["parity_max_abs_over_max_ref"] = err
    if not err <= 2e-2:
      raise SystemExit(f"parity failed in the benchmark run: {err}")
  print(json.dumps(rec))


if __name__ == "__main__":
  main()
