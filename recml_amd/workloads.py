"""Synthetic HSTU attention workloads (the benchmark configurations).

Every tensor comes from numpy.random.Generator(PCG64(seed)) with a fixed draw
order (lengths, q, k, v, pos_tab, ts_tab, timestamps) so that the GPU path,
the CPU oracle and the golden fixtures all see the same inputs.  Arrays are
fp32 masters; callers round to the storage dtype.

Shapes follow the HSTU layer's attention call: q, k, v are [B, L, H, d]
(recml/layers/keras/hstu.py:356-371) or, jagged, [sum(n_b), H, d].
"""

from __future__ import annotations

import dataclasses

import numpy as np


@dataclasses.dataclass
class Workload:
  name: str
  B: int
  L: int
  H: int
  d: int
  dtype: str                     # "fp32" | "bf16" | "fp8" (q and k float8_e4m3fn with per-head scales, v bf16)
  layout: str                    # "padded" | "jagged"
  seq_lens: np.ndarray           # int32 [B]
  q: np.ndarray                  # padded [B,L,H,d] or jagged [T,H,d], fp32
  k: np.ndarray
  v: np.ndarray
  n: int                         # normaliser N
  alpha: float = 1.0
  pos_tab: np.ndarray | None = None      # [H, 2L-1] fp32
  ts_tab: np.ndarray | None = None       # [H, num_buckets+1] fp32
  timestamps: np.ndarray | None = None   # int64, padded [B,L] or jagged [T]
  seq_offsets: np.ndarray | None = None  # int32 [B+1] (jagged)

  @property
  def flops(self) -> int:
    nn = self.seq_lens.astype(np.int64)
    return int((self.H * (nn * (nn + 1) // 2) * 4 * self.d).sum())

  def bytes_moved(self, elem_bytes: int, qk_bytes: int | None = None) -> int:
    """Q, K, V read once and O written once over the valid tokens."""
    tokens = int(self.seq_lens.astype(np.int64).sum())
    if self.layout == "padded":
      tokens = self.B * self.L
    qk = elem_bytes if qk_bytes is None else qk_bytes
    return tokens * self.H * self.d * (2 * qk + 2 * elem_bytes)


def power_law_lengths(rng, B, lo, hi, exponent):
  """Truncated power law p(n) ~ n^-exponent on [lo, hi] by inverse CDF."""
  e = 1.0 - exponent
  u = rng.random(B)
  x = (lo**e + u * (hi**e - lo**e)) ** (1.0 / e)
  return np.clip(np.floor(x), lo, hi).astype(np.int32)


def _normal(rng, shape, std):
  return (rng.standard_normal(shape, dtype=np.float32) * np.float32(std))


def _offsets(lens):
  off = np.zeros(len(lens) + 1, dtype=np.int32)
  off[1:] = np.cumsum(lens)
  return off


def make_timestamps(rng, lens, L, layout, t0=1_600_000_000, mean=3600.0):
  """int64 seconds: t0 + cumsum(ceil(Exp(mean))) per sequence.

  Padded rows repeat the last valid timestamp, which is what makes the padded
  and the jagged form of the same batch agree on the last row's "next item"
  timestamp (recml/layers/keras/hstu.py:194-202 reads ts[i+1]).
  """
  rows = []
  for n in lens:
    gaps = np.ceil(rng.exponential(mean, int(n))).astype(np.int64)
    rows.append(t0 + np.cumsum(gaps))
  if layout == "jagged":
    return np.concatenate(rows)
  out = np.zeros((len(lens), L), dtype=np.int64)
  for b, r in enumerate(rows):
    out[b, : len(r)] = r
    out[b, len(r):] = r[-1]
  return out


def config1(seed=1):
  """B=4, L=64, H=2, d=32 fp32, full lengths, causal, no bias, N=64."""
  rng = np.random.Generator(np.random.PCG64(seed))
  B, L, H, d = 4, 64, 2, 32
  lens = np.full(B, L, dtype=np.int32)
  q, k, v = (_normal(rng, (B, L, H, d), 0.1) for _ in range(3))
  return Workload("C1", B, L, H, d, "fp32", "padded", lens, q, k, v, n=L)


def config2(seed=2):
  """B=32, L=512, H=4, d=64 bf16, lens U{64..512}, padded, pos bias per head."""
  rng = np.random.Generator(np.random.PCG64(seed))
  B, L, H, d = 32, 512, 4, 64
  lens = rng.integers(64, L + 1, B).astype(np.int32)
  # padding rows hold noise on purpose: the op must ignore them
  q, k, v = (_normal(rng, (B, L, H, d), 0.1) for _ in range(3))
  pos = _normal(rng, (H, 2 * L - 1), 0.02)
  return Workload("C2", B, L, H, d, "bf16", "padded", lens, q, k, v, n=L,
                  pos_tab=pos)


def config3(seed=3, full=False, B=64, L=2048, H=8, d=128, bias=True):
  """B=64, L=2048, H=8, d=128 bf16, power-law lengths, jagged, pos + ts bias."""
  rng = np.random.Generator(np.random.PCG64(seed))
  lens = power_law_lengths(rng, B, 16, L, 1.2)
  if full:
    lens = np.full(B, L, dtype=np.int32)
  T = int(lens.sum())
  q, k, v = (_normal(rng, (T, H, d), 0.1) for _ in range(3))
  pos = _normal(rng, (H, 2 * L - 1), 0.02)
  tst = _normal(rng, (H, 129), 0.02)
  ts = make_timestamps(rng, lens, L, "jagged")
  w = Workload("C3-full" if full else "C3", B, L, H, d, "bf16", "jagged", lens,
               q, k, v, n=L, pos_tab=pos if bias else None,
               ts_tab=tst if bias else None, timestamps=ts if bias else None,
               seq_offsets=_offsets(lens))
  return w


def config4_attention(seed=4, B=128, L=1024, H=8, d=64):
  """Attention share of the end-to-end ranking forward: lens U{128..1024}."""
  rng = np.random.Generator(np.random.PCG64(seed))
  lens = rng.integers(128, L + 1, B).astype(np.int32)
  T = int(lens.sum())
  q, k, v = (_normal(rng, (T, H, d), 0.1) for _ in range(3))
  pos = _normal(rng, (H, 2 * L - 1), 0.02)
  return Workload("C4-attn", B, L, H, d, "bf16", "jagged", lens, q, k, v, n=L,
                  pos_tab=pos, seq_offsets=_offsets(lens))


def config5(seed=5, B=32, L=4096, H=8, d=128, fp8=True):
  """Low-precision shape: lens U{1024..4096}, pos bias, N=4096.  With fp8 the
  caller quantises q and k per head (scale = amax / 448) to float8_e4m3fn and
  keeps v in bf16; the masters here are fp32."""
  rng = np.random.Generator(np.random.PCG64(seed))
  lens = rng.integers(1024, L + 1, B).astype(np.int32)
  T = int(lens.sum())
  q, k, v = (_normal(rng, (T, H, d), 0.1) for _ in range(3))
  pos = _normal(rng, (H, 2 * L - 1), 0.02)
  return Workload("C5", B, L, H, d, "fp8" if fp8 else "bf16", "jagged", lens, q, k, v, n=L,
                  pos_tab=pos, seq_offsets=_offsets(lens))


def small_jagged(seed=7, B=3, L=24, H=2, d=32):
  """A tiny jagged case with both biases, for golden fixtures."""
  rng = np.random.Generator(np.random.PCG64(seed))
  lens = np.asarray([24, 5, 13][:B], dtype=np.int32)
  T = int(lens.sum())
  q, k, v = (_normal(rng, (T, H, d), 0.5) for _ in range(3))
  pos = _normal(rng, (H, 2 * L - 1), 0.2)
  tst = _normal(rng, (H, 129), 0.2)
  ts = make_timestamps(rng, lens, L, "jagged")
  return Workload("small-jagged", B, L, H, d, "fp32", "jagged", lens, q, k, v,
                  n=L, pos_tab=pos, ts_tab=tst, timestamps=ts,
                  seq_offsets=_offsets(lens))
