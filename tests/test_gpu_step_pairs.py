"""The step loops of the matrix-core kernels run in pairs of 32-key steps at d = 128 (forward) and
at every head dim (backward): these cases put every count of steps modulo 4 behind one tile, and an
odd first step under a sliding window, against the oracle."""

import numpy as np
import pytest
import torch

import recml_amd
from recml_amd import hstu_ops
from oracle import hstu_oracle as O

pytestmark = pytest.mark.gpu

BF16_TOL = 2e-2


def _dev(x, dtype=None):
  t = torch.from_numpy(np.ascontiguousarray(x)).to("cuda:0")
  return t if dtype is None else t.to(dtype)


def _rel(a, b):
  return np.abs(np.asarray(a, np.float64) - b).max() / max(np.abs(b).max(), 1e-30)


# lengths whose last tile ends after 1 .. 9 steps of 32 keys (and one that fills two tiles exactly)
LENS = np.array([1, 32, 33, 64, 65, 96, 97, 128, 129, 160, 161, 192, 223, 256, 257, 288], dtype=np.int32)


@pytest.mark.parametrize("d", [128, 64])
@pytest.mark.parametrize("bias", [False, True])
def test_forward_every_step_count(gpu, d, bias):
  rng = np.random.default_rng(900 + d + bias)
  H, L = 2, 288
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
  bf = torch.bfloat16
  a, keep = hstu_ops.build_args(_dev(q, bf), _dev(k, bf), _dev(v, bf), torch.empty((T, H, d), dtype=bf, device="cuda:0"),
                                seq_offsets=_dev(off), max_len=L, **gk)
  assert hstu_ops.kernel_variant(a) == "hstu_fwd_mfma_bf16"
  hstu_ops._run(a, keep)
  out = keep[3]
  ref = O.hstu_attention_jagged_ref(q, k, v, off, L, **kw)
  got = out.float().cpu().numpy()
  assert _rel(got, ref) <= BF16_TOL


@pytest.mark.parametrize("L,window,causal", [
    (300, 40, True),     # first step of the later tiles: (q0 - 40) / 32, odd for q0 = 128, even for q0 = 256
    (300, 70, False),
    (420, 5, True),
])
def test_window_first_step_parity_forward_and_backward(gpu, L, window, causal):
  rng = np.random.default_rng(950 + L + window)
  B, H, d = 3, 2, 128
  bf = torch.bfloat16
  lens = np.array([L, L - 37, 131], dtype=np.int32)
  q, k, v, dout = (O.round_bf16(rng.standard_normal((B, L, H, d)).astype(np.float32) * 0.4) for _ in range(4))
  pos = (rng.standard_normal((H, 2 * L - 1)) * 0.3).astype(np.float32)
  out = recml_amd.hstu_attention(_dev(q, bf), _dev(k, bf), _dev(v, bf), seq_lens=_dev(lens), causal=causal,
                                 sliding_window_size=window, pos_bias=_dev(pos))
  ref = O.hstu_attention_ref(q, k, v, seq_lens=lens, causal=causal, sliding_window_size=window, pos_tab=pos)
  assert _rel(out.float().cpu().numpy(), ref) <= BF16_TOL
  want = O.hstu_attention_bwd_ref(q, k, v, dout, seq_lens=lens, causal=causal, sliding_window_size=window, pos_tab=pos)
  variant = []
  got = recml_amd.hstu_attention_bwd(_dev(q, bf), _dev(k, bf), _dev(v, bf), _dev(dout, bf), seq_lens=_dev(lens),
                                     causal=causal, sliding_window_size=window, pos_bias=_dev(pos), _variant_out=variant)
  assert variant == ["hstu_bwd_mfma_bf16"]
  for nm, g, w in zip(("dq", "dk", "dv", "dpos"), got[:4], want[:4]):
    assert _rel(g.float().cpu().numpy().reshape(w.shape), w) <= BF16_TOL, nm
