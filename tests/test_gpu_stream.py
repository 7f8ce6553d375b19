"""The hand-scheduled instruction stream of the forward kernel's interior steps (d = 128, bf16): the same
arithmetic in the same order as the compiler-scheduled block code, so a call with
HSTU_FWD_COMPILER_SCHEDULED_BLOCKS must give the same bits, for both ways through the work list; and the
stream itself against the oracle on shapes where nearly every step is an interior one."""

import numpy as np
import pytest
import torch

from recml_amd import _lib, hstu_ops
from oracle import hstu_oracle as O

pytestmark = pytest.mark.gpu

BF16_TOL = 2e-2


def _run(q, k, v, flags, **kw):
  out = torch.full_like(v, float("nan"))
  a, keep = hstu_ops.build_args(q, k, v, out, **kw)
  assert hstu_ops.kernel_variant(a) == "hstu_fwd_mfma_bf16"
  a.flags |= flags
  hstu_ops._run(a, keep)
  torch.cuda.synchronize()
  return out


def _inputs(lens, L, H, pos, causal, jagged, timestamps=False, seed=0):
  g = torch.Generator(device="cuda:0").manual_seed(seed)
  d = 128
  lens = np.asarray(lens, np.int32)
  kw = dict(max_len=L, n=L, causal=causal)
  if jagged:
    offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    shape = (int(offs[-1]), H, d)
    kw["seq_offsets"] = torch.from_numpy(offs).to("cuda:0")
  else:
    shape = (len(lens), L, H, d)
    kw["seq_lens"] = torch.from_numpy(lens).to("cuda:0")
  q, k, v = (torch.randn(shape, device="cuda:0", generator=g).mul_(0.3).to(torch.bfloat16) for _ in range(3))
  if pos:
    kw["pos_bias"] = torch.randn((H, 2 * L - 1), device="cuda:0", generator=g) * 0.05
  if timestamps:
    rng = np.random.default_rng(seed)
    if jagged:
      ts = np.concatenate([1_600_000_000 + np.cumsum(np.ceil(rng.exponential(3600.0, n)).astype(np.int64)) for n in lens])
    else:
      ts = 1_600_000_000 + np.cumsum(np.ceil(rng.exponential(3600.0, (len(lens), L))).astype(np.int64), axis=1)
    kw["timestamps"] = torch.from_numpy(ts).to("cuda:0")
    kw["ts_bias"] = torch.randn((H, 129), device="cuda:0", generator=g) * 0.05
  return q, k, v, kw


CASES = [
    # name, lengths, L, H, position table, causal, jagged
    ("one long sequence", [2048], 2048, 8, False, True, True),
    ("one long sequence, table", [2048], 2048, 8, True, True, True),
    ("mixed lengths around every tile edge, table", [2048, 1655, 1000, 777, 513, 512, 511, 385, 384, 256, 129, 128, 127, 16, 1], 2048, 8, True, True, True),
    ("mixed lengths, no table", [2048, 1655, 1000, 777, 513, 512, 511, 385, 384, 256, 129, 128, 127, 16, 1], 2048, 8, False, True, True),
    ("padded with lengths, table", [2048, 1655, 1000, 640, 641, 639, 100], 2048, 4, True, True, False),
    ("no causal mask, jagged, table", [1024, 1000, 515, 300], 1024, 8, True, False, True),
    ("no causal mask, padded", [1024, 1023, 700], 1024, 2, False, False, False),
    ("two long sequences (tiles split by keys), table", [2048, 2048], 2048, 8, True, True, True),
]


@pytest.mark.parametrize("name,lens,L,H,pos,causal,jagged", CASES, ids=[c[0] for c in CASES])
@pytest.mark.parametrize("walk", ["one item per workgroup", "resident workgroups"])
def test_stream_gives_the_bits_of_the_block_code(gpu, walk, name, lens, L, H, pos, causal, jagged):
  q, k, v, kw = _inputs(lens, L, H, pos, causal, jagged)
  mode = _lib.FWD_ONE_ITEM_PER_WORKGROUP if walk == "one item per workgroup" else _lib.FWD_RESIDENT_WORKGROUPS
  ref = _run(q, k, v, mode | _lib.FWD_COMPILER_SCHEDULED_BLOCKS, **kw)
  got = _run(q, k, v, mode, **kw)
  assert not torch.isnan(got.float()).any()
  assert torch.equal(ref.view(torch.int16), got.view(torch.int16))


@pytest.mark.parametrize("pos", [False, True])
def test_stream_against_the_oracle(gpu, pos):
  # three sequences whose tiles have up to 15 quads of interior steps
  lens = [2048, 1300, 700]
  L, H = 2048, 2
  q, k, v, kw = _inputs(lens, L, H, pos, True, True, seed=7)
  got = _run(q, k, v, 0, **kw).float().cpu().numpy()
  off = kw["seq_offsets"].cpu().numpy()
  okw = {}
  if pos:
    okw["pos_tab"] = kw["pos_bias"].cpu().numpy()
  f = lambda t: t.float().cpu().numpy()
  ref = O.hstu_attention_jagged_ref(f(q), f(k), f(v), off, L, n=L, **okw)
  err = np.abs(got - ref).max() / np.abs(ref).max()
  assert err <= BF16_TOL, err
