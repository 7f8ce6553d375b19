"""The hand-scheduled instruction stream of the forward kernel's interior steps (d = 128, bf16): the same
arithmetic in the same order as the compiler-scheduled block code, so a call with
HSTU_FWD_COMPILER_SCHEDULED_BLOCKS must give the same bits, for both ways through the work list; and the
stream itself against the oracle on shapes where nearly every step is an interior one.  With a timestamp
bias the stream reads the per-(row, step) descriptors that a kernel of their own builds once per batch
(bucket of the nearest key, how many of the step's keys are one bucket further): timestamps a second and a
million seconds apart, out of order, and spans beyond 31 bits against the oracle as well."""

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


TS_CASES = [
    # name, lengths, L, H, position table, jagged
    ("one long sequence, timestamps", [2048], 2048, 8, False, True),
    ("one long sequence, table + timestamps", [2048], 2048, 8, True, True),
    ("mixed lengths, table + timestamps", [2048, 1655, 1000, 777, 513, 512, 511, 385, 384, 256, 129, 128, 127, 16, 1], 2048, 8, True, True),
    ("two long sequences (tiles split by keys), table + timestamps", [2048, 2048], 2048, 8, True, True),
    ("three sequences, two heads", [2048, 1300, 700], 2048, 2, True, True),
    ("padded with lengths, [B, L] timestamps", [1024, 1000, 640, 641, 100], 1024, 4, True, False),
    ("a small batch (no work list), padded", [512, 300], 512, 2, True, False),
    ("a small batch (no work list), jagged", [512, 300, 129], 512, 2, False, True),
]


@pytest.mark.parametrize("name,lens,L,H,pos,jagged", TS_CASES, ids=[c[0] for c in TS_CASES])
@pytest.mark.parametrize("walk", ["one item per workgroup", "resident workgroups"])
def test_stream_with_timestamps_gives_the_bits_of_the_block_code(gpu, walk, name, lens, L, H, pos, jagged):
  q, k, v, kw = _inputs(lens, L, H, pos, True, jagged, timestamps=True)
  mode = _lib.FWD_ONE_ITEM_PER_WORKGROUP if walk == "one item per workgroup" else _lib.FWD_RESIDENT_WORKGROUPS
  for _ in range(2):      # (twice: a race between the workgroups that write the descriptors would not show every time)
    ref = _run(q, k, v, mode | _lib.FWD_COMPILER_SCHEDULED_BLOCKS, **kw)
    got = _run(q, k, v, mode, **kw)
    assert not torch.isnan(got.float()).any()
    assert torch.equal(ref.view(torch.int16), got.view(torch.int16))


def _ts_oracle_case(lens, L, H, pos, ts, seed):
  g = torch.Generator(device="cuda:0").manual_seed(seed)
  offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
  shape = (int(offs[-1]), H, 128)
  q, k, v = (torch.randn(shape, device="cuda:0", generator=g).mul_(0.3).to(torch.bfloat16) for _ in range(3))
  ts_tab = torch.randn((H, 129), device="cuda:0", generator=g) * 0.2
  kw = dict(max_len=L, n=L, causal=True, seq_offsets=torch.from_numpy(offs).to("cuda:0"),
            timestamps=torch.from_numpy(ts).to("cuda:0"), ts_bias=ts_tab)
  okw = dict(timestamps=ts, ts_tab=ts_tab.cpu().numpy())
  if pos:
    kw["pos_bias"] = torch.randn((H, 2 * L - 1), device="cuda:0", generator=g) * 0.05
    okw["pos_tab"] = kw["pos_bias"].cpu().numpy()
  got = _run(q, k, v, 0, **kw).float().cpu().numpy()
  f = lambda t: t.float().cpu().numpy()
  ref = O.hstu_attention_jagged_ref(f(q), f(k), f(v), offs, L, n=L, **okw)
  return np.abs(got - ref).max() / np.abs(ref).max()


@pytest.mark.parametrize("mean_dt", [1.0, 3600.0, 1e6])
@pytest.mark.parametrize("pos", [False, True])
def test_stream_with_timestamps_against_the_oracle(gpu, mean_dt, pos):
  rng = np.random.default_rng(int(mean_dt) + pos)
  lens = np.asarray([1536, 900, 2048], np.int32)
  ts = np.concatenate([1_600_000_000 + np.cumsum(np.ceil(rng.exponential(mean_dt, n)).astype(np.int64)) for n in lens])
  assert _ts_oracle_case(lens, 2048, 2, pos, ts, seed=11) <= BF16_TOL


def test_timestamps_out_of_order_and_wide_spans_with_descriptors(gpu):
  # one sequence in order, one shuffled (every step flagged: the per-pair lookup), one with equal timestamps, one
  # whose span needs more than 31 bits (no 32-bit timestamps: the kernel's 64-bit path, descriptors unused)
  rng = np.random.default_rng(5)
  lens = np.asarray([1024, 1024, 700, 640], np.int32)
  a = 1_600_000_000 + np.cumsum(np.ceil(rng.exponential(3600.0, 1024)).astype(np.int64))
  b = rng.permutation(a)
  c = np.full(700, 1_700_000_000, np.int64)
  d = np.cumsum(rng.integers(1, 2**24, 640).astype(np.int64)) * 1000
  ts = np.concatenate([a, b, c, d])
  assert _ts_oracle_case(lens, 1024, 2, True, ts, seed=12) <= BF16_TOL


def test_stream_with_timestamps_in_the_padded_layout_against_the_oracle(gpu):
  # [B, L] timestamps (non-decreasing along the whole row, so the padding repeats nothing the rows read), lengths
  lens, L, H = [1024, 700, 333], 1024, 2
  q, k, v, kw = _inputs(lens, L, H, True, True, False, timestamps=True, seed=9)
  got = _run(q, k, v, 0, **kw).float().cpu().numpy()
  f = lambda t: t.float().cpu().numpy()
  ref = O.hstu_attention_ref(f(q), f(k), f(v), seq_lens=np.asarray(lens), n=L, pos_tab=kw["pos_bias"].cpu().numpy(),
                             timestamps=kw["timestamps"].cpu().numpy(), ts_tab=kw["ts_bias"].cpu().numpy())
  err = np.abs(got - ref).max() / np.abs(ref).max()
  assert err <= BF16_TOL, err
  for b, n in enumerate(lens):
    assert not got[b, n:].any()          # rows past a sequence's end: exactly 0


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


# ---- the backward's dK/dV kernel: pairs of unmasked blocks as one hand-scheduled stream (d = 128, no bias)

BWD_CASES = [
    # name, lengths, L, H, causal, jagged
    ("one long sequence", [2048], 2048, 2, True, True),
    ("mixed lengths around every tile edge", [2048, 1655, 1000, 777, 513, 512, 511, 385, 384, 256, 129, 128, 127, 16, 1], 2048, 2, True, True),
    ("no causal mask, jagged", [1024, 1000, 515, 300], 1024, 2, False, True),
    ("padded with lengths", [2048, 1655, 1000, 640, 641, 639, 100], 2048, 2, True, False),
    ("a first step that is odd", [1952, 700], 2048, 3, True, True),
]


@pytest.mark.parametrize("name,lens,L,H,causal,jagged", BWD_CASES, ids=[c[0] for c in BWD_CASES])
def test_backward_stream_gives_the_bits_of_the_block_code(gpu, name, lens, L, H, causal, jagged):
  q, k, v, kw = _inputs(lens, L, H, False, causal, jagged, seed=3)
  dout = torch.randn(v.shape, device="cuda:0", generator=torch.Generator(device="cuda:0").manual_seed(4)).mul_(0.5).to(torch.bfloat16)
  var = []
  ref = hstu_ops.hstu_attention_bwd(q, k, v, dout, _flags=_lib.FWD_COMPILER_SCHEDULED_BLOCKS, _variant_out=var, alpha=0.2, **kw)
  assert var[0] == "hstu_bwd_mfma_bf16"
  for _ in range(2):
    got = hstu_ops.hstu_attention_bwd(q, k, v, dout, alpha=0.2, **kw)
    torch.cuda.synchronize()
    for name_, a, b in zip(("dq", "dk", "dv"), ref[:3], got[:3]):
      assert not torch.isnan(b.float()).any(), name_
      assert torch.equal(a.view(torch.int16), b.view(torch.int16)), name_


def test_backward_stream_against_the_fp32_kernels(gpu):
  # every accumulator register of dK and dV: the general kernels in fp32 on the same inputs
  q, k, v, kw = _inputs([2048, 700], 2048, 2, False, True, True, seed=5)
  dout = torch.randn(v.shape, device="cuda:0", generator=torch.Generator(device="cuda:0").manual_seed(6)).mul_(0.5).to(torch.bfloat16)
  ref = hstu_ops.hstu_attention_bwd(q.float(), k.float(), v.float(), dout.float(), alpha=0.2, **kw)
  for flags in (0, _lib.FWD_COMPILER_SCHEDULED_BLOCKS):
    got = hstu_ops.hstu_attention_bwd(q, k, v, dout, alpha=0.2, _flags=flags, **kw)
    for name_, a, b in zip(("dq", "dk", "dv"), ref[:3], got[:3]):
      # per channel: a register that is read too early shows in one channel of every key
      err = (b.float() - a).abs().amax(dim=(0, 1)) / a.abs().amax()
      assert float(err.max()) <= 1e-2, (name_, flags, int(err.argmax()), float(err.max()))
