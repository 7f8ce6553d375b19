"""Properties of the op that hold at any size, checked at the benchmark's full sizes.

The oracle is too slow for whole batches of configuration 3; what does not depend on size is:

  * out is linear in V;
  * sequences do not see each other, whatever order the batch lists them in;
  * a row depends on no later key, value or timestamp (causal mask);
  * heads are independent and see only their own rows of the bias tables;
  * the jagged and the padded layout give the same rows;
  * backward: sum(q dq) = sum(k dk) (the logits are bilinear in q and k and the biases depend on
    neither), sum(v dv) = sum(out dout) (out is linear in v), gradients are linear in dout;
  * with dropout: all of the above for a fixed seed, the second backward identity tying the two
    directions' keep patterns together.

bf16 storage throughout: exact statements are asserted bit for bit, the others to the tolerance of
the parity tests (2e-2 of the largest value).
"""

import numpy as np
import pytest
import torch

import recml_amd
from recml_amd import workloads
from oracle import hstu_oracle as O

pytestmark = pytest.mark.gpu

TOL = 2e-2


def _dev(x, dtype=None):
  t = torch.from_numpy(np.ascontiguousarray(x)).to("cuda:0")
  return t if dtype is None else t.to(dtype)


def _bits(t):
  return t.contiguous().view(torch.int16)


class _C3:
  """Configuration 3 (B=64, max_len=2048, H=8, d=128, jagged, both biases) on the device."""

  def __init__(self):
    w = workloads.config3()
    self.w = w
    bf = torch.bfloat16
    self.q, self.k, self.v = (_dev(t, bf) for t in (w.q, w.k, w.v))
    self.off = _dev(w.seq_offsets)
    self.pos, self.tst, self.ts = _dev(w.pos_tab), _dev(w.ts_tab), _dev(w.timestamps)

  def kwargs(self, **over):
    kw = dict(seq_offsets=self.off, max_len=self.w.L, n=self.w.n, alpha=self.w.alpha,
              pos_bias=self.pos, timestamps=self.ts, ts_bias=self.tst)
    kw.update(over)
    return kw

  def run(self, q=None, k=None, v=None, **over):
    out = recml_amd.hstu_attention(self.q if q is None else q, self.k if k is None else k,
                                   self.v if v is None else v, **self.kwargs(**over))
    torch.cuda.synchronize()
    return out


@pytest.fixture(scope="module")
def c3(gpu):
  return _C3()


def test_linear_in_v(c3):
  g = torch.Generator(device="cuda:0").manual_seed(1)
  v2 = (torch.randn(c3.v.shape, device="cuda:0", generator=g) * 0.1).to(torch.bfloat16)
  # 0.5 and 2 scale bf16 values exactly; the sum of two bf16 tensors is rounded once
  mix = (0.5 * c3.v.float() + 2.0 * v2.float()).to(torch.bfloat16)
  a, b, m = c3.run().float(), c3.run(v=v2).float(), c3.run(v=mix).float()
  want = 0.5 * a + 2.0 * b
  assert (m - want).abs().max().item() <= TOL * want.abs().max().item()


def test_sequences_are_independent_and_order_free(c3):
  base = c3.run()
  w = c3.w
  # overwrite every other sequence with noise: the rest must not move by a bit
  q2, k2, v2 = c3.q.clone(), c3.k.clone(), c3.v.clone()
  for b in range(0, w.B, 2):
    s, e = int(w.seq_offsets[b]), int(w.seq_offsets[b + 1])
    for t in (q2, k2, v2):
      t[s:e].normal_(0.0, 0.3)
  out2 = c3.run(q=q2, k=k2, v=v2)
  for b in range(1, w.B, 2):
    s, e = int(w.seq_offsets[b]), int(w.seq_offsets[b + 1])
    assert torch.equal(_bits(out2[s:e]), _bits(base[s:e])), f"sequence {b} changed"
  # the same sequences listed in reverse order
  order = np.arange(w.B)[::-1]
  idx = np.concatenate([np.arange(w.seq_offsets[b], w.seq_offsets[b + 1]) for b in order])
  lens = w.seq_lens[order]
  off = _dev(np.concatenate([[0], np.cumsum(lens)]).astype(np.int32))
  it = _dev(idx.astype(np.int64))
  out3 = c3.run(q=c3.q[it], k=c3.k[it], v=c3.v[it], seq_offsets=off, timestamps=c3.ts[it])
  assert torch.equal(_bits(out3), _bits(base[it]))


def test_rows_do_not_depend_on_later_positions(c3):
  base = c3.run()
  w = c3.w
  k2, v2, ts2 = c3.k.clone(), c3.v.clone(), c3.ts.clone()
  cuts = {}
  for b in range(w.B):
    s, n = int(w.seq_offsets[b]), int(w.seq_lens[b])
    cut = n // 2 + 1            # positions >= cut change; the last kept row reads the timestamp at cut - 1 + 1
    cuts[b] = cut
    if cut < n:
      k2[s + cut:s + n].normal_(0.0, 0.3)
      v2[s + cut:s + n].normal_(0.0, 0.3)
    if cut + 1 < n:
      ts2[s + cut + 1:s + n] += 977
  out2 = c3.run(k=k2, v=v2, timestamps=ts2)
  for b in range(w.B):
    s = int(w.seq_offsets[b])
    assert torch.equal(_bits(out2[s:s + cuts[b]]), _bits(base[s:s + cuts[b]])), f"sequence {b}"


def test_heads_are_independent(c3):
  base = c3.run()
  perm = torch.tensor([3, 0, 7, 5, 1, 2, 6, 4], device="cuda:0")
  out = recml_amd.hstu_attention(c3.q[:, perm].contiguous(), c3.k[:, perm].contiguous(), c3.v[:, perm].contiguous(),
                                 **c3.kwargs(pos_bias=c3.pos[perm].contiguous(), ts_bias=c3.tst[perm].contiguous()))
  torch.cuda.synchronize()
  assert torch.equal(_bits(out), _bits(base[:, perm]))


def test_jagged_equals_padded_at_full_size(c3):
  base = c3.run()
  w = c3.w
  B, L, H, d = w.B, w.L, w.H, w.d
  qp, kp, vp = (torch.zeros((B, L, H, d), dtype=torch.bfloat16, device="cuda:0") for _ in range(3))
  tsp = torch.zeros((B, L), dtype=torch.int64, device="cuda:0")
  for b in range(B):
    s, n = int(w.seq_offsets[b]), int(w.seq_lens[b])
    qp[b, :n], kp[b, :n], vp[b, :n] = c3.q[s:s + n], c3.k[s:s + n], c3.v[s:s + n]
    tsp[b, :n] = c3.ts[s:s + n]
    tsp[b, n:] = c3.ts[s + n - 1]
  out = recml_amd.hstu_attention(qp, kp, vp, seq_lens=_dev(w.seq_lens), n=w.n, alpha=w.alpha,
                                 pos_bias=c3.pos, timestamps=tsp, ts_bias=c3.tst)
  torch.cuda.synchronize()
  for b in range(B):
    s, n = int(w.seq_offsets[b]), int(w.seq_lens[b])
    assert torch.equal(_bits(out[b, :n]), _bits(base[s:s + n])), f"sequence {b}"
    assert (out[b, n:] == 0).all()


def test_backward_identities_at_full_size(c3):
  g = torch.Generator(device="cuda:0").manual_seed(2)
  dout = (torch.randn(c3.v.shape, device="cuda:0", generator=g) * 0.1).to(torch.bfloat16)
  variant = []
  kw = c3.kwargs()
  kw.pop("n")
  dq, dk, dv, dpos, dts = recml_amd.hstu_attention_bwd(c3.q, c3.k, c3.v, dout, n=c3.w.n, _variant_out=variant, **kw)
  out = c3.run()
  torch.cuda.synchronize()
  assert variant == ["hstu_bwd_mfma_bf16"]
  dot = lambda a, b: (a.double() * b.double()).sum().item()
  # both sides are sums of 16.8 M products that mostly cancel: the tolerance is on the sums themselves
  # (observed: 3e-5 and 2e-4 of them), which a gradient off by a constant factor or one missing tile would break
  qdq, kdk = dot(c3.q, dq), dot(c3.k, dk)
  assert abs(qdq) > 1e-3 and abs(qdq - kdk) <= 5e-3 * abs(qdq), (qdq, kdk)
  vdv, odo = dot(c3.v, dv), dot(out, dout)
  assert abs(odo) > 1e-3 and abs(vdv - odo) <= 5e-3 * abs(odo), (vdv, odo)
  # linear in dout: twice the upstream gradient, twice every gradient (a power of two: exact in bf16, and the
  # table gradients differ only by the order of their atomic sums)
  dq2, dk2, dv2, dpos2, dts2 = recml_amd.hstu_attention_bwd(c3.q, c3.k, c3.v, (2 * dout.float()).to(torch.bfloat16),
                                                            n=c3.w.n, **kw)
  torch.cuda.synchronize()
  for a, b in ((dq, dq2), (dk, dk2), (dv, dv2)):
    assert torch.equal(_bits((2 * a.float()).to(torch.bfloat16)), _bits(b))
  for a, b in ((dpos, dpos2), (dts, dts2)):
    assert (2 * a - b).abs().max().item() <= 1e-3 * b.abs().max().item()


def test_backward_at_full_size_against_the_oracle(c3):
  """The matrix-core backward on the whole of configuration 3, sequence by sequence against the numpy
  oracle: every sequence of up to 320 tokens in fp64 and the longest one (1655 tokens) in fp32.  A
  sequence alone with its slice of the position table is the same problem as the sequence in the batch."""
  w = c3.w
  g = torch.Generator(device="cuda:0").manual_seed(3)
  dout = (torch.randn(c3.v.shape, device="cuda:0", generator=g) * 0.1).to(torch.bfloat16)
  kw = c3.kwargs()
  kw.pop("n")
  variant = []
  dq, dk, dv, _, _ = recml_amd.hstu_attention_bwd(c3.q, c3.k, c3.v, dout, n=w.n, table_grads=False, _variant_out=variant, **kw)
  torch.cuda.synchronize()
  assert variant == ["hstu_bwd_mfma_bf16"]
  got = [t.float().cpu().numpy() for t in (dq, dk, dv)]
  host = [t.float().cpu().numpy() for t in (c3.q, c3.k, c3.v, dout)]
  L = w.L
  lens = np.asarray(w.seq_lens)
  longest = int(np.argmax(lens))
  checked = 0
  for b in range(w.B):
    n = int(lens[b])
    if n == 0 or (n > 320 and b != longest):
      continue
    sl = slice(int(w.seq_offsets[b]), int(w.seq_offsets[b]) + n)
    qb, kb, vb, db = (x[sl][None] for x in host)
    pos = w.pos_tab[:, (L - 1) - (n - 1): (L - 1) + n]          # entries (L-1) + j - i for |j - i| < n
    want = O.hstu_attention_bwd_ref(qb, kb, vb, db, n=w.n, alpha=w.alpha, pos_tab=pos, ts_tab=w.ts_tab,
                                    timestamps=w.timestamps[sl][None], dtype=np.float64 if n <= 320 else np.float32)
    for name, gt, wt in zip(("dq", "dk", "dv"), got, want[:3]):
      err = np.abs(gt[sl] - wt[0]).max() / max(np.abs(wt).max(), 1e-30)
      assert err <= 2e-2, (b, n, name, err)
    checked += 1
  assert checked >= 40


def test_dropout_at_full_size(c3):
  """The training form at configuration 3's size: the pattern is a function of (sequence, head, i, j), so the
  padded layout drops the same pairs bit for bit; out stays linear in V; the backward's identities hold with the
  forward's output on one side -- which they only do when both directions drop the same pairs; and the sequences
  the oracle can afford agree with it."""
  w = c3.w
  B, L, H, d = w.B, w.L, w.H, w.d
  drop = dict(dropout_p=0.3, dropout_seed=0x5EED0123456789)
  base = c3.run(**drop)
  assert not torch.equal(_bits(base), _bits(c3.run()))
  qp, kp, vp = (torch.zeros((B, L, H, d), dtype=torch.bfloat16, device="cuda:0") for _ in range(3))
  tsp = torch.zeros((B, L), dtype=torch.int64, device="cuda:0")
  for b in range(B):
    s, n = int(w.seq_offsets[b]), int(w.seq_lens[b])
    qp[b, :n], kp[b, :n], vp[b, :n] = c3.q[s:s + n], c3.k[s:s + n], c3.v[s:s + n]
    tsp[b, :n] = c3.ts[s:s + n]
    tsp[b, n:] = c3.ts[s + n - 1]
  out = recml_amd.hstu_attention(qp, kp, vp, seq_lens=_dev(w.seq_lens), n=w.n, alpha=w.alpha,
                                 pos_bias=c3.pos, timestamps=tsp, ts_bias=c3.tst, **drop)
  torch.cuda.synchronize()
  for b in range(B):
    s, n = int(w.seq_offsets[b]), int(w.seq_lens[b])
    assert torch.equal(_bits(out[b, :n]), _bits(base[s:s + n])), f"sequence {b}"
  # linear in V with the pattern fixed
  g = torch.Generator(device="cuda:0").manual_seed(3)
  v2 = (torch.randn(c3.v.shape, device="cuda:0", generator=g) * 0.1).to(torch.bfloat16)
  mix = (0.5 * c3.v.float() + 2.0 * v2.float()).to(torch.bfloat16)
  want = 0.5 * base.float() + 2.0 * c3.run(v=v2, **drop).float()
  assert (c3.run(v=mix, **drop).float() - want).abs().max().item() <= TOL * want.abs().max().item()
  # the backward with the same rate and seed
  dout = (torch.randn(c3.v.shape, device="cuda:0", generator=g) * 0.1).to(torch.bfloat16)
  kw = c3.kwargs(**drop)
  dq, dk, dv, _, _ = recml_amd.hstu_attention_bwd(c3.q, c3.k, c3.v, dout, **kw)
  torch.cuda.synchronize()
  dot = lambda a, b: (a.double() * b.double()).sum().item()
  qdq, kdk = dot(c3.q, dq), dot(c3.k, dk)
  assert abs(qdq) > 1e-3 and abs(qdq - kdk) <= 5e-3 * abs(qdq), (qdq, kdk)
  vdv, odo = dot(c3.v, dv), dot(base, dout)
  assert abs(odo) > 1e-3 and abs(vdv - odo) <= 5e-3 * abs(odo), (vdv, odo)
  # ... and with another seed on the backward's side the second identity is gone
  dv_other = recml_amd.hstu_attention_bwd(c3.q, c3.k, c3.v, dout, **c3.kwargs(dropout_p=0.3, dropout_seed=1))[2]
  assert abs(dot(c3.v, dv_other) - odo) > 5e-2 * abs(odo)
  # the oracle on every sequence of up to 200 tokens
  short = [b for b in range(B) if int(w.seq_lens[b]) <= 200]
  assert len(short) >= 8
  f = lambda t: t.float().cpu().numpy()
  ref = O.hstu_attention_jagged_ref(f(c3.q), f(c3.k), f(c3.v), w.seq_offsets, L, n=w.n, alpha=w.alpha, pos_tab=w.pos_tab,
                                    timestamps=w.timestamps, ts_tab=w.ts_tab, sequences=short, **drop)
  got = f(base)
  scale = max(np.abs(ref[int(w.seq_offsets[b]):int(w.seq_offsets[b + 1])]).max() for b in short)
  for b in short:
    s, e = int(w.seq_offsets[b]), int(w.seq_offsets[b + 1])
    assert np.abs(got[s:e] - ref[s:e]).max() <= TOL * scale, b
