"""The entry points under HIP graph capture.

hstu_attn_fwd and hstu_attn_bwd only enqueue kernels on the caller's stream and
allocate nothing, so a caller may record them into a graph.  Every replay must
redo the whole call, the preparation kernel included: between replays the test
changes the tensors AND the sequence lengths (same token total, so the same
workspace size) in place, and compares each replay with an eager call on the
same buffers.  The forward and dq / dk / dv are deterministic: bit-exact.  The
table gradients are sums of float atomics: tolerance.
"""

import numpy as np
import pytest
import torch

import recml_amd
from recml_amd import hstu_ops, workloads
from oracle import hstu_oracle as O

pytestmark = pytest.mark.gpu

B, L, H, D = 6, 256, 2, 64
LENS = ([256, 40, 130, 1, 97, 200], [97, 256, 1, 200, 40, 130], [120, 121, 122, 119, 118, 124])
T = sum(LENS[0])
assert all(sum(l) == T for l in LENS)


def _batch(seed, lens):
  rng = np.random.Generator(np.random.PCG64(seed))
  lens = np.asarray(lens, np.int32)
  q, k, v, do = (O.round_bf16(rng.standard_normal((T, H, D)).astype(np.float32) * 0.3) for _ in range(4))
  ts = workloads.make_timestamps(rng, lens, L, "jagged")
  off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
  return dict(q=q, k=k, v=v, do=do, ts=ts, off=off)


class _Buffers:
  """Static device buffers a graph can be recorded against."""

  def __init__(self, dev):
    bf = dict(dtype=torch.bfloat16, device=dev)
    self.q, self.k, self.v, self.do = (torch.empty(T, H, D, **bf) for _ in range(4))
    self.ts = torch.empty(T, dtype=torch.int64, device=dev)
    self.off = torch.empty(B + 1, dtype=torch.int32, device=dev)
    rng = np.random.Generator(np.random.PCG64(99))
    self.pos = torch.from_numpy(rng.standard_normal((H, 2 * L - 1)).astype(np.float32) * 0.1).to(dev)
    self.tst = torch.from_numpy(rng.standard_normal((H, 129)).astype(np.float32) * 0.1).to(dev)

  def load(self, batch):
    for name in ("q", "k", "v", "do"):
      getattr(self, name).copy_(torch.from_numpy(batch[name]).to(torch.bfloat16))
    self.ts.copy_(torch.from_numpy(batch["ts"]))
    self.off.copy_(torch.from_numpy(batch["off"]))

  def kwargs(self):
    return dict(seq_offsets=self.off, max_len=L, n=L, pos_bias=self.pos, timestamps=self.ts, ts_bias=self.tst)


def test_forward_replays_in_a_graph(gpu):
  dev = torch.device("cuda:0")
  buf = _Buffers(dev)
  out = torch.empty(T, H, D, dtype=torch.bfloat16, device=dev)
  args, keep = hstu_ops.build_args(buf.q, buf.k, buf.v, out, **buf.kwargs())
  assert hstu_ops.kernel_variant(args) == "hstu_fwd_mfma_bf16"
  buf.load(_batch(0, LENS[0]))
  hstu_ops._run(args, keep)            # eager once: everything that happens on a first call happens here
  torch.cuda.synchronize()

  graph = torch.cuda.CUDAGraph()
  with torch.cuda.graph(graph):
    hstu_ops._run(args, keep)
  torch.cuda.synchronize()

  for rep, lens in enumerate(LENS):
    batch = _batch(10 + rep, lens)
    buf.load(batch)
    out.fill_(float("nan"))
    graph.replay()
    torch.cuda.synchronize()
    replayed = out.clone()
    out.fill_(float("nan"))
    hstu_ops._run(args, keep)
    torch.cuda.synchronize()
    assert torch.equal(replayed.view(torch.int16), out.view(torch.int16)), f"replay {rep} differs from the eager call"
    ref = O.hstu_attention_jagged_ref(batch["q"], batch["k"], batch["v"], batch["off"], L, n=L, alpha=1.0,
                                      pos_tab=buf.pos.cpu().numpy(), timestamps=batch["ts"],
                                      ts_tab=buf.tst.cpu().numpy(), dtype=np.float64)
    got = replayed.float().cpu().numpy()
    assert np.abs(got - ref).max() <= 2e-2 * np.abs(ref).max()


def test_backward_replays_in_a_graph(gpu):
  dev = torch.device("cuda:0")
  buf = _Buffers(dev)
  buf.load(_batch(1, LENS[0]))
  variant = []
  eager = recml_amd.hstu_attention_bwd(buf.q, buf.k, buf.v, buf.do, _variant_out=variant, **buf.kwargs())
  torch.cuda.synchronize()
  assert variant == ["hstu_bwd_mfma_bf16"]

  graph = torch.cuda.CUDAGraph()
  with torch.cuda.graph(graph):
    recorded = recml_amd.hstu_attention_bwd(buf.q, buf.k, buf.v, buf.do, **buf.kwargs())
  torch.cuda.synchronize()

  for rep, lens in enumerate(LENS):
    buf.load(_batch(20 + rep, lens))
    graph.replay()
    torch.cuda.synchronize()
    replayed = [t.clone() for t in recorded]
    eager = recml_amd.hstu_attention_bwd(buf.q, buf.k, buf.v, buf.do, **buf.kwargs())
    torch.cuda.synchronize()
    for name, a, b in zip(("dq", "dk", "dv"), replayed[:3], eager[:3]):
      assert torch.equal(a.view(torch.int16), b.view(torch.int16)), f"replay {rep}: {name} differs from the eager call"
    for name, a, b in zip(("dpos", "dts"), replayed[3:], eager[3:]):
      scale = b.abs().max().item()
      assert scale > 0
      assert (a - b).abs().max().item() <= 1e-4 * scale, f"replay {rep}: {name}"


def test_norm_gate_and_its_gradients_replay_in_a_graph(gpu):
  """The block's norm + gate step and its backward (two kernels: the rows' pass, then the column sums added in a
  fixed order, no memset) recorded into one graph: every replay, with the inputs changed in place between them,
  gives the bits of an eager call -- the column sums included."""
  from recml_amd import hstu_block_ops as B
  bf = torch.bfloat16
  gen = torch.Generator(device="cuda:0").manual_seed(77)
  rows, width = 3001, 512
  fused = torch.randn((rows, 4, width), device="cuda:0", generator=gen).to(bf)
  attn = (torch.randn((rows, width), device="cuda:0", generator=gen) * 3e-3).to(bf)
  dout = torch.randn((rows, width), device="cuda:0", generator=gen).to(bf)
  gamma = (1 + 0.2 * torch.randn(width, device="cuda:0", generator=gen)).to(bf)
  beta = (0.1 * torch.randn(width, device="cuda:0", generator=gen)).to(bf)
  dfused = torch.zeros_like(fused)

  def call():
    out = B.norm_gate(attn, fused[:, 0], gamma, beta, 1e-6)
    return (out,) + B.norm_gate_bwd(attn, fused[:, 0], gamma, beta, dout, 1e-6, du_out=dfused[:, 0])

  call()                                # (library loaded before capture)
  torch.cuda.synchronize()
  graph = torch.cuda.CUDAGraph()
  with torch.cuda.graph(graph):
    recorded = call()
  for rep in range(3):
    attn.mul_(1.5 if rep else 1.0).add_(1e-3 * rep)
    dout.neg_()
    fused.mul_(0.5)
    graph.replay()
    torch.cuda.synchronize()
    replayed = [t.clone() for t in recorded]
    eager = call()
    torch.cuda.synchronize()
    for name, a, b in zip(("out", "d_attn", "d_u", "d_gamma", "d_beta"), replayed, eager):
      assert torch.equal(a, b), f"replay {rep}: {name} differs from the eager call"
