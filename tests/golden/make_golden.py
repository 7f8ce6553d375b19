"""Writes the golden fixtures in this directory from the fp64 brute-force oracle.

  python tests/golden/make_golden.py

Nothing here touches the reference checkout: inputs come from
recml_amd.workloads (seeded numpy generators), outputs from the pure-Python
loops of oracle.hstu_oracle.hstu_attention_bruteforce.  The 3x3 mask literals
in mask_literals.json are the data of the reference's own test
(recml/layers/keras/utils_test.py:38-76).
"""

import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import hstu_oracle as O  # noqa: E402
from recml_amd import workloads  # noqa: E402


def jagged_bruteforce(w, q, k, v):
  out = np.zeros(q.shape, dtype=np.float64)
  L = w.L
  for b in range(w.B):
    s, e = int(w.seq_offsets[b]), int(w.seq_offsets[b + 1])
    m = e - s
    if m == 0:
      continue
    out[s:e] = O.hstu_attention_bruteforce(
        q[s:e][None], k[s:e][None], v[s:e][None], n=w.n, alpha=w.alpha,
        pos_tab=w.pos_tab[:, L - m: L + m - 1],
        timestamps=w.timestamps[s:e][None], ts_tab=w.ts_tab)[0]
  return out


def main():
  w = workloads.config1()
  out = O.hstu_attention_bruteforce(w.q, w.k, w.v, n=w.n)
  np.savez_compressed(os.path.join(HERE, "config1_fp64.npz"), out=out,
                      q_sum=np.float64(w.q.astype(np.float64).sum()))

  w = workloads.small_jagged()
  out = jagged_bruteforce(w, w.q, w.k, w.v)
  qb, kb, vb = (O.round_bf16(t) for t in (w.q, w.k, w.v))
  outb = jagged_bruteforce(w, qb, kb, vb)
  np.savez_compressed(os.path.join(HERE, "small_jagged_fp64.npz"), out=out,
                      out_bf16_inputs=outb, seq_offsets=w.seq_offsets)

  th = O.bucket_thresholds()
  np.savez_compressed(os.path.join(HERE, "bucket_table.npz"), thresholds=th,
                      boundary_set=O.bucket_boundary_set())

  with open(os.path.join(HERE, "mask_literals.json"), "w") as f:
    json.dump({
        "padding": [[1, 1, 1], [1, 0, 0], [1, 1, 0]],
        "attention": [[[1, 1, 1], [1, 1, 1], [1, 1, 1]],
                      [[1, 0, 0], [0, 0, 0], [0, 0, 0]],
                      [[1, 1, 0], [1, 1, 0], [0, 0, 0]]],
        "causal": [[[1, 0, 0], [1, 1, 0], [1, 1, 1]],
                   [[1, 0, 0], [0, 0, 0], [0, 0, 0]],
                   [[1, 0, 0], [1, 1, 0], [0, 0, 0]]],
    }, f, indent=1)


if __name__ == "__main__":
  main()
