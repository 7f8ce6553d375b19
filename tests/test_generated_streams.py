"""The hand-scheduled instruction streams that the kernels include are generated files kept in the tree: each must be
what its generator writes today, or the library is not built from the sources next to it."""

import os
import subprocess
import sys

import pytest

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "recml_amd", "csrc")


@pytest.mark.parametrize("gen,inc", [("gen_fwd_stream.py", "hstu_fwd_stream_d128.inc"), ("gen_bwd_stream.py", "hstu_bwd_stream_d128.inc")])
def test_generated_file_is_current(tmp_path, gen, inc):
  out = tmp_path / inc
  subprocess.run([sys.executable, os.path.join(CSRC, gen), "--out", str(out)], check=True, capture_output=True)
  assert out.read_text() == open(os.path.join(CSRC, inc)).read()


def test_backward_stream_pads_and_waits():
  # the emitter's own rules on a hand case: a vector read of a matrix result waits 11 states, a matrix read of a
  # vector result 2, and an LDS read is waited for with the count of the reads issued behind it
  sys.path.insert(0, CSRC)
  try:
    import gen_bwd_stream as G
  finally:
    sys.path.pop(0)
  em = G.Emitter()
  em.mfma("mfma v[0:15]", writes=tuple(range(16)))
  em.valu("v_mul v20, v0, v0", reads=(0,), writes=(20,))
  assert em.lines[1] == "s_nop 7" and em.lines[2] == "s_nop 2" and em.lines[3].startswith("v_mul")   # 11 states in between
  em.mfma("mfma v[32:47], v20", ab_reads=(20,), writes=tuple(range(32, 48)))
  assert em.lines[4] == "s_nop 1"                                                                      # 2 states in between
  em.lds("ds_read v50", "a", writes=(50,))
  em.lds("ds_read v51", "b", writes=(51,))
  em.need("a")
  assert em.lines[-1] == "s_waitcnt lgkmcnt(1)"
  em.need("a")                                   # already waited for
  assert em.lines[-1] == "s_waitcnt lgkmcnt(1)" and len(em.lines) == 9
