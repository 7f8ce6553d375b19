"""Host-side operator logic that needs no GPU: argument checks of the Python
entry points (same conditions and messages as the reference operator,
recml/core/ops/hstu_ops.py:903-979) and the mask helpers."""

import json
import os

import numpy as np
import pytest
import torch

import recml_amd
from recml_amd import hstu_ops, masks
from oracle import hstu_oracle as O

HERE = os.path.dirname(os.path.abspath(__file__))


def test_mask_helpers_match_reference_literals():
  lit = json.load(open(os.path.join(HERE, "golden", "mask_literals.json")))
  pad = torch.tensor(lit["padding"], dtype=torch.float32)
  np.testing.assert_array_equal(masks.make_attention_mask(pad).numpy(), np.array(lit["attention"], np.float32))
  np.testing.assert_array_equal(masks.make_causal_mask(pad).numpy(), np.array(lit["causal"], np.float32))
  np.testing.assert_array_equal(masks.make_causal_mask(pad).numpy(), O.make_causal_mask(pad.numpy()))
  assert masks.lengths_from_padding_mask(pad).tolist() == [3, 1, 2]
  with pytest.raises(ValueError):
    masks.lengths_from_padding_mask(torch.tensor([[1, 0, 1]]))


def test_mask_type_enum():
  assert recml_amd.MaskType.CAUSAL == "causal" and recml_amd.MaskType.FULL == "full"
  assert recml_amd.MaskType("causal") is recml_amd.MaskType.CAUSAL


def test_no_cpu_path():
  z = torch.zeros((1, 4, 1, 32))
  with pytest.raises(ValueError, match="no CPU path"):
    recml_amd.hstu_attention(z, z, z)
  with pytest.raises(TypeError):
    recml_amd.hstu_attention(np.zeros((1, 4, 1, 32)), z, z)


def test_bench_refuses_more_than_one_gpu():
  import subprocess
  import sys
  root = os.path.dirname(HERE)
  res = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, cwd=root)
  assert res.returncode != 0
  assert "one GPU" in (res.stderr + res.stdout)


def test_product_package_does_not_use_the_oracle():
  # the oracle is test infrastructure: nothing under recml_amd/ may import it
  pkg = os.path.join(os.path.dirname(HERE), "recml_amd")
  for dirpath, _, files in os.walk(pkg):
    for name in files:
      if name.endswith(".py"):
        text = open(os.path.join(dirpath, name)).read()
        assert "import oracle" not in text and "from oracle" not in text, os.path.join(dirpath, name)


def test_library_bucket_thresholds_equal_the_oracle_law():
  """The integer thresholds the kernels bucket time differences by (computed on the host, no GPU
  needed) are the oracle's, for the reference's bucket size and others."""
  import ctypes as C
  import numpy as np
  from recml_amd import _lib
  from oracle import hstu_oracle as O
  lib = _lib.load()
  for size in (0.301, 0.25, 0.4, 0.7, 1.0, 0.15):
    want = O.bucket_thresholds(size)
    out = (C.c_int32 * 256)()
    reach = lib.hstu_attn_bucket_thresholds(C.c_float(size), out, 256)
    assert reach == len(want), size
    got = np.frombuffer(out, dtype=np.int32)
    np.testing.assert_array_equal(got[:reach], want[:256])
    if reach < 256:
      assert (got[reach:] == 2**31 - 1).all()
  assert lib.hstu_attn_bucket_thresholds(C.c_float(-1.0), None, 0) == -4


def test_attention_batch_identity_of_inference_tensors():
  # tensors made under torch.inference_mode() have no version counter: reading it raises
  from recml_amd.hstu_ops import AttentionBatch
  with torch.inference_mode():
    t = torch.arange(5, dtype=torch.int32)
    a = AttentionBatch._ident(t)
    assert a == AttentionBatch._ident(t) and a[0] == t.data_ptr()
  assert AttentionBatch._ident(t) == a                    # read outside the mode as well
  u = torch.arange(5, dtype=torch.int32)
  before = AttentionBatch._ident(u)
  u.add_(1)
  assert AttentionBatch._ident(u) != before               # ordinary tensors: in-place changes are noticed
