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
