"""Mask helpers of the HSTU layer, for torch tensors.

make_attention_mask / make_causal_mask keep the reference's names and results
(recml/layers/keras/utils.py:29-41).  The attention kernel itself never needs
the [B, L, L] mask they build: for an end-padded batch it takes the per-
sequence lengths, which `lengths_from_padding_mask` extracts.
"""

from __future__ import annotations

import torch


def make_attention_mask(mask: torch.Tensor, dtype=torch.float32) -> torch.Tensor:
  """[B, L] padding mask -> [B, L, L] pairwise mask (utils.py:29-36)."""
  return (mask.unsqueeze(-1) * mask.unsqueeze(-2)).to(dtype)


def make_causal_mask(mask: torch.Tensor, dtype=torch.float32) -> torch.Tensor:
  """[B, L] padding mask -> [B, L, L] causal mask (utils.py:39-41)."""
  return torch.tril(make_attention_mask(mask, dtype=dtype))


def lengths_from_padding_mask(mask: torch.Tensor) -> torch.Tensor:
  """Lengths of an END-padded batch ([B, L] of 0/1 with all 1s first).

  Raises ValueError when a row is not a prefix of ones: such a batch needs
  the explicit-mask form of the op instead of lengths.
  """
  m = mask != 0
  lens = m.sum(dim=-1).to(torch.int32)
  L = m.shape[-1]
  prefix = torch.arange(L, device=m.device).unsqueeze(0) < lens.unsqueeze(-1)
  if not bool((prefix == m).all()):
    raise ValueError("padding mask is not end-padded; pass an explicit mask instead")
  return lens
