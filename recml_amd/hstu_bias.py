"""Trainable bias producers of the HSTU layer, as inputs of the attention kernel.

Mirrors, name for name:
  default_bucketization                        recml/layers/keras/hstu.py:33-55
  RelativePositionalBias                       recml/layers/keras/hstu.py:58-128
  RelativeBucketedTimeAndPositionBasedBias     recml/layers/keras/hstu.py:131-237

Each module holds the reference's weights (`_pos_biases [2 max_len - 1]`,
`_ts_w [num_buckets + 1]`, RandomNormal(0, 0.02)).  `forward(inputs)` returns
the dense bias the reference returns (`[1, n, n]` / `[B, n, n]`), for parity
and for callers that want the dense form.  The fast path never builds it:
`attention_kwargs(timestamps)` hands the tables themselves to
`recml_amd.hstu_attention` / `hstu_attention_autograd`, which fuse the
gathers into the kernel and return the table gradients.  A custom
`bucketization_fn` cannot be fused as a table (the kernels implement the
default law); `attention_kwargs` then hands over the dense bias, which the
kernels take as it is and whose gradient their backward returns, so the
weights behind it train all the same.
"""

from __future__ import annotations

import torch


def default_bucketization(x: torch.Tensor, bucket_size: float = 0.301) -> torch.Tensor:
  """log(clip(|x|, 1, 1e9)) / 0.301 truncated to int (recml/layers/keras/hstu.py:33-55).

  The clipped difference and the bucket size are rounded to float32 as in the
  reference; the logarithm and the quotient are taken in float64, which is the
  bucket law the fused kernels follow on every time difference, boundaries of
  buckets included.
  """
  x = x.abs().clamp(1, int(1e9)).to(torch.float32).to(torch.float64)
  size = float(torch.tensor(bucket_size, dtype=torch.float32))
  return torch.floor(torch.log(x) / size).to(torch.int64)


class RelativePositionalBias(torch.nn.Module):
  """bias[i, j] = w[(n - 1) + j - i], the closed form of the reference's
  pad / tile / reshape / slice recipe (recml/layers/keras/hstu.py:105-113)."""

  def __init__(self, max_len: int, stddev: float = 0.02, device=None, generator=None):
    super().__init__()
    w = torch.randn((2 * max_len - 1,), generator=generator) * stddev
    self._pos_biases = torch.nn.Parameter(w.to(device))
    self.max_len = max_len

  def table(self, n: int | None = None) -> torch.Tensor:
    """The [2n - 1] table the kernel indexes with (n - 1) + j - i: the reference reads the first
    2n - 1 weights for sequences of n <= max_len positions."""
    n = self.max_len if n is None else n
    return self._pos_biases[: 2 * n - 1]

  def forward(self, inputs: torch.Tensor) -> torch.Tensor:
    n = inputs.shape[-1]
    i = torch.arange(n, device=self._pos_biases.device)
    return self.table(n)[(n - 1) + i[None, :] - i[:, None]].unsqueeze(0)


class RelativeBucketedTimeAndPositionBasedBias(torch.nn.Module):
  """Position bias + ts_w[bucket(ts(next item of the query row) - ts(key))]
  (recml/layers/keras/hstu.py:190-235)."""

  def __init__(self, max_len: int, num_buckets: int = 128, bucketization_fn=default_bucketization,
               stddev: float = 0.02, position_bias_layer: RelativePositionalBias | None = None,
               device=None, generator=None):
    super().__init__()
    self._num_buckets = num_buckets
    self._bucketization_fn = bucketization_fn
    self._ts_w = torch.nn.Parameter((torch.randn((num_buckets + 1,), generator=generator) * stddev).to(device))
    self._positional_bias = position_bias_layer or RelativePositionalBias(max_len, stddev, device, generator)

  def time_bias(self, inputs: torch.Tensor) -> torch.Tensor:
    n = inputs.shape[1]
    ext = torch.cat([inputs, inputs[:, n - 1: n]], dim=1)
    diff = ext[:, 1:, None] - ext[:, None, :-1]
    bucket = self._bucketization_fn(diff).clamp(0, self._num_buckets).to(torch.int64)
    return self._ts_w[bucket]

  def forward(self, inputs: torch.Tensor) -> torch.Tensor:
    return self._positional_bias(inputs) + self.time_bias(inputs)

  def attention_kwargs(self, timestamps: torch.Tensor) -> dict:
    """Keyword arguments for hstu_attention / hstu_attention_autograd that apply this bias."""
    n = timestamps.shape[-1]
    if self._bucketization_fn is default_bucketization and self._num_buckets <= 128:
      return dict(pos_bias=self._positional_bias.table(n), timestamps=timestamps, ts_bias=self._ts_w)
    return dict(bias=self.forward(timestamps))
