"""MI355X-native HSTU pointwise-SiLU attention (forward).

Public surface mirrors the reference operator
(recml/core/ops/hstu_ops.py:829-851) and the layer-side call
(recml/layers/keras/hstu.py:356-390).
"""

from recml_amd.hstu_ops import (  # noqa: F401
    MaskType,
    hstu_attention,
    pointwise_attention,
    pointwise_splash_attention,
)
from recml_amd.masks import make_attention_mask, make_causal_mask  # noqa: F401
