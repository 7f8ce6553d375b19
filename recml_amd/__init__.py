"""MI355X-native HSTU pointwise-SiLU attention (forward and backward).

Public surface mirrors the reference operator
(recml/core/ops/hstu_ops.py:829-851), the layer-side call
(recml/layers/keras/hstu.py:356-390) and, as a harness around the kernel, the
HSTU block and model forward (recml/layers/keras/hstu.py:240-621).
"""

from recml_amd.hstu_ops import (  # noqa: F401
    AttentionBatch,
    MaskType,
    hstu_attention,
    hstu_attention_autograd,
    hstu_attention_bwd,
    pointwise_attention,
    pointwise_splash_attention,
)
from recml_amd.hstu_block_ops import embed_norm, gemm_silu, layer_norm, norm_gate, norm_gate_bwd  # noqa: F401
from recml_amd.masks import make_attention_mask, make_causal_mask  # noqa: F401
from recml_amd.hstu_layer import HSTU, HSTUBlock  # noqa: F401
from recml_amd.hstu_bias import (  # noqa: F401
    RelativeBucketedTimeAndPositionBasedBias,
    RelativePositionalBias,
    default_bucketization,
)
