"""Op-level seam: same names as the reference's ``fastfold.model.fastnn.kernel``
(kernel/__init__.py:1-13), every op a hand-written HIP kernel behind the C ABI."""
from .attention_core import fused_attention_core
from .jit.fused_ops import bias_dropout_add, bias_sigmod_ele, bias_ele_dropout_residual
from .layer_norm import FusedLayerNorm as LayerNorm
from .softmax import fused_softmax

__all__ = [
    "bias_dropout_add",
    "bias_sigmod_ele",
    "bias_ele_dropout_residual",
    "LayerNorm",
    "fused_softmax",
    "fused_attention_core",
]
