"""The one helper of ``megatron/model/utils.py`` that belongs to the softmax path."""
from .fused_softmax import SoftmaxFusionTypes


def get_fusion_type(neox_args):
    """Map the two fusion flags of the run configuration to a ``SoftmaxFusionTypes``:
    ``scaled_upper_triang_masked_softmax_fusion`` selects the causal kernel and takes
    precedence over ``scaled_masked_softmax_fusion`` (mask-tensor kernel); neither set means
    the unfused torch path.  Reference: megatron/model/utils.py:364-370."""
    if neox_args.scaled_upper_triang_masked_softmax_fusion:
        return SoftmaxFusionTypes.upper_triang
    if neox_args.scaled_masked_softmax_fusion:
        return SoftmaxFusionTypes.general
    return SoftmaxFusionTypes.none
