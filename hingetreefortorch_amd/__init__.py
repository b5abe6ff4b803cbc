"""MI355X-native hinge forest / hinge fern forward+backward path behind the HingeTreeForTorch operator API.

    hingetreefortorch_amd.hingetree_cpp   operator layer (tree_forward, tree_backward, ..., conv) over the C ABI
    hingetreefortorch_amd.functions       autograd Functions (HingeTree, HingeFern, HingeTreeConv*d, HingeFernConv*d)
    hingetreefortorch_amd.modules         nn.Modules (RandomHingeForest, RandomHingeFern, HingeTreeConv*d, ...)
    hingetreefortorch_amd.build           hipcc build of libhingetree_hip.so (csrc/, include/hingetree_hip.h)
"""
from . import hingetree_cpp  # noqa: F401
from .functions import HingeFern, HingeTree, LinearBatchNorm, LinearBatchNormForest  # noqa: F401
from .modules import (  # noqa: F401
    HingeFernConv1d,
    HingeFernConv2d,
    HingeFernConv3d,
    HingeTreeConv1d,
    HingeTreeConv2d,
    HingeTreeConv3d,
    LinearHingeForest,
    RandomHingeFernFusedLinear,
    RandomHingeForestFusedLinear,
    RandomHingeFernExpanded,
    RandomHingeForestExpanded,
    RandomHingeFern,
    RandomHingeForest,
)
