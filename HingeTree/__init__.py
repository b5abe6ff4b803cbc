"""Drop-in for the reference's `HingeTree` package (HingeTree/__init__.py): same public names for the forest / fern /
convolution path, implemented by hingetreefortorch_amd on the MI355X HIP library."""
from hingetreefortorch_amd.functions import (  # noqa: F401
    HingeTree,
    HingeFern,
    HingeTreeConv1d,
    HingeTreeConv2d,
    HingeTreeConv3d,
    HingeFernConv1d,
    HingeFernConv2d,
    HingeFernConv3d,
    LinearBatchNorm,
    LinearBatchNormForest,
    HingeTreeFusedLinear,
    HingeFernFusedLinear,
    HingeTreeExpanded,
    HingeFernExpanded,
    Contract,
    Expand,
    contract,
    expand,
)
