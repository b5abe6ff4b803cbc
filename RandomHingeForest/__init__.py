"""Drop-in for the reference's `RandomHingeForest` package (RandomHingeForest/__init__.py): same module names for the
forest / fern / convolution path, implemented by hingetreefortorch_amd on the MI355X HIP library."""
from hingetreefortorch_amd.modules import (  # noqa: F401
    RandomHingeForest,
    RandomHingeFern,
    HingeTreeConv1d,
    HingeTreeConv2d,
    HingeTreeConv3d,
    HingeFernConv1d,
    HingeFernConv2d,
    HingeFernConv3d,
    LinearHingeForest,
    RandomHingeForestFusedLinear,
    RandomHingeFernFusedLinear,
    RandomHingeForestExpanded,
    RandomHingeFernExpanded,
)
