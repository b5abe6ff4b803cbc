"""Drop-in for the reference's compiled `hingetree_cpp` module: `import hingetree_cpp` yields the host-side operator
layer of this package (the same module object, so its attributes can be inspected and patched under either name)."""
import sys

from hingetreefortorch_amd import hingetree_cpp as _impl

sys.modules[__name__] = _impl
