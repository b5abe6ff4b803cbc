"""Drop-in for the reference's compiled `hingetree_cpp` module: re-exports the host-side operator layer."""
from hingetreefortorch_amd.hingetree_cpp import *  # noqa: F401,F403
