"""MI355X-native implementation of PyTorch-BigGraph's per-bucket training step.

Import name: ``pytorch_biggraph_amd`` (the directory is ``pytorch-biggraph_amd``;
``__graft_entry__.load_package()`` registers it under the importable name).
"""
from . import _lib, native  # noqa: F401
from .native import StepRunner, StepSpec  # noqa: F401
