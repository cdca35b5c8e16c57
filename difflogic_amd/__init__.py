"""difflogic's LogicLayer kernel family for AMD MI355X (gfx950).

Same Python API as the reference package (difflogic/__init__.py:1-3): ``LogicLayer``,
``GroupSum``, ``PackBitsTensor`` and ``CompiledLogicNet``; ``difflogic_amd.difflogic_cuda`` stands in for the
reference's extension module of that name.  ``fuse_group_sum`` (not in the reference) merges a
model's last LogicLayer with the GroupSum after it for training, ``fuse_first_layers`` its first
two LogicLayers (``fuse_for_training``: both); ``FusedAdam`` (not in the
reference) is torch.optim.Adam's update for all weight tensors in one launch.  Importing the package loads
libdifflogic_hip.so; it raises ImportError if the library has not been built.
"""
from . import _lib

_lib.load()

from . import difflogic_cuda  # noqa: E402
from .difflogic import (FusedLogicLayerGroupSum, FusedLogicLayerPair, GroupSum, LogicLayer,  # noqa: E402
                        fuse_first_layers, fuse_for_training, fuse_group_sum)
from .packbitstensor import PackBitsTensor  # noqa: E402
from .compiled_model import CompiledLogicNet  # noqa: E402
from .optim import FusedAdam  # noqa: E402

__all__ = ["LogicLayer", "GroupSum", "PackBitsTensor", "CompiledLogicNet", "difflogic_cuda", "fuse_group_sum",
           "FusedLogicLayerGroupSum", "FusedAdam", "fuse_first_layers", "fuse_for_training", "FusedLogicLayerPair"]
