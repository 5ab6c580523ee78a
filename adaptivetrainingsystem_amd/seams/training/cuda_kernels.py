"""Import seam `training.cuda_kernels`.

The reference trainer does
    from training.cuda_kernels import FusedLoss, FusedGradClip
(Src/Main_Scripts/training/trainer.py:81).  With this directory's parent on sys.path (or this file
copied over the reference's training/cuda_kernels.py) those names resolve to the gfx950 kernels.
"""
from adaptivetrainingsystem_amd import _lib
from adaptivetrainingsystem_amd.training import FusedGradClip, FusedLoss  # noqa: F401

CUSTOM_KERNELS_AVAILABLE = _lib.is_built()
