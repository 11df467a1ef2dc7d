"""Device kernels: the contract (`api`) and its HIP implementation (`hip`)."""
from .api import AttnRows, Kernels

__all__ = ["AttnRows", "Kernels", "load_hip"]


def load_hip(build_if_missing: bool = True):
    """The HIP kernels of this package; raises when the library cannot be had."""
    from .hip import HipKernels
    return HipKernels.load(build_if_missing=build_if_missing)
