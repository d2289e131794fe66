"""MI355X-native compute half of the CATCCOS fused operators.

The package is a thin Python face over ``libcatccos_hip.so`` (HIP kernels behind the C ABI
of ``include/catccos_hip.h``).  Importing it does not load the library; the first op does,
and raises if the library has not been built.
"""
from ._abi import (FMT_E1M2, FMT_E2M1, FMT_E4M3, FMT_E5M2, ROUND_LUT, ROUND_RNE, CatccosError)  # noqa: F401
from .ops import *  # noqa: F401,F403
