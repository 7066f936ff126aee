"""MI355X-native Decoupled Dynamic Filter operator.

``from ddfnet_amd import ddf, DDFFunction, DDFPack, DDFUpPack, FilterNorm``
gives the reference's ``ddf`` package surface on hand-written gfx950 kernels.
"""
from .functional import DDFFunction, DDFUpFunction, OP_DICT, ddf, ddf_up  # noqa: F401
from .modules import (DDFPack, DDFUpPack, FilterNorm,  # noqa: F401
                      build_channel_branch, build_spatial_branch)
from ._lib import DDFHipError, LIB_PATH, is_built  # noqa: F401

__version__ = '0.1.0'
