"""Drop-in name for the reference's ``ddf`` package (its ``ddf/__init__.py:1``
star-imports ``ddf/ddf.py``): ``from ddf import ddf, DDFPack`` resolves to the
gfx950 implementation in ``ddfnet_amd``."""
from ddfnet_amd import (DDFFunction, DDFPack, DDFUpPack, FilterNorm, OP_DICT,  # noqa: F401
                        build_channel_branch, build_spatial_branch, ddf)
