"""Drop-in module name of the reference extension: ``import decdec_ext`` resolves here.

The reference's end-to-end/plugin.py, APLinear.py, LUTGEMMLinear.py and its evaluation code import
``decdec_ext`` and call the functions re-exported below; with this repository's root on
``sys.path`` they run against the gfx950 library unchanged.
"""
from decdec_amd.ext import *  # noqa: F401,F403
from decdec_amd.ext import REFERENCE_API, destroy_dec_context  # noqa: F401
