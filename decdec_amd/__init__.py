"""MI355X (gfx950) implementation of DecDEC's decode-time linear-layer path.

``decdec_amd.ext``     the reference's ``decdec_ext`` op surface (ctypes over libdecdec_hip.so)
``decdec_amd.formats`` packers / quantisers for the four on-device data formats
``decdec_amd.linear``  nn.Module wrappers with the reference's DECLinear interface
``decdec_amd.build``   hipcc build recipe
"""
__version__ = "0.1.0"
