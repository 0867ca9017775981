"""ferrite_amd: MI355X (gfx950) implementation of Ferrite's quantized linear path: the EXL3 trellis linear and the
NVFP4 prompt linear, behind the reference's fe-exl3 / fe-fp4 layer API. The product is the C-ABI library
(include/*.h, libferrite_amd.so); these modules are its Python mirror, with torch used only for device memory and
streams."""
from . import _lib  # noqa: F401
from ._lib import FeError  # noqa: F401
