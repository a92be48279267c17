"""MI355X-native Winograd / DWM convolution behind the API of huangdi95/pytorch_winoconv."""
from ._lib import build, load, LIB_PATH, WinoconvError  # noqa: F401
