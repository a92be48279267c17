"""MI355X-native Winograd / DWM convolution behind the API of huangdi95/pytorch_winoconv.

Same names as the reference package `MakePytorchPlusPlus` (reference: __init__.py:1-9):
AddGPU, Foo, WinoSplit, WinoConcat, DWM, add_gpu, wino_split, wino_concat, and the modules
dwm, matrix_conv, matrix_conv3d, WinoConv, network.  `backend` stands in for the compiled
extension `MakePytorchBackend`: the compiled pybind11 module of that name (csrc/host/, built by build()) where it
exists, else `backend`, a ctypes binding of the same C ABI with the same names and signatures.
"""
from ._lib import build, load, LIB_PATH, WinoconvError  # noqa: F401
from . import backend  # noqa: F401
try:
    from . import MakePytorchBackend  # noqa: F401
    from .MakePytorchBackend import AddGPU, Foo, WinoSplit, WinoConcat, DWM, winograd_conv, split_and_concat  # noqa: F401
except ImportError:
    from .backend import AddGPU, Foo, WinoSplit, WinoConcat, DWM, winograd_conv, split_and_concat  # noqa: F401
from .Add import add_gpu  # noqa: F401
from .Split_and_Concat import wino_split, wino_concat  # noqa: F401
from . import dwm, matrix_conv, matrix_conv3d, WinoConv, network, engine  # noqa: F401
from .WinoConv import Wino, WinoConv2d, WinoConv3d  # noqa: F401
from .network import Dwm  # noqa: F401
