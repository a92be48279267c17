"""The `Dwm` module of the reference (reference: network.py:17-35, whose __init__ names undefined
variables): forward(x, w) is dwm3d(x, w, None, (1, 1, 1)).  The scratch buffers the reference
tried to register are not needed - the engine takes its workspace from torch's allocator."""
from torch import nn

from . import dwm


class Dwm(nn.Module):
    def forward(self, x, w):
        return dwm.dwm3d(x, w, None, (1, 1, 1))
