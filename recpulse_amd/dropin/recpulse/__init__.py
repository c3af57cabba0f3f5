"""`recpulse` — the Python layer of the drop-in: Module, Linear, Conv2d, LSTMCell and GRUCell over `recpulse_cuda`.

Only the layers whose cost is the matmul path are provided here; the behaviour
each one keeps is cited in `recpulse.module`.
"""
__version__ = "0.2.0b1+mi355x"

from recpulse.module import Conv2d, GRUCell, Linear, LSTMCell, Module

__all__ = ["Module", "Linear", "Conv2d", "LSTMCell", "GRUCell"]
