"""lantern_amd: an MI355X (gfx950) tensor backend for Lantern behind the `Backend` operator API.

`BackendHIP` (backend.py) issues calls into lantern_amd/csrc/liblantern_hip.so, whose C ABI is
declared in include/lantern_hip.h; `Tensor` / `TensorR` (tensor.py) are the op surface models are
written against, with the names of the reference's TensorDifferentiation.scala.
"""
from .backend import BackendHIP, Backend, Buf                      # noqa: F401
from .tensor import (Tensor, TensorR, Random, gradR, gradR_loss,  # noqa: F401
                     set_backend, get_backend, int_array)
from .graph import StepGraph                                       # noqa: F401
