"""adhip: an MI355X (gfx950) execution backend behind the autodiff-ir-rust `Device` interface.

`adhip.autodiff`, `adhip.nn` and `adhip.Tensor` mirror the reference's caller-side API so that
programs read like the reference's own; `adhip.HipDevice` is the device: it serialises the IR,
hands it to the C-ABI library (`libadhip.so`) and serves `get_tensor`."""
from . import autodiff, ir, nn
from .core import Tensor, Value, ValueData, concat, constant, dot
from .device import Device, HipDevice, library_path

__all__ = ["autodiff", "ir", "nn", "Tensor", "Value", "ValueData", "concat", "constant", "dot",
           "Device", "HipDevice", "library_path"]
