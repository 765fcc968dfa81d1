"""MI355X (gfx950) backend for the mixture-of-experts layer of ml_dataflow's operator API.

The product is the C-ABI library under ml_dataflow_amd/lib (sources in ml_dataflow_amd/csrc, headers in
include/); this package only binds it for Python callers.
"""
from . import binding  # noqa: F401
from .backend import Backend, MoeLayer, DeviceBuffer  # noqa: F401
