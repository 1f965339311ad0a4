"""cyb_amd - MI355X (gfx950) backend for cyb's block-quantized matmul operator.

The package is a thin host-side mirror of the seam the reference runtime has
between its graph executor and a compute backend (cpu | wgpu | Metal -
/root/reference/decide/model-lifecycle.md:25-26,37): `Backend` owns a device,
`QWeight` is one quantised tensor of a loaded model, `QMatMul` is the graph
node, `Backend.run` executes it.  All arithmetic happens in libcybq.so
(hand-written HIP, C ABI in include/cybq.h); this package never computes the
op on the host and raises if the library is missing.
"""
from .backend import Backend, CybqError, QMatMul, QWeight, library_path
from . import container, driver, formats, stack, synth

__all__ = ["Backend", "CybqError", "QMatMul", "QWeight", "library_path", "formats", "synth", "container", "stack", "driver"]
__version__ = "0.1.0"
