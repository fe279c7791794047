"""lightcompress_amd — MI355X (gfx950) kernels behind the LightCompress (`llmc`)
layer-wise quantization API: quantizer primitives, RTN partials, int4 packing, GPTQ and AWQ.

The package is a thin Python mirror of the reference's class API over a C-ABI
shared library (``liblcq.so``, declared in ``include/lcq.h``) of hand-written
HIP kernels.  Build it with ``python -m lightcompress_amd.build``.
"""
from .quant import FloatQuantizer, IntegerQuantizer, Weight48IntegerQuantizer  # noqa: F401
