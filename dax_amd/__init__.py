"""dax_amd -- MI355X-native W8A8 (INT8 / FP8-e4m3fn) linear behind DAX's module-swap API.

The arithmetic runs in hand-written HIP kernels (``dax_amd/csrc``) reached through the C ABI
of ``dax_amd/lib/libdaxq.so`` (``include/daxq.h``) and registered as ``torch.ops.daxq.*``.
There is no CPU implementation: using the quantised modules without the built library and
a gfx950 device raises.
"""

__version__ = "0.1.0"
