"""MI355X-native decode engine for UV-50M: hand-written gfx950 HIP kernels behind the `ultraviolet.kernels`
decode-attention / KV-cache / sampler entry points of hliuson/ultraviolet.

Sub-packages
  csrc/      HIP kernels and the C-ABI library (libuvmi.so); `python -m ultraviolet_amd.csrc.build`
  kernels/   host-side mirror of `ultraviolet.kernels` (same names, arguments and error behaviour)
  engine/    UV-50M decode engine: weights, decode step, prefill, on-device continuous batching
"""
__version__ = "0.1.0"
