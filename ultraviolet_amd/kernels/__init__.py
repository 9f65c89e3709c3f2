"""Host-side mirror of `ultraviolet.kernels` (reference: ultraviolet/kernels/__init__.py:9-10): the same public names,
arguments and error behaviour, backed by the gfx950 HIP kernels in libuvmi.so through the C ABI of include/uvmi.h.
There is no CPU implementation here; device tensors are required."""
from .decode_attn import decode_attention, default_splits  # noqa: F401
from .kv_quant import dequantize_kv, kv_append, kv_write, kv_write_rows, quantize_kv  # noqa: F401
from .varlen_attn import packed_attention, varlen_attention  # noqa: F401
