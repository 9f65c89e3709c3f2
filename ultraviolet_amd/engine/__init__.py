"""UV-50M decode engine on the HIP kernels: configuration, weights, int8 KV state, decode step, packed prefill and the
on-device continuous-batching loop.  Mirrors the inference half of ultraviolet/model.py and
ultraviolet/kernels/fast_decode.py of the reference."""
from .config import PRESETS, UVConfig, as_uvconfig, make_config  # noqa: F401
from .evals import int8_check, teacher_forced_logits  # noqa: F401
from .model import KVState, UVEngine  # noqa: F401
from .weights import UVWeights, random_params  # noqa: F401
