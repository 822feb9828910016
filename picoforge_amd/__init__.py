"""MI355X-native MoE feed-forward path behind the entry points of picoforge's qwen4_moe.h.

The package is a thin host-side layer over picoforge_amd/libpicoforge_moe.so (C11
host + hand-written HIP kernels for gfx950).  Nothing here computes on the CPU:
if the library is missing, loading it raises.
"""
from . import abi  # noqa: F401
from .binding import LibraryMissing, Synth, load_product  # noqa: F401
from .layer import LayerWeights, MoeError, MoeLayer, rms_normalise  # noqa: F401
from .gguf import GgufError, GgufFile  # noqa: F401
