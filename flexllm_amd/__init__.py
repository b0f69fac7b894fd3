"""flexllm_amd: FlexLLM's quantized-transformer datapath on one MI355X (gfx950).

The compute lives in libflexllm_hip.so (hand-written HIP, C ABI in include/flexllm_hip.h); this
package is the thin Python host side: library loading, device buffers, synthetic inputs and the
Llama-3.2-1B W8A8 model wrapper.  There is no CPU fallback: importing works without a GPU, calling
an operator without the built library or without a device raises.
"""
from ._lib import lib, LibraryMissing, check, LIB_PATH  # noqa: F401
from .device import DeviceArray, Stream, Event, to_device, empty, zeros  # noqa: F401
from . import ops, synth  # noqa: F401
