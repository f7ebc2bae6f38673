"""MI355X-native (gfx950) quantized-weight linear path behind tinygrad's interfaces: hand-written HIP kernels reached through a
ctypes C-ABI shim.  Public surface mirrors the reference's names: gguf.ggml_data_to_tensor, nn.QuantLinear (nn.Linear.__call__
over raw GGUF blocks)."""
from tinygrad_amd import runtime  # noqa: F401
