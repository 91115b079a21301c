"""Host-side mirror of the reference's ``nanovllm/kernels`` compressors, running on HIP kernels."""
from .batched_compress import BatchedGEMMCompressor  # noqa: F401
from .kvpress_compressor import KVPressCompressor, create_kvpress_compressor  # noqa: F401
from .minicpm_compressor import MiniCPMKVCompressor  # noqa: F401
from .fused_compress import FusedCompressor, fused_linear_relu_dropout  # noqa: F401
