"""Host-side mirror of the reference's ``utils_ccm`` compressor modules, running on HIP kernels."""
from .module_ccm import CompressibleCache, KVCacheHybridCompressor, KVCacheLinearDecoupleCompressor  # noqa: F401
