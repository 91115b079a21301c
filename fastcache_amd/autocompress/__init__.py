"""The parts of the reference's ``nanovllm.autocompress`` package that sit on the compression hot path:
kernel factories, the stream manager and the hardware table (nanovllm/autocompress/__init__.py:60-107).
The method adapters and their registry (``get_method`` / ``list_methods``) come without the reference's cost
profiles; the cost model and scheduler are host-side policy and are not part of this build."""
from .context import GPUArch, HardwareProfile, WorkloadContext, detect_hardware, get_hardware_profile  # noqa: F401
from .execution import StreamManager, get_stream_manager  # noqa: F401
from .kernels import (KernelConfig, TileLangKernelGenerator, get_kernel_generator, get_mlp_kernel,  # noqa: F401
                      get_quantize_kernels, get_sparse_gather_kernel)
from .methods import (KVPressMethod, MethodRegistry, MLPCompressionMethod, QuantizationMethod,  # noqa: F401
                      get_method, list_methods)
