"""Host-side mirror of the reference's nano-vllm engine pieces that the compression path touches."""
from .block_manager import Block, BlockManager  # noqa: F401
from .sequence import Sequence, SequenceStatus  # noqa: F401
from .async_compress import AsyncCompressionManager, CompressionState, PipelineAsyncCompressor  # noqa: F401
from .scheduler import LlavaScheduler  # noqa: F401
