from .attention import Attention, decode_attention, store_kvcache  # noqa: F401
