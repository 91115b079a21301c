"""The compression-method adapters of the reference that carry device work: ``MLPCompressionMethod``
(nanovllm/autocompress/methods.py:122-220, a CCM compressor behind ``compress(keys, values, **kwargs)``),
``KVPressMethod`` (:227-495, a press by name) and ``QuantizationMethod`` (:520-757), computed by HIP kernels, and
the factory that hands them out by name (``MethodRegistry`` :787-843, ``get_method`` / ``list_methods`` :846-853).
The cost profiles and timing heuristics the reference attaches to them (A100 constants for its scheduler) are not
carried over.

Built: ``int8`` (one scale per row of the last dimension; ``symmetric=False`` gives uint8 codes with a
``(scale, zero point)`` pair per row), ``int4`` and ``nf4`` (one scale per group of ``group_size`` elements, two
codes per byte), ``fp8`` / ``fp8_e4m3`` / ``fp8_e5m2`` (float8 codes, one scale for the tensor).  Three expressions
of the reference do not run as written — the int4 packing applies ``|`` to floating tensors (:665), the NF4
look-up indexes a table with ``uint8`` tensors (:725-733), and de-quantising asymmetric int8 multiplies
``[..., D]`` codes by the ``[..., 2]`` parameter tensor (:726) — so for the first two the packing and look-up they
describe are what is built, and the third raises here as it does there.
"""
from __future__ import annotations

from enum import Enum, auto
from typing import Dict, List, Tuple

import torch

from .. import ops
from .._lib import FastcacheError


class QuantizationMethod:
    class QuantType(Enum):
        INT8 = auto()
        INT4 = auto()
        FP8_E4M3 = auto()
        FP8_E5M2 = auto()
        NF4 = auto()

    def __init__(self, quant_type: str = "int8", group_size: int = 128, symmetric: bool = True):
        self._quant_type = self._parse_quant_type(quant_type)
        self._group_size = group_size
        self._symmetric = symmetric

    def _parse_quant_type(self, quant_type: str) -> "QuantizationMethod.QuantType":
        mapping = {"int8": self.QuantType.INT8, "int4": self.QuantType.INT4, "fp8": self.QuantType.FP8_E4M3,
                   "fp8_e4m3": self.QuantType.FP8_E4M3, "fp8_e5m2": self.QuantType.FP8_E5M2, "nf4": self.QuantType.NF4}
        return mapping.get(quant_type.lower(), self.QuantType.INT8)     # unknown names mean int8, as in the reference

    @property
    def name(self) -> str:
        return f"quant_{self._quant_type.name.lower()}"

    @property
    def compression_ratio(self) -> float:
        return 4.0 if self._quant_type in (self.QuantType.INT4, self.QuantType.NF4) else 2.0

    def compress(self, keys: torch.Tensor, values: torch.Tensor, **kwargs):
        """``((quantised keys, key scales), (quantised values, value scales))`` (methods.py:604-620)."""
        return self._quantize(keys), self._quantize(values)

    def _quantize(self, tensor: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        t = self._quant_type
        if t == self.QuantType.INT8:
            return self._quantize_int8(tensor)
        if t == self.QuantType.INT4:
            return self._quantize_int4(tensor)
        if t == self.QuantType.NF4:
            return self._quantize_nf4(tensor)
        return self._quantize_fp8(tensor)

    def _quantize_int8(self, tensor: torch.Tensor):
        if not self._symmetric:
            return ops.quantize_rows_asym(tensor)       # (uint8 codes, [..., 2] = scale and zero point)
        return ops.quantize_rows(tensor, 8)

    def _quantize_fp8(self, tensor: torch.Tensor):
        """One scale for the tensor, handed out expanded to ``tensor[..., :1]``'s shape (methods.py:671-680)."""
        q, scale = ops.quantize_fp8(tensor, e5m2=self._quant_type == self.QuantType.FP8_E5M2)
        return q, scale.expand(tensor.shape[:-1] + (1,))

    def _quantize_int4(self, tensor: torch.Tensor):
        return ops.quantize_group4(tensor, self._group_size, nf4=False)

    def _quantize_nf4(self, tensor: torch.Tensor):
        return ops.quantize_group4(tensor, self._group_size, nf4=True)

    def dequantize(self, quantized: torch.Tensor, scale: torch.Tensor, dtype: torch.dtype = torch.float16) -> torch.Tensor:
        t = self._quant_type
        if t == self.QuantType.INT8:
            if quantized.dtype == torch.uint8:
                raise FastcacheError("asymmetric int8 codes cannot be de-quantised: the reference's expression "
                                     "multiplies [..., D] codes by the [..., 2] (scale, zero point) tensor")
            return ops.dequantize_rows(quantized, scale, dtype)
        if t in (self.QuantType.INT4, self.QuantType.NF4):
            return ops.dequantize_group4(quantized, scale, self._group_size, t == self.QuantType.NF4, dtype)
        return ops.dequantize_fp8(quantized, scale, dtype)


class MLPCompressionMethod:
    """A CCM MLP compressor (``BatchedGEMMCompressor``, ``KVCacheLinearDecoupleCompressor``, ...) as a method object.

    ``compress(keys, values, it_len=[image, text], layer_idx=0)`` takes one layer's ``[B, Hkv, S, D]`` tensors (that
    layer's MLP weights) or all layers' ``[L, B, Hkv, S, D]`` and returns tensors of the same rank with the token axis
    shortened.  The reference's body stacks keys and values into one ``[2, B, Hkv, S, D]`` tensor and hands it to a
    compressor that expects a list of per-layer ``(k, v)`` pairs (methods.py:196-207), which only unpacks for a batch
    of exactly two; what it means to do, the compressor applied to this K and V, is what is built."""

    def __init__(self, compressor=None, compression_ratio: float = 5.0, num_layers: int = 32):
        self._compressor = compressor
        self._compression_ratio = compression_ratio
        self._num_layers = num_layers

    @property
    def name(self) -> str:
        return "mlp_compress"

    @property
    def compression_ratio(self) -> float:
        return self._compression_ratio

    def compress(self, keys: torch.Tensor, values: torch.Tensor, **kwargs) -> Tuple[torch.Tensor, torch.Tensor]:
        if self._compressor is None:
            raise RuntimeError("MLP compressor not initialized")
        it_len = kwargs.get("it_len", [0, keys.shape[-2]])
        if keys.dim() == 5:
            out = self._compressor([(k, v) for k, v in zip(keys, values)], it_len=it_len)
            return torch.stack([k for k, _ in out]), torch.stack([v for _, v in out])
        if keys.dim() != 4:
            raise FastcacheError(f"keys must be [B, Hkv, S, D] or [L, B, Hkv, S, D], got {tuple(keys.shape)}")
        layer = int(kwargs.get("layer_idx", 0))
        if hasattr(self._compressor, "compress_layers"):
            # the chunked entry point addresses a layer's weights by its position in the full list
            padded = [(keys, values)] * (layer + 1)
            out = self._compressor.compress_layers(padded, layer, layer + 1, it_len=it_len)
        elif layer == 0:
            out = self._compressor([(keys, values)], it_len=it_len)
        else:
            raise FastcacheError(f"{type(self._compressor).__name__} has no per-layer entry point (layer_idx={layer})")
        return out[0][0], out[0][1]


class KVPressMethod:
    """A press chosen by name, called outside a model (methods.py:227-495).  The press runs on the HIP kernels of
    ``fastcache_amd.presses``; ``compress`` forwards ``module`` / ``hidden_states`` / ``attentions`` from the keyword
    arguments and hands all of them on as the press's ``kwargs`` (``queries``, ``position_embeddings``, ...)."""

    # the names the reference's registry lists (methods.py:244-330); 'h2o' and the others without a press class
    # are listed there and rejected at first use, here as well
    METHOD_NAMES = ("snapkv", "streaming_llm", "observed_attention", "expected_attention", "knorm", "tova", "think",
                    "simlayer", "h2o")

    @staticmethod
    def _press_map():
        from .. import presses
        return {"snapkv": presses.SnapKVPress, "streaming_llm": presses.StreamingLLMPress,
                "observed_attention": presses.ObservedAttentionPress,
                "expected_attention": presses.ExpectedAttentionPress, "knorm": presses.KnormPress,
                "tova": presses.TOVAPress, "think": presses.ThinKPress, "simlayer": presses.SimLayerKVPress,
                "random": presses.RandomPress}

    def __init__(self, method_name: str, compression_ratio: float = 0.5, **method_kwargs):
        self._method_name = method_name.lower()
        self._compression_ratio = compression_ratio
        self._method_kwargs = method_kwargs
        self._press = None

    def _init_press(self):
        if self._press is not None:
            return
        press_class = self._press_map().get(self._method_name)
        if press_class is None:
            raise ValueError(f"Unknown kvpress method: {self._method_name}")
        if self._method_name == "think":
            self._press = press_class(key_channel_compression_ratio=self._compression_ratio, **self._method_kwargs)
        elif self._method_name == "simlayer":
            # the reference passes compression_ratio= here as well, which this press (like kvpress's) cannot take:
            # its ratio is an outcome of the lazy-layer test
            self._press = press_class(**self._method_kwargs)
        else:
            self._press = press_class(compression_ratio=self._compression_ratio, **self._method_kwargs)

    @property
    def name(self) -> str:
        return f"kvpress_{self._method_name}"

    @property
    def press(self):
        self._init_press()
        return self._press

    def compress(self, keys: torch.Tensor, values: torch.Tensor, **kwargs) -> Tuple[torch.Tensor, torch.Tensor]:
        self._init_press()
        return self._press.compress(module=kwargs.get("module"), hidden_states=kwargs.get("hidden_states"),
                                    keys=keys, values=values, attentions=kwargs.get("attentions"), kwargs=kwargs)


class MethodRegistry:
    """Methods by name (methods.py:787-843): ``mlp`` / ``mlp_compress`` / ``batched_gemm``; ``kvpress_<press>`` or
    a bare press name; ``quant_<type>`` or ``int8`` / ``int4`` / ``fp8`` / ``nf4``; anything registered with
    ``register``.  Instances are cached per name and keyword arguments when the arguments are hashable (a compressor
    module is, by identity)."""
    _methods: Dict[str, type] = {}
    _instances: Dict[tuple, object] = {}

    @classmethod
    def register(cls, name: str, method_class: type) -> None:
        cls._methods[name] = method_class

    @classmethod
    def create(cls, name: str, **kwargs):
        try:
            key = (name, frozenset(kwargs.items()))
            hash(key)
        except TypeError:
            key = None
        if key is not None and key in cls._instances:
            return cls._instances[key]
        if name in ("mlp", "mlp_compress", "batched_gemm"):
            instance = MLPCompressionMethod(**kwargs)
        elif name.startswith("kvpress_") or name in KVPressMethod.METHOD_NAMES:
            instance = KVPressMethod(name.replace("kvpress_", ""), **kwargs)
        elif name.startswith("quant_") or name in ("int8", "int4", "fp8", "nf4"):
            instance = QuantizationMethod(name.replace("quant_", ""), **kwargs)
        elif name in cls._methods:
            instance = cls._methods[name](**kwargs)
        else:
            raise ValueError(f"Unknown compression method: {name}")
        if key is not None:
            cls._instances[key] = instance
        return instance

    @classmethod
    def list_methods(cls) -> List[str]:
        names = set(cls._methods) | {"mlp", "mlp_compress"}
        names |= {f"kvpress_{m}" for m in KVPressMethod.METHOD_NAMES}
        names |= {"quant_int8", "quant_int4", "quant_fp8", "quant_nf4"}
        return sorted(names)


def get_method(name: str, **kwargs):
    return MethodRegistry.create(name, **kwargs)


def list_methods() -> List[str]:
    return MethodRegistry.list_methods()
