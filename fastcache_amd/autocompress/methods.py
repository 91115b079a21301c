"""KV quantisation with the reference's call surface (``QuantizationMethod``,
nanovllm/autocompress/methods.py:520-757), computed by HIP kernels.

Built: ``int8`` (symmetric, one scale per row of the last dimension), ``int4`` and ``nf4`` (one scale per
group of ``group_size`` elements, two codes per byte).  Two expressions of the reference do not run as
written — the int4 packing applies ``|`` to floating tensors (:665) and the NF4 look-up indexes a table
with ``uint8`` tensors (:725-733) — so for those the packing and look-up they describe are what is built.
Not built: the fp8 cast variants and asymmetric int8 (``symmetric=False``), which raise.
"""
from __future__ import annotations

from enum import Enum, auto
from typing import Tuple

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
        raise FastcacheError(f"{self.name}: the fp8 cast variants are not part of this build")

    def _quantize_int8(self, tensor: torch.Tensor):
        if not self._symmetric:
            raise FastcacheError("asymmetric int8 quantisation is not part of this build")
        return ops.quantize_rows(tensor, 8)

    def _quantize_int4(self, tensor: torch.Tensor):
        return ops.quantize_group4(tensor, self._group_size, nf4=False)

    def _quantize_nf4(self, tensor: torch.Tensor):
        return ops.quantize_group4(tensor, self._group_size, nf4=True)

    def dequantize(self, quantized: torch.Tensor, scale: torch.Tensor, dtype: torch.dtype = torch.float16) -> torch.Tensor:
        t = self._quant_type
        if t == self.QuantType.INT8:
            return ops.dequantize_rows(quantized, scale, dtype)
        if t in (self.QuantType.INT4, self.QuantType.NF4):
            return ops.dequantize_group4(quantized, scale, self._group_size, t == self.QuantType.NF4, dtype)
        raise FastcacheError(f"{self.name}: the fp8 cast variants are not part of this build")
