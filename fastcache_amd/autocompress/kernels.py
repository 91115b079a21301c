"""Kernel factory with the reference's call surface (nanovllm/autocompress/kernels.py:37-454).

The reference generates TileLang / Triton / eager-torch variants at run time; here every factory
returns a thin callable over the one HIP implementation in libfastcache_hip:

* ``get_mlp_kernel(M, N, K, dtype) -> fn(X, W1, W2, W3)``: bias-free ``relu(relu(X@W1)@W2)@W3``,
  weights ``[in, out]``, each product rounded to the input dtype (kernels.py:158-266);
* ``get_sparse_gather_kernel(dtype) -> fn(X, indices)``: ``X[indices]`` (kernels.py:290-346);
* ``get_quantize_kernels(bits) -> (quantize, dequantize)`` (kernels.py:387-421).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict, Optional, Tuple

import torch

from .. import _lib, ops
from .._lib import FastcacheError


@dataclass
class KernelConfig:
    """kernels.py:37-55; the tile fields are accepted for compatibility and not used (the HIP
    kernels carry their own tiling)."""
    M: int = 640
    N: int = 128
    K: int = 640
    block_M: int = 128
    block_N: int = 128
    block_K: int = 32
    num_threads: int = 128
    num_warps: int = 4
    dtype: str = "float16"
    accum_dtype: str = "float32"
    use_tensor_core: bool = True
    num_stages: int = 3


def _mlp_compress(X: torch.Tensor, W1: torch.Tensor, W2: torch.Tensor, W3: torch.Tensor) -> torch.Tensor:
    """Three bias-free Linears with ReLU after the first two.  When the layer widths are the CCM ones
    (hidden 128, input a multiple of 128) the chain is one fused launch; otherwise one launch per layer."""
    M, K = X.shape
    N1, N2, N3 = W1.shape[1], W2.shape[1], W3.shape[1]
    if N1 == N2 == N3 == 128 and K % 128 == 0 and X.is_contiguous():
        cf = K // 128
        zeros = torch.zeros((1, 128), dtype=X.dtype, device=X.device)
        w = (W1.t().contiguous().unsqueeze(0), zeros, W2.t().contiguous().unsqueeze(0), zeros,
             W3.t().contiguous().unsqueeze(0), zeros)
        src = X.view(1, 1, M * cf, 128)          # row j of X = tokens [cf*j, cf*j + cf) of one head
        out = torch.empty((1, 1, M, 128), dtype=X.dtype, device=X.device)
        ops.ccm_mlp(_lib.dense_view(src), _lib.dense_view(out), w, cf, 0, M * cf, 0)
        return out.view(M, 128)
    y = ops.linear_act(X, W1.t().contiguous(), None, True)
    y = ops.linear_act(y, W2.t().contiguous(), None, True)
    return ops.linear_act(y, W3.t().contiguous(), None, False)


def _sparse_gather(X: torch.Tensor, indices: torch.Tensor) -> torch.Tensor:
    """``X[indices]`` for ``X [S, 128]`` and an ascending 1-D index tensor."""
    if X.dim() != 2 or X.shape[1] != 128:
        raise FastcacheError(f"sparse_gather: X must be [S, 128], got {tuple(X.shape)}")
    _lib.require_gpu(indices, "indices")
    n = indices.numel()
    Y = torch.empty((n, 128), dtype=X.dtype, device=X.device)
    if n == 0:
        return Y
    idx = indices.to(torch.int32).contiguous().view(1, 1, 1, n)
    src, dst = _lib.dense_view(X.contiguous().view(1, 1, X.shape[0], 128)), _lib.dense_view(Y.view(1, 1, n, 128))
    ops.compact(src, src, dst, dst, idx)
    return Y


class TileLangKernelGenerator:
    """Name kept from the reference (kernels.py:58-421); hands out the HIP-backed callables."""

    def __init__(self):
        self._kernel_cache: Dict[str, Any] = {}

    def generate_mlp_compress_kernel(self, config: KernelConfig) -> Callable:
        return self._kernel_cache.setdefault(f"mlp_{config.M}_{config.N}_{config.K}_{config.dtype}", _mlp_compress)

    def generate_sparse_gather_kernel(self, config: KernelConfig) -> Callable:
        return self._kernel_cache.setdefault(f"sparse_gather_{config.M}_{config.N}_{config.dtype}", _sparse_gather)

    def generate_quantize_kernel(self, bits: int = 4) -> Callable:
        def quantize(X, bits=bits):
            return ops.quantize_rows(X, bits)
        return self._kernel_cache.setdefault(f"quantize_{bits}", quantize)

    def generate_dequantize_kernel(self, bits: int = 4) -> Callable:
        def dequantize(X_quant, scale, dtype=None):
            return ops.dequantize_rows(X_quant, scale, torch.float16 if dtype is None else dtype)
        return self._kernel_cache.setdefault(f"dequantize_{bits}", dequantize)


_kernel_generator: Optional[TileLangKernelGenerator] = None


def get_kernel_generator() -> TileLangKernelGenerator:
    global _kernel_generator
    if _kernel_generator is None:
        _kernel_generator = TileLangKernelGenerator()
    return _kernel_generator


def get_mlp_kernel(M: int, N: int, K: int, dtype: str = "float16") -> Callable:
    return get_kernel_generator().generate_mlp_compress_kernel(KernelConfig(M=M, N=N, K=K, dtype=dtype))


def get_sparse_gather_kernel(dtype: str = "float16") -> Callable:
    return get_kernel_generator().generate_sparse_gather_kernel(KernelConfig(dtype=dtype))


def get_quantize_kernels(bits: int = 4) -> Tuple[Callable, Callable]:
    gen = get_kernel_generator()
    return gen.generate_quantize_kernel(bits), gen.generate_dequantize_kernel(bits)
