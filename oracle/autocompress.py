"""Oracle (test infrastructure): the single-layer fused Linear, the bias-free generated MLP, the
sparse gather and the per-row quantiser of the reference's kernel factories.

Restates ``fused_linear_relu_dropout`` in inference mode (nanovllm/kernels/fused_compress.py:21-178),
``FusedCompressor.compress_layer_fused`` (:307-377), and the eager variants of
``nanovllm/autocompress/kernels.py``: ``mlp_compress`` (:268-288), ``sparse_gather`` (:348-353),
``quantize`` / ``dequantize`` (:387-421).
"""
from __future__ import annotations

from typing import Tuple

import torch


def linear_act(x: torch.Tensor, weight_kn: torch.Tensor, bias, apply_relu: bool) -> torch.Tensor:
    """``act(x @ W + b)`` with ``W [K, N]``: operands in the storage dtype, fp32 accumulation, bias and
    ReLU applied on the fp32 accumulator, one rounding to the storage dtype (the Triton kernel's
    ``acc + b`` -> ``maximum`` -> ``tl.store(acc.to(dtype))``, fused_compress.py:93-118)."""
    acc = x.float() @ weight_kn.float()
    if bias is not None:
        acc = acc + bias.float()[None, :]
    if apply_relu:
        acc = torch.clamp_min(acc, 0.0)
    return acc.to(x.dtype)


def mlp_nobias(X: torch.Tensor, W1: torch.Tensor, W2: torch.Tensor, W3: torch.Tensor) -> torch.Tensor:
    """kernels.py:268-288: ``relu(X @ W1)``, ``relu(. @ W2)``, ``. @ W3`` with every product rounded to the dtype of X."""
    y = linear_act(X, W1, None, True)
    y = linear_act(y, W2, None, True)
    return linear_act(y, W3, None, False)


def fused_compress_layer(k: torch.Tensor, w, cf: int) -> torch.Tensor:
    """fused_compress.py:307-377 for one tensor ``[B, H, S, D]``; ``w = (w1 [cf*D, D], b1, w2, b2, w3, b3)``."""
    B, H, S, D = k.shape
    c = S // cf
    if c < 1:
        return k
    flat = k[:, :, :c * cf, :].reshape(B * H * c, cf * D)
    y = linear_act(flat, w[0], w[1], True)
    y = linear_act(y, w[2], w[3], True)
    y = linear_act(y, w[4], w[5], False).reshape(B, H, c, D)
    return torch.cat([y, k[:, :, c * cf:, :]], dim=2) if S > c * cf else y


def sparse_gather(X: torch.Tensor, indices: torch.Tensor) -> torch.Tensor:
    return X[indices.long()]


def quantize(X: torch.Tensor, bits: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """kernels.py:399-416, the same tensor expression evaluated by torch on the CPU."""
    x_max = X.abs().max(dim=-1, keepdim=True).values
    scale = x_max / (2 ** (bits - 1) - 1)
    scale = scale.clamp(min=1e-8)
    x_quant = (X / scale).round().clamp(-(2 ** (bits - 1)), 2 ** (bits - 1) - 1)
    return x_quant.to(torch.int8), scale


def dequantize(X_quant: torch.Tensor, scale: torch.Tensor, dtype=None) -> torch.Tensor:
    """kernels.py:418-421."""
    if dtype is None:
        dtype = torch.float16
    return X_quant.to(dtype) * scale


# ---- QuantizationMethod (nanovllm/autocompress/methods.py:636-757) ---------------------------------------
NF4_LEVELS = [-1.0, -0.6961928009986877, -0.5250730514526367, -0.39491748809814453, -0.28444138169288635,
              -0.18477343022823334, -0.09105003625154495, 0.0, 0.07958029955625534, 0.16093020141124725,
              0.24611230194568634, 0.33791524171829224, 0.44070982933044434, 0.5626170039176941,
              0.7229568362236023, 1.0]


def quantize_int8(tensor: torch.Tensor):
    """methods.py:639-643 (symmetric)."""
    scale = tensor.abs().amax(dim=-1, keepdim=True) / 127.0
    scale = scale.clamp(min=1e-8)
    return (tensor / scale).round().clamp(-128, 127).to(torch.int8), scale


def quantize_int8_asymmetric(tensor: torch.Tensor):
    """methods.py:644-651 (``symmetric=False``): uint8 codes and ``[..., 2]`` = (scale, zero point)."""
    x_min = tensor.amin(dim=-1, keepdim=True)
    x_max = tensor.amax(dim=-1, keepdim=True)
    scale = (x_max - x_min) / 255.0
    scale = scale.clamp(min=1e-8)
    zero_point = (-x_min / scale).round().clamp(0, 255)
    quantized = ((tensor - x_min) / scale).round().clamp(0, 255).to(torch.uint8)
    return quantized, torch.cat([scale, zero_point], dim=-1)


def quantize_fp8(tensor: torch.Tensor, e5m2: bool = False):
    """methods.py:671-680: one scale for the tensor (448 for both formats), torch's own float8 cast."""
    dtype = torch.float8_e5m2 if e5m2 else torch.float8_e4m3fn
    scale = tensor.abs().amax() / 448.0
    scale = scale.clamp(min=1e-8)
    quantized = (tensor / scale).to(dtype)
    return quantized, scale.expand_as(tensor[..., :1])


def dequantize_fp8(quantized: torch.Tensor, scale: torch.Tensor, dtype=torch.float16):
    """methods.py:735-736."""
    return quantized.to(dtype) * scale


def quantize_int4(tensor: torch.Tensor, group_size: int):
    """methods.py:654-669.  The reference packs with ``|`` on the floating ``quantized`` tensor, which torch
    rejects; the packing it describes (low nibble = even element + 8, high nibble = odd element + 8) is done
    on integers here."""
    shape = tensor.shape
    t = tensor.reshape(-1, group_size)
    scale = t.abs().amax(dim=-1, keepdim=True) / 7.0
    scale = scale.clamp(min=1e-8)
    q = (t / scale).round().clamp(-8, 7).to(torch.int32).view(-1, 2)
    packed = ((q[:, 0] + 8) | ((q[:, 1] + 8) << 4)).to(torch.uint8)
    return packed.view(*shape[:-1], -1), scale.view(*shape[:-1], -1)


def quantize_nf4(tensor: torch.Tensor, group_size: int):
    """methods.py:689-715."""
    table = torch.tensor(NF4_LEVELS, dtype=tensor.dtype)
    shape = tensor.shape
    t = tensor.reshape(-1, group_size)
    scale = t.abs().amax(dim=-1, keepdim=True)
    scale = scale.clamp(min=1e-8)
    normalized = t / scale
    diff = (normalized.unsqueeze(-1) - table).abs()
    q = diff.argmin(dim=-1).to(torch.uint8).view(-1, 2)
    packed = (q[:, 0] | (q[:, 1] << 4)).to(torch.uint8)
    return packed.view(*shape[:-1], -1), scale.view(*shape[:-1], -1)


def dequantize_4bit(packed: torch.Tensor, scale: torch.Tensor, group_size: int, nf4: bool, dtype=torch.float16):
    """methods.py:722-747.  ``unpacked * scale`` only broadcasts in the reference when there is one group per row;
    here every group is scaled by its own factor.  The NF4 look-up indexes with integer (not uint8) tensors."""
    low, high = (packed & 0x0F).long(), ((packed >> 4) & 0x0F).long()
    if nf4:
        table = torch.tensor(NF4_LEVELS, dtype=dtype)
        lo, hi = table[low], table[high]
    else:
        lo, hi = low.to(dtype) - 8, high.to(dtype) - 8
    unpacked = torch.stack([lo, hi], dim=-1).view(*packed.shape[:-1], -1)
    g = unpacked.reshape(-1, group_size) * scale.reshape(-1, 1)
    return g.view(*packed.shape[:-1], -1)
