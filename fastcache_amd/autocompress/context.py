"""Hardware and workload descriptions (reference: nanovllm/autocompress/context.py:14-380).

The reference ships roofline figures for NVIDIA parts only; this build adds the MI355X entry its
kernels are written for and detects it through the ROCm build of torch.
"""
from __future__ import annotations

from dataclasses import dataclass
from enum import Enum, auto
from typing import Dict, Optional


class GPUArch(Enum):
    AMPERE = auto()
    HOPPER = auto()
    ADA = auto()
    VOLTA = auto()
    TURING = auto()
    CDNA3 = auto()      # MI300 series
    CDNA4 = auto()      # MI350 series
    UNKNOWN = auto()


@dataclass
class HardwareProfile:
    """Peak figures of one GPU (the field list of the reference's profile, context.py:27-107) and the two-roof
    estimates built on them."""
    gpu_name: str = "Unknown"
    gpu_arch: GPUArch = GPUArch.UNKNOWN
    compute_capability: tuple = (0, 0)
    fp16_tflops: float = 0.0
    fp32_tflops: float = 0.0
    int8_tops: float = 0.0
    memory_bandwidth_gbps: float = 0.0
    memory_size_gb: float = 0.0
    l2_cache_mb: float = 0.0
    sm_count: int = 0
    max_threads_per_sm: int = 0

    DEFAULT_RIDGE = 150.0      # FLOP per byte assumed when the peaks are unknown

    @property
    def roofline_intensity(self) -> float:
        """The ridge of the roofline: FLOP per byte above which fp16 compute, not memory, is the limit."""
        if self.fp16_tflops <= 0 or self.memory_bandwidth_gbps <= 0:
            return self.DEFAULT_RIDGE
        return self.fp16_tflops * 1e3 / self.memory_bandwidth_gbps

    @staticmethod
    def _decode_work(batch_size: int, seq_len: int, num_heads: int, head_dim: int):
        """(FLOP, bytes) of one decode step's attention over a 16-bit cache: every cached element is read once
        for K and once for V and takes part in one multiply-add."""
        elems = batch_size * seq_len * num_heads * head_dim
        return 2 * elems, 4 * elems

    def is_decode_memory_bound(self, batch_size: int, seq_len: int, num_heads: int = 32, head_dim: int = 128) -> bool:
        flops, nbytes = self._decode_work(batch_size, seq_len, num_heads, head_dim)
        return flops < 0.5 * self.roofline_intensity * max(nbytes, 1)

    def estimate_decode_latency_ms(self, batch_size: int, seq_len: int, num_heads: int = 32,
                                   head_dim: int = 128) -> float:
        """The slower of the two roofs plus 10 microseconds of launch overhead."""
        if self.fp16_tflops <= 0 or self.memory_bandwidth_gbps <= 0:
            raise ValueError(f"{self.gpu_name}: peak figures unknown")
        flops, nbytes = self._decode_work(batch_size, seq_len, num_heads, head_dim)
        seconds = max(nbytes / (self.memory_bandwidth_gbps * 1e9), flops / (self.fp16_tflops * 1e12))
        return seconds * 1e3 + 0.01


@dataclass
class WorkloadContext:
    """Shape of the running inference job (context.py:110-176)."""
    batch_size: int = 1
    seq_len: int = 512
    expected_output_len: int = 100
    num_layers: int = 32
    num_kv_heads: int = 8
    head_dim: int = 128
    hidden_size: int = 4096
    memory_used_gb: float = 0.0
    memory_total_gb: float = 0.0
    avg_output_len: Optional[float] = None
    avg_decode_latency_ms: Optional[float] = None

    @property
    def memory_pressure(self) -> float:
        return 0.0 if self.memory_total_gb <= 0 else self.memory_used_gb / self.memory_total_gb

    @property
    def kv_cache_size_mb(self) -> float:
        return (self.batch_size * self.seq_len * self.num_layers * self.num_kv_heads * self.head_dim * 2 * 2) \
            / (1024 * 1024)

    def estimate_compressed_kv_size_mb(self, compression_ratio: float) -> float:
        return self.kv_cache_size_mb / compression_ratio

    def get_total_decode_time_ms(self, decode_latency_per_token_ms: float) -> float:
        n = self.expected_output_len if self.avg_output_len is None else int(self.avg_output_len)
        return decode_latency_per_token_ms * n


# The reference's table (context.py:181-286) plus the part this build targets.  MI355X: dense
# fp16/bf16 MFMA 2.5 PFLOP/s, fp32 157.3 TFLOP/s, int8 5.0 POP/s, 8 TB/s HBM3E, 288 GB,
# 8 XCDs x 4 MB L2, 256 CUs of 2048 threads; compute_capability carries the gfx number.
_GPU_PROFILES: Dict[str, HardwareProfile] = {
    "MI355X": HardwareProfile("AMD Instinct MI355X", GPUArch.CDNA4, (9, 5), 2500.0, 157.3, 5000.0, 8000.0, 288.0,
                              32.0, 256, 2048),
    "A100": HardwareProfile("NVIDIA A100", GPUArch.AMPERE, (8, 0), 312.0, 156.0, 624.0, 2039.0, 80.0, 40.0, 108, 2048),
    "A100-40GB": HardwareProfile("NVIDIA A100 40GB", GPUArch.AMPERE, (8, 0), 312.0, 156.0, 624.0, 1555.0, 40.0, 40.0,
                                 108, 2048),
    "H100": HardwareProfile("NVIDIA H100", GPUArch.HOPPER, (9, 0), 989.0, 494.0, 1979.0, 3350.0, 80.0, 50.0, 132, 2048),
    "RTX4090": HardwareProfile("NVIDIA RTX 4090", GPUArch.ADA, (8, 9), 165.0, 82.6, 330.0, 1008.0, 24.0, 72.0, 128,
                               1536),
    "RTX4080": HardwareProfile("NVIDIA RTX 4080", GPUArch.ADA, (8, 9), 97.5, 48.7, 195.0, 716.8, 16.0, 64.0, 76, 1536),
    "RTX3090": HardwareProfile("NVIDIA RTX 3090", GPUArch.AMPERE, (8, 6), 71.0, 35.6, 142.0, 936.2, 24.0, 6.0, 82,
                               1536),
    "V100": HardwareProfile("NVIDIA V100", GPUArch.VOLTA, (7, 0), 125.0, 15.7, 62.0, 900.0, 32.0, 6.0, 80, 2048),
}


def detect_hardware() -> HardwareProfile:
    """Match the visible GPU against the table (context.py:289-358); a CPU-only host gives the
    'CPU' profile, an unlisted GPU a profile with the properties torch reports and no peaks."""
    import torch
    if not torch.cuda.is_available():
        return HardwareProfile(gpu_name="CPU", gpu_arch=GPUArch.UNKNOWN)
    name = torch.cuda.get_device_name(0)
    props = torch.cuda.get_device_properties(0)
    arch_name = getattr(props, "gcnArchName", "")
    flat = name.upper().replace(" ", "")
    for key, profile in _GPU_PROFILES.items():
        if key.upper() in flat or (key == "MI355X" and arch_name.startswith("gfx950")):
            profile.memory_size_gb = props.total_memory / (1024 ** 3)
            return profile
    return HardwareProfile(gpu_name=name, compute_capability=torch.cuda.get_device_capability(0),
                           memory_size_gb=props.total_memory / (1024 ** 3), sm_count=props.multi_processor_count,
                           max_threads_per_sm=props.max_threads_per_multi_processor)


def get_hardware_profile(name: Optional[str] = None) -> HardwareProfile:
    """context.py:361-378."""
    if name is not None:
        if name in _GPU_PROFILES:
            return _GPU_PROFILES[name]
        raise ValueError(f"Unknown GPU: {name}. Available: {list(_GPU_PROFILES.keys())}")
    return detect_hardware()
