"""``MiniCPMKVCompressor`` (nanovllm/kernels/minicpm_compressor.py:16-192): the Hybrid compressor
with its image MLPs and ``attention`` heads present, as nano-vllm loads it for MiniCPM-V."""
from __future__ import annotations

import torch
import torch.nn as nn

from ..utils_ccm.module_ccm import _CCMBase, _mlp_list


class MiniCPMKVCompressor(_CCMBase):
    def __init__(self, src_config, compression_factor: int = 5, min_seq_len: int = 2):
        super().__init__()
        self.n_layer = src_config.num_hidden_layers
        self.nhead = src_config.num_key_value_heads
        self.d_model = src_config.hidden_size
        self.head_dim = src_config.hidden_size // src_config.num_attention_heads
        self.compression_factor = compression_factor
        self.min_seq_len = min_seq_len
        self.compress_tk = _mlp_list(self.n_layer, self.head_dim, compression_factor)
        self.compress_tv = _mlp_list(self.n_layer, self.head_dim, compression_factor)
        self.compress_ik = _mlp_list(self.n_layer, self.head_dim, compression_factor)
        self.compress_iv = _mlp_list(self.n_layer, self.head_dim, compression_factor)
        self.attention = nn.ModuleList([nn.Linear(self.head_dim, 1) for _ in range(self.n_layer)])

    @torch.no_grad()
    def forward(self, kv_cache, it_len=[0, 1], forward_mode: str = "val"):
        """``it_len[0] == 0``: the whole sequence through the text MLPs (:154-162); otherwise the
        image/text split (:163-182)."""
        if forward_mode == "train":
            raise NotImplementedError("inference-only build: forward_mode='train' is not supported")
        layers = [kv_cache[i] for i in range(self.n_layer)]
        return self._forward_split(layers, it_len, split=it_len[0] != 0)

    def _paged_segments(self, seq_len, it_len):
        if it_len[0] == 0:
            return [("compress_tk", "compress_tv", 0, seq_len)]
        return super()._paged_segments(seq_len, it_len)
