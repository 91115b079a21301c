"""The engine loop around the compression hooks, and the lazy (threshold-triggered) compression policy.

``CompressionEngine.step`` follows ``LlavaLLMEngine.step`` (nanovllm/engine/llava_engine.py:187-272):
schedule, run the model, compress after prefill (synchronously, or on the side stream with the wait moved
in front of the first decode of those sequences), release the freed blocks, post-process.  The model
forward is not part of this build: ``model_step(seqs, is_prefill) -> token ids`` is supplied by the caller
(a real model writing its KV through the runner's pool, or a synthetic stand-in).

``LazyCompressionEngine`` plays the part of nanovllm_fastapi_server.py:54-153: no compression after prefill;
when the free blocks fall under a fraction of the pool, every running sequence not yet compressed is
compressed in one batch and its tail blocks are released.  It keeps no set of its own: the scheduler's
running queue and ``Sequence.is_compressed`` are the state.
"""
from __future__ import annotations

import time
from dataclasses import dataclass
from typing import Callable, Dict, List, Optional, Tuple

from .kv_runner import PagedKVRunner
from .llm_hooks import free_compressed_blocks
from .scheduler import LlavaScheduler
from .sequence import Sequence, SequenceStatus


@dataclass
class SamplingParams:
    temperature: float = 1.0
    max_tokens: int = 64
    ignore_eos: bool = False


class CompressionEngine:
    def __init__(self, scheduler: LlavaScheduler, model_runner: PagedKVRunner,
                 model_step: Callable[[List[Sequence], bool], List[int]], enable_compression: bool = True,
                 async_compression: bool = False, decode_overlap=None):
        self.scheduler = scheduler
        self.model_runner = model_runner
        if getattr(model_runner, "block_manager", False) is None:      # lets the runner un-share pages it rewrites
            model_runner.block_manager = scheduler.block_manager
        self.model_step = model_step
        self.enable_compression = enable_compression
        self.async_compression = async_compression
        self.decode_overlap = decode_overlap          # a DecodeOverlapCompressor: compress a few layers per decode step
        self._pending_compression_events: Dict[int, object] = {}
        self.total_compression_time = 0.0
        self.total_freed_blocks = 0

    def add_request(self, prompt: List[int], sampling_params: Optional[SamplingParams] = None) -> Sequence:
        seq = Sequence(prompt, sampling_params or SamplingParams())
        self.scheduler.add(seq)
        return seq

    def is_finished(self) -> bool:
        return self.scheduler.is_finished()

    def step(self, apply_compression: bool = False) -> Tuple[list, int]:
        seqs, is_prefill = self.scheduler.schedule()
        if not is_prefill and self.async_compression and self.enable_compression:
            self._wait_pending_compressions(seqs)
            self._free_compressed_blocks(seqs)
        token_ids = self.model_step(seqs, is_prefill)
        compress_now = apply_compression and is_prefill and self.enable_compression
        if self.decode_overlap is not None and self.enable_compression:
            # kv-cache pipeline/nanovllm/engine/llava_engine.py: start after prefill, advance after every decode step
            if compress_now:
                self.decode_overlap.start_decode_overlap_compression(seqs)
            elif not is_prefill:
                self._free_compressed_blocks(self.decode_overlap.step_decode_overlap_compression(seqs))
            compress_now = False
        if compress_now and not self.async_compression:
            sec, _ = self.model_runner.compress_kv_cache_batch(seqs)
            self.total_compression_time += sec
            self._free_compressed_blocks(seqs)
        if compress_now and self.async_compression:
            self._start_pipeline_compression(seqs)
        self.scheduler.postprocess(seqs, token_ids)
        outputs = [(seq.seq_id, seq[seq.num_prompt_tokens:]) for seq in seqs if seq.status == SequenceStatus.FINISHED]
        for seq_id, _ in outputs:
            self.model_runner.clear_compressed_lens([seq_id])
        num_tokens = sum(len(seq) for seq in seqs) if is_prefill else -len(seqs)
        return outputs, num_tokens

    def _start_pipeline_compression(self, seqs: List[Sequence]) -> None:
        event = self.model_runner.start_background_compression(seqs)
        if event is not None:
            for seq in seqs:
                self._pending_compression_events[seq.seq_id] = event

    def _wait_pending_compressions(self, seqs: List[Sequence]) -> None:
        for seq in seqs:
            event = self._pending_compression_events.pop(seq.seq_id, None)
            if event is not None:
                event.synchronize()

    def _free_compressed_blocks(self, seqs: List[Sequence]) -> None:
        todo = [s for s in seqs if not s.is_compressed]      # a sequence is shortened once
        self.total_freed_blocks += free_compressed_blocks(self.scheduler.block_manager, self.model_runner, todo)


class LazyCompressionEngine:
    """Memory-pressure policy on top of a ``CompressionEngine`` (the role of nanovllm_fastapi_server.py:54-153):
    prefills leave the caches whole; before a step, if fewer than ``compression_threshold`` of the pool's pages are
    free, every running sequence that still holds its full cache is compressed in ONE batched pass and its tail
    pages go back to the pool, where the same step's scheduler can hand them to waiting requests.

    Nothing is remembered between steps: the candidates are read off the scheduler's running queue (a sequence is
    there only after its prefill ran, and ``Sequence.is_compressed`` says whether it was shortened), so a pre-empted
    or finished sequence needs no bookkeeping here.  A sequence that has decoded since its prefill holds
    ``len(seq) - 1`` KV rows (the last token's row is written by the next step); like the reference this pass hands
    ``len(seq)`` rows to the compressor there."""

    def __init__(self, llm: CompressionEngine, compression_threshold: float = 0.3,
                 compression_backend: str = "kvpress"):
        self.llm = llm
        self.compression_threshold = compression_threshold
        self.compression_backend = compression_backend
        self._pass_seconds: List[float] = []          # wall time of every batched pass so far

    # -- the pool, as the policy sees it ---------------------------------------------------------------
    @property
    def total_blocks(self) -> int:
        return len(self.llm.scheduler.block_manager.blocks)

    @property
    def threshold_blocks(self) -> int:
        return int(self.total_blocks * self.compression_threshold)

    def candidates(self) -> List[Sequence]:
        return [s for s in self.llm.scheduler.running if not s.is_compressed]

    @property
    def uncompressed_seqs(self) -> set:
        """Ids of the running sequences with a full cache (the reference keeps this as a mutable set)."""
        return {s.seq_id for s in self.candidates()}

    def under_pressure(self) -> bool:
        return len(self.llm.scheduler.block_manager.free_block_ids) < self.threshold_blocks

    # -- engine surface -----------------------------------------------------------------------------------
    def add_request(self, prompt, sampling_params=None):
        return self.llm.add_request(prompt, sampling_params)

    def is_finished(self) -> bool:
        return self.llm.is_finished()

    def step(self):
        if self.under_pressure():
            self.compress_running()
        return self.llm.step(apply_compression=False)

    def compress_running(self) -> int:
        """Compress every candidate now; returns how many sequences were shortened."""
        todo = self.candidates()
        if not todo:
            return 0
        t0 = time.perf_counter()
        self.llm.model_runner.compress_kv_cache_batch(todo)
        self.llm._free_compressed_blocks(todo)
        self._pass_seconds.append(time.perf_counter() - t0)
        return len(todo)

    _do_batch_compression = compress_running          # the reference's name for the pass

    # -- statistics ---------------------------------------------------------------------------------------
    @property
    def compression_count(self) -> int:
        return len(self._pass_seconds)

    @property
    def total_compression_time(self) -> float:
        return sum(self._pass_seconds)

    def get_stats(self) -> dict:
        n, total_ms = self.compression_count, self.total_compression_time * 1000
        return {"compression_count": n, "total_compression_time_ms": total_ms,
                "avg_compression_time_ms": total_ms / n if n else 0}
