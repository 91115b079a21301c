"""Compressor checkpoint files in the reference's layout.

Training saves ``{'epoch', 'model_state_dict': {'compressor': state_dict}, 'optimizer_state_dict',
'scheduler_state_dict', 'loss'}`` (scripts/finetune_llava.py:29-47); the runner accepts that, a flat
``{'model_state_dict': state_dict}`` or a raw state dict, the last two non-strictly
(nanovllm/engine/llava_model_runner.py:447-456, nanovllm/kernels/minicpm_compressor.py:215-223).
Parameter names are ``compress_{tk,tv,ik,iv}.{layer}.{0,3,6}.{weight,bias}`` and
``attention.{layer}.{weight,bias}``, so a file written by the reference loads into this build's modules and
the other way round.  Files are read with ``weights_only=True``: nothing in them is executed.
"""
from __future__ import annotations

import os
from typing import Optional, Tuple

import torch


def save_checkpoint(epoch: int, model, optimizer=None, scheduler=None, loss: float = 0.0, is_best: bool = False,
                    filefoldname: str = "ckpt_store", filename: str = "checkpoint.pth") -> str:
    """scripts/finetune_llava.py:29-47: writes ``last_<filename>`` (and ``best_<filename>``)."""
    os.makedirs(filefoldname, exist_ok=True)
    checkpoint = {
        "epoch": epoch,
        "model_state_dict": {"compressor": model.state_dict()},
        "optimizer_state_dict": optimizer.state_dict() if optimizer is not None else None,
        "scheduler_state_dict": scheduler.state_dict() if scheduler is not None else None,
        "loss": loss,
    }
    path = os.path.join(filefoldname, f"last_{filename}")
    torch.save(checkpoint, path)
    if is_best:
        torch.save(checkpoint, os.path.join(filefoldname, f"best_{filename}"))
    return path


def load_compressor_state(module, path: str, map_location="cpu") -> Tuple[list, list]:
    """Load compressor weights with the runner's fallbacks; returns ``(missing, unexpected)`` key lists
    (both empty for the strict first form)."""
    checkpoint = torch.load(path, map_location=map_location, weights_only=True)
    if isinstance(checkpoint, dict) and "model_state_dict" in checkpoint:
        msd = checkpoint["model_state_dict"]
        if isinstance(msd, dict) and "compressor" in msd:
            module.load_state_dict(msd["compressor"])
            return [], []
        res = module.load_state_dict(msd, strict=False)
    else:
        res = module.load_state_dict(checkpoint, strict=False)
    return list(res.missing_keys), list(res.unexpected_keys)


def load_checkpoint_only_model(model, filename: str = "checkpoint.pth") -> bool:
    """scripts/finetune_llava.py:68-80: model weights only; False when the file does not exist."""
    if not os.path.isfile(filename):
        return False
    load_compressor_state(model, filename)
    return True


def load_checkpoint(model, optimizer=None, scheduler=None, filename: str = "checkpoint.pth") -> Tuple[int, float]:
    """scripts/finetune_llava.py:50-66: ``(start_epoch, loss)``, or ``(0, inf)`` when the file does not exist."""
    if not os.path.isfile(filename):
        return 0, float("inf")
    checkpoint = torch.load(filename, map_location="cpu", weights_only=True)
    model.load_state_dict(checkpoint["model_state_dict"]["compressor"])
    if optimizer is not None and checkpoint.get("optimizer_state_dict") is not None:
        optimizer.load_state_dict(checkpoint["optimizer_state_dict"])
    if scheduler is not None and checkpoint.get("scheduler_state_dict"):
        scheduler.load_state_dict(checkpoint["scheduler_state_dict"])
    return checkpoint["epoch"], checkpoint["loss"]
