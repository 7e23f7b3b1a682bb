"""Shared helpers for the parity tests."""
import numpy as np
import torch


def bits(t: torch.Tensor) -> np.ndarray:
    """Raw 16-bit patterns of a bf16/fp16 tensor as a numpy uint16 array."""
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def from_bits(b: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(b.view(np.int16).copy()).view(torch.bfloat16)


def announce(msg: str) -> None:
    """Name the case before it touches the GPU (flushed, so it survives a lost box)."""
    print(f"[case] {msg}", flush=True)
