"""Helpers shared by the GPU parity tests: move an oracle problem to the device and
call the HIP path through the package's ctypes binding of the C ABI."""
import numpy as np
import torch


def to_dev(p, dev="cuda:0", scale_dtype=torch.bfloat16):
    A = torch.from_numpy(p["A"]).to(dev)
    B = torch.from_numpy(p["B"].view(np.int8)).to(dev)
    s = torch.from_numpy(p["s"].reshape(-1, 1).copy()).to(dev)
    ws = torch.from_numpy(p["ws"].view(np.int16).copy()).view(scale_dtype).to(dev)
    return A, B, s, ws


def bf16_bits(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def bf16_ordinal(bits: np.ndarray) -> np.ndarray:
    """Maps bf16 bit patterns to integers whose difference counts representable values."""
    b = bits.astype(np.int32)
    return np.where(b & 0x8000, -(b & 0x7FFF), b & 0x7FFF)
