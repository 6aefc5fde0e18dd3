"""Shared helpers for the parity tests: torch <-> oracle conversions and input makers."""
import numpy as np
import torch


def bits_of(t: torch.Tensor) -> np.ndarray:
    """bf16 tensor -> uint16 bit patterns (host)."""
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def bf16_from_bits(bits: np.ndarray, device="cpu") -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).view(torch.bfloat16).to(device)


def u8(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().contiguous().numpy()


def randn_bits(rng: np.random.Generator, shape, std=1.0, outliers=0.0) -> np.ndarray:
    from oracle import mx_oracle as mo

    x = rng.standard_normal(shape, dtype=np.float32) * np.float32(std)
    if outliers:
        x = np.where(rng.random(shape) < outliers, x * np.float32(100.0), x)
    return mo.f32_to_bf16_bits(x)


def rel_l2(a: np.ndarray, b: np.ndarray) -> float:
    a = a.astype(np.float64)
    b = b.astype(np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-300))
