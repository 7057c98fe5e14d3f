"""bfloat16 at the NumPy boundary.  NumPy has no bfloat16 type, so buffers of HLO type bf16 travel as uint16 arrays
holding the bit patterns: the upper 16 bits of the float32 pattern of the same value."""
import numpy as np


def from_bits(bits) -> np.ndarray:
    """uint16 bit patterns -> float32 values (exact)."""
    return (np.asarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def to_bits(values) -> np.ndarray:
    """float values -> uint16 bit patterns, rounded to nearest with ties to even; NaN stays a quiet NaN."""
    f = np.ascontiguousarray(values, dtype=np.float32)
    u = f.view(np.uint32)
    rounded = ((u + np.uint32(0x7FFF) + ((u >> 16) & np.uint32(1))) >> 16).astype(np.uint16)
    return np.where(np.isnan(f), ((u >> 16) | np.uint32(0x40)).astype(np.uint16), rounded)
