"""Element types carried through the IR.

bf16 has no numpy dtype: on the host it rides as ``uint16`` bit patterns,
exactly like the reference (emmy/compiler/dtype.py:69); on the device it is
``__bf16`` storage converted to/from fp32 with round-to-nearest-even.
"""

from __future__ import annotations

from dataclasses import dataclass

import numpy as np


@dataclass(frozen=True)
class DType:
    name: str  # "f32" | "bf16" | "f16" | "i32" — the canonical token a render target spells as a C type
    nbytes: int
    np: np.dtype  # host carrier dtype

    def __repr__(self) -> str:
        return self.name


F32 = DType("f32", 4, np.dtype(np.float32))
BF16 = DType("bf16", 2, np.dtype(np.uint16))
F16 = DType("f16", 2, np.dtype(np.float16))
I32 = DType("i32", 4, np.dtype(np.int32))
I64 = DType("i64", 8, np.dtype(np.int64))

_BY_NAME = {d.name: d for d in (F32, BF16, F16, I32, I64)}


def by_name(name: str) -> DType:
    return _BY_NAME[name]


def from_torch(t) -> DType:
    import torch

    table = {torch.float32: F32, torch.bfloat16: BF16, torch.float16: F16, torch.int32: I32, torch.int64: I64}
    try:
        return table[t]
    except KeyError as exc:
        raise TypeError(f"unsupported torch dtype {t}") from exc


def to_torch(d: DType):
    import torch

    return {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16, "i32": torch.int32, "i64": torch.int64}[d.name]


def bf16_bits_from_f32(x: np.ndarray) -> np.ndarray:
    """fp32 → bf16 bit patterns, round-to-nearest-even (NaN kept quiet).

    Same closed form the reference uses for bf16 constants
    (emmy/compiler/backend/cuda/program.py:259-263)."""
    bits = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    rounded = (bits + 0x7FFF + ((bits >> 16) & 1)) >> 16
    nan = np.isnan(x)
    out = rounded.astype(np.uint16)
    if np.any(nan):
        out = np.where(nan, np.uint16(0x7FC0), out)
    return out


def f32_from_bf16_bits(bits: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)
