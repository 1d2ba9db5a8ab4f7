"""What the readers of designs with their own ``config.json`` schema (uzu_amd.lazolix, uzu_amd.relulix, uzu_amd.begasun) share: bf16 tensors of a safetensors file by name with
shape checks, bf16 bit patterns, and a full-precision linear of the engine's description."""
from __future__ import annotations

from typing import Optional, Tuple

import numpy as np

from . import desc as D


def f32_to_bf16_bits(a: np.ndarray) -> np.ndarray:
    """round-to-nearest-even bf16 bit patterns of an f32 array"""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    return r


def bits_to_f32(bits: np.ndarray) -> np.ndarray:
    return (bits.astype(np.uint32) << 16).view(np.float32)


class Tensors:
    """bf16 tensors of a safetensors file by name: `bits(name)` = uint16 patterns, `f32(name)` = their values; shapes are checked where the caller knows them."""

    def __init__(self, st, err):
        self.st, self.err = st, err

    def has(self, name: str) -> bool:
        return name in self.st.index

    def shape(self, name: str) -> Tuple[int, ...]:
        if name not in self.st.index:
            raise self.err(f"{self.st.path}: tensor '{name}' not found")
        return tuple(self.st.index[name][1])

    def bits(self, name: str, shape: Optional[Tuple[int, ...]] = None) -> np.ndarray:
        have = self.shape(name)
        dtype = self.st.index[name][0]
        if shape is not None and tuple(shape) != have:
            raise self.err(f"{self.st.path}: tensor '{name}' is {list(have)}, the configuration implies {list(shape)}")
        if dtype == "BF16":
            return np.ascontiguousarray(self.st.tensor(name, have, "BF16"))
        if dtype == "F32":
            return f32_to_bf16_bits(self.st.tensor(name, have, "F32"))
        raise self.err(f"{self.st.path}: tensor '{name}' is {dtype}: bf16 (or f32) expected")

    def f32(self, name: str, shape: Optional[Tuple[int, ...]] = None) -> np.ndarray:
        have = self.shape(name)
        if self.st.index[name][0] == "F32":
            if shape is not None and tuple(shape) != have:
                raise self.err(f"{self.st.path}: tensor '{name}' is {list(have)}, the configuration implies {list(shape)}")
            return np.ascontiguousarray(self.st.tensor(name, have, "F32"))
        return np.ascontiguousarray(bits_to_f32(self.bits(name, shape)))


def full_linear(bits: np.ndarray, bias: Optional[np.ndarray] = None) -> D.LinearWeights:
    n, k = bits.shape
    return D.LinearWeights(n=int(n), k=int(k), bits=16, group_size=0, method=D.QUANT_NONE, weights=np.ascontiguousarray(bits), out_biases=bias)
