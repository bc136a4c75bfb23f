"""Host-side encodings of the three storage dtypes (numpy has no bfloat16).

bf16 rounding is IEEE round-to-nearest-even, what `half::bf16::from_f32` does on
the reference side (crates/incin-backends/src/cpu/storage.rs:163-168) and what
the device's float -> bf16 conversion does.
"""
import numpy as np

from .capi import BF16, F16, F32

NAMES = {F32: "f32", F16: "f16", BF16: "bf16"}
ITEMSIZE = {F32: 4, F16: 2, BF16: 2}


def f32_to_bf16_bits(x):
    x = np.asarray(x, dtype=np.float32, order="C")
    u = x.view(np.uint32).astype(np.uint64)
    rounded = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    nan = np.isnan(x)
    if nan.any():
        rounded = np.where(nan, np.uint16(0x7FC0), rounded)
    return rounded.reshape(x.shape)


def bf16_bits_to_f32(b):
    b = np.asarray(b, dtype=np.uint16, order="C")
    return (b.astype(np.uint32) << 16).view(np.float32).reshape(b.shape)


def encode(x, dtype):
    """f32 array -> array holding the storage encoding (f32, f16, or bf16 bits as uint16)."""
    x = np.asarray(x, dtype=np.float32)
    if dtype == F32:
        return np.asarray(x, order="C")
    if dtype == F16:
        with np.errstate(over="ignore"):
            return np.asarray(x.astype(np.float16), order="C")
    return f32_to_bf16_bits(x)


def decode(raw, dtype):
    """storage encoding -> f32 array."""
    if dtype == F32:
        return np.asarray(raw, dtype=np.float32)
    if dtype == F16:
        return np.asarray(raw, dtype=np.float16).astype(np.float32)
    return bf16_bits_to_f32(raw)


def storage_numpy_dtype(dtype):
    return {F32: np.float32, F16: np.float16, BF16: np.uint16}[dtype]


def round_to(x, dtype):
    """f32 values rounded to the storage dtype, kept as f32 (what the f32 oracle is fed)."""
    return decode(encode(x, dtype), dtype)
