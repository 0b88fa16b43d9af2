"""Helpers shared by the GPU parity tests."""
import numpy as np
import torch

from oracle import glif3_oracle as orc
from bmtk_amd import ops, synthetic


def prop_pair(par, h):
    """(fp64 oracle propagators, fp32 device propagators from the HIP precompute)."""
    return orc.precompute(par, h), ops.glif3_precompute(par, h)


def rel_err(got, want, floor):
    """max |got-want| / max(|want|, floor) -- `floor` is the scale below which
    differences count absolutely (stated at each call site)."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    return float(np.max(np.abs(got - want) / np.maximum(np.abs(want), floor))) if got.size else 0.0


def to_dev(a):
    return torch.as_tensor(np.ascontiguousarray(a), device="cuda")


def bits_of(z):
    """uint8 flags -> int64 spike-bit words (+1 padding word) on the host."""
    n = z.size
    words = (n + 63) // 64
    padded = np.zeros(words * 64, np.uint8)
    padded[:n] = z
    packed = np.packbits(padded.reshape(words, 64), axis=1, bitorder="little").view(np.uint64).reshape(-1)
    return np.concatenate([packed, np.zeros(1, np.uint64)]).view(np.int64)
