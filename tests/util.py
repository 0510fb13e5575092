"""Helpers shared by the GPU parity tests: seeded host inputs from the oracle's PRNG,
moved to the device as the exact same bytes the oracle sees."""
from __future__ import annotations

import numpy as np
import torch

import oracle


def to_dev_f16(bits: np.ndarray, dev) -> torch.Tensor:
    return torch.from_numpy(bits.view(np.float16)).to(dev)


def to_dev_bf16(bits: np.ndarray, dev) -> torch.Tensor:
    return torch.from_numpy(bits.view(np.int16)).to(dev).view(torch.bfloat16)


def from_dev_f16_bits(t: torch.Tensor) -> np.ndarray:
    return t.cpu().numpy().view(np.uint16)


def from_dev_bf16_bits(t: torch.Tensor) -> np.ndarray:
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def normal_f16_bits(shape, seed, std=1.0) -> np.ndarray:
    return oracle.f32_to_f16_bits(oracle.normal_f32(shape, seed, 0.0, std))


def normal_bf16_bits(shape, seed, std=1.0) -> np.ndarray:
    return oracle.f32_to_bf16_bits(oracle.normal_f32(shape, seed, 0.0, std))


def f16_ulp_diff(a_bits: np.ndarray, b_bits: np.ndarray) -> np.ndarray:
    """Distance in units of f16 representable values (sign-magnitude -> ordered ints)."""
    def ordered(u):
        u = u.astype(np.int32)
        return np.where(u & 0x8000, -(u & 0x7FFF), u)
    return np.abs(ordered(a_bits) - ordered(b_bits))


def rel_l2(got: np.ndarray, ref: np.ndarray) -> float:
    return float(np.linalg.norm(got.astype(np.float64) - ref.astype(np.float64)) /
                 max(np.linalg.norm(ref.astype(np.float64)), 1e-30))


def assert_rounded_close(got: np.ndarray, ref: np.ndarray, tile, rel_ulp: float = 2.0 ** -7, atol_frac: float = 2e-5, what: str = "",
                         mag: np.ndarray | None = None) -> None:
    """Elementwise: every output within one unit in the last place of the 16-bit output type (relative `rel_ulp`:
    2^-7 for bf16, 2^-10 for f16) of the f32 reference, plus a small absolute term for sums that cancel; asserted on the
    whole matrix and, separately, on the rows and columns of the last (partial) tile, where a wrong tail would hide in
    a whole-matrix norm.  The absolute term is `atol_frac` of `mag`, the element's own sum of |products| (what the
    rounding of an f32 accumulation in another order scales with: one missing product of K is mag/K, far above it),
    or of the largest |ref| where no `mag` is given."""
    got64, ref64 = got.astype(np.float64), ref.astype(np.float64)
    bound = np.abs(ref64) * rel_ulp + atol_frac * (np.max(np.abs(ref64)) if mag is None else mag.astype(np.float64))
    bad = np.abs(got64 - ref64) > bound
    assert not bad.any(), f"{what}: {int(bad.sum())} elements off by more than one ulp, first at {np.argwhere(bad)[0]}"
    bm, bn = tile
    r0, c0 = (got.shape[0] - 1) // bm * bm, (got.shape[1] - 1) // bn * bn
    assert not bad[r0:, :].any() and not bad[:, c0:].any(), f"{what}: last tile rows/columns"
