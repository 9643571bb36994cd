"""Shared helpers of the parity tests: oracle operands <-> device tensors."""

from __future__ import annotations

import numpy as np
import torch

from oracle import int4_oracle as oracle


def bits_to_bf16(bits: np.ndarray, device="cpu") -> torch.Tensor:
    """uint16 bit patterns -> torch bfloat16 tensor (no value conversion)."""
    t = torch.from_numpy(np.ascontiguousarray(bits).view(np.int16).copy())
    return t.view(torch.bfloat16).to(device)


def bf16_to_bits(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def to_device(ops: dict, device) -> dict:
    """numpy operand dict of the oracle -> torch tensors on ``device``."""
    return {
        "x": bits_to_bf16(ops["x_bits"], device),
        "qweight": torch.from_numpy(ops["qweight"].copy()).to(device),
        "scales": bits_to_bf16(ops["scales_bits"], device),
        "qzeros": torch.from_numpy(ops["qzeros"].copy()).to(device),
    }


def assert_gemv_close(y_bits: np.ndarray, ops: dict, G: int, what: str = ""):
    """The operator tolerance, stated once.

    |y - y_ref| <= max(1 bf16 ulp at y_ref, 1e-2 |y_ref|) + 2^-18 sum|x w|, with
    y_ref the float64 product over the canonical (bit-exact) bf16 weights.
    Returns the worst backward error |y - y_ref| / sum|x w| for reporting.
    """
    y = oracle.bf16_bits_to_f32(y_bits).astype(np.float64)
    y_ref = oracle.gemv_f64(ops["x_bits"], ops["qweight"], ops["scales_bits"], ops["qzeros"], G)
    a_ref = oracle.gemv_abs_f64(ops["x_bits"], ops["qweight"], ops["scales_bits"], ops["qzeros"], G)
    assert y.shape == y_ref.shape, f"{what}: shape {y.shape} vs {y_ref.shape}"
    err = np.abs(y - y_ref)
    tol = oracle.gemv_tolerance(y_ref, a_ref)
    bad = err > tol
    assert not bad.any(), (
        f"{what}: {int(bad.sum())} of {bad.size} outputs out of tolerance; worst at "
        f"{np.unravel_index(np.argmax(err - tol), err.shape)}: got {y.flat[np.argmax(err - tol)]!r} "
        f"ref {y_ref.flat[np.argmax(err - tol)]!r}")
    return float((err / np.maximum(a_ref, 1e-300)).max())
