"""numpy restatement of the reference's scale / zero-point semantics.

TEST INFRASTRUCTURE ONLY.  Follows algorithm/quantize/quantizer.py:37-186
(UniformAffineQuantizer): __init__ (:57-68) fixes qmin/qmax, per_token_dynamic_calibration
(:149-179) derives scale and zero point from the min/max of the last axis (after an optional
reshape into groups), fake_quant (:111-132) rounds, shifts, clamps and dequantizes.
Learnable clipping (lwc) and the "fix0to1" metric are training-only and not restated.

Pinned by: closed-form cases in tests/test_oracle.py (a row that is exactly representable
quantizes to itself; the max-abs element of a symmetric row maps to +/-(2^(n-1)-1); the
min / max of an asymmetric row map to qmin / qmax; the dequantization error of every
in-range element is at most scale/2).
"""
import numpy as np

CLIPMIN = 1e-5  # quantizer.py:24


class QuantParams:
    def __init__(self, n_bits, symmetric=False, disable_zero_point=False, group_size=None):
        self.n_bits = n_bits
        self.symmetric = symmetric
        self.disable_zero_point = disable_zero_point
        self.group_size = group_size
        if disable_zero_point:  # quantizer.py:60-62
            self.qmin = -(2 ** (n_bits - 1))
            self.qmax = 2 ** (n_bits - 1) - 1
        else:  # quantizer.py:63-68, "bit balance" widens 1- and 2-bit ranges by one level
            self.qmin = 0
            self.qmax = 2 ** n_bits - 1
            if n_bits in (1, 2):
                self.qmax += 1


def calibrate(x, qp):
    """quantizer.py:149-179.  x: float [rows, cols].  Returns (scale, round_zero_point|None),
    each of shape [rows * cols/group, 1] (or [rows, 1] without groups)."""
    x = np.asarray(x, dtype=np.float64)
    if qp.group_size:
        assert x.shape[-1] % qp.group_size == 0, "deficiency padding is not restated"
        x = x.reshape(-1, qp.group_size)
    xmin = x.min(axis=-1, keepdims=True)
    xmax = x.max(axis=-1, keepdims=True)
    n = qp.n_bits
    if qp.symmetric:
        abs_max = np.maximum(np.abs(xmax), np.abs(xmin))
        scale = np.clip(abs_max / (2 ** (n - 1) - 1), CLIPMIN, 1e4)
        zero_point = (2 ** (n - 1) - 1) * np.ones_like(scale)
    else:
        rng = xmax - xmin
        scale = rng / (2 ** n) if n in (1, 2) else rng / (2 ** n - 1)
        scale = np.clip(scale, CLIPMIN, 1e4)
        zero_point = -xmin / scale
    if qp.disable_zero_point:
        return scale, None
    return scale, np.round(np.clip(zero_point, -1e4, 1e4))


def quantize(x, qp, scale, zp):
    """Integer codes of fake_quant (quantizer.py:120-123): clamp(round(x/scale) + zp)."""
    x = np.asarray(x, dtype=np.float64)
    shape = x.shape
    if qp.group_size:
        x = x.reshape(-1, qp.group_size)
    xi = np.round(x / scale)
    if zp is not None:
        xi = xi + zp
    xi = np.clip(xi, qp.qmin, qp.qmax)
    return xi.reshape(shape)


def dequantize(xi, qp, scale, zp):
    """quantizer.py:124-128."""
    shape = xi.shape
    xi = np.asarray(xi, dtype=np.float64)
    if qp.group_size:
        xi = xi.reshape(-1, qp.group_size)
    if zp is not None:
        xi = xi - zp
    return (xi * scale).reshape(shape)


def fake_quant(x, qp):
    scale, zp = calibrate(x, qp)
    return dequantize(quantize(x, qp, scale, zp), qp, scale, zp)
