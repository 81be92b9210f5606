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


def per_token_codes_f32(x, n_bits, symmetric):
    """calibrate + quantize for one scale per row (no groups), in float32 round-half-even
    arithmetic, with codes expressed as signed integers: x ~ scale * (code - zero).

    symmetric: the disable_zero_point range [-2^(n-1), 2^(n-1)-1], zero = 0.
    asymmetric: unsigned code u in [0, 2^n - 1] and zero point zp as the reference derives them
    (quantizer.py:165-179, without the 1-/2-bit "bit balance" widening), returned shifted by
    2^(n-1): code = u - 2^(n-1), zero = zp - 2^(n-1).
    Returns (codes int32 [rows, cols], scale float32 [rows], zero float32 [rows])."""
    f = np.float32
    x = np.asarray(x).astype(f)
    xmin = x.min(axis=-1, keepdims=True)
    xmax = x.max(axis=-1, keepdims=True)
    half = 1 << (n_bits - 1)
    if symmetric:
        scale = np.maximum(np.abs(xmax), np.abs(xmin)) / f(half - 1)
        scale = np.clip(scale, f(CLIPMIN), f(1e4)).astype(f)
        codes = np.clip(np.rint(x / scale), -half, half - 1)
        zero = np.zeros_like(scale)
    else:
        scale = (xmax - xmin) / f(2 * half - 1)
        scale = np.clip(scale, f(CLIPMIN), f(1e4)).astype(f)
        zp = np.rint(np.clip(-xmin / scale, f(-1e4), f(1e4))).astype(f)
        codes = np.clip(np.rint(x / scale) + zp, 0, 2 * half - 1) - half
        zero = zp - f(half)
    return codes.astype(np.int32), scale[:, 0].astype(f), zero[:, 0].astype(f)


def group_affine_codes(w, n_bits, group_size):
    """Weights [N, K] -> asymmetric codes per (row, group of group_size along K), the reference's
    weight configuration (per_channel_axes=[0] + group_size, main.py:280-288 of the reference)
    with the plain 2^n - 1 level range.  Signed representation as in per_token_codes_f32.
    Returns (codes int32 [N, K], scale float64 [N, K/g], zero float64 [N, K/g])."""
    w = np.asarray(w, dtype=np.float64)
    n, k = w.shape
    g = w.reshape(n, k // group_size, group_size)
    wmin = g.min(axis=-1, keepdims=True)
    wmax = g.max(axis=-1, keepdims=True)
    half = 1 << (n_bits - 1)
    scale = np.clip((wmax - wmin) / (2 * half - 1), CLIPMIN, 1e4)
    zp = np.round(np.clip(-wmin / scale, -1e4, 1e4))
    codes = np.clip(np.round(g / scale) + zp, 0, 2 * half - 1) - half
    return codes.reshape(n, k).astype(np.int32), scale[..., 0], zp[..., 0] - half


def dequant_matmul(x_codes, x_scale, x_zero, w_codes, w_scale, w_zero, group_size):
    """fp64 x_dq @ w_dq.T of the dequantised operands (the reference's fake-quant forward,
    int_linear.py:25-84 with quantizer.py:124-128).  w_scale / w_zero are [N, K/g] (or [N, 1]
    with group_size = K); x_scale / x_zero are [M]."""
    xd = (x_codes.astype(np.float64) - np.asarray(x_zero, dtype=np.float64)[:, None]) * \
        np.asarray(x_scale, dtype=np.float64)[:, None]
    ws = np.repeat(np.asarray(w_scale, dtype=np.float64), group_size, axis=1)
    wz = np.repeat(np.asarray(w_zero, dtype=np.float64), group_size, axis=1)
    wd = (w_codes.astype(np.float64) - wz) * ws
    return xd @ wd.T
