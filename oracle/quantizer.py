"""numpy restatement of the reference's scale / zero-point semantics.

TEST INFRASTRUCTURE ONLY.  Follows algorithm/quantize/quantizer.py:37-186
(UniformAffineQuantizer): __init__ (:57-68) fixes qmin/qmax, per_token_dynamic_calibration
(:149-179) derives scale and zero point from the min/max of the last axis (after an optional
reshape into groups), fake_quant (:111-132) rounds, shifts, clamps and dequantizes.
Learnable clipping (lwc) and the "fix0to1" metric are training-only and not restated.

Pinned by: closed-form cases in tests/test_oracle.py (a row that is exactly representable
quantizes to itself; the max-abs element of a symmetric row maps to +/-(2^(n-1)-1); the
min / max of an asymmetric row map to qmin / qmax; the dequantization error of every
in-range element is at most scale/2; bit balance: five levels at 2 bits, a row spanning [0, 4 s] maps to
0..4 exactly; rows padded to whole groups: the padded group's scale is that of its real elements).
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


def _into_groups(x, qp):
    """quantizer.py:151-156 / :112-118: rows reshaped into groups; a row whose length is not a multiple of the
    group size is padded with zeros first (the "deficiency", :82-91; the reference allows it for symmetric
    quantisation only)."""
    deficiency = (-x.shape[-1]) % qp.group_size
    if deficiency:
        assert qp.symmetric, "the reference pads rows to whole groups only for symmetric quantisation"
        x = np.concatenate([x, np.zeros((x.shape[0], deficiency), dtype=x.dtype)], axis=1)
    return x.reshape(-1, qp.group_size), deficiency


def calibrate(x, qp):
    """quantizer.py:149-179.  x: float [rows, cols].  Returns (scale, round_zero_point|None),
    each of shape [rows * ceil(cols/group), 1] (or [rows, 1] without groups)."""
    x = np.asarray(x, dtype=np.float64)
    if qp.group_size:
        x, _ = _into_groups(x, qp)
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
    deficiency = 0
    if qp.group_size:
        x, deficiency = _into_groups(x, qp)
    xi = np.round(x / scale)
    if zp is not None:
        xi = xi + zp
    xi = np.clip(xi, qp.qmin, qp.qmax)
    if deficiency:  # the padding is cut off again (quantizer.py:130-131)
        return xi.reshape(shape[0], -1)[:, :shape[1]]
    return xi.reshape(shape)


def dequantize(xi, qp, scale, zp):
    """quantizer.py:124-128."""
    shape = xi.shape
    xi = np.asarray(xi, dtype=np.float64)
    deficiency = 0
    if qp.group_size:
        xi, deficiency = _into_groups(xi, qp)
    if zp is not None:
        xi = xi - zp
    if deficiency:
        return (xi * scale).reshape(shape[0], -1)[:, :shape[1]]
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


def group_affine_codes_bit_balance(w, n_bits, group_size):
    """The reference's default weight quantiser at 1 and 2 bits ("bit balance", quantizer.py:66-68,169-171): the
    asymmetric range is widened by one level, qmax = 2^n and scale = range / 2^n, so a 2-bit weight takes five
    values u in [0, 4].  Goes through calibrate / quantize above (QuantParams applies the widening).  The codes need
    n + 1 bits; they are returned in the signed representation of that width: code = u - 2^n, zero = zp - 2^n.
    Returns (codes int32 [N, K], scale float64 [N, K/g], zero float64 [N, K/g], storage bits n + 1)."""
    assert n_bits in (1, 2)
    w = np.asarray(w, dtype=np.float64)
    n, k = w.shape
    qp = QuantParams(n_bits, symmetric=False, group_size=group_size)
    scale, zp = calibrate(w, qp)
    u = quantize(w, qp, scale, zp)
    half = 1 << n_bits
    return ((u - half).astype(np.int32), scale.reshape(n, k // group_size), zp.reshape(n, k // group_size) - half, n_bits + 1)


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
