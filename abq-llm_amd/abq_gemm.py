"""ctypes binding of libabq_gemm.so (the C ABI in include/abq_gemm.h).

Plumbing for the tests, the smoke check and the benchmark: device buffers are torch tensors,
their data_ptr() goes straight through the C ABI.  There is no CPU fallback here: if the
shared library is missing or the HIP launch fails, the call raises.

Import torch before this module so that the library binds to the HIP runtime torch loaded.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libabq_gemm.so")

ABQ_OK = 0
STATUS_NAMES = {
    0: "ABQ_OK", 1: "ABQ_ERR_INVALID_ARG", 2: "ABQ_ERR_BAD_K", 3: "ABQ_ERR_UNSUPPORTED",
    4: "ABQ_ERR_NOT_INITIALIZED", 5: "ABQ_ERR_LAUNCH", 6: "ABQ_ERR_NO_DEVICE", 7: "ABQ_ERR_TOO_LARGE",
}
globals().update({name: code for code, name in STATUS_NAMES.items()})
OUT_I32, OUT_F16_TENSOR, OUT_F16_SCALED, OUT_F16_TENSOR_F32SCALE = 0, 1, 2, 3
(STRATEGY_AUTO, STRATEGY_BCNT, STRATEGY_MFMA16, STRATEGY_MFMA32, STRATEGY_GENERIC, STRATEGY_DECODE, STRATEGY_TILED, STRATEGY_FP6,
 STRATEGY_DECODE_TILED) = range(9)
STRATEGY_NAMES = ["auto", "bcnt", "mfma16", "mfma32", "generic", "decode", "tiled", "fp6", "decode_tiled"]
LAYOUT_PLANES, LAYOUT_TILED, LAYOUT_FP6, LAYOUT_F16 = 0, 1, 2, 3
ACT_NONE, ACT_SILU_GATE = 0, 1

# every symbol include/abq_gemm.h declares
EXPORTED = [
    "abq_status_string", "abq_last_hip_error", "abq_version",
    "abq_pack_i32", "abq_pack_u4", "abq_pack_f16", "abq_pack_f16_tiled",
    "abq_parse_kernel_name", "abq_format_kernel_name",
    "abq_native_config_count", "abq_native_config_get",
    "abq_gemm_init", "abq_gemm_set_scales", "abq_gemm_exec", "abq_gemm_launch",
    "abq_planes_bytes", "abq_relayout_planes", "abq_gemm_set_operand_layout", "abq_gemm_workspace_bytes",
    "abq_gemm_set_workspace", "abq_fp6_bytes", "abq_fp6_eligible", "abq_prepared_decode_pays", "abq_gemm_set_dynamic_f16_activations", "abq_relayout_planes_fp6",
    "abq_gemm_set_zero_points", "abq_weight_zero_term", "abq_quant_pack_f16", "abq_gemm_set_activation",
    "abq_gemm_exec_static", "abq_gemm_set_f16_activations",
    "abq_row_sums", "abq_gemm_set_row_sums", "abq_gemm_row_sums_ready",
    "abq_tuning_load", "abq_tuning_add", "abq_tuning_clear", "abq_tuning_enable_builtin", "abq_tuning_lookup",
    "abq_preferred_weight_layout", "abq_preferred_weight_records", "abq_padded_bits", "abq_folded_bits", "abq_relayout_planes_folded", "abq_relayout_planes_fp6_folded", "abq_relayout_planes_padded", "abq_gemm_set_value_bits",
    "abq_gemm_set_padded_activations",
    "abq_relayout_planes_biased", "abq_gemm_set_biased_records", "abq_pack_f16_fp6",
]


class TileConfig(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int) for n in (
        "x_bits", "w_bits", "is_signed", "block_m", "block_n", "block_k",
        "warp_m", "warp_n", "warp_k", "mma_m", "mma_n", "mma_k", "nstage")]

    def as_tuple(self):
        return tuple(getattr(self, n) for n, _ in self._fields_)

    def __repr__(self):
        return "TileConfig(%s)" % ", ".join("%s=%d" % (n, getattr(self, n)) for n, _ in self._fields_)


class Dim3(ctypes.Structure):
    _fields_ = [("x", ctypes.c_uint), ("y", ctypes.c_uint), ("z", ctypes.c_uint)]


class GemmState(ctypes.Structure):
    _fields_ = [
        ("shared_mem_size", ctypes.c_size_t),
        ("grid_dim", Dim3), ("block_dim", Dim3),
        ("init_success", ctypes.c_int),
        ("M", ctypes.c_int), ("N", ctypes.c_int), ("K", ctypes.c_int),
        ("X", ctypes.c_void_p), ("W", ctypes.c_void_p), ("C", ctypes.c_void_p), ("D", ctypes.c_void_p),
        ("bias", ctypes.c_int),
        ("cfg", TileConfig),
        ("strategy", ctypes.c_int), ("variant", ctypes.c_int), ("out_kind", ctypes.c_int),
        ("x_scale", ctypes.c_void_p), ("w_scale", ctypes.c_void_p),
        ("group_size", ctypes.c_int),
        ("reserved", ctypes.c_int * 5),
        ("x_layout", ctypes.c_int), ("w_layout", ctypes.c_int), ("auto_chosen", ctypes.c_int),
        ("workspace", ctypes.c_void_p), ("workspace_bytes", ctypes.c_size_t),
        ("x_zero", ctypes.c_void_p), ("w_zero", ctypes.c_void_p),
        ("x_group_sums", ctypes.c_void_p), ("w_zero_term", ctypes.c_void_p),
        ("act", ctypes.c_int),
        ("x_pack_scale", ctypes.c_void_p),
        ("x_row_sums", ctypes.c_void_p), ("w_row_sums", ctypes.c_void_p),
    ]


class AbqError(RuntimeError):
    def __init__(self, status, what):
        self.status = status
        super().__init__("%s failed: %s (%d)" % (what, STATUS_NAMES.get(status, "?"), status))


_lib = None


def lib():
    """Loads libabq_gemm.so; raises if it has not been built (no fallback)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "libabq_gemm.so is not built: run `make -C %s` (or __graft_entry__.build())" % _HERE)
        L = ctypes.CDLL(LIB_PATH)
        vp, ci = ctypes.c_void_p, ctypes.c_int
        L.abq_status_string.restype = ctypes.c_char_p
        L.abq_status_string.argtypes = [ci]
        L.abq_last_hip_error.restype = ci
        L.abq_version.restype = ci
        L.abq_pack_i32.argtypes = [vp, vp, ci, ci, ci, vp]
        L.abq_pack_u4.argtypes = [vp, vp, ci, ci, ci, vp]
        L.abq_pack_f16.argtypes = [vp, vp, vp, ci, ci, ci, vp]
        L.abq_pack_f16_tiled.argtypes = [vp, vp, vp, ci, ci, ci, vp]
        L.abq_pack_f16_fp6.argtypes = [vp, vp, vp, ci, ci, ci, ci, vp]
        L.abq_parse_kernel_name.argtypes = [ctypes.c_char_p, ctypes.POINTER(TileConfig), ctypes.POINTER(ci)]
        L.abq_format_kernel_name.argtypes = [ctypes.POINTER(TileConfig), ci, ctypes.c_char_p, ctypes.c_size_t]
        L.abq_native_config_count.argtypes = [ci, ci, ci]
        L.abq_native_config_count.restype = ci
        L.abq_native_config_get.argtypes = [ci, ci, ci, ci, ctypes.POINTER(TileConfig)]
        L.abq_gemm_init.argtypes = [ctypes.POINTER(TileConfig), ci, ci, ci, vp, vp, ci, ci, ci, vp, vp, ci, ci,
                                    ctypes.POINTER(GemmState)]
        L.abq_gemm_set_scales.argtypes = [ctypes.POINTER(GemmState), vp, vp, ci]
        L.abq_gemm_exec.argtypes = [ctypes.POINTER(GemmState), vp]
        L.abq_gemm_exec_static.argtypes = [ctypes.POINTER(GemmState), vp]
        L.abq_gemm_set_f16_activations.argtypes = [ctypes.POINTER(GemmState), vp, vp]
        L.abq_gemm_set_dynamic_f16_activations.argtypes = [ctypes.POINTER(GemmState), vp, ci]
        L.abq_gemm_launch.argtypes = [ctypes.POINTER(TileConfig), vp, vp, vp, vp, ci, ci, ci, ci, vp]
        L.abq_planes_bytes.argtypes = [ci, ci, ci]
        L.abq_planes_bytes.restype = ctypes.c_size_t
        L.abq_relayout_planes.argtypes = [vp, vp, ci, ci, ci, vp]
        L.abq_relayout_planes_fp6.argtypes = [vp, vp, ci, ci, ci, ci, vp]
        L.abq_fp6_bytes.argtypes = [ci, ci]
        L.abq_fp6_bytes.restype = ctypes.c_size_t
        L.abq_fp6_eligible.argtypes = [ci, ci, ci, ci]
        L.abq_prepared_decode_pays.argtypes = [ci] * 8
        L.abq_prepared_decode_pays.restype = ci
        L.abq_gemm_set_operand_layout.argtypes = [ctypes.POINTER(GemmState), ci, ci]
        L.abq_gemm_workspace_bytes.argtypes = [ctypes.POINTER(GemmState)]
        L.abq_gemm_workspace_bytes.restype = ctypes.c_size_t
        L.abq_gemm_set_workspace.argtypes = [ctypes.POINTER(GemmState), vp, ctypes.c_size_t]
        L.abq_gemm_set_zero_points.argtypes = [ctypes.POINTER(GemmState), vp, vp, vp, vp]
        L.abq_row_sums.argtypes = [vp, ci, ci, ci, vp, vp]
        L.abq_gemm_set_row_sums.argtypes = [ctypes.POINTER(GemmState), vp, vp]
        L.abq_tuning_load.argtypes = [ctypes.c_char_p, ctypes.POINTER(ci)]
        L.abq_tuning_add.argtypes = [ctypes.POINTER(TileConfig), ci, ci, ci, ci, ctypes.c_float]
        L.abq_tuning_clear.restype = None
        L.abq_tuning_enable_builtin.argtypes = [ci]
        L.abq_tuning_enable_builtin.restype = None
        L.abq_tuning_lookup.argtypes = [ci, ci, ci, ci, ci, ci, ci, ci, ctypes.POINTER(TileConfig), ctypes.POINTER(ctypes.c_float)]
        L.abq_preferred_weight_layout.argtypes = [ci] * 7
        L.abq_preferred_weight_layout.restype = ci
        L.abq_preferred_weight_records.argtypes = [ci] * 7 + [ctypes.POINTER(ci)]
        L.abq_preferred_weight_records.restype = ci
        L.abq_relayout_planes_biased.argtypes = [vp, vp, ci, ci, vp]
        L.abq_gemm_set_biased_records.argtypes = [ctypes.POINTER(GemmState), ci, ci]
        L.abq_padded_bits.argtypes = [ci]
        L.abq_padded_bits.restype = ci
        L.abq_relayout_planes_padded.argtypes = [vp, vp, ci, ci, ci, ci, vp]
        L.abq_relayout_planes_folded.argtypes = [vp, vp, ci, vp, ci, ci, ci, ci, vp, vp]
        L.abq_relayout_planes_fp6_folded.argtypes = [vp, vp, ci, vp, ci, ci, ci, ci, vp, vp]
        L.abq_folded_bits.argtypes = [ci]
        L.abq_gemm_set_value_bits.argtypes = [ctypes.POINTER(GemmState), ci, ci]
        L.abq_gemm_set_padded_activations.argtypes = [ctypes.POINTER(GemmState), ci]
        L.abq_gemm_row_sums_ready.argtypes = [ctypes.POINTER(GemmState)]
        L.abq_gemm_row_sums_ready.restype = ci
        L.abq_gemm_set_activation.argtypes = [ctypes.POINTER(GemmState), ci]
        L.abq_weight_zero_term.argtypes = [vp, ci, ci, ci, ci, vp, vp, ci, vp, vp]
        L.abq_quant_pack_f16.argtypes = [vp, ci, ci, ci, ci, ci, vp, vp, vp, vp, ci, vp]
        _lib = L
    return _lib


def _check(status, what):
    if status != ABQ_OK:
        raise AbqError(status, what)


def _stream_ptr(stream):
    if stream is None:
        import torch
        return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    if isinstance(stream, int):
        return ctypes.c_void_p(stream)
    return ctypes.c_void_p(stream.cuda_stream)


def parse_kernel_name(name):
    cfg, wmma = TileConfig(), ctypes.c_int(0)
    _check(lib().abq_parse_kernel_name(name.encode(), ctypes.byref(cfg), ctypes.byref(wmma)), "abq_parse_kernel_name")
    return cfg, bool(wmma.value)


def format_kernel_name(cfg, is_wmma=False):
    buf = ctypes.create_string_buffer(160)
    _check(lib().abq_format_kernel_name(ctypes.byref(cfg), int(is_wmma), buf, 160), "abq_format_kernel_name")
    return buf.value.decode()


def native_configs(x_bits, w_bits, signed):
    n = lib().abq_native_config_count(x_bits, w_bits, int(signed))
    out = []
    for i in range(n):
        c = TileConfig()
        _check(lib().abq_native_config_get(x_bits, w_bits, int(signed), i, ctypes.byref(c)), "abq_native_config_get")
        out.append(c)
    return out


def planes_empty(bits, rows, k, device="cuda"):
    import torch
    return torch.empty((bits, rows, k // 32), dtype=torch.int32, device=device)


def pack_i32(values, bits, out=None, stream=None):
    """values: int32 device tensor [rows, k] -> planes int32 tensor [bits, rows, k/32]."""
    import torch
    assert values.dtype == torch.int32 and values.is_cuda and values.is_contiguous()
    rows, k = values.shape
    if out is None:
        out = planes_empty(bits, rows, k, values.device)
    _check(lib().abq_pack_i32(values.data_ptr(), out.data_ptr(), rows, k, bits, _stream_ptr(stream)), "abq_pack_i32")
    return out


def pack_u4(words, rows, k, bits=4, out=None, stream=None):
    import torch
    assert words.dtype == torch.int32 and words.is_cuda and words.is_contiguous()
    assert words.numel() == rows * k // 8
    if out is None:
        out = planes_empty(bits, rows, k, words.device)
    _check(lib().abq_pack_u4(words.data_ptr(), out.data_ptr(), rows, k, bits, _stream_ptr(stream)), "abq_pack_u4")
    return out


def pack_f16(values, scale, bits, out=None, stream=None, tiled=False):
    """values: fp16 device tensor [rows, k]; scale: float32 device tensor with one element.
    tiled: write the K-tiled layout (what relayout_planes makes of the planes) directly."""
    import torch
    assert values.dtype == torch.float16 and values.is_cuda and values.is_contiguous()
    assert scale.dtype == torch.float32 and scale.is_cuda
    rows, k = values.shape
    if out is None:
        out = (torch.empty((k // 128, rows, bits, 4), dtype=torch.int32, device=values.device) if tiled
               else planes_empty(bits, rows, k, values.device))
    fn, name = (lib().abq_pack_f16_tiled, "abq_pack_f16_tiled") if tiled else (lib().abq_pack_f16, "abq_pack_f16")
    _check(fn(values.data_ptr(), scale.data_ptr(), out.data_ptr(), rows, k, bits, _stream_ptr(stream)), name)
    return out


def pack_f16_fp6(values, scale, bits, signed, stream=None):
    """The same values as pack_f16 written as FP6 records [k/128, rows, 24] (bits <= 5 signed, <= 4 unsigned)."""
    import torch
    assert values.dtype == torch.float16 and values.is_cuda and values.is_contiguous()
    rows, k = values.shape
    out = torch.empty((k // 128, rows, 24), dtype=torch.int32, device=values.device)
    _check(lib().abq_pack_f16_fp6(values.data_ptr(), scale.data_ptr(), out.data_ptr(), rows, k, bits, int(bool(signed)),
                                  _stream_ptr(stream)), "abq_pack_f16_fp6")
    return out


def relayout_planes(planes, out=None, stream=None):
    """planes int32 tensor [bits, rows, k/32] -> K-tiled tensor [k/128, rows, bits, 4]."""
    import torch
    bits, rows, kw = planes.shape
    assert planes.is_cuda and planes.is_contiguous() and kw % 4 == 0
    if out is None:
        out = torch.empty((kw // 4, rows, bits, 4), dtype=torch.int32, device=planes.device)
    _check(lib().abq_relayout_planes(planes.data_ptr(), out.data_ptr(), rows, kw * 32, bits, _stream_ptr(stream)),
           "abq_relayout_planes")
    return out


def row_sums(planes, stream=None):
    """planes int32 tensor [bits, rows, k/32] -> int32 [rows]: the sum over k of each row's unsigned codes (what the
    staged kernel wants handed in for pairs with an unsigned 8-bit operand)."""
    import torch
    bits, rows, kw = planes.shape
    assert planes.is_cuda and planes.is_contiguous()
    out = torch.empty(rows, dtype=torch.int32, device=planes.device)
    _check(lib().abq_row_sums(planes.data_ptr(), rows, kw * 32, bits, out.data_ptr(), _stream_ptr(stream)), "abq_row_sums")
    return out


def relayout_planes_biased(planes, stream=None):
    """planes int32 tensor [8, rows, k/32] of unsigned codes -> K-tiled records [k/128, rows, 8, 4] holding code - 128."""
    import torch
    bits, rows, kw = planes.shape
    assert bits == 8 and planes.is_cuda and planes.is_contiguous() and kw % 4 == 0
    out = torch.empty((kw // 4, rows, 8, 4), dtype=torch.int32, device=planes.device)
    _check(lib().abq_relayout_planes_biased(planes.data_ptr(), out.data_ptr(), rows, kw * 32, _stream_ptr(stream)),
           "abq_relayout_planes_biased")
    return out


def padded_bits(bits):
    return lib().abq_padded_bits(bits)


def relayout_planes_padded(planes, signed, stream=None):
    """planes int32 tensor [bits, rows, k/32] -> K-tiled records of the next width of one field (2, 4 or 8 bits),
    [k/128, rows, padded bits, 4], the codes extended to that width."""
    import torch
    bits, rows, kw = planes.shape
    assert planes.is_cuda and planes.is_contiguous() and kw % 4 == 0
    out = torch.empty((kw // 4, rows, padded_bits(bits), 4), dtype=torch.int32, device=planes.device)
    _check(lib().abq_relayout_planes_padded(planes.data_ptr(), out.data_ptr(), rows, kw * 32, bits, int(bool(signed)),
                                            _stream_ptr(stream)), "abq_relayout_planes_padded")
    return out


def relayout_planes_folded(planes, w_zero, group_size, signed, stream=None):
    """Weight planes [bits, rows, k/32] and their zero points [rows, k/group_size] (whole numbers) -> K-tiled records of
    the signed differences code - zero point, [k/128, rows, folded bits, 4]; a GEMM on them needs no weight zero points.
    Raises if a zero point is no whole number or a difference does not fit the records."""
    import torch
    bits, rows, kw = planes.shape
    rb = lib().abq_folded_bits(bits)
    assert planes.is_cuda and planes.is_contiguous() and kw % 4 == 0 and rb
    assert w_zero.dtype == torch.float32 and w_zero.is_contiguous() and tuple(w_zero.shape) == (rows, kw * 32 // group_size)
    out = torch.empty((kw // 4, rows, rb, 4), dtype=torch.int32, device=planes.device)
    misfit = torch.zeros(1, dtype=torch.int32, device=planes.device)
    _check(lib().abq_relayout_planes_folded(planes.data_ptr(), w_zero.data_ptr(), group_size, out.data_ptr(), rows, kw * 32, bits,
                                            int(bool(signed)), misfit.data_ptr(), _stream_ptr(stream)), "abq_relayout_planes_folded")
    if int(misfit.item()):
        raise ValueError("zero points that are no whole numbers, or differences that do not fit the records")
    return out


def relayout_planes_fp6_folded(planes, w_zero, group_size, signed, stream=None):
    """The same as FP6 records [k/128, rows, 24] (codes of at most 4 bits); used under the pair's own widths on a signed GEMM."""
    import torch
    bits, rows, kw = planes.shape
    assert planes.is_cuda and planes.is_contiguous() and kw % 4 == 0
    assert w_zero.dtype == torch.float32 and w_zero.is_contiguous() and tuple(w_zero.shape) == (rows, kw * 32 // group_size)
    out = torch.empty((kw // 4, rows, 24), dtype=torch.int32, device=planes.device)
    misfit = torch.zeros(1, dtype=torch.int32, device=planes.device)
    _check(lib().abq_relayout_planes_fp6_folded(planes.data_ptr(), w_zero.data_ptr(), group_size, out.data_ptr(), rows, kw * 32, bits,
                                                int(bool(signed)), misfit.data_ptr(), _stream_ptr(stream)), "abq_relayout_planes_fp6_folded")
    if int(misfit.item()):
        raise ValueError("zero points that are no whole numbers, or differences without an FP6 code")
    return out


def fp6_eligible(x_bits, w_bits, signed, k):
    """Whether the FP6 matrix-core route is exact for this bit pair and K (host-side check)."""
    return bool(lib().abq_fp6_eligible(x_bits, w_bits, int(bool(signed)), k))


def prepared_decode_pays(x_bits, w_bits, signed, m, n, k, group_size=0, act=ACT_NONE):
    """Whether a GEMM of this shape on operands that are both K-tiled runs the decode kernel of that layout."""
    return bool(lib().abq_prepared_decode_pays(x_bits, w_bits, int(bool(signed)), m, n, k, group_size, act))


def relayout_planes_fp6(planes, signed, out=None, stream=None):
    """planes int32 tensor [bits, rows, k/32] -> FP6 records [k/128, rows, 24] (6-bit sign-magnitude codes)."""
    import torch
    bits, rows, kw = planes.shape
    assert planes.is_cuda and planes.is_contiguous() and kw % 4 == 0
    if out is None:
        out = torch.empty((kw // 4, rows, 24), dtype=torch.int32, device=planes.device)
    _check(lib().abq_relayout_planes_fp6(planes.data_ptr(), out.data_ptr(), rows, kw * 32, bits, int(bool(signed)),
                                         _stream_ptr(stream)), "abq_relayout_planes_fp6")
    return out


def quant_pack_f16(x, bits, symmetric=True, tiled=False, group_size=0, stream=None, fp6=False):
    """Per-token dynamic quantisation + packing of fp16 activations [rows, k].

    Returns (planes, scale[rows], zero[rows] or None, group_sums[rows, k/group_size] or None);
    planes hold signed codes, [bits, rows, k/32], K-tiled [k/128, rows, bits, 4] or FP6 records
    [k/128, rows, 24] (bits <= 5)."""
    import torch
    assert x.dtype == torch.float16 and x.is_cuda and x.is_contiguous() and not (tiled and fp6)
    rows, k = x.shape
    shape = (k // 128, rows, 24) if fp6 else (k // 128, rows, bits, 4) if tiled else (bits, rows, k // 32)
    planes = torch.empty(shape, dtype=torch.int32, device=x.device)
    scale = torch.empty(rows, dtype=torch.float32, device=x.device)
    zero = None if symmetric else torch.empty(rows, dtype=torch.float32, device=x.device)
    sums = torch.empty((rows, k // group_size), dtype=torch.int32, device=x.device) if group_size else None
    _check(lib().abq_quant_pack_f16(x.data_ptr(), rows, k, bits, int(bool(symmetric)), LAYOUT_FP6 if fp6 else int(bool(tiled)),
                                    planes.data_ptr(), scale.data_ptr(),
                                    zero.data_ptr() if zero is not None else None,
                                    sums.data_ptr() if sums is not None else None, group_size,
                                    _stream_ptr(stream)), "abq_quant_pack_f16")
    return planes, scale, zero, sums


def weight_zero_term(w_planes, signed, w_scale, w_zero, group_size, stream=None):
    """[N] rank-one term of the activation zero-point correction, from reference-layout planes."""
    import torch
    bits, n, kw = w_planes.shape
    out = torch.empty(n, dtype=torch.float32, device=w_planes.device)
    _check(lib().abq_weight_zero_term(w_planes.data_ptr(), n, kw * 32, bits, int(bool(signed)), w_scale.data_ptr(),
                                      w_zero.data_ptr() if w_zero is not None else None, group_size,
                                      out.data_ptr(), _stream_ptr(stream)), "abq_weight_zero_term")
    return out


class Gemm:
    """One initialised GEMM (the role of AqBMMAOpState + InitFn/ExecFn in the reference).

    x_planes / w_planes are in the reference layout [bits, rows, k/32] unless x_tiled / w_tiled
    say they were converted with relayout_planes ([k/128, rows, bits, 4]), or x_fp6 / w_fp6 give the
    bit width of an operand converted with relayout_planes_fp6 ([k/128, rows, 24])."""

    def __init__(self, x_planes, w_planes, signed, out=None, cfg=None, out_kind=OUT_I32, c_scale=None,
                 x_scale=None, w_scale=None, group_size=0, x_tiled=False, w_tiled=False, workspace=None,
                 x_zero=None, w_zero=None, x_group_sums=None, w_zero_term=None, act=ACT_NONE,
                 x_fp6=0, w_fp6=0, x_row_sums=None, w_row_sums=None, value_bits=None, biased=None, x_padded_from=None,
                 x_planes_of=None):
        import torch
        if x_fp6:
            kt, M, _ = x_planes.shape
            q, kw = int(x_fp6), kt * 4
        elif x_tiled:
            kt, M, q, _ = x_planes.shape
            kw = kt * 4
            if x_padded_from is not None:  # records of padded_bits(q) bits holding codes of q = x_padded_from bits
                assert q == padded_bits(int(x_padded_from))
                q = int(x_padded_from)
        else:
            q, M, kw = x_planes.shape
            if x_planes_of is not None:  # planes of fewer bits than the state's width (value_bits says how many)
                assert q == int(value_bits[0]) and q <= int(x_planes_of)
                q = int(x_planes_of)
        if w_fp6:
            kt2, N, _ = w_planes.shape
            p, kw2 = int(w_fp6), kt2 * 4
        elif w_tiled:
            kt2, N, p, _ = w_planes.shape
            kw2 = kt2 * 4
        else:
            p, N, kw2 = w_planes.shape
        assert kw == kw2 and x_planes.is_cuda and w_planes.is_cuda
        assert x_planes.is_contiguous() and w_planes.is_contiguous()
        K = kw * 32
        if out is None:
            out = torch.empty((M, N // 2 if act == ACT_SILU_GATE else N),
                              dtype=torch.int32 if out_kind == OUT_I32 else torch.float16, device=x_planes.device)
        self.out, self.x_planes, self.w_planes = out, x_planes, w_planes
        self.c_scale, self.x_scale, self.w_scale = c_scale, x_scale, w_scale
        self.state = GemmState()
        cfg_ptr = ctypes.byref(cfg) if cfg is not None else None
        st = lib().abq_gemm_init(cfg_ptr, q, p, int(bool(signed)), x_planes.data_ptr(), w_planes.data_ptr(),
                                 M, N, K, out.data_ptr(), c_scale.data_ptr() if c_scale is not None else None,
                                 0, out_kind, ctypes.byref(self.state))
        _check(st, "abq_gemm_init")
        if out_kind == OUT_F16_SCALED:
            _check(lib().abq_gemm_set_scales(ctypes.byref(self.state), x_scale.data_ptr(), w_scale.data_ptr(),
                                             group_size), "abq_gemm_set_scales")
        self.zero_operands = (x_zero, w_zero, x_group_sums, w_zero_term)
        if any(t is not None for t in self.zero_operands):
            _check(lib().abq_gemm_set_zero_points(ctypes.byref(self.state),
                                                  *[t.data_ptr() if t is not None else None
                                                    for t in self.zero_operands]), "abq_gemm_set_zero_points")
        if x_padded_from is not None:
            _check(lib().abq_gemm_set_padded_activations(ctypes.byref(self.state), 1), "abq_gemm_set_padded_activations")
        if x_tiled or w_tiled or x_fp6 or w_fp6:
            xl = LAYOUT_FP6 if x_fp6 else int(x_tiled)
            wl = LAYOUT_FP6 if w_fp6 else int(w_tiled)
            _check(lib().abq_gemm_set_operand_layout(ctypes.byref(self.state), xl, wl), "abq_gemm_set_operand_layout")
        if act != ACT_NONE:
            _check(lib().abq_gemm_set_activation(ctypes.byref(self.state), act), "abq_gemm_set_activation")
        if value_bits is not None:  # (x, w): the codes' real widths inside padded records
            _check(lib().abq_gemm_set_value_bits(ctypes.byref(self.state), int(value_bits[0]), int(value_bits[1])),
                   "abq_gemm_set_value_bits")
        if biased is not None:  # (x, w): which K-tiled operands of an unsigned W8A8 pair hold code - 128
            _check(lib().abq_gemm_set_biased_records(ctypes.byref(self.state), int(bool(biased[0])), int(bool(biased[1]))),
                   "abq_gemm_set_biased_records")
        self.row_sums = (x_row_sums, w_row_sums)
        if x_row_sums is not None or w_row_sums is not None:
            _check(lib().abq_gemm_set_row_sums(ctypes.byref(self.state), x_row_sums.data_ptr() if x_row_sums is not None else None,
                                               w_row_sums.data_ptr() if w_row_sums is not None else None), "abq_gemm_set_row_sums")
        self.workspace = workspace
        if workspace is not None:
            _check(lib().abq_gemm_set_workspace(ctypes.byref(self.state), workspace.data_ptr(),
                                                workspace.numel() * workspace.element_size()), "abq_gemm_set_workspace")

    @property
    def workspace_bytes(self):
        return lib().abq_gemm_workspace_bytes(ctypes.byref(self.state))

    @property
    def row_sums_ready(self):
        """True if run() launches the staged kernel that takes the row sums of an unsigned 8-bit pair handed in."""
        return bool(lib().abq_gemm_row_sums_ready(ctypes.byref(self.state)))

    @property
    def strategy(self):
        return STRATEGY_NAMES[self.state.strategy]

    @property
    def config_name(self):
        return format_kernel_name(self.state.cfg)

    def run(self, stream=None):
        _check(lib().abq_gemm_exec(ctypes.byref(self.state), _stream_ptr(stream)), "abq_gemm_exec")
        return self.out

    def set_f16_activations(self, x_f16, scale):
        """Decode on prepared weights without a packing launch: the kernel quantises the fp16 activations [M, K]
        itself with the static scale (one float on the device).  Raises ABQ_ERR_UNSUPPORTED where that kernel does
        not apply."""
        import torch
        assert x_f16.dtype == torch.float16 and x_f16.is_cuda and x_f16.is_contiguous() and scale.dtype == torch.float32
        _check(lib().abq_gemm_set_f16_activations(ctypes.byref(self.state), x_f16.data_ptr(), scale.data_ptr()),
               "abq_gemm_set_f16_activations")
        self.x_f16, self.x_pack_scale = x_f16, scale

    def set_dynamic_f16_activations(self, x_f16, symmetric, w_zero=None, w_zero_term=None):
        """Group-scale decode on prepared weights without a quantising launch: the kernel quantises the fp16
        activations [M, K] per token itself (symmetric, or with a zero point, which needs w_zero_term).  w_zero: the
        weight zero points, if any (group sums are made inside the kernel).  Raises ABQ_ERR_UNSUPPORTED where that
        kernel does not apply."""
        import torch
        assert x_f16.dtype == torch.float16 and x_f16.is_cuda and x_f16.is_contiguous()
        _check(lib().abq_gemm_set_dynamic_f16_activations(ctypes.byref(self.state), x_f16.data_ptr(), int(bool(symmetric))),
               "abq_gemm_set_dynamic_f16_activations")
        self.x_f16 = x_f16
        if w_zero is not None or w_zero_term is not None:
            self.zero_operands = (None, w_zero, None, w_zero_term)
            _check(lib().abq_gemm_set_zero_points(ctypes.byref(self.state), None, w_zero.data_ptr() if w_zero is not None else None,
                                                  None, w_zero_term.data_ptr() if w_zero_term is not None else None),
                   "abq_gemm_set_zero_points")

    def run_static(self, stream=None):
        """The same through the entry point that allocates nothing (conversions into the library's static array)."""
        _check(lib().abq_gemm_exec_static(ctypes.byref(self.state), _stream_ptr(stream)), "abq_gemm_exec_static")
        return self.out


def gemm(x_planes, w_planes, signed, **kw):
    return Gemm(x_planes, w_planes, signed, **kw).run()
