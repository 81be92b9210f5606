"""The packed weight file and the offline converter (host code, no GPU): the tool's codes, scales
and zero points against the oracle's restatement of the reference quantiser, the file layout,
the headerless plane dump for the reference's FasterTransformer loader, and the error paths."""
import os
import struct
import subprocess

import numpy as np
import pytest

from conftest import PKG

TOOL = os.path.join(PKG, "build", "abq_convert_weights")


def _need_tool():
    if not os.path.exists(TOOL):
        pytest.fail("%s is not built: run `make -C abq-llm_amd` (or __graft_entry__.build())" % TOOL)


def read_abqw(path):
    raw = open(path, "rb").read()
    magic, version, n, k, bits, is_signed, group, has_zero = struct.unpack_from("<8sIIIIIII", raw, 0)
    assert magic == b"ABQWGT1\0" and version == 1
    groups = k // group if group else 1
    off = 64
    planes = np.frombuffer(raw, dtype=np.uint32, count=bits * n * k // 32, offset=off).reshape(bits, n, k // 32)
    off += planes.nbytes
    scale = np.frombuffer(raw, dtype=np.float32, count=n * groups, offset=off).reshape(n, groups)
    off += scale.nbytes
    zero = None
    if has_zero:
        zero = np.frombuffer(raw, dtype=np.float32, count=n * groups, offset=off).reshape(n, groups)
        off += zero.nbytes
    assert off == len(raw)
    return dict(n=n, k=k, bits=bits, signed=is_signed, group=group, planes=planes, scale=scale, zero=zero)


@pytest.mark.parametrize("bits,group,fp16", [(2, 128, True), (4, 64, False), (3, 128, False), (8, 128, True)])
def test_converter_asymmetric_matches_the_restated_quantizer(tmp_path, oracle, bits, group, fp16):
    from oracle import quantizer as Q
    _need_tool()
    rng = np.random.default_rng(bits + group)
    n, k = 48, 384
    w = rng.normal(0, 0.02, (n, k)).astype(np.float16 if fp16 else np.float32)
    src, dst, ft = tmp_path / "w.bin", tmp_path / "w.abqw", tmp_path / "w.ft.bin"
    w.tofile(src)
    cmd = [TOOL, str(src), str(n), str(k), str(bits), str(group), "asym", str(dst), "--ft-bin", str(ft)]
    out = subprocess.run(cmd + (["--fp16"] if fp16 else []), capture_output=True, text=True, timeout=60)
    assert out.returncode == 0, out.stdout + out.stderr
    f = read_abqw(dst)
    codes, scale, zero = Q.group_affine_codes(w, bits, group)
    assert (f["n"], f["k"], f["bits"], f["signed"], f["group"]) == (n, k, bits, 1, group)
    assert np.array_equal(f["planes"], oracle.pack_i32(codes, bits))
    assert np.array_equal(f["scale"], scale.astype(np.float32))
    assert np.array_equal(f["zero"], zero.astype(np.float32))
    # the reference's loader reads the plane bytes with no header (LlamaDecoderLayerWeight.cc:377-400):
    # w_bits * K * N / 16 two-byte elements
    raw = open(ft, "rb").read()
    assert raw == f["planes"].tobytes() and len(raw) == bits * k * n // 16 * 2


@pytest.mark.parametrize("bits", [2, 1])
def test_converter_bit_balance_matches_the_restated_quantizer(tmp_path, oracle, bits):
    """--bit-balance: the reference's default for asymmetric 1- and 2-bit weights (quantizer.py:66-68,169-171):
    2^bits + 1 levels, scale = range / 2^bits, stored with one more plane."""
    from oracle import quantizer as Q
    _need_tool()
    rng = np.random.default_rng(40 + bits)
    n, k, group = 48, 384, 128
    w = rng.normal(0, 0.02, (n, k)).astype(np.float32)
    src, dst = tmp_path / "w.bin", tmp_path / "w.abqw"
    w.tofile(src)
    out = subprocess.run([TOOL, str(src), str(n), str(k), str(bits), str(group), "asym", str(dst), "--bit-balance"],
                         capture_output=True, text=True, timeout=60)
    assert out.returncode == 0, out.stdout + out.stderr
    f = read_abqw(dst)
    codes, scale, zero, store_bits = Q.group_affine_codes_bit_balance(w, bits, group)
    assert store_bits == bits + 1 and (f["n"], f["k"], f["bits"], f["signed"], f["group"]) == (n, k, bits + 1, 1, group)
    assert set(np.unique(codes + (1 << bits))) == set(range((1 << bits) + 1))  # all 2^bits + 1 levels occur
    assert np.array_equal(f["planes"], oracle.pack_i32(codes, bits + 1))
    assert np.array_equal(f["scale"], scale.astype(np.float32))
    assert np.array_equal(f["zero"], zero.astype(np.float32))
    # refused where the reference has no such mode
    for extra in (["3", str(group), "asym"], ["2", str(group), "sym"]):
        out = subprocess.run([TOOL, str(src), str(n), str(k)] + extra + [str(dst), "--bit-balance"], capture_output=True, text=True)
        assert out.returncode == 1 and "bit balance" in out.stdout


def test_converter_symmetric_per_channel(tmp_path, oracle):
    from oracle import quantizer as Q
    _need_tool()
    rng = np.random.default_rng(5)
    n, k, bits = 20, 256, 4
    w = rng.normal(0, 1, (n, k)).astype(np.float32)
    src, dst = tmp_path / "w.bin", tmp_path / "w.abqw"
    w.tofile(src)
    out = subprocess.run([TOOL, str(src), str(n), str(k), str(bits), "0", "sym", str(dst)], capture_output=True, text=True)
    assert out.returncode == 0, out.stdout + out.stderr
    f = read_abqw(dst)
    qp = Q.QuantParams(bits, symmetric=True, disable_zero_point=True)
    scale, _ = Q.calibrate(w, qp)
    codes = Q.quantize(w, qp, scale, None).astype(np.int32)
    assert f["zero"] is None and f["group"] == 0
    assert np.array_equal(f["scale"][:, 0], scale[:, 0].astype(np.float32))
    assert np.array_equal(f["planes"], oracle.pack_i32(codes, bits))


def test_converter_error_paths(tmp_path):
    _need_tool()
    src = tmp_path / "w.bin"
    np.zeros((4, 100), dtype=np.float32).tofile(src)
    out = subprocess.run([TOOL, str(src), "4", "100", "2", "0", "sym", str(tmp_path / "o")], capture_output=True, text=True)
    assert out.returncode == 1 and "K must be >= 128" in out.stdout
    np.zeros((4, 128), dtype=np.float32).tofile(src)
    out = subprocess.run([TOOL, str(src), "5", "128", "2", "0", "sym", str(tmp_path / "o")], capture_output=True, text=True)
    assert out.returncode == 1 and "does not hold exactly" in out.stdout
    out = subprocess.run([TOOL, str(src), "4", "128", "2", "96", "asym", str(tmp_path / "o")], capture_output=True, text=True)
    assert out.returncode == 1 and "group_size" in out.stdout
    out = subprocess.run([TOOL], capture_output=True, text=True)
    assert out.returncode == 2 and "Usage" in out.stdout
