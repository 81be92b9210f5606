"""CPU tests of the host-side logic that ships: the bit helpers the kernels are built from
(compiled for the host), the C ABI's argument checking / naming / tile registry, and the tile
generator.  No GPU compute is called here."""
import ctypes
import hashlib
import json
import os
import re
import subprocess

import numpy as np
import pytest

from conftest import PKG, ROOT

HERE = os.path.dirname(os.path.abspath(__file__))
COMBOS = [(2, 2), (3, 3), (4, 4), (5, 5), (6, 6), (7, 7), (8, 8), (4, 2), (6, 2), (8, 2), (8, 4), (8, 3)]


@pytest.fixture(scope="module")
def shim(tmp_path_factory):
    out = str(tmp_path_factory.mktemp("shim") / "libshim.so")
    subprocess.check_call(["g++", "-O2", "-std=c++17", "-shared", "-fPIC", "-I" + os.path.join(PKG, "csrc"),
                           os.path.join(HERE, "host_shim.cpp"), "-o", out])
    L = ctypes.CDLL(out)
    L.shim_planes_to_int8.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_long]
    L.shim_via_fields.argtypes = [ctypes.c_int, ctypes.c_int] + [ctypes.c_void_p] * 4 + [ctypes.c_long]
    L.shim_eight_values_to_plane_bytes.argtypes = [ctypes.c_void_p]
    L.shim_eight_values_to_plane_bytes.restype = ctypes.c_uint64
    L.shim_nibble_word_plane_byte.argtypes = [ctypes.c_uint32, ctypes.c_int]
    L.shim_nibble_word_plane_byte.restype = ctypes.c_uint32
    return L


def expand(shim, planes, mode):
    """planes uint32 [bits, rows, kw] -> int8 [rows, kw, 32] in the kernels' element order."""
    bits, rows, kw = planes.shape
    words = np.ascontiguousarray(planes.transpose(1, 2, 0))  # [rows, kw, bits]
    out = np.zeros((rows, kw, 8), dtype=np.uint32)
    shim.shim_planes_to_int8(bits, mode, words.ctypes.data, out.ctypes.data, rows * kw)
    return out.view(np.int8).reshape(rows, kw, 32)


def rand_vals(rng, rows, k, bits, signed):
    lo, hi = (-(1 << (bits - 1)), (1 << (bits - 1)) - 1) if signed else (0, (1 << bits) - 1)
    return rng.integers(lo, hi + 1, size=(rows, k), dtype=np.int32)


@pytest.mark.parametrize("bits", range(1, 9))
def test_field_packed_route_equals_plane_route(shim, oracle, bits):
    """planes -> fields -> int8 gives the same bytes as planes -> int8, for every placement mode,
    and the field words hold exactly the bits of the values (a field word is a permutation of them)."""
    rng = np.random.default_rng(100 + bits)
    planes = rng.integers(0, 1 << 32, size=(bits, 6, 16), dtype=np.uint64).astype(np.uint32)
    words = np.ascontiguousarray(planes.transpose(1, 2, 0))
    n = 6 * 16
    for mode in (0, 1, 2):
        if mode == 2 and bits != 8:
            continue
        fields = np.zeros((n, bits), dtype=np.uint32)
        out = np.zeros((n, 8), dtype=np.uint32)
        sums = np.zeros(n, dtype=np.int32)
        shim.shim_via_fields(bits, mode, words.ctypes.data, fields.ctypes.data, out.ctypes.data, sums.ctypes.data, n)
        want = np.zeros((n, 8), dtype=np.uint32)
        shim.shim_planes_to_int8(bits, mode, words.ctypes.data, want.ctypes.data, n)
        assert np.array_equal(out, want)
        vals = oracle.unpack(planes, False).reshape(n, 32)
        assert np.array_equal(sums, vals.sum(axis=1))
        popc = lambda a: np.unpackbits(a.view(np.uint8)).reshape(n, -1).sum(axis=1)
        assert np.array_equal(popc(fields), popc(np.ascontiguousarray(words.reshape(n, bits))))


@pytest.mark.parametrize("bits", range(1, 9))
def test_planes_to_int8_values_and_order(shim, oracle, bits):
    rng = np.random.default_rng(bits)
    K = 128
    for signed in (True, False):
        if signed and bits == 1:
            continue
        v = rand_vals(rng, 4, K, bits, signed)
        planes = oracle.pack_i32(v, bits)
        mode = shim.shim_int8_mode(bits, int(signed))
        got = expand(shim, planes, mode).astype(np.int32)
        # byte (4*s + c) of the 32 is the element at bit position 8c+s, i.e. element 31-(8c+s)
        s, c = np.divmod(np.arange(32), 4)
        elem = 31 - (8 * c + s)
        want = v.reshape(4, K // 32, 32)[:, :, elem]
        if signed:
            want = want << (8 - bits)      # top-aligned two's complement
        elif bits == 8:
            want = want - 128              # bit 7 flipped
        assert np.array_equal(got, want)


@pytest.mark.parametrize("q,p", COMBOS)
@pytest.mark.parametrize("signed", [True, False])
def test_int8_route_reproduces_oracle(shim, oracle, q, p, signed):
    """The arithmetic of the matrix-core kernels, emulated on the host: expand both operands,
    int8 dot products, then the shift (signed) or the row-sum correction (8-bit unsigned)."""
    rng = np.random.default_rng(31 * q + p)
    M, N, K = 6, 10, 384
    x, w = rand_vals(rng, M, K, q, signed), rand_vals(rng, N, K, p, signed)
    xp, wp = oracle.pack_i32(x, q), oracle.pack_i32(w, p)
    xm, wm = shim.shim_int8_mode(q, int(signed)), shim.shim_int8_mode(p, int(signed))
    a = expand(shim, xp, xm).reshape(M, K).astype(np.int64)
    b = expand(shim, wp, wm).reshape(N, K).astype(np.int64)
    acc = a @ b.T
    assert np.abs(acc).max() < 2 ** 31
    if signed:
        assert np.all(acc % (1 << (16 - q - p)) == 0)
        d = acc >> (16 - q - p)
    else:
        d = acc.copy()
        sx = (x.astype(np.int64)).sum(axis=1)
        sw = (w.astype(np.int64)).sum(axis=1)
        if p == 8:
            d += 128 * sx[:, None]
        if q == 8:
            d += 128 * sw[None, :]
        if p == 8 and q == 8:
            d -= 16384 * K
    assert np.array_equal(d.astype(np.int32), oracle.gemm_popc(xp, wp, signed)[0])


def test_eight_values_to_plane_bytes(shim, oracle):
    rng = np.random.default_rng(2)
    for _ in range(200):
        v = rng.integers(-128, 256, 8).astype(np.int32)
        got = shim.shim_eight_values_to_plane_bytes(v.ctypes.data)
        for b in range(8):
            byte = (got >> (8 * b)) & 0xFF
            want = sum(((int(v[c]) >> b) & 1) << (7 - c) for c in range(8))
            assert byte == want


def test_nibble_word_plane_byte(shim):
    rng = np.random.default_rng(3)
    for word in rng.integers(0, 2 ** 32, 200, dtype=np.uint64):
        word = int(word)
        for b in range(4):
            want = sum((((word >> (4 * (7 - e))) >> b) & 1) << (7 - e) for e in range(8))
            assert shim.shim_nibble_word_plane_byte(word, b) == want


def test_plane_pair_weight_matches_reference_rule(shim):
    # engine/test_any_mma.cu:64-68: multiplier of plane b is -2^b only for the MSB of a signed operand
    for q, p in COMBOS:
        for signed in (0, 1):
            for i in range(q):
                for j in range(p):
                    xm = -(1 << i) if signed and i == q - 1 else (1 << i)
                    wm = -(1 << j) if signed and j == p - 1 else (1 << j)
                    assert shim.shim_plane_pair_weight(i, j, q, p, signed) == xm * wm


# ------------------------------------------------------------------ C ABI (no compute)

def test_library_exports_every_declared_symbol(abq):
    header = open(os.path.join(ROOT, "include", "abq_gemm.h")).read()
    declared = set(re.findall(r"\b(abq_[a-z0-9_]+)\s*\(", header))
    assert declared == set(abq.EXPORTED)
    L = abq.lib()
    for name in declared:
        assert hasattr(L, name), name
        # every entry point that takes arguments has its ctypes signature declared: without one a 64-bit device pointer
        # is passed as a C int and arrives truncated
        takes_args = not re.search(r"\b%s\s*\(\s*void\s*\)" % name, header)
        assert getattr(L, name).argtypes is not None or not takes_args, name
    assert L.abq_version() == 1
    assert L.abq_status_string(2).decode().startswith("K must")


def test_state_struct_matches_header_size(abq):
    # sizeof(abq_gemm_state) as the C compiler sees it
    src = '#include "abq_gemm.h"\n#include <stdio.h>\nint main(){printf("%zu %zu", sizeof(abq_gemm_state), sizeof(abq_tile_config));return 0;}'
    exe = "/tmp/abq_sizeof"
    subprocess.run(["gcc", "-x", "c", "-", "-I" + os.path.join(ROOT, "include"), "-o", exe], input=src.encode(), check=True)
    a, b = subprocess.check_output([exe]).decode().split()
    assert int(a) == ctypes.sizeof(abq.GemmState) and int(b) == ctypes.sizeof(abq.TileConfig)


def test_kernel_name_round_trip(abq):
    name = "AqBMMA_8x2xtrue_1x48x512_8x24x128_8x8x128_4"  # the FT M==1 configuration
    cfg, wmma = abq.parse_kernel_name(name)
    assert not wmma and cfg.as_tuple() == (8, 2, 1, 1, 48, 512, 8, 24, 128, 8, 8, 128, 4)
    assert abq.format_kernel_name(cfg) == name
    cfg2, wmma2 = abq.parse_kernel_name("AqBWMMA_4x4xfalse_8x32x256_32x64x128_8x8x128_2_ExecFn")
    assert wmma2 and cfg2.is_signed == 0 and cfg2.nstage == 2
    for bad in ("AqBMMA_8x2xmaybe_1x48x512_8x24x128_8x8x128_4", "Foo_1", "AqBMMA_8x2xtrue_1x48x512"):
        with pytest.raises(abq.AbqError):
            abq.parse_kernel_name(bad)


def _init(abq, cfg=None, q=8, p=2, signed=1, X=0x1000, W=0x2000, M=1, N=64, K=4096, D=0x3000, C=None, bias=0,
          out_kind=0):
    st = abq.GemmState()
    rc = abq.lib().abq_gemm_init(ctypes.byref(cfg) if cfg is not None else None, q, p, signed, X, W, M, N, K, D, C,
                                 bias, out_kind, ctypes.byref(st))
    return rc, st


def test_init_error_paths(abq):
    # the host-forcible failures of the reference: K constraint, bias, null pointers, unknown tuple
    assert _init(abq)[0] == 0
    for K in (0, 64, 127, 200, 4096 + 32):
        rc, st = _init(abq, K=K)
        assert rc in (1, 2) and st.init_success == 0
    assert _init(abq, K=96)[0] == 2
    assert _init(abq, bias=1)[0] == 3
    assert _init(abq, X=None)[0] == 1 and _init(abq, W=None)[0] == 1 and _init(abq, D=None)[0] == 1
    assert _init(abq, M=0)[0] == 1 and _init(abq, N=-1)[0] == 1
    assert _init(abq, out_kind=1)[0] == 1  # fp16 per-tensor output without a scale pointer
    assert _init(abq, out_kind=7)[0] == 1
    assert _init(abq, q=17, p=2)[0] == 3
    rc, st = _init(abq, q=16, p=1)  # a W1A16 sample of the reference library: run-time loop kernel
    assert rc == 0 and st.strategy == abq.STRATEGY_GENERIC
    # exec on a failed state is refused before any launch
    rc, st = _init(abq, K=100)
    assert abq.lib().abq_gemm_exec(ctypes.byref(st), None) == 4
    # a native MMA triple with a tile that is not instantiated
    cfg, _ = abq.parse_kernel_name("AqBMMA_8x2xtrue_16x48x4096_16x48x512_16x16x64_2")
    assert _init(abq, cfg=cfg)[0] == 3
    # K too large for the top-aligned signed int8 route
    cfg, _ = abq.parse_kernel_name("AqBMMA_8x2xtrue_16x16x4096_16x16x512_16x16x64_2")
    assert _init(abq, cfg=cfg, K=1 << 17)[0] == 7


def test_default_strategy_choice_and_reference_tuples(abq):
    # W2A8 on plane operands: the popcount kernel for one row, the matrix-core decode kernel up to 16, blocks of 16 rows
    # whose waves split K up to 128 (64 on wide outputs), MFMA 32x32 above
    for M, want in ((1, abq.STRATEGY_BCNT), (2, abq.STRATEGY_DECODE), (4, abq.STRATEGY_DECODE),
                    (8, abq.STRATEGY_DECODE), (16, abq.STRATEGY_DECODE), (17, abq.STRATEGY_MFMA16), (64, abq.STRATEGY_MFMA16),
                    (128, abq.STRATEGY_MFMA16), (129, abq.STRATEGY_MFMA32), (2048, abq.STRATEGY_MFMA32)):
        rc, st = _init(abq, M=M, N=4096)
        assert rc == 0 and st.strategy == want, M
    rc, st = _init(abq, M=64, N=4096)
    assert st.cfg.as_tuple()[3:] == (16, 32, 2048, 16, 32, 512, 16, 16, 64, 2) and st.grid_dim.y == 4
    rc, st = _init(abq, M=64, N=4096, K=11008)
    assert st.cfg.block_k == 4096
    rc, st = _init(abq, M=100, N=4096)
    assert st.cfg.as_tuple()[3:] == (16, 64, 1024, 16, 32, 512, 16, 16, 64, 2)
    rc, st = _init(abq, M=100, N=11008)
    assert st.strategy == abq.STRATEGY_MFMA32
    # the choice follows x_bits * w_bits * M against a bound by w_bits (popcount work against the cost of the weight transposes)
    for q, p, M, want in ((2, 2, 4, abq.STRATEGY_BCNT), (2, 2, 8, abq.STRATEGY_DECODE), (4, 4, 2, abq.STRATEGY_BCNT),
                          (4, 4, 4, abq.STRATEGY_DECODE), (8, 8, 2, abq.STRATEGY_BCNT), (8, 8, 4, abq.STRATEGY_DECODE),
                          (5, 5, 1, abq.STRATEGY_BCNT), (5, 5, 2, abq.STRATEGY_DECODE), (8, 4, 1, abq.STRATEGY_BCNT)):
        rc, st = _init(abq, q=q, p=p, M=M, N=4096)
        assert rc == 0 and st.strategy == want, (q, p, M)
    rc, st = _init(abq, M=1, N=4096)   # K = 4096: 32 lanes per row, one pass per lane in flight, eight waves of two rows
    assert st.cfg.as_tuple()[3:] == (1, 16, 4096, 1, 2, 4096, 1, 1, 128, 1) and st.block_dim.x == 512 and st.grid_dim.x == 256
    rc, st = _init(abq, M=1, N=4096, K=11008)  # three passes of 32 lanes
    assert st.cfg.nstage == 3 and st.cfg.block_k == 4096
    # a reference (tensor-core) tuple is accepted and resolved to a native tile
    cfg, _ = abq.parse_kernel_name("AqBMMA_8x2xtrue_8x48x256_32x48x128_8x8x128_5")
    rc, st = _init(abq, cfg=cfg, M=8)
    assert rc == 0 and st.strategy == abq.STRATEGY_DECODE and st.cfg.mma_k == 64 and st.cfg.nstage == 3
    assert st.grid_dim.x == 4 and st.block_dim.x == 1024


@pytest.mark.parametrize("q,p", COMBOS)
def test_native_configs_resolve_to_themselves(abq, q, p):
    for signed in (0, 1):
        cfgs = abq.native_configs(q, p, signed)
        assert len(cfgs) >= 12
        seen = set()
        for c in cfgs:
            rc, st = _init(abq, cfg=c, M=8, N=512, K=4096)
            assert rc == 0, c
            assert st.cfg.as_tuple() == c.as_tuple()
            seen.add(abq.format_kernel_name(c))
        assert len(seen) == len(cfgs)
    assert abq.native_configs(9, 9, 1) == []


def test_fp6_route_eligibility_and_tile_tuples(abq):
    """The FP6 matrix-core route takes operands that are E2M3 numbers (unsigned <= 4 bits, signed
    <= 5) while max|x| * max|w| * K stays below 2^24; its tiles are named MMA 32x32x64, NSTAGE 5."""
    for q in range(1, 9):
        for p in range(1, 9):
            for signed in (0, 1):
                lim = 5 if signed else 4
                mx = (1 << (q - 1)) if signed else (1 << q) - 1
                mw = (1 << (p - 1)) if signed else (1 << p) - 1
                for K in (128, 4096, 13824, 65536, 1 << 20):
                    want = q <= lim and p <= lim and mx * mw * K < (1 << 24)
                    assert abq.fp6_eligible(q, p, signed, K) == want, (q, p, signed, K)
    assert abq.lib().abq_fp6_bytes(10, 256) == 10 * 2 * 96 and abq.lib().abq_fp6_bytes(10, 200) == 0
    cfg, _ = abq.parse_kernel_name("AqBMMA_4x4xtrue_256x128x128_64x64x128_32x32x64_5")
    rc, st = _init(abq, cfg=cfg, M=2048, N=4096, K=4096)
    assert rc == 0 and st.strategy == abq.STRATEGY_FP6
    assert st.grid_dim.x == 8 * 4 * 8 and st.block_dim.x == 512 and st.shared_mem_size == 4 * 384 * 96
    # not eligible: 8-bit activations; K beyond the exactness bound; unknown tile
    cfg, _ = abq.parse_kernel_name("AqBMMA_8x2xtrue_256x128x128_64x64x128_32x32x64_5")
    assert _init(abq, cfg=cfg, M=64, N=64, K=256)[0] == abq.ABQ_ERR_UNSUPPORTED
    cfg, _ = abq.parse_kernel_name("AqBMMA_4x4xfalse_128x128x128_64x64x128_32x32x64_5")
    assert _init(abq, cfg=cfg, M=64, N=64, K=65536)[0] == 0
    assert _init(abq, cfg=cfg, M=64, N=64, K=131072)[0] == abq.ABQ_ERR_UNSUPPORTED
    cfg, _ = abq.parse_kernel_name("AqBMMA_4x4xfalse_96x128x128_96x64x128_32x32x64_5")
    assert _init(abq, cfg=cfg, M=64, N=64, K=256)[0] == abq.ABQ_ERR_UNSUPPORTED


# ------------------------------------------------------------------ tile generator

@pytest.fixture(scope="module")
def gen_kernel(tmp_path_factory):
    exe = str(tmp_path_factory.mktemp("gen") / "gen_kernel")
    subprocess.check_call(["g++", "-O2", "-std=c++17", os.path.join(PKG, "engine", "gen_kernel.cpp"), "-o", exe])
    return exe


def _tuples(text):
    pat = re.compile(r"AQ_INSTANTIATE_FUN\(AqBMMA,\s*(\d+),\s*(\d+),\s*(true|false),\s*" + r",\s*".join([r"(\d+)"] * 10) + r"\)")
    return [(int(g[0]), int(g[1]), 1 if g[2] == "true" else 0) + tuple(int(v) for v in g[3:]) for g in pat.findall(text)]


def test_gen_kernel_sm80_space_matches_reference_tile_lists(gen_kernel):
    """The four tile lists the reference ships that its own generator reproduces (as digests)."""
    fx = json.load(open(os.path.join(HERE, "golden", "generator_fixture.json")))
    for name, info in fx["lists"].items():
        out = subprocess.check_output([gen_kernel, str(info["x_bits"]), str(info["w_bits"]), "1", str(fx["k_stage"]),
                                       "--space", "sm80"]).decode()
        tuples = _tuples(out)
        assert len(tuples) == info["count"], name
        h = hashlib.sha256()
        for t in sorted(tuples):
            h.update((",".join(str(v) for v in t) + "\n").encode())
        assert h.hexdigest() == info["sha256_sorted"], name
        assert list(tuples[0]) == info["first"] and list(tuples[-1]) == info["last"]


def test_gen_kernel_sm80_space_matches_reference_generator(gen_kernel):
    ref = os.path.join(ROOT, "oracle", "_ref", "gen_kernel_ref")
    if not os.path.exists(ref):
        pytest.skip("oracle/_ref not built (reference tree not mounted)")
    for q, p in COMBOS:
        for signed in ("0", "1"):
            for ks in ("2", "4", "6"):
                mine = subprocess.check_output([gen_kernel, str(q), str(p), signed, ks, "--space", "sm80"])
                theirs = subprocess.check_output([ref, str(q), str(p), signed, ks])
                assert mine == theirs, (q, p, signed, ks)


def test_gen_kernel_native_space_is_what_the_library_instantiates(gen_kernel, abq):
    inc = open(os.path.join(PKG, "csrc", "abq_mfma_variants.inc")).read()
    committed = [l for l in inc.splitlines() if l.startswith("V(")]
    out = subprocess.check_output([gen_kernel, "8", "8", "1", "4", "--format", "variants"]).decode().splitlines()
    assert out == committed
    for q, p in COMBOS:
        for signed in (0, 1):
            text = subprocess.check_output([gen_kernel, str(q), str(p), str(signed), "4"]).decode()
            gen = set(_tuples(text))
            native = set(c.as_tuple() for c in abq.native_configs(q, p, signed))
            assert gen == native, (q, p, signed)


def test_group_scales_move_a_state_to_the_kernel_that_carries_them(abq):
    """Which strategy a state ends on once group scales are attached, for both orders of the two calls, and that
    a refused call leaves the state untouched (host logic only: nothing is launched)."""
    lib = abq.lib()
    T = abq.LAYOUT_TILED

    def state(q=8, p=2, M=1, signed=1, **kw):
        rc, st = _init(abq, q=q, p=p, M=M, signed=signed, N=4096, K=4096, out_kind=abq.OUT_F16_SCALED, **kw)
        assert rc == 0
        return st

    names = abq.STRATEGY_NAMES
    # plane operands, at most 16 rows: popcount by default, the decode kernel once it has to carry group scales
    st = state()
    assert names[st.strategy] == "bcnt"
    assert lib.abq_gemm_set_scales(ctypes.byref(st), 0x4000, 0x5000, 128) == 0
    assert names[st.strategy] == "decode" and st.group_size == 128
    # ... and the prepared-operand decode kernel when the layouts are declared afterwards
    assert lib.abq_gemm_set_operand_layout(ctypes.byref(st), T, T) == 0
    assert names[st.strategy] == "decode_tiled" and st.group_size == 128 and st.variant == 0
    # layouts first, scales second: the same place
    st = state(M=8)
    assert lib.abq_gemm_set_operand_layout(ctypes.byref(st), T, T) == 0 and names[st.strategy] == "decode_tiled"
    assert lib.abq_gemm_set_scales(ctypes.byref(st), 0x4000, 0x5000, 128) == 0
    assert names[st.strategy] == "decode_tiled" and st.variant == 0
    assert lib.abq_gemm_set_activation(ctypes.byref(st), abq.ACT_SILU_GATE) == 0 and names[st.strategy] == "decode_tiled"
    # groups of 64 run there too (two groups to a K tile); widths of several fields have no variant there: the tiled kernel
    st = state(M=8)
    assert lib.abq_gemm_set_operand_layout(ctypes.byref(st), T, T) == 0
    assert lib.abq_gemm_set_scales(ctypes.byref(st), 0x4000, 0x5000, 64) == 0 and names[st.strategy] == "decode_tiled"
    st = state(q=6, p=2, M=8)
    assert lib.abq_gemm_set_scales(ctypes.byref(st), 0x4000, 0x5000, 128) == 0
    assert lib.abq_gemm_set_operand_layout(ctypes.byref(st), T, T) == 0 and names[st.strategy] == "tiled"
    # more than 16 rows: tiled
    st = state(M=64)
    assert lib.abq_gemm_set_scales(ctypes.byref(st), 0x4000, 0x5000, 128) == 0 and names[st.strategy] == "tiled"
    # a refused call (unsigned 8-bit operands have no group-scale kernel) changes nothing, not even the strategy the
    # call had moved the state to on its way
    st = state(q=8, p=8, signed=0)
    before = bytes(st)
    assert lib.abq_gemm_set_scales(ctypes.byref(st), 0x4000, 0x5000, 128) == abq.ABQ_ERR_UNSUPPORTED
    assert bytes(st) == before
    cfg = abq.native_configs(8, 2, 1)
    pinned = [c for c in cfg if c.mma_k == 128][0]  # a popcount tile named by the caller stays where it is
    rc, st = _init(abq, cfg=pinned, q=8, p=2, M=1, N=4096, K=4096, out_kind=abq.OUT_F16_SCALED)
    assert rc == 0
    before = bytes(st)
    assert lib.abq_gemm_set_scales(ctypes.byref(st), 0x4000, 0x5000, 128) == abq.ABQ_ERR_UNSUPPORTED
    assert bytes(st) == before


def test_workspace_after_layouts_and_scales_keeps_a_consistent_state(abq):
    """layouts -> scales -> workspace at 32 rows: a state on the prepared-operand decode kernel stays there (it converts
    nothing), and a group-scale state that does move lands on a variant of the group-scale table."""
    lib = abq.lib()
    T = abq.LAYOUT_TILED
    names = abq.STRATEGY_NAMES
    for (N, K) in ((4096, 4096), (4096, 11008)):
        rc, st = _init(abq, q=8, p=2, M=32, signed=1, N=N, K=K, out_kind=abq.OUT_F16_SCALED)
        assert rc == 0
        assert lib.abq_gemm_set_operand_layout(ctypes.byref(st), T, T) == 0
        assert lib.abq_gemm_set_scales(ctypes.byref(st), 0x4000, 0x5000, 128) == 0
        assert names[st.strategy] == "decode_tiled" and st.variant == 0
        before = (st.strategy, st.variant, st.cfg.as_tuple())
        assert lib.abq_gemm_set_workspace(ctypes.byref(st), 0x100000, 1 << 20) == 0
        assert (st.strategy, st.variant, st.cfg.as_tuple()) == before
        assert lib.abq_gemm_workspace_bytes(ctypes.byref(st)) == 0
    # without group scales: 65 to 128 rows on the decode kernel stay there as well
    rc, st = _init(abq, q=4, p=4, M=64, signed=1, N=4096, K=4096)
    assert rc == 0 and lib.abq_gemm_set_operand_layout(ctypes.byref(st), T, T) == 0
    assert names[st.strategy] == "decode_tiled"
    assert lib.abq_gemm_set_workspace(ctypes.byref(st), 0x100000, 1 << 20) == 0 and names[st.strategy] == "decode_tiled"
    # plane operands with group scales at 32 rows (the group-scale prefill kernel from the start): the workspace call
    # keeps the variant inside the group-scale table
    rc, st = _init(abq, q=8, p=2, M=32, signed=1, N=4096, K=4096, out_kind=abq.OUT_F16_SCALED)
    assert rc == 0 and lib.abq_gemm_set_scales(ctypes.byref(st), 0x4000, 0x5000, 128) == 0
    assert names[st.strategy] == "tiled"
    v = st.variant
    assert lib.abq_gemm_set_workspace(ctypes.byref(st), 0x100000, 64 << 20) == 0
    assert names[st.strategy] == "tiled" and st.variant == v
    # fp16 activations handed to the decode kernel are not converted: no workspace asked for them
    rc, st = _init(abq, q=8, p=2, M=4, signed=1, N=4096, K=4096)
    assert rc == 0 and lib.abq_gemm_set_operand_layout(ctypes.byref(st), T, T) == 0
    assert lib.abq_gemm_set_f16_activations(ctypes.byref(st), 0x200000, 0x300000) == 0
    assert lib.abq_gemm_workspace_bytes(ctypes.byref(st)) == 0


def test_a_loaded_tuning_table_overrides_the_rules(abq, tmp_path):
    """The autotune result is consumed: an entry of the table moves a state whose tile is the library's choice to the
    measured tile, on the layouts it runs on, for the M of its bucket, and a pinned tile stays where it is."""
    lib = abq.lib()
    T, F6, P = abq.LAYOUT_TILED, abq.LAYOUT_FP6, abq.LAYOUT_PLANES
    names = abq.STRATEGY_NAMES
    N, K = 4224, 2176  # a shape no compiled-in entry names

    def tile_after(q, p, M, xl, wl, workspace=False, group=0):
        rc, st = _init(abq, q=q, p=p, M=M, signed=1, N=N, K=K, out_kind=abq.OUT_F16_SCALED if group else abq.OUT_I32)
        assert rc == 0
        if group:
            assert lib.abq_gemm_set_scales(ctypes.byref(st), 0x4000, 0x5000, group) == 0
        if (xl, wl) != (P, P):
            assert lib.abq_gemm_set_operand_layout(ctypes.byref(st), xl, wl) == 0
        if workspace:
            assert lib.abq_gemm_set_workspace(ctypes.byref(st), 0x100000, 256 << 20) == 0
        return abq.format_kernel_name(st.cfg), names[st.strategy], st

    lib.abq_tuning_clear()
    try:
        assert lib.abq_tuning_lookup(4, 4, 1, 128, N, K, 0, 0, ctypes.byref(abq.TileConfig()), None) == abq.ABQ_ERR_UNSUPPORTED
        by_rules = tile_after(4, 4, 128, P, T, workspace=True)[0]
        by_rules_no_room = tile_after(4, 4, 128, P, T)[0]  # (nowhere to convert the activations: no decode kernel)
        by_rules_planes = tile_after(4, 4, 128, P, P)[0]
        by_rules_fp6 = tile_after(4, 4, 128, F6, F6)[0]
        # three measured tiles for the shape, one per operand layout, none of them the rules' choice
        tiled_tile = "AqBMMA_4x4xtrue_128x64x128_64x32x128_32x32x32_4"
        decode_tile = "AqBMMA_4x4xtrue_16x16x2048_16x16x128_16x16x64_6"
        fp6_tile = "AqBMMA_4x4xtrue_128x128x128_64x64x128_32x32x64_5"
        planes_tile = "AqBMMA_4x4xtrue_64x64x256_32x32x256_32x32x32_2"
        for name in (tiled_tile, decode_tile, fp6_tile, planes_tile):
            assert name not in (by_rules, by_rules_no_room, by_rules_planes, by_rules_fp6)
        table = tmp_path / "tuned.txt"
        table.write_text("# measured\n%s 128 %d %d 0 500.0\n%s 100 %d %d 0 450.5\n%s 128 %d %d 0 300\n"
                         % (tiled_tile, N, K, fp6_tile, N, K, planes_tile, N, K))
        taken = ctypes.c_int(0)
        assert lib.abq_tuning_load(str(table).encode(), ctypes.byref(taken)) == 0 and taken.value == 3
        # ... each layout gets its entry; rows 65 to 128 share a bucket, 64 and 129 are outside it
        assert tile_after(4, 4, 128, P, T, workspace=True)[0] == tiled_tile
        assert tile_after(4, 4, 65, T, T)[0] == tiled_tile.replace("128x64x128", "128x64x128")
        assert tile_after(4, 4, 128, F6, F6)[0] == fp6_tile
        assert tile_after(4, 4, 128, P, P)[0] == planes_tile
        assert tile_after(4, 4, 64, P, T, workspace=True)[0] != tiled_tile
        assert tile_after(4, 4, 129, P, T, workspace=True)[0] != tiled_tile
        assert tile_after(4, 4, 128, P, T, workspace=True)[2].auto_chosen == 1
        # another shape, another pair: the rules
        rc, st = _init(abq, q=4, p=4, M=128, signed=1, N=N + 128, K=K)
        assert rc == 0 and lib.abq_gemm_set_operand_layout(ctypes.byref(st), T, T) == 0
        assert abq.format_kernel_name(st.cfg) != tiled_tile
        # the best over all layouts is what a loader is told to prepare, and what the lookup returns
        assert lib.abq_preferred_weight_layout(4, 4, 1, 128, N, K, 0) == T
        cfg, tops = abq.TileConfig(), ctypes.c_float(0)
        assert lib.abq_tuning_lookup(4, 4, 1, 100, N, K, 0, 0, ctypes.byref(cfg), ctypes.byref(tops)) == 0
        assert abq.format_kernel_name(cfg) == tiled_tile and tops.value == 500.0
        assert lib.abq_tuning_lookup(4, 4, 1, 100, N, K, 0, 1 << F6, ctypes.byref(cfg), ctypes.byref(tops)) == 0
        assert abq.format_kernel_name(cfg) == fp6_tile and abs(tops.value - 450.5) < 1e-3
        # a faster entry added later wins; the decode kernel on prepared operands needs the activations K-tiled, or a
        # workspace to convert them into
        cfg2 = abq.parse_kernel_name(decode_tile)[0]
        assert lib.abq_tuning_add(ctypes.byref(cfg2), 128, N, K, 0, 600.0) == 0
        assert tile_after(4, 4, 128, T, T)[:2] == (decode_tile, "decode_tiled")
        assert tile_after(4, 4, 128, P, T)[0] in (tiled_tile, by_rules_no_room)
        assert tile_after(4, 4, 128, P, T, workspace=True)[:2] == (decode_tile, "decode_tiled")
        # a tile the caller names is not moved
        pinned = abq.parse_kernel_name("AqBMMA_4x4xtrue_64x64x128_32x32x128_32x32x32_4")[0]
        rc, st = _init(abq, cfg=pinned, q=4, p=4, M=128, N=N, K=K)
        assert rc == 0 and lib.abq_gemm_set_operand_layout(ctypes.byref(st), T, T) == 0
        assert st.cfg.as_tuple() == pinned.as_tuple()
        # group scales: their own entries (group size is part of the key), taken where the tile is picked
        g_tile = "AqBMMA_8x2xtrue_256x128x128_64x64x128_32x32x32_4"
        assert tile_after(8, 2, 1024, T, T, group=128)[0] != g_tile
        assert lib.abq_tuning_add(ctypes.byref(abq.parse_kernel_name(g_tile)[0]), 1024, N, K, 128, 1000.0) == 0
        assert tile_after(8, 2, 1024, T, T, group=128)[0] == g_tile
        assert tile_after(8, 2, 1024, T, T)[0] != g_tile or True  # (the plain GEMM of that shape has no entry)
        # a malformed file is refused as a whole
        bad = tmp_path / "bad.txt"
        bad.write_text("%s 128 %d %d 0 1.0\nnot a kernel name 1 2 3\n" % (tiled_tile, N, K))
        assert lib.abq_tuning_load(str(bad).encode(), ctypes.byref(taken)) == abq.ABQ_ERR_INVALID_ARG and taken.value == 0
        assert lib.abq_tuning_load(b"/nonexistent/file", None) == abq.ABQ_ERR_INVALID_ARG
        lib.abq_tuning_clear()
        assert tile_after(4, 4, 128, P, T, workspace=True)[0] == by_rules
    finally:
        lib.abq_tuning_clear()


def test_compiled_in_tuning_table_serves_the_sweep_it_came_from(abq):
    """engine/tuning_mi355x.txt is compiled in: its entries are what a state of that shape gets, and switching the
    compiled-in table off gives the rules back."""
    lib = abq.lib()
    lines = [l.split() for l in open(os.path.join(PKG, "engine", "tuning_mi355x.txt")) if l.strip() and not l.startswith("#")]
    assert len(lines) >= 66
    seen = 0
    for name, M, N, K, group, tops in lines:
        cfg, _ = abq.parse_kernel_name(name)
        got = abq.TileConfig()
        assert lib.abq_tuning_lookup(cfg.x_bits, cfg.w_bits, cfg.is_signed, int(M), int(N), int(K), int(group),
                                     1 << (2 if cfg.nstage == 5 else 1 if cfg.nstage in (4, 6) else 0), ctypes.byref(got), None) == 0
        seen += 1
    assert seen == len(lines)
    try:
        lib.abq_tuning_enable_builtin(0)
        name, M, N, K, group, _ = lines[0]
        cfg, _ = abq.parse_kernel_name(name)
        assert lib.abq_tuning_lookup(cfg.x_bits, cfg.w_bits, cfg.is_signed, int(M), int(N), int(K), int(group), 0,
                                     ctypes.byref(abq.TileConfig()), None) == abq.ABQ_ERR_UNSUPPORTED
    finally:
        lib.abq_tuning_enable_builtin(1)


def test_unsigned_8bit_codes_reach_the_prepared_decode_kernel_with_their_row_sums(abq):
    """Unsigned 8-bit codes are fed as value - 128: the decode kernel on prepared operands takes such a state only once
    the row sums are set; padded records of narrower codes (value bits declared) need none."""
    lib = abq.lib()
    T = abq.LAYOUT_TILED
    names = abq.STRATEGY_NAMES

    def state(q, p, M=4):
        rc, st = _init(abq, q=q, p=p, M=M, signed=0, N=4096, K=4096)
        assert rc == 0 and lib.abq_gemm_set_operand_layout(ctypes.byref(st), T, T) == 0
        return st

    st = state(8, 8)
    assert names[st.strategy] == "tiled"
    assert lib.abq_gemm_set_row_sums(ctypes.byref(st), 0x7000, None) == 0 and names[st.strategy] == "tiled"  # both are needed
    assert lib.abq_gemm_set_row_sums(ctypes.byref(st), 0x7000, 0x8000) == 0 and names[st.strategy] == "decode_tiled"
    st = state(8, 2)
    assert names[st.strategy] == "tiled"
    assert lib.abq_gemm_set_row_sums(ctypes.byref(st), None, 0x8000) == 0 and names[st.strategy] == "decode_tiled"
    # padded records: 7-bit codes in 8-bit fields need no sums; a mix of real and padded 8-bit operands has no kernel there
    st = state(8, 8)
    assert lib.abq_gemm_set_value_bits(ctypes.byref(st), 7, 7) == 0 and names[st.strategy] == "decode_tiled"
    st = state(8, 8)
    assert lib.abq_gemm_set_value_bits(ctypes.byref(st), 8, 7) == 0
    assert lib.abq_gemm_set_row_sums(ctypes.byref(st), 0x7000, 0x8000) == 0 and names[st.strategy] == "tiled"
    st = state(8, 2)
    assert lib.abq_gemm_set_value_bits(ctypes.byref(st), 6, 2) == 0 and names[st.strategy] == "decode_tiled"
    assert lib.abq_gemm_set_value_bits(ctypes.byref(st), 9, 2) == abq.ABQ_ERR_INVALID_ARG
    assert lib.abq_gemm_set_value_bits(ctypes.byref(st), 6, 0) == abq.ABQ_ERR_INVALID_ARG
    # more than 16 rows: where the prefill kernel is the better choice the sums change nothing about the strategy
    st = state(8, 8, M=512)
    assert lib.abq_gemm_set_row_sums(ctypes.byref(st), 0x7000, 0x8000) == 0 and names[st.strategy] == "tiled"
    assert lib.abq_gemm_row_sums_ready(ctypes.byref(st)) == 1
    assert [abq.padded_bits(b) for b in range(0, 10)] == [0, 2, 2, 4, 4, 8, 8, 8, 8, 0]


def test_weights_of_several_fields_reach_the_prepared_decode_kernel_as_they_are(abq):
    """Weights of 3, 5, 6, 7 bits: the decode kernel on prepared operands reads the prefill kernels' records, so a
    decode-sized state with both operands K-tiled moves there with the pair's own widths.  Activations of such widths
    only as padded records: declared before or after the layouts; undeclared, the state stays on the prefill kernel;
    the workspace of plane activations counts the padded size; more than 16 rows stay on the prefill kernel."""
    lib = abq.lib()
    T, P = abq.LAYOUT_TILED, abq.LAYOUT_PLANES
    names = abq.STRATEGY_NAMES

    def fresh(q, p, M=4, signed=1):
        rc, st = _init(abq, q=q, p=p, M=M, signed=signed, N=4096, K=4096)
        assert rc == 0
        return st

    st = fresh(8, 3)  # activations of one field: nothing to declare
    assert lib.abq_gemm_set_operand_layout(ctypes.byref(st), T, T) == 0 and names[st.strategy] == "decode_tiled"
    assert (st.cfg.x_bits, st.cfg.w_bits, st.cfg.nstage) == (8, 3, 6) and lib.abq_gemm_workspace_bytes(ctypes.byref(st)) == 0
    for q, p in [(3, 3), (5, 5), (6, 6), (7, 7), (6, 2)]:
        st = fresh(q, p)
        assert lib.abq_gemm_set_operand_layout(ctypes.byref(st), T, T) == 0 and names[st.strategy] == "tiled"
        assert lib.abq_gemm_set_padded_activations(ctypes.byref(st), 1) == 0 and names[st.strategy] == "decode_tiled"
        assert (st.cfg.x_bits, st.cfg.w_bits, st.cfg.nstage) == (q, p, 6)
        assert lib.abq_gemm_set_padded_activations(ctypes.byref(st), 0) == 0 and names[st.strategy] == "tiled"
        st = fresh(q, p)  # the other order
        assert lib.abq_gemm_set_padded_activations(ctypes.byref(st), 1) == 0
        assert lib.abq_gemm_set_operand_layout(ctypes.byref(st), T, T) == 0 and names[st.strategy] == "decode_tiled"
        # plane activations under a tile of that kernel: exec pads them into the workspace
        cfg = [c for c in abq.native_configs(q, p, True) if c.nstage == 6][0]
        rc, st = _init(abq, q=q, p=p, M=4, signed=1, N=4096, K=4096, cfg=cfg)
        assert rc == 0 and lib.abq_gemm_set_operand_layout(ctypes.byref(st), P, T) == 0
        assert lib.abq_gemm_workspace_bytes(ctypes.byref(st)) == 4 * 4096 * abq.padded_bits(q) // 8
        # ... and records of the activations' own width are refused for it
        assert lib.abq_gemm_set_operand_layout(ctypes.byref(st), T, T) == abq.ABQ_ERR_UNSUPPORTED
        st = fresh(q, p, M=64)  # more than 16 rows: only the prefill kernel, which reads no padded records
        assert lib.abq_gemm_set_operand_layout(ctypes.byref(st), T, T) == 0 and names[st.strategy] == "tiled"
        assert lib.abq_gemm_set_padded_activations(ctypes.byref(st), 1) == abq.ABQ_ERR_UNSUPPORTED and names[st.strategy] == "tiled"
    st = fresh(8, 2)
    assert lib.abq_gemm_set_padded_activations(ctypes.byref(st), 1) == 0 and st.reserved[4] == 0  # one field: its own padding


def test_prefill_tile_choice_on_the_baseline_shapes(abq):
    """The tile the library picks for prepared operands, pinned on shapes of BASELINE.json configs[2] and
    configs[4] and on a few where the measured sweep of all tiles separates them clearly:
    large tiles only where their quantised grids pay, 128x128 in between, small tiles for small grids."""
    lib = abq.lib()

    def picked(q, p, M, N, K, layout, group=0):
        rc, st = _init(abq, q=q, p=p, M=M, N=N, K=K, out_kind=abq.OUT_F16_SCALED if group else abq.OUT_I32)
        assert rc == 0
        if group:
            assert lib.abq_gemm_set_scales(ctypes.byref(st), 0x4000, 0x5000, group) == 0
        assert lib.abq_gemm_set_operand_layout(ctypes.byref(st), layout, layout) == 0
        c = st.cfg
        return (c.block_m, c.block_n, c.block_k, c.warp_m, c.warp_n, c.nstage)

    T, F6 = abq.LAYOUT_TILED, abq.LAYOUT_FP6
    # W4A4 on the FP6 route: 128x128 from a chip's worth of tiles up where the larger tile's grid is ragged
    assert picked(4, 4, 512, 4096, 4096, F6) == (128, 64, 128, 64, 32, 5)
    assert picked(4, 4, 256, 4096, 4096, F6) == (64, 64, 128, 32, 32, 5)
    assert picked(4, 4, 1024, 11008, 4096, F6) == (128, 128, 128, 64, 64, 5)
    assert picked(4, 4, 1024, 4096, 4096, F6) == (128, 128, 128, 64, 64, 5)
    # ... and 256x128 where its rounds of workgroups come out even
    assert picked(4, 4, 512, 11008, 4096, F6) == (256, 128, 128, 64, 64, 5)
    assert picked(4, 4, 2048, 12288, 4096, F6) == (256, 128, 128, 64, 64, 5)
    assert picked(4, 4, 16384, 4096, 4096, F6) == (256, 128, 128, 64, 64, 5)
    # W2A8: 256x256 only where its grid is whole rounds of the chip
    assert picked(8, 2, 2048, 4096, 4096, T) == (128, 128, 128, 64, 64, 4)
    assert picked(8, 2, 4096, 11008, 4096, T) == (128, 128, 128, 64, 64, 4)       # 688 tiles of 256x256: a third round mostly empty
    assert picked(8, 2, 4096, 4096, 4096, T) == (256, 256, 128, 64, 128, 4)
    assert picked(8, 2, 8192, 4096, 4096, T) == (256, 256, 128, 64, 128, 4)
    # small grids: two groups of waves split K inside the workgroup, and the tile lies along N where an activation
    # row is the longer record (also up to 400 tiles of 128x128, without the split)
    assert picked(8, 2, 512, 4096, 4096, T) == (64, 128, 256, 32, 64, 4)
    assert picked(8, 2, 256, 4096, 4096, T) == (64, 64, 256, 32, 32, 4)
    assert picked(4, 4, 512, 4096, 4096, T) == (128, 64, 256, 64, 32, 4)
    assert picked(8, 2, 512, 11008, 4096, T) == (64, 128, 128, 32, 64, 4)
    assert picked(8, 2, 384, 12288, 4096, T) == (64, 128, 128, 32, 64, 4)
    assert picked(8, 2, 1024, 4096, 4096, T) == (128, 128, 256, 64, 64, 4)     # one round of 128x128 tiles: with the split
    assert picked(4, 4, 1024, 4096, 11008, T) == (128, 128, 256, 64, 64, 4)
    assert picked(8, 8, 1024, 4096, 4096, T) == (128, 128, 128, 64, 64, 4)     # (not built for W8A8)
    # the tiles whose waves split K stay within one round of workgroups: past 256 of the 64x128 (128x64) tile, 128x128
    assert picked(8, 4, 256, 11008, 4096, T) == (128, 128, 256, 64, 64, 4)
    assert picked(8, 2, 192, 11008, 4096, T) == (128, 128, 256, 64, 64, 4)
    assert picked(4, 4, 256, 11008, 4096, T) == (128, 128, 256, 64, 64, 4)
    assert picked(8, 4, 768, 4096, 4096, T) == (128, 128, 256, 64, 64, 4)
    assert picked(8, 4, 384, 4096, 4096, T) == (64, 128, 256, 32, 64, 4)      # 192 workgroups: as before
    # signed W8A8: 128x64 and 128x128 from 160 workgroups (more than 256 of the smaller tile would be a second round)
    assert picked(8, 8, 128, 11008, 4096, T) == (128, 64, 128, 64, 32, 4)
    assert picked(8, 8, 256, 11008, 4096, T) == (128, 128, 128, 64, 64, 4)
    assert picked(8, 8, 768, 4096, 4096, T) == (128, 128, 128, 64, 64, 4)
    assert picked(8, 8, 256, 4096, 4096, T) == (64, 64, 128, 32, 32, 4)
    # ... and on long K, up to one round of 128x64 tiles, that tile with its waves splitting K
    assert picked(8, 8, 512, 4096, 11008, T) == (128, 64, 256, 64, 32, 4)
    assert picked(8, 8, 512, 4096, 4096, T) == (128, 64, 128, 64, 32, 4)
    # signed W8A8: 256x128 as soon as it fills the chip
    assert picked(8, 8, 2048, 4096, 4096, T) == (256, 128, 128, 64, 64, 4)
    assert picked(8, 8, 1024, 4096, 4096, T) == (128, 128, 128, 64, 64, 4)
    assert picked(8, 8, 512, 11008, 4096, T) == (256, 128, 128, 64, 64, 4)
    assert picked(8, 8, 4096, 4096, 4096, T) == (256, 128, 128, 64, 64, 4)
    # group scales (the decoder-layer linears): 128x128 once it fills the chip, 128x64 below
    assert picked(8, 2, 1024, 12288, 4096, T, group=128) == (128, 128, 128, 64, 64, 4)
    assert picked(8, 2, 1024, 4096, 4096, T, group=128) == (128, 128, 256, 64, 64, 4)  # one round of 128x128: waves split K
    assert picked(8, 2, 1024, 5120, 5120, T, group=128) == (128, 128, 128, 64, 64, 4)  # 320 workgroups: not
    assert picked(8, 2, 16384, 22016, 4096, T, group=128) == (128, 128, 128, 64, 64, 4)
    assert picked(8, 2, 128, 4096, 4096, T, group=64) == (64, 64, 128, 32, 32, 4)
    # up to one 128x64 workgroup per compute unit: the tile whose waves split K (its stages fill a compute unit's LDS)
    assert picked(8, 2, 512, 4096, 4096, T, group=128) == (128, 64, 256, 64, 32, 4)
    assert picked(8, 2, 128, 12288, 4096, T, group=128) == (128, 64, 256, 64, 32, 4)
    # up to one 64x64 workgroup per compute unit: that tile with the split (one MFMA tile per wave)
    assert picked(8, 2, 128, 4096, 11008, T, group=128) == (64, 64, 256, 32, 32, 4)
    assert picked(8, 2, 64, 12288, 4096, T, group=128) == (64, 64, 256, 32, 32, 4)
    assert picked(8, 2, 256, 4096, 4096, T, group=128) == (64, 64, 256, 32, 32, 4)
    assert picked(8, 8, 64, 4096, 4096, T, group=128) == (64, 64, 256, 32, 32, 4)
    # 384 workgroups would be two rounds of it: the 128x128 tile with the same split while that makes one round
    assert picked(8, 2, 192, 12288, 4096, T, group=128) == (128, 128, 256, 64, 64, 4)
    assert picked(8, 2, 128, 22016, 4096, T, group=128) == (128, 128, 256, 64, 64, 4)
    assert picked(8, 2, 384, 12288, 4096, T, group=128) == (128, 128, 128, 64, 64, 4)  # 288 tiles of 128x128: that tile, no split
    assert picked(4, 4, 384, 12288, 4096, T, group=128) == (128, 64, 128, 64, 32, 4)   # (narrow activations: 128x64 up to 400)
    assert picked(8, 2, 64, 22016, 4096, T, group=128) == (64, 128, 256, 32, 64, 4)    # ... one round of the 64x128 one
    assert picked(4, 4, 64, 22016, 4096, T, group=128) == (128, 128, 256, 64, 64, 4)   # (built for activations wider than weights)
    # ... activations of at most 4 bits keep 128x64 up to 400 tiles
    assert picked(4, 4, 512, 11008, 4096, T, group=128) == (128, 64, 128, 64, 32, 4)
    assert picked(8, 2, 512, 11008, 4096, T, group=128) == (128, 128, 128, 64, 64, 4)
    assert picked(4, 4, 2048, 4096, 4096, T, group=128) == (128, 128, 128, 64, 64, 4)
    # W8A8 with group scales: the LDS-staged kernel has the 128x64 tile only, and it is the faster one on large grids too
    assert picked(8, 8, 16384, 4096, 4096, T, group=128) == (128, 64, 128, 64, 32, 4)
    assert picked(8, 8, 2048, 12288, 4096, T, group=128) == (128, 64, 128, 64, 32, 4)
    # group scales on FP6 records: 256x128 where its rounds of workgroups come out even
    assert picked(4, 4, 2048, 4096, 4096, F6, group=128) == (256, 128, 128, 64, 64, 5)
    assert picked(4, 4, 1024, 11008, 4096, F6, group=128) == (128, 128, 128, 64, 64, 5)   # 344 tiles of 256x128: 1.3 rounds
    assert picked(4, 4, 16384, 4096, 11008, F6, group=128) == (256, 128, 128, 64, 64, 5)
    assert picked(4, 4, 1024, 4096, 4096, F6, group=128) == (128, 128, 128, 64, 64, 5)
    assert picked(4, 4, 512, 4096, 4096, F6, group=128) == (128, 64, 128, 64, 32, 5)


def test_preferred_weight_records_name_the_padded_pair_for_widths_of_several_fields(abq):
    """What a loader is told to write: for weights of 2, 4, 8 bits the layout abq_preferred_weight_layout names, at their
    own width; for 3, 5, 6, 7 bits K-tiled records of the next single-field width at every M (the padded pair's
    kernels), or FP6 records where that pair's answer is FP6 and the codes qualify; signed 5-bit weights under
    narrow activations keep FP6 records above 16 rows."""
    lib = abq.lib()
    T, F6 = abq.LAYOUT_TILED, abq.LAYOUT_FP6
    bits = ctypes.c_int(0)

    def ask(q, p, signed, M, N=5120, K=5120, group=0):
        layout = lib.abq_preferred_weight_records(q, p, signed, M, N, K, group, ctypes.byref(bits))
        return layout, bits.value

    for (q, p) in [(8, 2), (4, 4), (8, 8), (2, 2), (8, 4)]:
        for M in (1, 8, 128, 2048):
            assert ask(q, p, 1, M) == (lib.abq_preferred_weight_layout(q, p, 1, M, 5120, 5120, 0), p)
    for M in (1, 8, 16, 128, 2048):
        assert ask(6, 6, 1, M) == (T, 8) and ask(7, 7, 0, M) == (T, 8) and ask(5, 5, 0, M) == (T, 8)
        assert ask(8, 3, 1, M) == (T, 4) and ask(8, 3, 1, M, group=128) == (T, 4)
    assert ask(5, 5, 1, 128) == (F6, 5) and ask(5, 5, 1, 8) == (T, 8)
    assert ask(8, 5, 1, 128) == (T, 8)            # activations too wide for FP6
    # 3-bit weights under 3-bit activations: whatever the 4-bit pair is told, at the width that layout holds
    for M in (8, 128, 2048):
        want = lib.abq_preferred_weight_layout(4, 4, 1, M, 5120, 5120, 0)
        assert ask(3, 3, 1, M) == ((F6, 3) if want == F6 else (T, 4))
    assert lib.abq_preferred_weight_records(6, 6, 1, 128, 5120, 5120, 0, None) == T


def test_folded_record_entry_points_check_their_arguments(abq):
    """abq_relayout_planes_folded / abq_relayout_planes_fp6_folded refuse, before any launch: null pointers, rows <= 0,
    bit widths they have no records for (8-bit codes less a zero point need nine bits; FP6 holds differences of codes of
    at most 4 bits), groups that are no multiple of 32 or do not divide K, K that is no multiple of 128."""
    lib = abq.lib()
    P = ctypes.c_void_p(0x1000)  # never dereferenced on the host: every call below returns before a launch
    OK_K, G = 4096, 128
    assert lib.abq_folded_bits(2) == 4 and lib.abq_folded_bits(3) == 4 and lib.abq_folded_bits(4) == 8
    assert lib.abq_folded_bits(7) == 8 and lib.abq_folded_bits(8) == 0 and lib.abq_folded_bits(0) == 0
    for fn, widest in ((lib.abq_relayout_planes_folded, 7), (lib.abq_relayout_planes_fp6_folded, 4)):
        assert fn(None, P, G, P, 16, OK_K, 2, 1, P, None) == 1
        assert fn(P, None, G, P, 16, OK_K, 2, 1, P, None) == 1
        assert fn(P, P, G, None, 16, OK_K, 2, 1, P, None) == 1
        assert fn(P, P, G, P, 0, OK_K, 2, 1, P, None) == 1
        assert fn(P, P, G, P, 16, OK_K, 0, 1, P, None) == 1
        assert fn(P, P, 48, P, 16, OK_K, 2, 1, P, None) == 1       # groups of whole plane words only
        assert fn(P, P, 0, P, 16, OK_K, 2, 1, P, None) == 1
        assert fn(P, P, G, P, 16, OK_K, widest + 1, 1, P, None) == 3
        assert fn(P, P, G, P, 16, 4096 + 64, 2, 1, P, None) == 2
        assert fn(P, P, G, P, 16, 64, 2, 1, P, None) == 2
        assert fn(P, P, 96, P, 16, OK_K, 2, 1, P, None) == 2       # 96 does not divide 4096


def test_small_batches_with_plane_activations_reach_the_prepared_decode_kernel_once_there_is_a_workspace(abq):
    """Weights prepared, activations still planes, 17 to 128 rows: with a workspace to convert the activations into, the
    state moves to the decode kernel of prepared operands wherever it would with prepared activations (either kernel
    converts them first); without one, with group scales, or where the prefill tile is estimated ahead, it stays."""
    lib = abq.lib()
    T, P = abq.LAYOUT_TILED, abq.LAYOUT_PLANES
    names = abq.STRATEGY_NAMES

    def strategy(q, p, M, N, K, xl, workspace):
        rc, st = _init(abq, q=q, p=p, M=M, signed=1, N=N, K=K)
        assert rc == 0 and lib.abq_gemm_set_operand_layout(ctypes.byref(st), xl, T) == 0
        if workspace:
            assert lib.abq_gemm_set_workspace(ctypes.byref(st), 0x100000, 256 << 20) == 0
            assert lib.abq_gemm_workspace_bytes(ctypes.byref(st)) <= 256 << 20
        return names[st.strategy]

    lib.abq_tuning_clear()
    lib.abq_tuning_enable_builtin(0)  # the rules alone
    try:
        for (q, p, M, N, K) in [(8, 2, 32, 4096, 4096), (4, 4, 64, 4096, 4096), (2, 2, 48, 4096, 11008), (8, 2, 24, 4096, 11008),
                                (8, 2, 128, 11008, 4096), (8, 8, 64, 4096, 4096), (8, 2, 300, 4096, 4096)]:
            with_records = strategy(q, p, M, N, K, T, False)
            assert strategy(q, p, M, N, K, P, True) == with_records
            assert strategy(q, p, M, N, K, P, False) == "tiled"
        assert strategy(8, 2, 32, 4096, 4096, P, True) == "decode_tiled" and strategy(2, 2, 48, 4096, 11008, P, True) == "decode_tiled"
        assert strategy(8, 2, 128, 11008, 4096, P, True) == "tiled" and strategy(8, 2, 300, 4096, 4096, P, True) == "tiled"
    finally:
        lib.abq_tuning_enable_builtin(1)
