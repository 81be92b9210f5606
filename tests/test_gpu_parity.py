"""GPU parity tests: every kernel is called through the C ABI (libabq_gemm.so) and compared
bit for bit with the CPU oracle on the same seeded inputs.  Inputs are packed by the oracle on
the host, so the GEMM tests do not depend on the pack kernels."""
import json
import os

import numpy as np
import pytest

torch = pytest.importorskip("torch")

pytestmark = pytest.mark.gpu

COMBOS = [(2, 2), (3, 3), (4, 4), (5, 5), (6, 6), (7, 7), (8, 8), (4, 2), (6, 2), (8, 2), (8, 4), (8, 3)]
BASELINE_COMBOS = [c for c in COMBOS if c != (8, 3)]  # the 11 of BASELINE.json configs[3]


def rand_vals(rng, rows, k, bits, signed):
    lo, hi = (-(1 << (bits - 1)), (1 << (bits - 1)) - 1) if signed else (0, (1 << bits) - 1)
    return rng.integers(lo, hi + 1, size=(rows, k), dtype=np.int32)


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int32) if a.dtype == np.uint32 else np.ascontiguousarray(a)).cuda()


def planes_dev(planes):
    return torch.from_numpy(np.ascontiguousarray(planes).view(np.int32)).cuda()


def run_cfg(abq, xd, wd, signed, cfg=None, **kw):
    """Runs one configuration; kernels on the K-tiled layout get the workspace they ask for."""
    g = abq.Gemm(xd, wd, signed, cfg=cfg, **kw)
    if g.strategy in ("tiled", "fp6", "decode_tiled") and g.workspace_bytes and "workspace" not in kw:
        ws = torch.empty(g.workspace_bytes, dtype=torch.uint8, device="cuda")
        g = abq.Gemm(xd, wd, signed, cfg=cfg, workspace=ws, **kw)
    return g.run()


@pytest.fixture(scope="module", autouse=True)
def _need_gpu():
    if not torch.cuda.is_available():
        pytest.fail("marked gpu but no GPU is visible")


# ------------------------------------------------------------------ packing

@pytest.mark.parametrize("rows,k,bits", [(1, 128, 8), (3, 128, 2), (8, 4096, 8), (17, 384, 5), (64, 4096, 4),
                                         (5, 11008, 8), (2, 256, 13), (1, 128, 32), (130, 1152, 7)])
def test_pack_i32_bit_exact(abq, oracle, rows, k, bits):
    rng = np.random.default_rng(rows * 1000 + k + bits)
    v = rng.integers(-(1 << 31), (1 << 31) - 1, size=(rows, k), dtype=np.int64).astype(np.int32) if bits > 8 \
        else rand_vals(rng, rows, k, 8, True)  # values wider than `bits` must alias like the reference
    got = abq.pack_i32(dev(v), bits).cpu().numpy().view(np.uint32)
    assert np.array_equal(got, oracle.pack_i32(v, bits))


def test_pack_i32_large_and_round_trip(abq, oracle):
    rng = np.random.default_rng(11)
    v = rand_vals(rng, 2048, 4096, 8, True)
    got = abq.pack_i32(dev(v), 8).cpu().numpy().view(np.uint32)
    assert np.array_equal(got, oracle.pack_i32(v, 8))
    assert np.array_equal(oracle.unpack(got, True), v)


@pytest.mark.parametrize("rows,k", [(1, 128), (16, 256), (64, 4096)])
def test_pack_u4_bit_exact(abq, oracle, rows, k):
    rng = np.random.default_rng(rows + k)
    words = rng.integers(0, 1 << 32, size=rows * k // 8, dtype=np.uint64).astype(np.uint32)
    got = abq.pack_u4(dev(words), rows, k, 4).cpu().numpy().view(np.uint32)
    assert np.array_equal(got, oracle.pack_u4(words, rows, k, 4))


@pytest.mark.parametrize("scale", [1.0, 0.5, 127.0 / 6.0, 100.0, 1e-3])
def test_pack_f16_all_finite_bit_patterns(abq, oracle, scale):
    x = np.arange(65536, dtype=np.uint16).view(np.float16)
    x = np.where(np.isfinite(x), x, np.float16(0)).astype(np.float16).reshape(512, 128)
    s = torch.tensor([scale], dtype=torch.float32, device="cuda")
    for bits in (8, 17):
        got = abq.pack_f16(torch.from_numpy(x).cuda(), s, bits).cpu().numpy().view(np.uint32)
        want = oracle.pack_f16(x, scale, bits)
        with np.errstate(over="ignore"):
            finite = np.isfinite((x * np.float16(scale)).astype(np.float16))  # inf -> int is device defined
        mask = np.packbits(finite.reshape(512, 4, 32), axis=2, bitorder="big").view(">u4").astype(np.uint32).reshape(512, 4)
        assert np.array_equal(got & mask, want & mask)


@pytest.mark.parametrize("rows,k", [(1, 128), (5, 4096), (16, 11008), (300, 512), (1024, 4096)])
def test_pack_f16_tiled_equals_the_relayout_of_the_planes(abq, rows, k):
    """abq_pack_f16_tiled writes in one pass what abq_relayout_planes makes of abq_pack_f16's planes."""
    g = torch.Generator(device="cuda").manual_seed(rows + k)
    x = (torch.randn((rows, k), generator=g, device="cuda") * 3).to(torch.float16)
    s = torch.tensor([127.0 / 6.0], dtype=torch.float32, device="cuda")
    for bits in range(1, 9):
        want = abq.relayout_planes(abq.pack_f16(x, s, bits))
        got = abq.pack_f16(x, s, bits, tiled=True)
        torch.cuda.synchronize()
        assert torch.equal(got.view(-1), want.view(-1)), bits


@pytest.mark.parametrize("rows,k", [(1, 128), (5, 4096), (300, 512), (1024, 4096)])
def test_pack_f16_fp6_equals_the_fp6_relayout_of_the_planes(abq, rows, k):
    """abq_pack_f16_fp6 writes in one pass what abq_relayout_planes_fp6 makes of abq_pack_f16's planes, values that
    overflow the code width included (the reference packs the low bits and does not clamp)."""
    g = torch.Generator(device="cuda").manual_seed(rows + k + 1)
    x = (torch.randn((rows, k), generator=g, device="cuda") * 3).to(torch.float16)
    s = torch.tensor([2.5], dtype=torch.float32, device="cuda")
    for bits, signed in [(4, True), (5, True), (2, True), (3, True), (4, False), (2, False), (1, False)]:
        want = abq.relayout_planes_fp6(abq.pack_f16(x, s, bits), signed)
        got = abq.pack_f16_fp6(x, s, bits, signed)
        torch.cuda.synchronize()
        assert torch.equal(got, want), (bits, signed)
    with pytest.raises(abq.AbqError):
        abq.pack_f16_fp6(x, s, 6, True)


@pytest.mark.parametrize("p", [2, 4, 8])
def test_decode_quantises_fp16_activations_itself(abq, oracle, p):
    """abq_gemm_set_f16_activations: the decode kernel on prepared weights reads fp16 activations and quantises them
    with the static scale inside the kernel; bit for bit abq_pack_f16 followed by the GEMM, on every shape class
    (several passes over long rows, row blocks, ragged N, every instance the default picks)."""
    rng = np.random.default_rng(70 + p)
    scale = torch.tensor([127.0 / 6.0], dtype=torch.float32, device="cuda")
    for (M, N, K) in [(1, 4096, 4096), (4, 11008, 4096), (8, 4096, 11008), (16, 200, 384), (3, 16, 128), (16, 1040, 11008),
                      (2, 4096, 11008), (13, 4100, 2176)]:
        x = (torch.randn((M, K), device="cuda") * 3).to(torch.float16)
        x[0, :4] = torch.tensor([0.0, -0.0, 6.0, -6.0], dtype=torch.float16)
        w = rand_vals(rng, N, K, p, True)
        wt = abq.relayout_planes(planes_dev(oracle.pack_i32(w, p)))
        xt = abq.pack_f16(x, scale, 8, tiled=True)
        for kw in (dict(), dict(out_kind=abq.OUT_F16_TENSOR_F32SCALE, c_scale=torch.tensor([0.0123], dtype=torch.float32, device="cuda"))):
            want = abq.Gemm(xt, wt, True, x_tiled=True, w_tiled=True, **kw)
            assert want.strategy == "decode_tiled"
            want_out = want.run().clone()
            g = abq.Gemm(xt, wt, True, x_tiled=True, w_tiled=True, **kw)
            g.set_f16_activations(x, scale)
            got = g.run()
            torch.cuda.synchronize()
            assert torch.equal(got, want_out), (M, N, K, p, kw.keys())
    # states the kernel does not serve are refused and stay usable
    x = (torch.randn((64, 256), device="cuda")).to(torch.float16)
    xt = abq.pack_f16(x, scale, 8, tiled=True)
    wt = abq.relayout_planes(planes_dev(oracle.pack_i32(rand_vals(rng, 32, 256, p, True), p)))
    g = abq.Gemm(xt, wt, True, x_tiled=True, w_tiled=True)  # 64 rows: the prefill kernel
    with pytest.raises(abq.AbqError) as e:
        g.set_f16_activations(x, scale)
    assert e.value.status == abq.ABQ_ERR_UNSUPPORTED
    g.run()


def field_packed(patterns, bits):
    """The K-tiled, field-packed layout written out from its definition: patterns [rows, K] are the
    elements' bit patterns (low `bits` bits).  A row's K tile of 128 elements is one record of
    bits*4 words.  Inside a 32-element word-set, "expanded" dword s, byte c is element
    31 - (8c + s).  8 bits: the expanded dwords themselves.  Otherwise one field per set bit f of
    `bits` (4, then 2, then 1), covering value bits [bits & (f-1), +f), starting at word
    4 * (bits & ~(2f-1)) of the record with f words per word-set: word j, byte c, bits
    [f*s, f*s+f) = field of the element at expanded dword (8/f)*j + s, byte c."""
    rows, K = patterns.shape
    kt = K // 128
    v = patterns.astype(np.uint32).reshape(rows, kt, 4, 32)
    s_idx, c_idx = np.meshgrid(np.arange(8), np.arange(4), indexing="ij")
    E = v[..., 31 - (8 * c_idx + s_idx)]  # [rows, kt, ws, s, c]
    rec = np.zeros((kt, rows, bits * 4), dtype=np.uint32)
    shifts8 = (8 * np.arange(4)).astype(np.uint32)
    if bits == 8:
        words = (E << shifts8).sum(axis=-1, dtype=np.uint32)  # [rows, kt, ws, s]
        rec[:] = words.reshape(rows, kt, 32).transpose(1, 0, 2)
        return rec
    for f in (4, 2, 1):
        if not bits & f:
            continue
        base, off, per = bits & (f - 1), 4 * (bits & ~(2 * f - 1)), 8 // f
        fv = (E >> np.uint32(base)) & np.uint32((1 << f) - 1)
        for ws in range(4):
            for j in range(f):
                word = np.zeros((rows, kt), dtype=np.uint32)
                for s in range(per):
                    word |= (fv[:, :, ws, per * j + s, :] << (shifts8 + np.uint32(f * s))).sum(axis=-1, dtype=np.uint32)
                rec[:, :, off + f * ws + j] = word.T
    return rec


def test_relayout_planes_matches_closed_form(abq, oracle):
    rng = np.random.default_rng(12)
    for bits, rows, k in [(2, 1, 128), (8, 37, 1152), (4, 300, 4096), (3, 64, 13824), (1, 5, 256), (5, 33, 384),
                          (6, 130, 512), (7, 9, 640)]:
        planes = rng.integers(0, 1 << 32, size=(bits, rows, k // 32), dtype=np.uint64).astype(np.uint32)
        got = abq.relayout_planes(planes_dev(planes)).cpu().numpy().view(np.uint32)
        want = field_packed(oracle.unpack(planes, False), bits)
        assert np.array_equal(got.reshape(want.shape), want), (bits, rows, k)


def test_row_sums_of_plane_operands(abq, oracle):
    rng = np.random.default_rng(14)
    for bits, rows, k in [(8, 1, 128), (8, 37, 1152), (2, 300, 4096), (4, 5, 13824), (3, 66, 384), (8, 2048, 4096)]:
        v = rng.integers(0, 1 << bits, size=(rows, k), dtype=np.int32)
        if rows > 1:
            v[1] = (1 << bits) - 1  # a row of maximal codes
        got = abq.row_sums(planes_dev(oracle.pack_i32(v, bits))).cpu().numpy()
        assert np.array_equal(got, v.sum(axis=1)), (bits, rows, k)


def test_tiled_kernels_with_prepared_operands(abq, oracle):
    """K-tiled kernels fed tiled activations and/or tiled weights directly, ragged shapes."""
    rng = np.random.default_rng(13)
    for q, p, signed, M, N, K in [(8, 2, True, 300, 200, 640), (4, 4, False, 70, 513, 1152), (8, 8, False, 257, 129, 384),
                                  (8, 4, True, 130, 200, 768), (8, 8, True, 70, 129, 128), (8, 2, False, 300, 290, 640),
                                  (8, 4, False, 130, 200, 768), (8, 8, False, 300, 513, 1152)]:
        x, w = rand_vals(rng, M, K, q, signed), rand_vals(rng, N, K, p, signed)
        xd, wd = planes_dev(oracle.pack_i32(x, q)), planes_dev(oracle.pack_i32(w, p))
        xt, wt = abq.relayout_planes(xd), abq.relayout_planes(wd)
        want = oracle.np_gemm(x, w)
        for cfg in [c for c in abq.native_configs(q, p, signed) if c.nstage == 4]:
            got = abq.gemm(xt, wt, signed, cfg=cfg, x_tiled=True, w_tiled=True).cpu().numpy()
            assert np.array_equal(got, want), abq.format_kernel_name(cfg)
            ws = torch.empty(xd.numel() * 4, dtype=torch.uint8, device="cuda")
            got = abq.gemm(xd, wt, signed, cfg=cfg, w_tiled=True, workspace=ws).cpu().numpy()
            assert np.array_equal(got, want), abq.format_kernel_name(cfg)
            if not signed and 8 in (q, p):
                # unsigned 8-bit operands with their row sums handed in: the staged kernel where it has the tile
                # (the other tiles keep the kernel that gathers the sums itself, whatever is handed in)
                g = abq.Gemm(xt, wt, signed, cfg=cfg, x_tiled=True, w_tiled=True, x_row_sums=abq.row_sums(xd), w_row_sums=abq.row_sums(wd))
                staged_tile = cfg.warp_k == 128 and cfg.block_k == 128 and (cfg.block_m, cfg.block_n, cfg.warp_m, cfg.warp_n) in (
                    (128, 128, 64, 64), (128, 64, 64, 32), (64, 64, 32, 32), (256, 128, 64, 64)) + (
                    ((256, 256, 64, 128),) if (q, p) != (8, 8) else ())
                assert g.row_sums_ready == staged_tile, abq.format_kernel_name(cfg)
                assert np.array_equal(g.run().cpu().numpy(), want), abq.format_kernel_name(cfg)
                # activations as planes with a workspace that holds their sums too, weight sums handed in
                ws2 = torch.empty(xd.numel() * 4 + 4 * M + 512, dtype=torch.uint8, device="cuda")
                g = abq.Gemm(xd, wt, signed, cfg=cfg, w_tiled=True, workspace=ws2, w_row_sums=abq.row_sums(wd))
                assert g.row_sums_ready == staged_tile and g.workspace_bytes <= ws2.numel()
                assert np.array_equal(g.run().cpu().numpy(), want), abq.format_kernel_name(cfg)
                if (q, p) == (8, 8):
                    # biased records (code - 128 written at preparation): the signed pair's staged kernel runs them, the
                    # activations arriving biased too or as planes (converted that way into the workspace); a tile that
                    # kernel is not built for is refused
                    xb_, wb_ = abq.relayout_planes_biased(xd), abq.relayout_planes_biased(wd)
                    assert torch.equal(wb_, abq.relayout_planes(wd) ^ torch.tensor(-2139062144, dtype=torch.int32, device="cuda"))
                    g1 = abq.Gemm(xb_, wb_, signed, cfg=cfg, x_tiled=True, w_tiled=True, x_row_sums=abq.row_sums(xd),
                                  w_row_sums=abq.row_sums(wd), biased=(True, True))
                    g2 = abq.Gemm(xd, wb_, signed, cfg=cfg, w_tiled=True, workspace=ws2, w_row_sums=abq.row_sums(wd), biased=(False, True))
                    for gb in (g1, g2):
                        if staged_tile:
                            gb.out.fill_(-7)
                            assert np.array_equal(gb.run().cpu().numpy(), want), abq.format_kernel_name(cfg)
                        else:
                            with pytest.raises(abq.AbqError):
                                gb.run()
                    with pytest.raises(abq.AbqError):  # plain activations against biased weights
                        abq.Gemm(xt, wb_, signed, cfg=cfg, x_tiled=True, w_tiled=True, x_row_sums=abq.row_sums(xd),
                                 w_row_sums=abq.row_sums(wd), biased=(False, True)).run()
        # a state with an explicit non-tiled tile refuses tiled operands; exec without workspace is refused
        cfg = [c for c in abq.native_configs(q, p, signed) if c.nstage == 2][0]
        with pytest.raises(abq.AbqError):
            abq.Gemm(xd, wt, signed, cfg=cfg, w_tiled=True)
        cfg = [c for c in abq.native_configs(q, p, signed) if c.nstage == 4][0]
        with pytest.raises(abq.AbqError):
            abq.Gemm(xd, wd, signed, cfg=cfg).run()


# ------------------------------------------------------------------ FP6 matrix-core route

def fp6_records(values):
    """FP6 records written out from their definition: values [rows, K] -> uint32 [K/128, rows, 24].
    An element's code is (sign << 5) | |value|.  A word-set (32 consecutive K elements) is a string
    of 192 bits, position p (bits [6p, 6p+6)) holding element 31 - 8*(p % 4) - p // 4; a record has
    word-set ws at words [12*(ws & 1) + 6*(ws >> 1), +6)."""
    rows, K = values.shape
    kt = K // 128
    v = values.astype(np.int64).reshape(rows, kt, 4, 32)
    code = (np.where(v < 0, 32, 0) | np.abs(v)).astype(np.uint64)
    pos = np.arange(32)
    ordered = code[..., 31 - 8 * (pos % 4) - pos // 4]  # [rows, kt, ws, p]
    rec = np.zeros((kt, rows, 24), dtype=np.uint32)
    for ws in range(4):
        words = np.zeros((rows, kt, 6), dtype=np.uint64)
        for pp in range(32):
            bit = 6 * pp
            w0, sh = bit // 32, bit % 32
            words[..., w0] |= (ordered[:, :, ws, pp] << np.uint64(sh)) & np.uint64(0xFFFFFFFF)
            if sh > 26:
                words[..., w0 + 1] |= ordered[:, :, ws, pp] >> np.uint64(32 - sh)
        off = 12 * (ws & 1) + 6 * (ws >> 1)
        rec[:, :, off:off + 6] = words.astype(np.uint32).transpose(1, 0, 2)
    return rec


FP6_OPERANDS = [(1, False), (2, False), (3, False), (4, False), (2, True), (3, True), (4, True), (5, True)]


def test_relayout_planes_fp6_matches_closed_form(abq, oracle):
    rng = np.random.default_rng(61)
    for bits, signed in FP6_OPERANDS:
        for rows, k in [(1, 128), (5, 256), (40, 1152), (67, 4096)]:
            vals = rand_vals(rng, rows, k, bits, signed)
            vals[0, :4] = [oracle.value_range(bits, signed)[0], oracle.value_range(bits, signed)[1], 0, vals[0, 3]]
            got = abq.relayout_planes_fp6(planes_dev(oracle.pack_i32(vals, bits)), signed).cpu().numpy().view(np.uint32)
            assert np.array_equal(got, fp6_records(vals)), (bits, signed, rows, k)
    with pytest.raises(abq.AbqError):  # 5 bits unsigned / 6 bits signed have no exact FP6 form
        abq.relayout_planes_fp6(planes_dev(oracle.pack_i32(rand_vals(rng, 4, 128, 5, False), 5)), False)
    with pytest.raises(abq.AbqError):
        abq.relayout_planes_fp6(planes_dev(oracle.pack_i32(rand_vals(rng, 4, 128, 6, True), 6)), True)


def test_fp6_gemm_every_eligible_pair_and_tile(abq, oracle):
    """FP6 route against the oracle: every eligible bit pair (also pairs without a popcount / int8
    specialisation), every tile, ragged shapes, prepared and per-call converted operands."""
    rng = np.random.default_rng(62)
    shapes = [(33, 70, 128), (100, 200, 384), (300, 129, 640), (64, 257, 1152)]
    cfg44 = [c for c in abq.native_configs(4, 4, True) if c.nstage == 5]
    assert len(cfg44) >= 4 and all(c.mma_k == 64 for c in cfg44)
    for signed in (True, False):
        widths = [b for b, s in FP6_OPERANDS if s == signed]
        for q in widths:
            for p in widths:
                M, N, K = shapes[(q + p) % len(shapes)]
                assert abq.fp6_eligible(q, p, signed, K)
                x, w = rand_vals(rng, M, K, q, signed), rand_vals(rng, N, K, p, signed)
                xd, wd = planes_dev(oracle.pack_i32(x, q)), planes_dev(oracle.pack_i32(w, p))
                xf, wf = abq.relayout_planes_fp6(xd, signed), abq.relayout_planes_fp6(wd, signed)
                want = oracle.np_gemm(x, w)
                for c in cfg44:
                    cfg = abq.TileConfig(q, p, int(signed), c.block_m, c.block_n, c.block_k, c.warp_m, c.warp_n,
                                         c.warp_k, c.mma_m, c.mma_n, c.mma_k, c.nstage)
                    out = torch.full((M, N), -777, dtype=torch.int32, device="cuda")
                    got = abq.gemm(xf, wf, signed, cfg=cfg, x_fp6=q, w_fp6=p, out=out).cpu().numpy()
                    assert np.array_equal(got, want), (abq.format_kernel_name(cfg), M, N, K)
                # activations converted inside the call, weights prepared; the library picks the tile
                g = abq.Gemm(xd, wf, signed, w_fp6=p)
                assert g.strategy == "fp6" and g.workspace_bytes == (K // 128) * M * 96
                ws = torch.empty(g.workspace_bytes, dtype=torch.uint8, device="cuda")
                got = abq.gemm(xd, wf, signed, w_fp6=p, workspace=ws).cpu().numpy()
                assert np.array_equal(got, want), (q, p, signed)
                with pytest.raises(abq.AbqError):  # no workspace for the activations
                    g.run()


def test_fp6_gemm_range_ends_and_limits(abq, oracle):
    """Largest magnitudes over the longest K the route accepts: the fp32 accumulation stays exact."""
    for q, p, signed, K in [(4, 4, False, 65536), (5, 5, True, 65536 - 128), (4, 4, True, 13824), (5, 2, True, 13824)]:
        assert abq.fp6_eligible(q, p, signed, K)
        xlo, xhi = oracle.value_range(q, signed)
        wlo, whi = oracle.value_range(p, signed)
        M, N = 40, 72
        x = np.full((M, K), xlo if signed else xhi, dtype=np.int32)
        w = np.full((N, K), wlo if signed else whi, dtype=np.int32)
        x[1::2] = xhi
        w[1::3] = whi
        x[5, ::7] = 0
        xd, wd = planes_dev(oracle.pack_i32(x, q)), planes_dev(oracle.pack_i32(w, p))
        got = abq.gemm(abq.relayout_planes_fp6(xd, signed), abq.relayout_planes_fp6(wd, signed), signed,
                       x_fp6=q, w_fp6=p).cpu().numpy()
        assert np.array_equal(got, oracle.np_gemm(x, w)), (q, p, signed, K)
    rng = np.random.default_rng(63)
    # beyond the exactness bound, wider operands, group scales and mixed layouts are refused
    assert not abq.fp6_eligible(4, 4, False, 131072 - 128) and not abq.fp6_eligible(5, 5, True, 65536)
    assert not abq.fp6_eligible(5, 4, False, 128) and not abq.fp6_eligible(6, 2, True, 128)
    x, w = rand_vals(rng, 32, 256, 8, True), rand_vals(rng, 64, 256, 2, True)
    xd, wd = planes_dev(oracle.pack_i32(x, 8)), planes_dev(oracle.pack_i32(w, 2))
    wf = abq.relayout_planes_fp6(wd, True)
    with pytest.raises(abq.AbqError):
        abq.Gemm(xd, wf, True, w_fp6=2)  # 8-bit activations
    x4 = rand_vals(rng, 32, 256, 4, True)
    x4d = planes_dev(oracle.pack_i32(x4, 4))
    with pytest.raises(abq.AbqError):
        abq.Gemm(abq.relayout_planes(x4d), wf, True, x_tiled=True, w_fp6=2)  # tiled and FP6 together
    sc = torch.ones(64 * 2, dtype=torch.float32, device="cuda")
    with pytest.raises(abq.AbqError):  # group scales on the FP6 route: groups of 128 only
        abq.Gemm(x4d, wf, True, w_fp6=2, out_kind=abq.OUT_F16_SCALED, x_scale=sc, w_scale=sc, group_size=64)


def test_fp6_fp16_epilogues(abq, oracle):
    rng = np.random.default_rng(64)
    M, N, K, q, p = 130, 200, 512, 4, 4
    x, w = rand_vals(rng, M, K, q, True), rand_vals(rng, N, K, p, True)
    xf = abq.relayout_planes_fp6(planes_dev(oracle.pack_i32(x, q)), True)
    wf = abq.relayout_planes_fp6(planes_dev(oracle.pack_i32(w, p)), True)
    acc = oracle.np_gemm(x, w)
    xs = torch.rand(M, device="cuda") * 0.01 + 0.001
    ws = torch.rand(N, device="cuda") * 0.01 + 0.001
    got = abq.gemm(xf, wf, True, x_fp6=q, w_fp6=p, out_kind=abq.OUT_F16_SCALED, x_scale=xs, w_scale=ws).float().cpu().numpy()
    want = acc.astype(np.float64) * xs.cpu().numpy().astype(np.float64)[:, None] * ws.cpu().numpy().astype(np.float64)[None, :]
    assert np.all(np.abs(got - want) <= 1e-2 * np.abs(want) + 1e-6)  # tolerance of the fp16 dequantised output: 1e-2 relative
    c = torch.tensor([0.03125], dtype=torch.float16, device="cuda")
    got = abq.gemm(xf, wf, True, x_fp6=q, w_fp6=p, out_kind=abq.OUT_F16_TENSOR, c_scale=c).cpu().numpy()
    want16 = (acc.astype(np.float32).astype(np.float16) * np.float16(0.03125)).astype(np.float16)
    assert np.array_equal(got.view(np.uint16), want16.view(np.uint16))


@pytest.mark.parametrize("q,p,fp6,signed", [(4, 4, True, True), (8, 2, False, True), (4, 4, False, True), (8, 8, False, True),
                                             (2, 2, False, True), (6, 6, False, True), (8, 8, False, False), (4, 4, True, False)])
def test_scaled_fp16_epilogue_every_staged_tile(abq, oracle, q, p, fp6, signed):
    """Per-token x per-channel scales with fp16 output on every tile of the LDS-staged kernels: once with
    an output width the whole-line store takes (multiple of 8) and once with one it does not, ragged M."""
    rng = np.random.default_rng(900 + 10 * q + p + fp6 + 2 * signed)
    tiles = [c for c in abq.native_configs(q, p, signed) if c.nstage == (5 if fp6 else 4) and c.warp_k == 128]
    assert tiles
    for (M, N, K) in [(130, 328, 384), (70, 203, 256)]:
        x, w = rand_vals(rng, M, K, q, signed), rand_vals(rng, N, K, p, signed)
        xd, wd = planes_dev(oracle.pack_i32(x, q)), planes_dev(oracle.pack_i32(w, p))
        if fp6:
            xo, wo, kw = abq.relayout_planes_fp6(xd, signed), abq.relayout_planes_fp6(wd, signed), dict(x_fp6=q, w_fp6=p)
        else:
            xo, wo, kw = abq.relayout_planes(xd), abq.relayout_planes(wd), dict(x_tiled=True, w_tiled=True)
        xs = torch.rand(M, device="cuda") * 0.01 + 0.001
        ws = torch.rand(N, device="cuda") * 0.01 + 0.001
        want = (oracle.np_gemm(x, w).astype(np.float64) * xs.cpu().numpy().astype(np.float64)[:, None]
                * ws.cpu().numpy().astype(np.float64)[None, :])
        c16 = torch.tensor([0.03125], dtype=torch.float16, device="cuda")
        with np.errstate(over="ignore"):  # beyond fp16's range both sides give infinity
            want16 = (oracle.np_gemm(x, w).astype(np.float32).astype(np.float16) * np.float16(0.03125)).astype(np.float16)
        for cfg in tiles:
            g = abq.Gemm(xo, wo, signed, cfg=cfg, out_kind=abq.OUT_F16_SCALED, x_scale=xs, w_scale=ws, **kw)
            got = g.run().float().cpu().numpy()
            # tolerance of the fp16 dequantised output: 1e-2 relative
            assert np.all(np.abs(got - want) <= 1e-2 * np.abs(want) + 1e-6), (g.config_name, M, N, K)
            # one fp16 scale for the whole output: half(acc) * scale, bit for bit
            got16 = abq.Gemm(xo, wo, signed, cfg=cfg, out_kind=abq.OUT_F16_TENSOR, c_scale=c16, **kw).run().cpu().numpy()
            assert np.array_equal(got16.view(np.uint16), want16.view(np.uint16)), (g.config_name, M, N, K)


@pytest.mark.parametrize("q,p,fp6,signed", [(8, 2, False, True), (4, 4, True, True), (8, 8, False, True), (7, 7, False, False),
                                             (4, 4, False, False)])
def test_workgroup_numbering_covers_every_tile(abq, oracle, q, p, fp6, signed):
    """Every tile of the LDS-staged kernels on grids whose number of m blocks is not a multiple of the four
    the workgroup numbering groups them by (4 + 2, and 4 + 4 + 1), with n blocks that do not fill the eight
    bands (18 blocks in bands of 3): every output element written once, with the right value."""
    rng = np.random.default_rng(4100 + 10 * q + p + fp6)
    tiles = [c for c in abq.native_configs(q, p, signed) if c.nstage == (5 if fp6 else 4) and c.warp_k == 128]
    assert tiles
    K = 256
    for cfg in tiles:
        for m_blocks, n_blocks in ((6, 18), (9, 5)):
            M, N = (m_blocks - 1) * cfg.block_m + 9, (n_blocks - 1) * cfg.block_n + 40
            x, w = rand_vals(rng, M, K, q, signed), rand_vals(rng, N, K, p, signed)
            xd, wd = planes_dev(oracle.pack_i32(x, q)), planes_dev(oracle.pack_i32(w, p))
            if fp6:
                xo, wo, kw = abq.relayout_planes_fp6(xd, signed), abq.relayout_planes_fp6(wd, signed), dict(x_fp6=q, w_fp6=p)
            else:
                xo, wo, kw = abq.relayout_planes(xd), abq.relayout_planes(wd), dict(x_tiled=True, w_tiled=True)
            want = (x.astype(np.float64) @ w.astype(np.float64).T).astype(np.int32)  # exact: |sums| < 2^53
            out = torch.full((M, N), -12345, dtype=torch.int32, device="cuda")
            g = abq.Gemm(xo, wo, signed, cfg=cfg, out=out, **kw)
            got = g.run().cpu().numpy()
            assert np.array_equal(got, want), (g.config_name, M, N, K)


@pytest.mark.parametrize("signed", [True, False])
def test_config2_w4a4_prefill_full_size_fp6(abq, oracle, signed):
    """W4A4 at M in {512, 2048} on the LLaMA-7B shapes through the FP6 route: exact against the fp64
    closed form and the CPU oracle on sampled rows, and identical to the int8 tiled kernel."""
    rng = np.random.default_rng(2000 + int(signed))
    for (N, K) in [(4096, 4096), (11008, 4096), (4096, 11008)]:
        w = rand_vals(rng, N, K, 4, signed)
        wp = oracle.pack_i32(w, 4)
        wd = planes_dev(wp)
        wf6 = abq.relayout_planes_fp6(wd, signed)
        wfd = torch.from_numpy(w).cuda().double()
        for M in (512, 2048):
            x = rand_vals(rng, M, K, 4, signed)
            xp = oracle.pack_i32(x, 4)
            xd = planes_dev(xp)
            ws = torch.empty((K // 128) * M * 96, dtype=torch.uint8, device="cuda")
            g = abq.Gemm(xd, wf6, signed, w_fp6=4, workspace=ws)
            assert g.strategy == "fp6"
            got_d = g.run()
            ref = torch.from_numpy(x).cuda().double() @ wfd.T
            assert torch.equal(got_d.double(), ref), (signed, M, N, K)
            _sampled_oracle_check(oracle, xp, wp, signed, got_d.cpu().numpy(), rng, rows=2)
            del ref


# ------------------------------------------------------------------ GEMM: every native tile, every combination

SMALL_SHAPES = [(1, 64, 128), (3, 37, 384), (8, 130, 1152), (17, 64, 512), (33, 96, 256)]


@pytest.mark.parametrize("q,p", COMBOS)
@pytest.mark.parametrize("signed", [True, False])
def test_gemm_every_native_config_small_shapes(abq, oracle, q, p, signed):
    rng = np.random.default_rng(97 * q + 13 * p + int(signed))
    cfgs = abq.native_configs(q, p, signed)
    assert cfgs
    for (M, N, K) in SMALL_SHAPES:
        x, w = rand_vals(rng, M, K, q, signed), rand_vals(rng, N, K, p, signed)
        xp, wp = oracle.pack_i32(x, q), oracle.pack_i32(w, p)
        want = oracle.np_gemm(x, w)
        assert np.array_equal(oracle.gemm_popc(xp, wp, signed)[0], want)
        xd, wd = planes_dev(xp), planes_dev(wp)
        for cfg in cfgs:
            out = torch.full((M, N), -12345, dtype=torch.int32, device="cuda")
            got = run_cfg(abq, xd, wd, signed, cfg=cfg, out=out).cpu().numpy()
            assert np.array_equal(got, want), (abq.format_kernel_name(cfg), M, N, K)
        got = abq.gemm(xd, wd, signed).cpu().numpy()  # library's own choice
        assert np.array_equal(got, want)


def test_gemm_extreme_values_do_not_overflow(abq, oracle):
    """All operands at the range ends, K = 13824 (the longest K of the baseline configurations)."""
    K = 13824
    for q, p, signed in [(8, 8, False), (8, 8, True), (8, 2, True), (4, 4, False), (7, 7, False)]:
        xlo, xhi = oracle.value_range(q, signed)
        wlo, whi = oracle.value_range(p, signed)
        x = np.array([[xlo] * K, [xhi] * K, [xlo, xhi] * (K // 2)], dtype=np.int32)
        w = np.array([[wlo] * K, [whi] * K, [whi, wlo] * (K // 2), [0] * K], dtype=np.int32)
        xd, wd = planes_dev(oracle.pack_i32(x, q)), planes_dev(oracle.pack_i32(w, p))
        want = oracle.np_gemm(x, w)
        for cfg in abq.native_configs(q, p, signed):
            got = run_cfg(abq, xd, wd, signed, cfg=cfg).cpu().numpy()
            assert np.array_equal(got, want), (q, p, signed, abq.format_kernel_name(cfg))


def test_decode_kernel_k_chunking_and_many_tiles(abq, oracle):
    """Decode kernel corner cases: activations too large for one LDS chunk (M=16, long K), a
    partial last K step, more weight tiles than workgroups, and several 16-row blocks of M."""
    rng = np.random.default_rng(21)
    for q, p, signed, M, N, K in [(8, 2, True, 16, 100, 11008), (8, 8, False, 13, 70, 13824), (4, 4, False, 16, 333, 8320),
                                  (8, 2, True, 8, 16 * 256 * 3 + 5, 128), (8, 8, False, 40, 4200, 384)]:
        x, w = rand_vals(rng, M, K, q, signed), rand_vals(rng, N, K, p, signed)
        xd, wd = planes_dev(oracle.pack_i32(x, q)), planes_dev(oracle.pack_i32(w, p))
        want = oracle.np_gemm(x, w)
        for cfg in abq.native_configs(q, p, signed):
            if cfg.nstage != 3:
                continue
            got = abq.gemm(xd, wd, signed, cfg=cfg).cpu().numpy()
            assert np.array_equal(got, want), (abq.format_kernel_name(cfg), M, N, K)


DECODE_TILED_PAIRS = COMBOS  # all twelve pairs of the reference's library


@pytest.mark.parametrize("q,p", DECODE_TILED_PAIRS)
@pytest.mark.parametrize("signed", [True, False])
def test_decode_on_prepared_operands(abq, oracle, q, p, signed):
    """Decode-sized GEMM with both operands K-tiled: the library moves to the decode kernel of that layout by
    itself (no workspace, one launch); every tile tuple of that kernel on ragged shapes: partial tiles of N, an odd
    number of K tiles (half-filled last step), M past 16 (several row blocks), long K (rows per workgroup limited
    by the LDS), more steps than the waves hold in flight.  Widths made of several fields (3, 5, 6, 7 bits) come as
    padded records of the next single-field width; unsigned 8-bit codes bring their row sums."""
    qp, pp = abq.padded_bits(q), abq.padded_bits(p)
    padded = (qp, pp) != (q, p)
    rng = np.random.default_rng(500 + 10 * q + p + int(signed))
    shapes = [(1, 64, 128), (1, 4096, 4096), (3, 37, 384), (4, 200, 1408), (8, 130, 1152), (8, 64, 11008), (13, 72, 4096),
              (16, 100, 13824), (16, 48, 2048), (17, 64, 512), (40, 96, 640), (2, 300, 24576)]
    for (M, N, K) in shapes:
        x, w = rand_vals(rng, M, K, q, signed), rand_vals(rng, N, K, p, signed)
        if M > 1:
            x[1] = (1 << (q - 1)) - 1 if signed else (1 << q) - 1  # a row of the largest code ...
            w[0] = -(1 << (p - 1)) if signed else (1 << p) - 1      # ... against one of the code furthest from zero
        xd, wd = planes_dev(oracle.pack_i32(x, q)), planes_dev(oracle.pack_i32(w, p))
        xt, wt = abq.relayout_planes_padded(xd, signed), abq.relayout_planes_padded(wd, signed)
        assert xt.shape == (K // 128, M, qp, 4) and wt.shape == (K // 128, N, pp, 4)
        if not padded:  # for the widths of one field the padded records are the K-tiled records
            assert torch.equal(xt, abq.relayout_planes(xd)) and torch.equal(wt, abq.relayout_planes(wd))
        want = oracle.np_gemm(x, w)
        kw = dict(x_tiled=True, w_tiled=True)
        if padded:
            kw["value_bits"] = (q, p)
        needs_sums = not signed and 8 in (q, p)
        if needs_sums:
            # without the row sums a state of unsigned 8-bit codes stays on the prefill kernel, which takes them itself
            g = abq.Gemm(xt, wt, signed, **kw)
            assert g.strategy == "tiled"
            assert np.array_equal(g.run().cpu().numpy(), want), (g.config_name, M, N, K)
            kw.update(x_row_sums=abq.row_sums(xd), w_row_sums=abq.row_sums(wd))
        g = abq.Gemm(xt, wt, signed, **kw)
        assert (g.state.cfg.x_bits, g.state.cfg.w_bits) == (qp, pp)
        # up to 16 rows always; up to 128 rows where the library estimates the decode kernel ahead (several blocks of rows)
        assert g.strategy == "decode_tiled" if M <= 16 else g.strategy in ("decode_tiled", "tiled"), (g.strategy, M, N, K)
        assert g.workspace_bytes == 0
        assert np.array_equal(g.run().cpu().numpy(), want), (g.config_name, M, N, K)
        ran = 0
        for cfg in abq.native_configs(qp, pp, signed):
            if cfg.nstage != 6:
                continue
            out = torch.full((M, N), -12345, dtype=torch.int32, device="cuda")
            got = abq.Gemm(xt, wt, signed, cfg=cfg, out=out, **kw).run().cpu().numpy()
            assert np.array_equal(got, want), (abq.format_kernel_name(cfg), M, N, K)
            ran += 1
        assert ran == 7
        if needs_sums:  # a tile of this kernel named by the caller, but no sums: refused before any launch
            cfg = [c for c in abq.native_configs(qp, pp, signed) if c.nstage == 6][0]
            with pytest.raises(abq.AbqError) as e:
                abq.Gemm(xt, wt, signed, cfg=cfg, x_tiled=True, w_tiled=True, **({"value_bits": (q, p)} if padded else {})).run()
            assert e.value.status == abq.ABQ_ERR_INVALID_ARG


@pytest.mark.parametrize("q,p", [(3, 3), (5, 5), (6, 6), (7, 7), (8, 3), (6, 2)])
@pytest.mark.parametrize("signed", [True, False])
def test_prefill_on_padded_weight_records(abq, oracle, q, p, signed):
    """Weights of 3, 5, 6 or 7 bits held as padded records serve the prefill as well: the state is initialised with
    the padded pair and told the codes' widths, the activations arrive as planes of their own width and exec extends
    them to the records' width in the workspace (sign extension for signed codes; the row sums of unsigned codes in
    8-bit records are those of the codes)."""
    qp, pp = abq.padded_bits(q), abq.padded_bits(p)
    rng = np.random.default_rng(900 + 10 * q + p + int(signed))
    for (M, N, K) in [(17, 64, 512), (40, 200, 1408), (128, 256, 4096), (300, 130, 1152)]:
        x, w = rand_vals(rng, M, K, q, signed), rand_vals(rng, N, K, p, signed)
        x[1] = (1 << (q - 1)) - 1 if signed else (1 << q) - 1
        x[2] = -(1 << (q - 1)) if signed else 0
        w[0] = -(1 << (p - 1)) if signed else (1 << p) - 1
        xd, wd = planes_dev(oracle.pack_i32(x, q)), planes_dev(oracle.pack_i32(w, p))
        wt = abq.relayout_planes_padded(wd, signed)
        want = oracle.np_gemm(x, w)
        ws = torch.empty(M * K * qp // 8 + 4 * (M + N) + 1024, dtype=torch.uint8, device="cuda")
        g = abq.Gemm(xd, wt, signed, w_tiled=True, value_bits=(q, p), x_planes_of=qp, workspace=ws)
        assert (g.state.cfg.x_bits, g.state.cfg.w_bits) == (qp, pp) and g.strategy in ("tiled", "decode_tiled")
        assert g.workspace_bytes <= ws.numel()
        assert np.array_equal(g.run().cpu().numpy(), want), (g.config_name, M, N, K)
        assert np.array_equal(g.run().cpu().numpy(), want)
        if not signed and 8 in (qp, pp):  # the same with the weights' sums from their preparation
            g = abq.Gemm(xd, wt, signed, w_tiled=True, value_bits=(q, p), x_planes_of=qp, workspace=ws, w_row_sums=abq.row_sums(wd))
            assert np.array_equal(g.run().cpu().numpy(), want), (g.config_name, M, N, K)


def test_prefill_pads_activations_of_several_fields_by_itself(abq, oracle):
    """Signed W2A6 above 16 rows, activations as planes, weights as their own K-tiled records: the library runs the pair
    as W2A8 (exec extends the activation codes while it converts them), says so in the state, and sizes the workspace
    for the wider records.  Unsigned pairs and decode-sized calls keep the pair's own kernels."""
    rng = np.random.default_rng(77)
    for (M, N, K) in [(17, 64, 512), (128, 200, 1408), (300, 130, 1152)]:
        x, w = rand_vals(rng, M, K, 6, True), rand_vals(rng, N, K, 2, True)
        x[1], x[2], w[0] = 31, -32, -2
        xd, wd = planes_dev(oracle.pack_i32(x, 6)), planes_dev(oracle.pack_i32(w, 2))
        g = abq.Gemm(xd, abq.relayout_planes(wd), True, w_tiled=True)
        assert (g.state.cfg.x_bits, g.state.cfg.w_bits, g.strategy) == (8, 2, "tiled")
        assert g.workspace_bytes >= M * K
        ws = torch.empty(g.workspace_bytes, dtype=torch.uint8, device="cuda")
        g = abq.Gemm(xd, abq.relayout_planes(wd), True, w_tiled=True, workspace=ws)
        assert np.array_equal(g.run().cpu().numpy(), oracle.np_gemm(x, w)), (g.config_name, M, N, K)
    x, w = rand_vals(rng, 40, 512, 6, False), rand_vals(rng, 64, 512, 2, False)
    g = abq.Gemm(planes_dev(oracle.pack_i32(x, 6)), abq.relayout_planes(planes_dev(oracle.pack_i32(w, 2))), False, w_tiled=True)
    assert g.state.cfg.x_bits == 6
    x = rand_vals(rng, 8, 512, 6, True)
    g = abq.Gemm(planes_dev(oracle.pack_i32(x, 6)), abq.relayout_planes(planes_dev(oracle.pack_i32(w, 2))), True, w_tiled=True)
    assert g.state.cfg.x_bits == 6


@pytest.mark.parametrize("q,p,signed", [(8, 2, True), (4, 4, True), (2, 2, True), (8, 8, True), (4, 4, False), (8, 4, True)])
def test_small_batches_from_planes_on_the_prepared_decode_kernel(abq, oracle, q, p, signed):
    """Weights prepared, activations handed over as planes, 17 to 128 rows: once the state has a workspace it runs the
    decode kernel of prepared operands wherever it would on prepared activations (exec converts the planes first, over
    several blocks of rows); without a workspace it stays on the prefill kernel.  Bit exact either way."""
    rng = np.random.default_rng(1700 + 10 * q + p + int(signed))
    took_decode = 0
    for (M, N, K) in [(17, 64, 512), (40, 200, 1408), (64, 4096, 1024), (100, 130, 4096), (128, 264, 1152), (33, 96, 11008)]:
        x, w = rand_vals(rng, M, K, q, signed), rand_vals(rng, N, K, p, signed)
        xd, wt = planes_dev(oracle.pack_i32(x, q)), abq.relayout_planes(planes_dev(oracle.pack_i32(w, p)))
        want = oracle.np_gemm(x, w)
        on_records = abq.Gemm(abq.relayout_planes(xd), wt, signed, x_tiled=True, w_tiled=True)
        g = abq.Gemm(xd, wt, signed, w_tiled=True)
        assert g.strategy == "tiled"
        ws = torch.empty(max(g.workspace_bytes, M * K * q // 8 + 4096), dtype=torch.uint8, device="cuda")
        g = abq.Gemm(xd, wt, signed, w_tiled=True, workspace=ws)
        assert g.strategy == on_records.strategy, (M, N, K, g.strategy, on_records.strategy)
        assert g.workspace_bytes <= ws.numel()
        took_decode += g.strategy == "decode_tiled"
        assert np.array_equal(g.run().cpu().numpy(), want), (g.config_name, M, N, K)
        assert np.array_equal(on_records.run().cpu().numpy(), want), (on_records.config_name, M, N, K)
    assert took_decode >= 2


FIELD_PAIRS = [(3, 3), (5, 5), (6, 6), (7, 7), (8, 3), (6, 2)]  # a width of several fields on either side


@pytest.mark.parametrize("q,p", FIELD_PAIRS)
@pytest.mark.parametrize("signed", [True, False])
def test_decode_on_prepared_operands_of_several_fields(abq, oracle, q, p, signed):
    """Weights of 3, 5, 6 or 7 bits on the decode kernel as the records the prefill kernels read (no padded copy), the
    state initialised with the pair's own widths; activations of such widths as padded records, declared so, or as
    planes, which exec converts.  Every tile tuple of the kernel on ragged shapes (partial tiles of N, numbers of K
    tiles that leave the last step of the 2-bit and of the 1-bit field partly empty, long K), the rows of the largest
    codes against the code furthest from zero, unsigned 8-bit activations with the weights' row sums."""
    qp = abq.padded_bits(q)
    rng = np.random.default_rng(900 + 10 * q + p + int(signed))
    shapes = [(1, 64, 128), (1, 4096, 4096), (3, 37, 384), (4, 200, 1408), (8, 130, 1152), (8, 64, 11008), (13, 72, 4096),
              (16, 100, 13824), (16, 48, 2048), (2, 300, 24576), (5, 16, 640), (7, 1000, 896), (17, 64, 512), (40, 96, 640)]
    for (M, N, K) in shapes:
        x, w = rand_vals(rng, M, K, q, signed), rand_vals(rng, N, K, p, signed)
        if M > 1:
            x[1] = (1 << (q - 1)) - 1 if signed else (1 << q) - 1
            w[0] = -(1 << (p - 1)) if signed else (1 << p) - 1
        xd, wd = planes_dev(oracle.pack_i32(x, q)), planes_dev(oracle.pack_i32(w, p))
        wt = abq.relayout_planes(wd)                      # the weights' own records
        xt = abq.relayout_planes_padded(xd, signed)       # activations: records of one field
        assert wt.shape == (K // 128, N, p, 4) and xt.shape == (K // 128, M, qp, 4)
        want = oracle.np_gemm(x, w)
        kw = dict(x_tiled=True, w_tiled=True)
        if qp != q:
            kw["x_padded_from"] = q
        needs_sums = not signed and q == 8
        if needs_sums:
            g = abq.Gemm(xt, wt, signed, **kw)  # no sums: the prefill kernel, which takes them itself
            assert g.strategy == "tiled"
            assert np.array_equal(g.run().cpu().numpy(), want), (g.config_name, M, N, K)
            kw["w_row_sums"] = abq.row_sums(wd)
        if M <= 16 or qp == q:
            g = abq.Gemm(xt, wt, signed, **kw)
            assert (g.state.cfg.x_bits, g.state.cfg.w_bits) == (q, p)
            # (several blocks of rows: the decode kernel only where the library estimates it ahead, weights of one field)
            assert (g.strategy == "decode_tiled" if M <= 16 else g.strategy in ("decode_tiled", "tiled")) and g.workspace_bytes == 0, (g.strategy, M, N, K)
            assert np.array_equal(g.run().cpu().numpy(), want), (g.config_name, M, N, K)
        else:  # more than 16 rows: the library picks the prefill kernel, which does not read padded activation records
            with pytest.raises(abq.AbqError):
                abq.Gemm(xt, wt, signed, **kw)
        ran = 0
        for cfg in abq.native_configs(q, p, signed):
            if cfg.nstage != 6:
                continue
            out = torch.full((M, N), -12345, dtype=torch.int32, device="cuda")
            got = abq.Gemm(xt, wt, signed, cfg=cfg, out=out, **kw).run().cpu().numpy()
            assert np.array_equal(got, want), (abq.format_kernel_name(cfg), M, N, K)
            ran += 1
        assert ran == (7 if p == 2 else 3)
        # activations handed over as planes: exec writes the padded records into the workspace
        cfg = [c for c in abq.native_configs(q, p, signed) if c.nstage == 6][0]
        sums = {"w_row_sums": kw["w_row_sums"]} if needs_sums else {}
        g = abq.Gemm(xd, wt, signed, cfg=cfg, w_tiled=True, **sums)
        assert g.workspace_bytes == xt.numel() * 4
        g = abq.Gemm(xd, wt, signed, cfg=cfg, w_tiled=True, workspace=torch.empty(g.workspace_bytes, dtype=torch.uint8, device="cuda"), **sums)
        assert np.array_equal(g.run().cpu().numpy(), want), ("planes in", M, N, K)
    if qp != q:
        # records of the activations' own width are what the prefill kernel reads: the state stays there, and a tile of
        # the decode kernel named by the caller is refused on them
        M, N, K = 4, 64, 256
        x, w = rand_vals(rng, M, K, q, signed), rand_vals(rng, N, K, p, signed)
        xe = abq.relayout_planes(planes_dev(oracle.pack_i32(x, q)))
        wt = abq.relayout_planes(planes_dev(oracle.pack_i32(w, p)))
        g = abq.Gemm(xe, wt, signed, x_tiled=True, w_tiled=True)
        assert g.strategy == "tiled"
        assert np.array_equal(g.run().cpu().numpy(), oracle.np_gemm(x, w))
        cfg = [c for c in abq.native_configs(q, p, signed) if c.nstage == 6][0]
        with pytest.raises(abq.AbqError):
            abq.Gemm(xe, wt, signed, cfg=cfg, x_tiled=True, w_tiled=True).run()


def test_decode_kernel_over_row_blocks_is_the_default_where_it_pays(abq, oracle):
    """Between 17 and 128 rows on prepared operands the library weighs the decode kernel over blocks of 16 rows
    against the prefill kernel's 64 x 64 tile: the choices its fit makes on the LLaMA-7B width, the result either
    way, and the per-token x per-channel epilogue over several row blocks."""
    rng = np.random.default_rng(640)
    N = K = 4096
    for q, p, M, want in [(4, 4, 64, "decode_tiled"), (8, 2, 32, "decode_tiled"), (8, 2, 128, "tiled"), (8, 8, 64, "tiled"),
                          (4, 4, 200, "tiled"), (2, 2, 48, "decode_tiled")]:
        x, w = rand_vals(rng, M, K, q, True), rand_vals(rng, N, K, p, True)
        xt = abq.relayout_planes(planes_dev(oracle.pack_i32(x, q)))
        wt = abq.relayout_planes(planes_dev(oracle.pack_i32(w, p)))
        g = abq.Gemm(xt, wt, True, x_tiled=True, w_tiled=True)
        assert g.strategy == want, (q, p, M, g.strategy, g.config_name)
        assert np.array_equal(g.run().cpu().numpy(), oracle.np_gemm(x, w)), (q, p, M)
    M, N, K = 40, 200, 1152
    x, w = rand_vals(rng, M, K, 8, True), rand_vals(rng, N, K, 2, True)
    xt = abq.relayout_planes(planes_dev(oracle.pack_i32(x, 8)))
    wt = abq.relayout_planes(planes_dev(oracle.pack_i32(w, 2)))
    xs = (rng.random(M) * 0.05 + 0.01).astype(np.float32)
    ws = (rng.random(N) * 0.01 + 0.001).astype(np.float32)
    g = abq.Gemm(xt, wt, True, out_kind=abq.OUT_F16_SCALED, x_scale=dev(xs), w_scale=dev(ws), x_tiled=True, w_tiled=True)
    assert g.strategy == "decode_tiled" and g.state.grid_dim.y == 3
    got = g.run().cpu().numpy().astype(np.float64)
    want = oracle.np_gemm(x, w).astype(np.float64) * xs[:, None].astype(np.float64) * ws[None, :].astype(np.float64)
    assert np.all(np.abs(got - want) <= 1e-2 * np.abs(want) + 1e-6)  # 1e-2 relative (fp16 rounding is 2^-11)


def test_decode_on_prepared_operands_epilogues(abq, oracle):
    """The fp16 epilogues of the decode kernel on K-tiled operands: the reference's per-tensor formula bit for bit,
    per-token x per-channel scales within 1e-2 relative."""
    rng = np.random.default_rng(77)
    M, N, K = 8, 200, 1152
    x, w = rand_vals(rng, M, K, 8, True), rand_vals(rng, N, K, 2, True)
    xp, wp = oracle.pack_i32(x, 8), oracle.pack_i32(w, 2)
    xt, wt = abq.relayout_planes(planes_dev(xp)), abq.relayout_planes(planes_dev(wp))
    acc = oracle.np_gemm(x, w)
    scale = torch.tensor([0.0123], dtype=torch.float16, device="cuda")
    g = abq.Gemm(xt, wt, True, out_kind=abq.OUT_F16_TENSOR, c_scale=scale, x_tiled=True, w_tiled=True)
    assert g.strategy == "decode_tiled"
    got = g.run().cpu().numpy()
    assert np.array_equal(got.view(np.uint16), oracle.epilogue_f16(acc, np.float16(0.0123)).view(np.uint16))
    xs = (rng.random(M) * 0.05 + 0.01).astype(np.float32)
    ws = (rng.random(N) * 0.01 + 0.001).astype(np.float32)
    g = abq.Gemm(xt, wt, True, out_kind=abq.OUT_F16_SCALED, x_scale=dev(xs), w_scale=dev(ws), x_tiled=True, w_tiled=True)
    assert g.strategy == "decode_tiled"
    got = g.run().cpu().numpy().astype(np.float64)
    want = acc.astype(np.float64) * xs[:, None].astype(np.float64) * ws[None, :].astype(np.float64)
    assert np.all(np.abs(got - want) <= 1e-2 * np.abs(want) + 1e-6)  # 1e-2 relative (fp16 rounding is 2^-11)


def test_gemm_generic_bit_widths(abq, oracle):
    """Bit pairs without a specialised kernel (the W1A1 / W1A4 / W1A8 / W1A16 / W2A16 samples)."""
    rng = np.random.default_rng(5)
    for q, p, signed in [(1, 1, False), (4, 1, False), (8, 1, False), (16, 1, False), (16, 2, True), (5, 3, True)]:
        M, N, K = 3, 70, 256
        x = rand_vals(rng, M, K, q, signed and q > 1)
        w = rand_vals(rng, N, K, p, signed and p > 1)
        xp, wp = oracle.pack_i32(x, q), oracle.pack_i32(w, p)
        g = abq.Gemm(planes_dev(xp), planes_dev(wp), signed)
        assert g.strategy == "generic"
        assert np.array_equal(g.run().cpu().numpy(), oracle.gemm_bitserial(xp, wp, signed))


def test_reference_kernel_names_run(abq, oracle):
    """The two production tiles of the FT wrapper (abq_gemm_wrapper.cu:106-124) by name."""
    rng = np.random.default_rng(6)
    for name, M in (("AqBMMA_8x2xtrue_1x48x512_8x24x128_8x8x128_4", 1), ("AqBMMA_8x2xtrue_8x48x256_32x48x128_8x8x128_5", 8),
                    ("AqBWMMA_8x2xfalse_8x48x256_32x48x128_8x8x128_5", 6)):
        cfg, _ = abq.parse_kernel_name(name)
        signed = bool(cfg.is_signed)
        x, w = rand_vals(rng, M, 4096, 8, signed), rand_vals(rng, 1000, 4096, 2, signed)
        got = abq.gemm(planes_dev(oracle.pack_i32(x, 8)), planes_dev(oracle.pack_i32(w, 2)), signed, cfg=cfg)
        assert np.array_equal(got.cpu().numpy(), oracle.np_gemm(x, w))


# ------------------------------------------------------------------ output stages

def test_fp16_per_tensor_epilogue_matches_reference_rounding(abq, oracle):
    rng = np.random.default_rng(7)
    M, N, K = 8, 256, 1024
    x, w = rand_vals(rng, M, K, 8, True), rand_vals(rng, N, K, 2, True)
    xd, wd = planes_dev(oracle.pack_i32(x, 8)), planes_dev(oracle.pack_i32(w, 2))
    acc = oracle.np_gemm(x, w)
    for scale in (np.float16(0.0123), np.float16(1.0), np.float16(3.5e-3)):
        c = torch.tensor([float(scale)], dtype=torch.float16, device="cuda")
        for cfg in [None] + abq.native_configs(8, 2, True):
            got = run_cfg(abq, xd, wd, True, cfg=cfg, out_kind=abq.OUT_F16_TENSOR, c_scale=c).cpu().numpy()
            want = oracle.epilogue_f16(acc, scale)
            assert np.array_equal(got.view(np.uint16), want.view(np.uint16))


def test_fp16_per_token_per_channel_epilogue(abq, oracle):
    """out = acc * x_scale[m] * w_scale[n]; tolerance 1e-2 relative (BASELINE.json north_star)."""
    rng = np.random.default_rng(8)
    for M in (1, 8, 48):
        N, K = 384, 2048
        x, w = rand_vals(rng, M, K, 8, True), rand_vals(rng, N, K, 2, True)
        sx = rng.uniform(0.01, 0.05, M).astype(np.float32)
        sw = rng.uniform(0.005, 0.02, N).astype(np.float32)
        xd, wd = planes_dev(oracle.pack_i32(x, 8)), planes_dev(oracle.pack_i32(w, 2))
        got = abq.gemm(xd, wd, True, out_kind=abq.OUT_F16_SCALED, x_scale=torch.from_numpy(sx).cuda(),
                       w_scale=torch.from_numpy(sw).cuda()).cpu().numpy().astype(np.float64)
        want = (x.astype(np.float64) * sx[:, None]) @ (w.astype(np.float64) * sw[:, None]).T
        denom = np.maximum(np.abs(want), np.abs(want).mean())
        assert np.max(np.abs(got - want) / denom) < 1e-2


# ------------------------------------------------------------------ BASELINE.json configurations at full size

def _sampled_oracle_check(oracle, xp, wp, signed, got, rng, rows=4):
    M = xp.shape[1]
    pick = np.sort(rng.choice(M, size=min(rows, M), replace=False))
    want = oracle.gemm_popc(np.ascontiguousarray(xp[:, pick]), wp, signed)[0]
    assert np.array_equal(got[pick], want)


def test_config0_w4a4_unsigned_m64(abq, oracle):
    rng = np.random.default_rng(0)
    M, N, K = 64, 4096, 4096
    x, w = rand_vals(rng, M, K, 4, False), rand_vals(rng, N, K, 4, False)
    xp, wp = oracle.pack_i32(x, 4), oracle.pack_i32(w, 4)
    got = abq.gemm(planes_dev(xp), planes_dev(wp), False).cpu().numpy()
    assert np.array_equal(got, oracle.gemm_popc(xp, wp, False)[0])


@pytest.mark.parametrize("N,K", [(4096, 4096), (11008, 4096), (4096, 11008)])
def test_config1_w2a8_decode_full_size(abq, oracle, N, K):
    rng = np.random.default_rng(N + K)
    w = rand_vals(rng, N, K, 2, True)
    wp = oracle.pack_i32(w, 2)
    wd = planes_dev(wp)
    for M in (1, 4, 8):
        x = np.clip(np.rint(rng.normal(0, 32, (M, K))), -128, 127).astype(np.int32)
        xp = oracle.pack_i32(x, 8)
        want = oracle.gemm_popc(xp, wp, True)[0]
        xd = planes_dev(xp)
        for cfg in [None] + abq.native_configs(8, 2, True):
            if cfg is not None and cfg.mma_m == 32:
                continue
            got = run_cfg(abq, xd, wd, True, cfg=cfg).cpu().numpy()
            assert np.array_equal(got, want), (M, cfg)
        # prepared operands (weights converted once, activations as the quantising kernel hands them over)
        g = abq.Gemm(abq.relayout_planes(xd), abq.relayout_planes(wd), True, x_tiled=True, w_tiled=True)
        assert g.strategy == "decode_tiled"
        assert np.array_equal(g.run().cpu().numpy(), want), (M, g.config_name)


@pytest.mark.parametrize("q,p,signed", [(4, 4, True), (4, 4, False), (8, 8, True), (8, 8, False)])
def test_config2_prefill_full_size(abq, oracle, q, p, signed):
    """M in {512, 2048} on the LLaMA-7B shapes: exact against the fp64 closed form X.W^T
    (every product and sum is an integer below 2^53) and against the CPU oracle on sampled rows."""
    rng = np.random.default_rng(1000 + q + int(signed))
    for (N, K) in [(4096, 4096), (11008, 4096), (4096, 11008)]:
        w = rand_vals(rng, N, K, p, signed)
        wp = oracle.pack_i32(w, p)
        wd = planes_dev(wp)
        wt = abq.relayout_planes(wd)  # weights prepared once in the K-tiled layout
        wf = torch.from_numpy(w).cuda().double()
        for M in (512, 2048):
            x = rand_vals(rng, M, K, q, signed)
            xp = oracle.pack_i32(x, q)
            xd = planes_dev(xp)
            ws = torch.empty(xd.numel() * 4 + 4 * M + 512, dtype=torch.uint8, device="cuda")
            # (unsigned 8-bit operands: the weights' row sums come with the prepared weights, the activations' are
            # taken per call into the workspace; the staged kernel then runs them like the signed pairs)
            g = abq.Gemm(xd, wt, signed, w_tiled=True, workspace=ws, w_row_sums=None if signed else abq.row_sums(wd))
            assert g.strategy == "tiled" and g.row_sums_ready == ((q, p, signed) == (8, 8, False))
            got_d = g.run()
            if (q, p, signed) == (8, 8, False):  # the same on weights prepared as biased records (code - 128)
                gb = abq.Gemm(xd, abq.relayout_planes_biased(wd), signed, w_tiled=True, workspace=ws, w_row_sums=abq.row_sums(wd),
                              biased=(False, True))
                assert gb.strategy == "tiled" and gb.config_name == g.config_name
                assert torch.equal(gb.run(), got_d)
            ref = torch.from_numpy(x).cuda().double() @ wf.T
            assert torch.equal(got_d.double(), ref), (q, p, signed, M, N, K)
            _sampled_oracle_check(oracle, xp, wp, signed, got_d.cpu().numpy(), rng, rows=2)
            if M == 512:  # the kernel that needs no workspace
                g2 = abq.Gemm(xd, wd, signed)
                assert g2.strategy == "mfma32"
                assert torch.equal(g2.run().double(), ref)
            del ref


def _config3_best_tiles():
    """(x_bits, w_bits, signed, N, K) -> the tile tuple the autotune harness measured as fastest on MI355X (the
    'fastest tile' column of the kept sweep), from tests/golden/config3_best_tiles.json."""
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "config3_best_tiles.json")) as f:
        return {(e["x_bits"], e["w_bits"], e["signed"], e["N"], e["K"]): tuple(e["tile"]) for e in json.load(f)["best"]}


@pytest.mark.parametrize("q,p", BASELINE_COMBOS)
def test_config3_bit_combo_sweep_m128(abq, oracle, q, p):
    """BASELINE configs[3]: every combination at M = 128 on the LLaMA-13B shapes, signed and unsigned, bit exact on
    the library's own choice and on the autotuned tile (the fastest one of the harness sweep for that case)."""
    rng = np.random.default_rng(3000 + 10 * q + p)
    best = _config3_best_tiles()
    M = 128
    for (N, K) in [(5120, 5120), (13824, 5120), (5120, 13824)]:
        for signed in (True, False):
            x, w = rand_vals(rng, M, K, q, signed), rand_vals(rng, N, K, p, signed)
            xp, wp = oracle.pack_i32(x, q), oracle.pack_i32(w, p)
            xd, wd = planes_dev(xp), planes_dev(wp)
            got_d = run_cfg(abq, xd, wd, signed,
                            workspace=torch.empty((xp.size + wp.size) * 4, dtype=torch.uint8, device="cuda"))
            ref = torch.from_numpy(x).cuda().double() @ torch.from_numpy(w).cuda().double().T
            assert torch.equal(got_d.double(), ref), (q, p, signed, N, K)
            _sampled_oracle_check(oracle, xp, wp, signed, got_d.cpu().numpy(), rng, rows=2)
            tile = best[(q, p, signed, N, K)]
            cfg = [c for c in abq.native_configs(q, p, signed) if c.as_tuple()[3:] == tile]
            assert len(cfg) == 1, tile  # the autotuned tile is one the library builds
            got_t = run_cfg(abq, xd, wd, signed, cfg=cfg[0])
            assert torch.equal(got_t.double(), ref), (q, p, signed, N, K, tile)
