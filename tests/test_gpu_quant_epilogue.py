"""GPU tests of the dequantisation side of the path: per-token dynamic quantisation fused with
packing, group-wise weight scales, zero-point corrections, and the decoder-layer linears of
BASELINE.json configs[4].  Expected values are fp64 matmuls of the dequantised operands; the
tolerance is the 1e-2 relative error the task states for the fp16 output."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

pytestmark = pytest.mark.gpu

REL_TOL = 1e-2


@pytest.fixture(scope="module", autouse=True)
def _need_gpu():
    if not torch.cuda.is_available():
        pytest.fail("marked gpu but no GPU is visible")


def planes_dev(planes):
    return torch.from_numpy(np.ascontiguousarray(planes).view(np.int32)).cuda()


def fdev(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).cuda()


def assert_close_rel(got, want):
    """|got - want| <= REL_TOL * |want| elementwise (BASELINE: 1e-2 relative), plus a much tighter norm-wise bound.
    The only slack is an absolute 1e-3 of the matrix's RMS for entries that cancel to nearly zero: the fp32 epilogue
    adds group terms and zero-point corrections that are each up to a few hundred times the matrix's RMS (asymmetric
    activations, K = 11008), so their rounding (6e-8 relative each) leaves about 1e-4 of the RMS as absolute noise,
    which no relative bound on a vanishing entry can absorb (measured worst case: 1.5e-4 of the RMS)."""
    got = got.astype(np.float64)
    rms = np.sqrt(np.mean(want ** 2))
    err = np.abs(got - want)
    assert np.all(np.isfinite(got))
    assert np.all(err <= REL_TOL * np.abs(want) + 1e-3 * rms), float((err / (np.abs(want) + 1e-1 * rms)).max())
    assert np.linalg.norm(got - want) <= 2e-3 * np.linalg.norm(want)


def run_grouped(abq, xp, wp, signed, strategy="tiled", **kw):
    g = abq.Gemm(xp, wp, signed, out_kind=abq.OUT_F16_SCALED, **kw)
    assert g.strategy == strategy
    if g.workspace_bytes:
        ws = torch.empty(g.workspace_bytes, dtype=torch.uint8, device="cuda")
        g = abq.Gemm(xp, wp, signed, out_kind=abq.OUT_F16_SCALED, workspace=ws, **kw)
    out = g.run()
    torch.cuda.synchronize()
    return out.cpu().numpy()


# ------------------------------------------------------------------ quantise + pack

@pytest.mark.parametrize("rows,k,bits,symmetric", [(1, 128, 8, True), (5, 4096, 8, True), (33, 11008, 8, False),
                                                   (7, 256, 4, True), (16, 1152, 4, False), (3, 384, 2, True),
                                                   (64, 4096, 6, False), (9, 640, 5, False), (12, 512, 3, True),
                                                   (3, 24576, 8, True), (2, 24704, 8, False),  # last row kept in LDS / first not
                                                   # a workgroup per row up to here; beyond, one wave per row:
                                                   (1100, 4096, 8, True), (2100, 5120, 8, False), (1030, 1024, 4, False),
                                                   # the longest rows a workgroup's four waves hold in registers
                                                   (20, 13824, 8, False), (4, 16384, 8, True), (300, 2048, 8, False)])
def test_quant_pack_matches_the_restated_quantizer(abq, oracle, rows, k, bits, symmetric):
    from oracle import quantizer as Q
    rng = np.random.default_rng(rows + k + bits)
    x = (rng.normal(0, 1, (rows, k)) * rng.uniform(0.1, 8, (rows, 1))).astype(np.float16)
    x[0, :7] = [0, -0.0, 1, -1, 0.5, 65504, -3]  # an outlier row
    codes, scale, zero = Q.per_token_codes_f32(x, bits, symmetric)
    for gs in (64, 128):
        planes, s, z, sums = abq.quant_pack_f16(torch.from_numpy(x).cuda(), bits, symmetric=symmetric, group_size=gs)
        torch.cuda.synchronize()
        assert np.array_equal(s.cpu().numpy(), scale)
        if not symmetric:
            assert np.array_equal(z.cpu().numpy(), zero)
        assert np.array_equal(planes.cpu().numpy().view(np.uint32), oracle.pack_i32(codes, bits))
        assert np.array_equal(sums.cpu().numpy(), codes.reshape(rows, k // gs, gs).sum(axis=2))
    # K-tiled output equals the relayout of the plane output
    tiled, _, _, _ = abq.quant_pack_f16(torch.from_numpy(x).cuda(), bits, symmetric=symmetric, tiled=True)
    assert torch.equal(tiled, abq.relayout_planes(planes))
    # ... also when the group sums are taken in the same pass
    tiled, s_t, _, sums_t = abq.quant_pack_f16(torch.from_numpy(x).cuda(), bits, symmetric=symmetric, tiled=True, group_size=128)
    assert torch.equal(tiled, abq.relayout_planes(planes)) and torch.equal(s_t, s)
    assert np.array_equal(sums_t.cpu().numpy(), codes.reshape(rows, k // 128, 128).sum(axis=2))
    # FP6 records (codes of at most 5 bits) equal the FP6 relayout of the plane output
    if bits <= 5:
        rec, s6, _, _ = abq.quant_pack_f16(torch.from_numpy(x).cuda(), bits, symmetric=symmetric, fp6=True)
        assert torch.equal(rec, abq.relayout_planes_fp6(planes, True)) and torch.equal(s6, s)
    else:
        with pytest.raises(abq.AbqError):
            abq.quant_pack_f16(torch.from_numpy(x).cuda(), bits, symmetric=symmetric, fp6=True)


@pytest.mark.parametrize("symmetric", [True, False])
def test_quant_pack_rows_with_infinities(abq, oracle, symmetric):
    """A row that holds an infinity: the scale saturates at its upper clamp and the infinite elements take the
    end codes, as a division would leave them (the kernel's quotient without a division needs its fix-up here)."""
    from oracle import quantizer as Q
    rng = np.random.default_rng(77 + symmetric)
    x = (rng.normal(0, 300, (4, 512))).astype(np.float16)
    x[0, 3], x[0, 100] = np.inf, -np.inf
    x[1, 511] = np.inf
    x[2, 0] = -np.inf
    with np.errstate(invalid="ignore", over="ignore"):
        codes, scale, zero = Q.per_token_codes_f32(x, 8, symmetric)
    planes, s, z, _ = abq.quant_pack_f16(torch.from_numpy(x).cuda(), 8, symmetric=symmetric)
    torch.cuda.synchronize()
    assert np.array_equal(s.cpu().numpy(), scale)
    if not symmetric:
        assert np.array_equal(z.cpu().numpy(), zero)
    assert np.array_equal(planes.cpu().numpy().view(np.uint32), oracle.pack_i32(codes, 8))


@pytest.mark.parametrize("absmax,bits", [(127.0, 8), (381.0, 8), (63.5, 8), (21.0, 4), (889.0, 8), (3.0, 2), (77.0, 4),
                                         (35.0, 4), (91.0, 4)])
def test_quant_pack_rounds_exact_ties_like_the_division(abq, oracle, absmax, bits):
    """Rows whose scale is 1, 3, 0.5, 7 ... exactly and whose values are odd multiples of half a scale: every
    quotient is a tie, so a quotient that is off by one ulp rounds to the other neighbour."""
    from oracle import quantizer as Q
    qmax = (1 << (bits - 1)) - 1
    step = absmax / qmax
    k = 256
    x = np.zeros((4, k), dtype=np.float16)
    odd = np.arange(k) * 2 + 1
    x[0] = ((odd % (2 * qmax)) * step / 2)
    x[1] = -x[0]
    x[2] = (np.arange(k) % (qmax + 1)) * step
    x[3] = x[0] * np.where(np.arange(k) % 3 == 0, -1, 1)
    x[:, -1] = absmax
    assert np.array_equal(x.astype(np.float64)[0, :-1], (odd % (2 * qmax))[:-1] * step / 2)  # exact in fp16
    codes, scale, _ = Q.per_token_codes_f32(x, bits, True)
    assert np.all(scale == np.float32(step))
    planes, s, _, _ = abq.quant_pack_f16(torch.from_numpy(x).cuda(), bits, symmetric=True)
    torch.cuda.synchronize()
    assert np.array_equal(s.cpu().numpy(), scale)
    assert np.array_equal(planes.cpu().numpy().view(np.uint32), oracle.pack_i32(codes, bits))


# ------------------------------------------------------------------ group scales, zero points

@pytest.mark.parametrize("q,p,signed", [(8, 2, True), (4, 4, True), (8, 4, True), (4, 4, False), (6, 2, False),
                                        (2, 2, True), (7, 7, False)])
@pytest.mark.parametrize("group_size", [128, 64])
def test_group_scale_epilogue(abq, oracle, q, p, signed, group_size):
    from oracle import quantizer as Q
    rng = np.random.default_rng(q * 10 + p + group_size)
    for (M, N, K) in [(70, 200, 384), (256, 1024, 1024)]:
        lo_x, hi_x = (-(1 << (q - 1)), 1 << (q - 1)) if signed else (0, 1 << q)
        lo_w, hi_w = (-(1 << (p - 1)), 1 << (p - 1)) if signed else (0, 1 << p)
        x = rng.integers(lo_x, hi_x, (M, K)).astype(np.int32)
        w = rng.integers(lo_w, hi_w, (N, K)).astype(np.int32)
        xs = rng.uniform(0.01, 0.05, M)
        wsc = rng.uniform(0.001, 0.02, (N, K // group_size))
        want = Q.dequant_matmul(x, xs, np.zeros(M), w, wsc, np.zeros_like(wsc), group_size)
        got = run_grouped(abq, planes_dev(oracle.pack_i32(x, q)), planes_dev(oracle.pack_i32(w, p)), signed,
                          x_scale=fdev(xs), w_scale=fdev(wsc), group_size=group_size)
        assert_close_rel(got, want)


@pytest.mark.parametrize("group_size", [128, 64])
@pytest.mark.parametrize("with_x_zero", [False, True])
def test_zero_point_corrections(abq, oracle, group_size, with_x_zero):
    from oracle import quantizer as Q
    rng = np.random.default_rng(group_size + with_x_zero)
    for (q, p, signed) in [(8, 2, True), (4, 4, False)]:
        M, N, K = 150, 330, 5 * 1152  # 45 (or 90) groups: more than one LDS staging pass
        lo_x, hi_x = (-(1 << (q - 1)), 1 << (q - 1)) if signed else (0, 1 << q)
        lo_w, hi_w = (-(1 << (p - 1)), 1 << (p - 1)) if signed else (0, 1 << p)
        x = rng.integers(lo_x, hi_x, (M, K)).astype(np.int32)
        w = rng.integers(lo_w, hi_w, (N, K)).astype(np.int32)
        xs = rng.uniform(0.01, 0.05, M)
        xz = rng.integers(lo_x // 2, hi_x // 2, M).astype(np.float64) if with_x_zero else np.zeros(M)
        wsc = rng.uniform(0.001, 0.02, (N, K // group_size))
        wz = rng.integers(lo_w, hi_w, (N, K // group_size)).astype(np.float64)
        want = Q.dequant_matmul(x, xs, xz, w, wsc, wz, group_size)
        wp = planes_dev(oracle.pack_i32(w, p))
        kw = dict(x_scale=fdev(xs), w_scale=fdev(wsc), group_size=group_size, w_zero=fdev(wz),
                  x_group_sums=torch.from_numpy(x.reshape(M, K // group_size, group_size).sum(axis=2).astype(np.int32)).cuda())
        if with_x_zero:
            term = abq.weight_zero_term(wp, signed, kw["w_scale"], kw["w_zero"], group_size)
            want_term = (wsc * (w.reshape(N, -1, group_size).sum(axis=2) - group_size * wz)).sum(axis=1)
            assert np.allclose(term.cpu().numpy(), want_term, rtol=1e-5, atol=1e-5)
            kw.update(x_zero=fdev(xz), w_zero_term=term)
        got = run_grouped(abq, planes_dev(oracle.pack_i32(x, q)), wp, signed, **kw)
        assert_close_rel(got, want)


@pytest.mark.parametrize("q,p,signed", [(8, 2, True), (4, 4, True), (8, 4, True), (4, 4, False), (6, 2, False)])
@pytest.mark.parametrize("group_size", [128, 64])
def test_decode_kernel_with_group_scales_and_zero_points(abq, oracle, q, p, signed, group_size):
    """At most 16 activation rows on plane operands run the decode kernel's group-scale variant."""
    from oracle import quantizer as Q
    rng = np.random.default_rng(q + 7 * p + group_size)
    for (M, N, K, zeros) in [(1, 64, 128, 0), (5, 200, 384, 1), (16, 4096 + 8, 4096, 2), (8, 300, 11008, 2), (3, 4096, 1152, 1)]:
        lo_x, hi_x = (-(1 << (q - 1)), 1 << (q - 1)) if signed else (0, 1 << q)
        lo_w, hi_w = (-(1 << (p - 1)), 1 << (p - 1)) if signed else (0, 1 << p)
        x = rng.integers(lo_x, hi_x, (M, K)).astype(np.int32)
        w = rng.integers(lo_w, hi_w, (N, K)).astype(np.int32)
        G = K // group_size
        xs = rng.uniform(0.01, 0.05, M)
        wsc = rng.uniform(0.001, 0.02, (N, G))
        wz = rng.integers(lo_w, hi_w, (N, G)).astype(np.float64) if zeros >= 1 else np.zeros((N, G))
        xz = rng.integers(lo_x // 2, hi_x // 2, M).astype(np.float64) if zeros >= 2 else np.zeros(M)
        want = Q.dequant_matmul(x, xs, xz, w, wsc, wz, group_size)
        wp = planes_dev(oracle.pack_i32(w, p))
        kw = dict(x_scale=fdev(xs), w_scale=fdev(wsc), group_size=group_size)
        if zeros >= 1:
            kw.update(w_zero=fdev(wz),
                      x_group_sums=torch.from_numpy(x.reshape(M, G, group_size).sum(axis=2).astype(np.int32)).cuda())
        if zeros >= 2:
            kw.update(x_zero=fdev(xz), w_zero_term=abq.weight_zero_term(wp, signed, kw["w_scale"], kw["w_zero"], group_size))
        out = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
        got = run_grouped(abq, planes_dev(oracle.pack_i32(x, q)), wp, signed, strategy="decode", out=out, **kw)
        assert_close_rel(got, want)
        # the same state moved to the tiled kernel by declaring prepared weights gives the same values
        got2 = run_grouped(abq, planes_dev(oracle.pack_i32(x, q)), abq.relayout_planes(wp), signed, w_tiled=True, **kw)
        assert_close_rel(got2, want)
        assert np.abs(got.astype(np.float64) - got2.astype(np.float64)).max() <= 2e-3 * np.abs(want).max()


@pytest.mark.parametrize("q,p,signed", [(8, 2, True), (8, 4, True), (8, 8, True), (4, 4, True), (4, 2, True), (2, 2, True),
                                        (4, 4, False), (4, 2, False), (2, 2, False)])
@pytest.mark.parametrize("group_size", [128, 64])
def test_decode_on_prepared_operands_with_group_scales(abq, oracle, q, p, signed, group_size):
    """At most 16 activation rows with both operands K-tiled and groups of 128 or 64: the prepared-operand decode
    kernel's group-scale variant (one K tile = one or two scale groups per step), with zero points on both sides."""
    from oracle import quantizer as Q
    rng = np.random.default_rng(3 * q + 11 * p + signed)
    for (M, N, K, zeros) in [(1, 64, 128, 0), (5, 200, 384, 1), (16, 4096 + 8, 4096, 2), (8, 300, 11008, 2), (3, 4096, 1152, 1),
                             (1, 11008, 4096, 2), (16, 48, 11008, 2), (2, 16, 2176, 1), (13, 20, 256, 2)]:
        lo_x, hi_x = (-(1 << (q - 1)), 1 << (q - 1)) if signed else (0, 1 << q)
        lo_w, hi_w = (-(1 << (p - 1)), 1 << (p - 1)) if signed else (0, 1 << p)
        x = rng.integers(lo_x, hi_x, (M, K)).astype(np.int32)
        w = rng.integers(lo_w, hi_w, (N, K)).astype(np.int32)
        G = K // group_size
        xs = rng.uniform(0.01, 0.05, M)
        wsc = rng.uniform(0.001, 0.02, (N, G))
        wz = rng.integers(lo_w, hi_w, (N, G)).astype(np.float64) if zeros >= 1 else np.zeros((N, G))
        xz = rng.integers(lo_x // 2, hi_x // 2, M).astype(np.float64) if zeros >= 2 else np.zeros(M)
        want = Q.dequant_matmul(x, xs, xz, w, wsc, wz, group_size)
        wp = planes_dev(oracle.pack_i32(w, p))
        kw = dict(x_scale=fdev(xs), w_scale=fdev(wsc), group_size=group_size, x_tiled=True, w_tiled=True)
        if zeros >= 1:
            kw.update(w_zero=fdev(wz), x_group_sums=torch.from_numpy(x.reshape(M, G, group_size).sum(axis=2).astype(np.int32)).cuda())
        if zeros >= 2:
            kw.update(x_zero=fdev(xz), w_zero_term=abq.weight_zero_term(wp, signed, kw["w_scale"], kw["w_zero"], group_size))
        out = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
        xt, wt = abq.relayout_planes(planes_dev(oracle.pack_i32(x, q))), abq.relayout_planes(wp)
        got = run_grouped(abq, xt, wt, signed, strategy="decode_tiled", out=out, **kw)
        assert_close_rel(got, want)


@pytest.mark.parametrize("q,p,signed", [(8, 2, True), (4, 4, True), (8, 4, True), (4, 4, False)])
def test_group_scale_decode_kernel_over_row_blocks(abq, oracle, q, p, signed):
    """17 to 128 rows on prepared operands with groups of 128: where the library estimates it ahead of the prefill
    kernel, the decode kernel's group-scale variant runs over blocks of 16 rows (8 where a block's activations would
    not fit the LDS); zero points on both sides, ragged last block, the fused SiLU gate, either order of the calls."""
    from oracle import quantizer as Q
    rng = np.random.default_rng(900 + 10 * q + p + signed)
    lo_x, hi_x = (-(1 << (q - 1)), 1 << (q - 1)) if signed else (0, 1 << q)
    lo_w, hi_w = (-(1 << (p - 1)), 1 << (p - 1)) if signed else (0, 1 << p)
    for (M, N, K, act) in [(24, 192, 1152, False), (40, 330, 1152, False), (33, 192, 1152, True), (17, 64, 11008, False),
                           (32, 4096, 4096, False)]:
        G = K // 128
        x = rng.integers(lo_x, hi_x, (M, K)).astype(np.int32)
        w = rng.integers(lo_w, hi_w, (N, K)).astype(np.int32)
        xs = rng.uniform(0.01, 0.05, M)
        xz = rng.integers(lo_x // 2, hi_x // 2 + 1, M).astype(np.float64)
        wsc = rng.uniform(0.001, 0.02, (N, G))
        wz = rng.integers(lo_w, hi_w, (N, G)).astype(np.float64)
        want = Q.dequant_matmul(x, xs, xz, w, wsc, wz, 128)
        if act:  # rows of W come in blocks of 16 gate rows followed by their 16 up rows
            blocks = want.reshape(M, N // 32, 2, 16)
            gate, up = blocks[:, :, 0, :], blocks[:, :, 1, :]
            want = (gate / (1.0 + np.exp(-gate)) * up).reshape(M, N // 2)
        wp = planes_dev(oracle.pack_i32(w, p))
        kw = dict(x_scale=fdev(xs), w_scale=fdev(wsc), group_size=128, w_zero=fdev(wz), x_zero=fdev(xz), x_tiled=True, w_tiled=True,
                  x_group_sums=torch.from_numpy(x.reshape(M, G, 128).sum(axis=2).astype(np.int32)).cuda())
        kw["w_zero_term"] = abq.weight_zero_term(wp, signed, kw["w_scale"], kw["w_zero"], 128)
        if act:
            kw["act"] = abq.ACT_SILU_GATE
        xt, wt = abq.relayout_planes(planes_dev(oracle.pack_i32(x, q))), abq.relayout_planes(wp)
        assert abq.prepared_decode_pays(q, p, signed, M, N, K, 128, abq.ACT_SILU_GATE if act else abq.ACT_NONE)
        g = abq.Gemm(xt, wt, signed, out_kind=abq.OUT_F16_SCALED, **kw)
        assert g.strategy == "decode_tiled", (g.strategy, M, N, K)
        got = g.run()
        torch.cuda.synchronize()
        assert_close_rel(got.cpu().numpy(), want)
        if (M, N, K) == (32, 4096, 4096):
            # layouts -> scales -> workspace: a workspace the state does not need leaves it on the same kernel
            ws = torch.empty(1 << 20, dtype=torch.uint8, device="cuda")
            g2 = abq.Gemm(xt, wt, signed, out_kind=abq.OUT_F16_SCALED, workspace=ws, **kw)
            assert (g2.strategy, g2.config_name) == (g.strategy, g.config_name)
            assert torch.equal(g2.run(), got)
    # what the estimate decides on the decoder-layer linears (W2A8: the narrow outputs only)
    if (q, p, signed) == (8, 2, True):
        assert abq.prepared_decode_pays(8, 2, True, 32, 4096, 4096, 128) and abq.prepared_decode_pays(8, 2, True, 32, 4096, 11008, 128)
        assert not abq.prepared_decode_pays(8, 2, True, 32, 12288, 4096, 128)
        assert not abq.prepared_decode_pays(8, 2, True, 96, 4096, 4096, 128)
        assert not abq.prepared_decode_pays(8, 2, True, 200, 4096, 4096, 128)
        assert abq.prepared_decode_pays(8, 2, True, 32, 4096, 4096, 64)  # groups of 64: two to a K tile


def test_decode_kernel_quantises_fp16_activations_per_token_itself(abq, oracle):
    """abq_gemm_set_dynamic_f16_activations: the group-scale decode kernel on prepared weights takes fp16 activations and
    quantises them per token in the kernel, symmetric or with a zero point.  Same formulas and rounding as the
    quantise-and-pack kernel, so the output equals that of the two launches bit for bit (and through it the oracle,
    which the two-launch path is checked against); rows with outliers, a constant row, ragged N, the fused gate."""
    rng = np.random.default_rng(4242)
    for (M, N, K, p, symmetric, with_wz, act) in [(1, 4096, 4096, 2, True, True, False), (1, 4096, 4096, 2, False, True, False),
                                                  (4, 200, 4096, 2, False, True, False), (3, 330, 1152, 4, True, False, False),
                                                  (1, 192, 11008, 2, False, True, True), (2, 12288, 4096, 2, False, True, False),
                                                  (1, 22016, 4096, 2, True, True, True), (4, 64, 128, 8, False, True, False),
                                                  (16, 96, 1024, 2, False, True, False)]:
        G = K // 128
        lo_w, hi_w = -(1 << (p - 1)), 1 << (p - 1)
        w = rng.integers(lo_w, hi_w, (N, K)).astype(np.int32)
        wp = planes_dev(oracle.pack_i32(w, p))
        wt = abq.relayout_planes(wp)
        wsc = fdev(rng.uniform(0.001, 0.02, (N, G)))
        wz = fdev(rng.integers(lo_w, hi_w, (N, G)).astype(np.float64)) if with_wz else None
        xg = torch.Generator(device="cuda").manual_seed(M + N + K)
        x = torch.randn((M, K), generator=xg, device="cuda", dtype=torch.float32)
        x[:, ::97] *= 8.0
        if M > 1:
            x[M - 1] = 0.25  # a constant row: the scale clamps, the codes saturate
        x = x.to(torch.float16)
        xt, xs, xz, sums = abq.quant_pack_f16(x, 8, symmetric=symmetric, tiled=True, group_size=128)
        term = abq.weight_zero_term(wp, True, wsc, wz, 128) if (with_wz and not symmetric) else None
        kw = dict(x_scale=xs, w_scale=wsc, group_size=128, x_tiled=True, w_tiled=True, out_kind=abq.OUT_F16_SCALED,
                  act=abq.ACT_SILU_GATE if act else abq.ACT_NONE)
        if with_wz:
            kw.update(w_zero=wz, x_group_sums=sums)
        if not symmetric:
            if term is None:
                term = abq.weight_zero_term(wp, True, wsc, torch.zeros_like(wsc), 128)
                kw.update(w_zero=torch.zeros_like(wsc), x_group_sums=sums)
            kw.update(x_zero=xz, w_zero_term=term)
        ref = abq.Gemm(xt, wt, True, **kw)
        assert ref.strategy == "decode_tiled"
        want = ref.run().clone()
        # the same state, fed the fp16 rows
        kw2 = {k: v for k, v in kw.items() if k not in ("x_zero", "w_zero_term", "w_zero", "x_group_sums")}
        out = torch.full_like(want, float("nan"))
        g = abq.Gemm(xt, wt, True, out=out, **kw2)
        g.set_dynamic_f16_activations(x, symmetric, w_zero=kw.get("w_zero"), w_zero_term=kw.get("w_zero_term"))
        got = g.run()
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), (M, N, K, p, symmetric, with_wz, act)
    # shapes and states the kernel does not take: 8 x 4096 elements are too many for one workgroup's registers,
    # and a state without group scales has no such variant
    K, N = 4096, 64
    wt = abq.relayout_planes(planes_dev(oracle.pack_i32(rng.integers(-2, 2, (N, K)).astype(np.int32), 2)))
    wsc = fdev(rng.uniform(0.001, 0.02, (N, K // 128)))
    x = torch.randn((8, K), device="cuda", dtype=torch.float16)
    xt, xs, _, _ = abq.quant_pack_f16(x, 8, symmetric=True, tiled=True, group_size=128)
    g = abq.Gemm(xt, wt, True, x_scale=xs, w_scale=wsc, group_size=128, x_tiled=True, w_tiled=True, out_kind=abq.OUT_F16_SCALED)
    with pytest.raises(abq.AbqError):
        g.set_dynamic_f16_activations(x, True)
    g = abq.Gemm(xt[:, :4].contiguous(), wt, True, x_scale=xs[:4].contiguous(), w_scale=fdev(rng.uniform(0.001, 0.02, N)),
                 x_tiled=True, w_tiled=True, out_kind=abq.OUT_F16_SCALED)
    with pytest.raises(abq.AbqError):
        g.set_dynamic_f16_activations(x[:4].contiguous(), True)


def test_decode_on_prepared_operands_group_scales_either_call_order(abq, oracle):
    """Layouts declared before the scales are attached (the C ABI allows both orders) lands on the same kernel."""
    import ctypes
    from oracle import quantizer as Q
    rng = np.random.default_rng(5)
    M, N, K = 4, 96, 512
    x = rng.integers(-128, 128, (M, K)).astype(np.int32)
    w = rng.integers(-2, 2, (N, K)).astype(np.int32)
    xs, wsc = rng.uniform(0.01, 0.05, M), rng.uniform(0.001, 0.02, (N, K // 128))
    xt = abq.relayout_planes(planes_dev(oracle.pack_i32(x, 8)))
    wt = abq.relayout_planes(planes_dev(oracle.pack_i32(w, 2)))
    g = abq.Gemm(xt, wt, True, out_kind=abq.OUT_F16_SCALED, x_scale=fdev(xs), w_scale=fdev(wsc), x_tiled=True, w_tiled=True)
    assert g.strategy == "decode_tiled"  # per-channel state on prepared operands
    wsc_d = fdev(wsc)
    st = abq.lib().abq_gemm_set_scales(ctypes.byref(g.state), g.x_scale.data_ptr(), wsc_d.data_ptr(), 128)
    assert st == 0 and g.strategy == "decode_tiled"
    out = g.run()
    torch.cuda.synchronize()
    assert_close_rel(out.cpu().numpy(), Q.dequant_matmul(x, xs, np.zeros(M), w, wsc, np.zeros_like(wsc), 128))
    # groups of 64 run on the same kernel (two groups to a K tile)
    g2 = abq.Gemm(xt, wt, True, out_kind=abq.OUT_F16_SCALED, x_scale=fdev(xs), w_scale=fdev(np.repeat(wsc, 2, axis=1)),
                  group_size=64, x_tiled=True, w_tiled=True)
    assert g2.strategy == "decode_tiled"
    out2 = g2.run()
    torch.cuda.synchronize()
    assert_close_rel(out2.cpu().numpy(), Q.dequant_matmul(x, xs, np.zeros(M), w, wsc, np.zeros_like(wsc), 128))


def interleave16(gate, up):
    """[I, ...] gate rows and [I, ...] up rows -> [2I, ...] in blocks of 16 gate rows followed by their 16 up rows."""
    I = gate.shape[0]
    assert I % 16 == 0
    out = np.empty((2 * I,) + gate.shape[1:], dtype=gate.dtype)
    blocks = out.reshape((I // 16, 2, 16) + gate.shape[1:])
    blocks[:, 0] = gate.reshape((I // 16, 16) + gate.shape[1:])
    blocks[:, 1] = up.reshape((I // 16, 16) + up.shape[1:])
    return out


@pytest.mark.parametrize("M,strategy", [(1, "decode"), (7, "decode"), (16, "decode"), (100, "tiled"), (300, "tiled"),
                                        (1, "decode_tiled"), (7, "decode_tiled"), (16, "decode_tiled")])
@pytest.mark.parametrize("group_size", [128, 64])
def test_silu_gate_epilogue(abq, oracle, M, strategy, group_size):
    """gate / up pair fused into one GEMM: D = silu(x Wg^T) * (x Wu^T) on the dequantised values."""
    from oracle import quantizer as Q
    rng = np.random.default_rng(M + group_size)
    q, p, I, K = 8, 2, 11008 if M == 7 else 176, 4096 if M == 7 else 640
    G = K // group_size
    x = rng.integers(-128, 128, (M, K)).astype(np.int32)
    xs, xz = rng.uniform(0.005, 0.02, M), rng.integers(-20, 20, M).astype(np.float64)
    parts = []
    for _ in range(2):  # gate, up
        w = rng.integers(-2, 2, (I, K)).astype(np.int32)
        parts.append((w, rng.uniform(0.002, 0.02, (I, G)), rng.integers(-2, 2, (I, G)).astype(np.float64)))
    full = [Q.dequant_matmul(x, xs, xz, w, sc, z, group_size) for (w, sc, z) in parts]
    want = full[0] / (1.0 + np.exp(-full[0])) * full[1]
    w_cat, sc_cat, z_cat = (interleave16(parts[0][i], parts[1][i]) for i in range(3))
    wp = planes_dev(oracle.pack_i32(w_cat, p))
    kw = dict(x_scale=fdev(xs), w_scale=fdev(sc_cat), group_size=group_size, w_zero=fdev(z_cat), x_zero=fdev(xz),
              x_group_sums=torch.from_numpy(x.reshape(M, G, group_size).sum(axis=2).astype(np.int32)).cuda(),
              act=abq.ACT_SILU_GATE)
    kw["w_zero_term"] = abq.weight_zero_term(wp, True, kw["w_scale"], kw["w_zero"], group_size)
    out = torch.full((M, I), float("nan"), dtype=torch.float16, device="cuda")
    if strategy == "tiled":
        got = run_grouped(abq, planes_dev(oracle.pack_i32(x, q)), abq.relayout_planes(wp), True, w_tiled=True, out=out, **kw)
    elif strategy == "decode_tiled":
        got = run_grouped(abq, abq.relayout_planes(planes_dev(oracle.pack_i32(x, q))), abq.relayout_planes(wp), True,
                          strategy="decode_tiled", x_tiled=True, w_tiled=True, out=out, **kw)
    else:
        got = run_grouped(abq, planes_dev(oracle.pack_i32(x, q)), wp, True, strategy="decode", out=out, **kw)
    assert got.shape == (M, I)
    assert_close_rel(got, want)


def test_group_scale_argument_checks(abq, oracle):
    rng = np.random.default_rng(0)
    x = planes_dev(oracle.pack_i32(rng.integers(0, 256, (32, 256)).astype(np.int32), 8))
    w = planes_dev(oracle.pack_i32(rng.integers(0, 256, (64, 256)).astype(np.int32), 8))
    s = torch.ones(64 * 4, dtype=torch.float32, device="cuda")
    with pytest.raises(abq.AbqError) as e:  # 8-bit unsigned operands have no group-scale kernel
        abq.Gemm(x, w, False, out_kind=abq.OUT_F16_SCALED, x_scale=s, w_scale=s, group_size=128)
    assert e.value.status == abq.ABQ_ERR_UNSUPPORTED
    with pytest.raises(abq.AbqError) as e:  # only 64 and 128
        abq.Gemm(x, w, True, out_kind=abq.OUT_F16_SCALED, x_scale=s, w_scale=s, group_size=32)
    assert e.value.status == abq.ABQ_ERR_UNSUPPORTED
    with pytest.raises(abq.AbqError) as e:  # zero points need group scales
        abq.Gemm(x, w, True, out_kind=abq.OUT_F16_SCALED, x_scale=s, w_scale=s, group_size=0, w_zero=s, x_group_sums=s)
    assert e.value.status == abq.ABQ_ERR_UNSUPPORTED
    with pytest.raises(abq.AbqError) as e:  # the fused activation lives in the group-scale epilogues
        abq.Gemm(x, w, True, out_kind=abq.OUT_F16_SCALED, x_scale=s, w_scale=s, group_size=0, act=abq.ACT_SILU_GATE)
    assert e.value.status == abq.ABQ_ERR_UNSUPPORTED
    with pytest.raises(abq.AbqError) as e:  # w_zero without the activation group sums
        abq.Gemm(x, w, True, out_kind=abq.OUT_F16_SCALED, x_scale=s, w_scale=s, group_size=128, w_zero=s)
    assert e.value.status == abq.ABQ_ERR_INVALID_ARG

def _staged_grouped_lds(cfg):
    """LDS of the staged kernel's group-scale variant for a tile: 3 or 4 stages of the packed records
    (16 bytes per bit of width per row and K tile) plus the tile's scales (at least 512 bytes) each."""
    buf = 16 * (cfg.block_m * cfg.x_bits + cfg.block_n * cfg.w_bits) + max(512, 4 * cfg.block_n)
    buf *= cfg.block_k // cfg.warp_k  # groups of waves that split K: a stage holds a K tile for each
    two_per_cu = cfg.block_m * cfg.block_n <= 128 * 128 and 2 * 4 * buf > 160 * 1024 >= 2 * 3 * buf
    return buf * (3 if two_per_cu or 4 * buf > 160 * 1024 else 4)


@pytest.mark.parametrize("q,p,signed", [(8, 2, True), (4, 4, True), (4, 4, False), (8, 4, True), (2, 2, True),
                                        (2, 2, False), (4, 2, True), (8, 8, True)])
def test_group_scale_staged_kernel_every_tile(abq, oracle, q, p, signed):
    """Groups of 128 on pairs of 2-, 4- and 8-bit fields run on the kernel that loads the records and
    the scales straight into LDS; every tile it is built for, picked by its tuple, with zero points
    on both sides, on shapes with ragged edges, fewer K tiles than LDS stages, odd and even tile counts (the 64 x 64
    tile, one MFMA tile per wave, alternates between two accumulators) and a K of 86 groups (three chunks of the
    zero-point term, rows of the scale arrays that start off 16-byte boundaries)."""
    from oracle import quantizer as Q
    rng = np.random.default_rng(100 * q + 10 * p + signed)
    tiles = [c for c in abq.native_configs(q, p, signed)
             if c.nstage == 4 and c.warp_k == 128 and (c.warp_m, c.warp_n) in ((64, 64), (64, 32), (32, 64), (32, 32)) and
             (c.block_m, c.block_n) in ((256, 128), (128, 128), (128, 64), (128, 256), (64, 128), (64, 64))]
    assert ((128, 256) in [(c.block_m, c.block_n) for c in tiles]) == (q > p)
    assert [c.block_k for c in tiles if (c.block_m, c.block_n) == (64, 128)] == ([128, 256] if q > p else [])
    if (q, p) == (8, 8):
        tiles = [c for c in tiles if (c.block_m, c.block_n) in ((128, 64), (64, 64))]
    assert tiles
    assert [c.block_k for c in tiles if (c.block_m, c.block_n) == (64, 64)] == [128, 256]
    assert [c.block_k for c in tiles if (c.block_m, c.block_n) == (128, 64)] == [128, 256]  # plain, and waves that split K
    lo_x, hi_x = (-(1 << (q - 1)), 1 << (q - 1)) if signed else (0, 1 << q)
    lo_w, hi_w = (-(1 << (p - 1)), 1 << (p - 1)) if signed else (0, 1 << p)
    for (M, N, K) in [(300, 200, 640), (70, 330, 256), (129, 65, 128), (200, 136, 1536), (70, 100, 11008)]:
        G = K // 128
        x = rng.integers(lo_x, hi_x, (M, K)).astype(np.int32)
        w = rng.integers(lo_w, hi_w, (N, K)).astype(np.int32)
        xs = rng.uniform(0.01, 0.05, M)
        xz = rng.integers(lo_x // 2, hi_x // 2 + 1, M).astype(np.float64)
        wsc = rng.uniform(0.001, 0.02, (N, G))
        wz = rng.integers(lo_w, hi_w, (N, G)).astype(np.float64)
        want = Q.dequant_matmul(x, xs, xz, w, wsc, wz, 128)
        wp = planes_dev(oracle.pack_i32(w, p))
        kw = dict(x_scale=fdev(xs), w_scale=fdev(wsc), group_size=128, w_zero=fdev(wz), x_zero=fdev(xz),
                  x_group_sums=torch.from_numpy(x.reshape(M, G, 128).sum(axis=2).astype(np.int32)).cuda())
        kw["w_zero_term"] = abq.weight_zero_term(wp, signed, kw["w_scale"], kw["w_zero"], 128)
        xt, wt = abq.relayout_planes(planes_dev(oracle.pack_i32(x, q))), abq.relayout_planes(wp)
        for cfg in tiles:
            g = abq.Gemm(xt, wt, signed, cfg=cfg, out_kind=abq.OUT_F16_SCALED, x_tiled=True, w_tiled=True, **kw)
            assert g.strategy == "tiled" and (g.state.cfg.block_m, g.state.cfg.block_n, g.state.cfg.block_k) == (
                cfg.block_m, cfg.block_n, cfg.block_k)
            assert g.state.shared_mem_size == _staged_grouped_lds(cfg), (g.config_name, g.state.shared_mem_size)
            got = g.run()
            torch.cuda.synchronize()
            assert_close_rel(got.cpu().numpy(), want)

@pytest.mark.parametrize("q,p", [(8, 2), (4, 4), (8, 8)])
def test_group_scale_decode_kernel_on_wide_outputs_of_more_than_eight_rows(abq, oracle, q, p):
    """9 to 16 rows on outputs of at least 512 tiles of 16 weight rows: the decode kernel's group-scale variant takes two
    tiles per workgroup (the staged rows serve twice the weights); an output whose width is no multiple of 32 and a
    last workgroup with one tile keep working, zero points on both sides."""
    from oracle import quantizer as Q
    rng = np.random.default_rng(8800 + 10 * q + p)
    lo_x, hi_x, lo_w, hi_w = -(1 << (q - 1)), 1 << (q - 1), -(1 << (p - 1)), 1 << (p - 1)
    for (M, N, K) in [(16, 8224, 1152), (12, 8208, 1536), (9, 8200, 2048)]:
        G = K // 128
        x = rng.integers(lo_x, hi_x, (M, K)).astype(np.int32)
        w = rng.integers(lo_w, hi_w, (N, K)).astype(np.int32)
        xs = rng.uniform(0.01, 0.05, M)
        xz = rng.integers(lo_x // 2, hi_x // 2 + 1, M).astype(np.float64)
        wsc = rng.uniform(0.001, 0.02, (N, G))
        wz = rng.integers(lo_w, hi_w, (N, G)).astype(np.float64)
        want = Q.dequant_matmul(x, xs, xz, w, wsc, wz, 128)
        wp = planes_dev(oracle.pack_i32(w, p))
        kw = dict(x_scale=fdev(xs), w_scale=fdev(wsc), group_size=128, w_zero=fdev(wz), x_zero=fdev(xz), x_tiled=True, w_tiled=True,
                  x_group_sums=torch.from_numpy(x.reshape(M, G, 128).sum(axis=2).astype(np.int32)).cuda())
        kw["w_zero_term"] = abq.weight_zero_term(wp, True, kw["w_scale"], kw["w_zero"], 128)
        xt, wt = abq.relayout_planes(planes_dev(oracle.pack_i32(x, q))), abq.relayout_planes(wp)
        g = abq.Gemm(xt, wt, True, out_kind=abq.OUT_F16_SCALED, **kw)
        assert g.strategy == "decode_tiled", (M, N, K, g.strategy)
        got = g.run()
        torch.cuda.synchronize()
        assert_close_rel(got.float().cpu().numpy(), want)


@pytest.mark.parametrize("q,p,act", [(8, 2, False), (4, 4, False), (8, 2, True)])
def test_group_scale_tiles_whose_waves_split_k_are_the_default_on_grids_of_one_round(abq, oracle, q, p, act):
    """Grids of at most one workgroup per compute unit run the tile with two groups of waves that split K inside the
    workgroup: 64x64 while that makes at most 256 workgroups, then 128x64, 128x128 beyond while that does, 64x128 for wide outputs
    of at most 64 rows (activations wider than the weights); an odd number of K tiles (the last trip has one group
    without a tile), zero points on both sides, ragged edges, the fused SiLU gate."""
    from oracle import quantizer as Q
    rng = np.random.default_rng(7100 + 10 * q + p + act)
    lo_x, hi_x, lo_w, hi_w = -(1 << (q - 1)), 1 << (q - 1), -(1 << (p - 1)), 1 << (p - 1)
    cases = [(300, 192, 640, (64, 64, 256)), (300, 3840, 384, (128, 64, 256)), (1040, 2144, 384, (128, 128, 256)),
             (130, 16000, 256, (128, 128, 256))]
    if q > p:
        cases.append((40, 16640, 384, (64, 128, 256)))
    for (M, N, K, tile) in cases:
        G = K // 128
        x = rng.integers(lo_x, hi_x, (M, K)).astype(np.int32)
        w = rng.integers(lo_w, hi_w, (N, K)).astype(np.int32)
        xs = rng.uniform(0.01, 0.05, M)
        xz = rng.integers(lo_x // 2, hi_x // 2 + 1, M).astype(np.float64)
        wsc = rng.uniform(0.001, 0.02, (N, G))
        wz = rng.integers(lo_w, hi_w, (N, G)).astype(np.float64)
        want = Q.dequant_matmul(x, xs, xz, w, wsc, wz, 128)
        if act:  # rows of W come in blocks of 16 gate rows followed by their 16 up rows
            blocks = want.reshape(M, N // 32, 2, 16)
            gate, up = blocks[:, :, 0, :], blocks[:, :, 1, :]
            want = (gate / (1.0 + np.exp(-gate)) * up).reshape(M, N // 2)
        wp = planes_dev(oracle.pack_i32(w, p))
        kw = dict(x_scale=fdev(xs), w_scale=fdev(wsc), group_size=128, w_zero=fdev(wz), x_zero=fdev(xz), x_tiled=True, w_tiled=True,
                  x_group_sums=torch.from_numpy(x.reshape(M, G, 128).sum(axis=2).astype(np.int32)).cuda())
        kw["w_zero_term"] = abq.weight_zero_term(wp, True, kw["w_scale"], kw["w_zero"], 128)
        if act:
            kw["act"] = abq.ACT_SILU_GATE
        xt, wt = abq.relayout_planes(planes_dev(oracle.pack_i32(x, q))), abq.relayout_planes(wp)
        g = abq.Gemm(xt, wt, True, out_kind=abq.OUT_F16_SCALED, **kw)
        c = g.state.cfg
        assert g.strategy == "tiled" and (c.block_m, c.block_n, c.block_k) == tile, (M, N, K, g.config_name)
        got = g.run()
        torch.cuda.synchronize()
        assert_close_rel(got.float().cpu().numpy(), want)


@pytest.mark.parametrize("p,signed_codes", [(2, True), (3, True), (4, True), (2, False), (3, False), (6, True)])
@pytest.mark.parametrize("group_size", [128, 64])
def test_zero_points_folded_into_the_weight_records(abq, oracle, p, signed_codes, group_size):
    """Weights with whole-number zero points as records of code - zero point, one field wider: the GEMM runs the signed
    pair of that width with group scales and no weight zero points, and gives what the zero-point term gives: against
    the dequantised reference, and against the same GEMM on the plain records with the zero points handed in.
    Decode- and prefill-sized calls, activation zero points (whose weight-side term comes from the original weights),
    ragged shapes; zero points that are no whole numbers or push a difference out of the records are reported."""
    from oracle import quantizer as Q
    rng = np.random.default_rng(4000 + 10 * p + signed_codes + group_size)
    q, rb = 8, abq.lib().abq_folded_bits(p)
    assert rb == (4 if p <= 3 else 8)
    lo_w, hi_w = (-(1 << (p - 1)), 1 << (p - 1)) if signed_codes else (0, 1 << p)
    for (M, N, K) in [(4, 96, 512), (40, 200, 640), (300, 130, 1152), (130, 264, 4096)]:
        G = K // group_size
        x = rng.integers(-128, 128, (M, K)).astype(np.int32)
        w = rng.integers(lo_w, hi_w, (N, K)).astype(np.int32)
        xs = rng.uniform(0.01, 0.05, M)
        xz = rng.integers(-64, 65, M).astype(np.float64)
        wsc = rng.uniform(0.001, 0.02, (N, G))
        wz = rng.integers(lo_w, hi_w + (0 if signed_codes else 1), (N, G)).astype(np.float64)
        want = Q.dequant_matmul(x, xs, xz, w, wsc, wz, group_size)
        wp = planes_dev(oracle.pack_i32(w, p))
        folded = abq.relayout_planes_folded(wp, fdev(wz), group_size, signed_codes)
        assert folded.shape == (K // 128, N, rb, 4)
        xsum = torch.from_numpy(x.reshape(M, G, group_size).sum(axis=2).astype(np.int32)).cuda()
        term = abq.weight_zero_term(wp, signed_codes, fdev(wsc), fdev(wz), group_size)
        xt = abq.relayout_planes(planes_dev(oracle.pack_i32(x, q)))
        g = abq.Gemm(xt, folded, True, out_kind=abq.OUT_F16_SCALED, x_tiled=True, w_tiled=True, x_scale=fdev(xs), w_scale=fdev(wsc),
                     group_size=group_size, x_zero=fdev(xz), w_zero_term=term)
        assert (g.state.cfg.x_bits, g.state.cfg.w_bits) == (8, rb)
        got = g.run().float().cpu().numpy()
        assert_close_rel(got, want)
        if signed_codes and p in (2, 4):  # the same through the zero-point term, on the weights' own records
            ref = abq.Gemm(xt, abq.relayout_planes(wp), True, out_kind=abq.OUT_F16_SCALED, x_tiled=True, w_tiled=True, x_scale=fdev(xs),
                           w_scale=fdev(wsc), group_size=group_size, x_zero=fdev(xz), w_zero=fdev(wz), x_group_sums=xsum,
                           w_zero_term=term).run().float().cpu().numpy()
            assert_close_rel(got, ref)
    wz_bad = wz.copy()
    wz_bad[3, 1] += 0.25
    with pytest.raises(ValueError):
        abq.relayout_planes_folded(wp, fdev(wz_bad), group_size, signed_codes)
    wz_bad = wz.copy()
    wz_bad[5, 0] = -(1 << rb)
    with pytest.raises(ValueError):
        abq.relayout_planes_folded(wp, fdev(wz_bad), group_size, signed_codes)


@pytest.mark.parametrize("q,p,signed_codes", [(4, 4, True), (4, 2, True), (3, 3, True), (4, 4, False), (4, 2, False)])
def test_zero_points_folded_into_fp6_records(abq, oracle, q, p, signed_codes):
    """The same on the FP6 route: FP6 records of code - zero point (magnitudes of at most 16), a signed GEMM without
    weight zero points under the pair's own widths; unsigned codes and activations ride along as the signed numbers
    they are (their records hold the values).  Against the
    dequantised reference; a difference of magnitude 17 is reported."""
    from oracle import quantizer as Q
    rng = np.random.default_rng(4600 + 10 * q + p + signed_codes)
    lo_w, hi_w = (-(1 << (p - 1)), 1 << (p - 1)) if signed_codes else (0, 1 << p)
    lo_x, hi_x = (-(1 << (q - 1)), 1 << (q - 1)) if signed_codes else (0, 1 << q)
    for (M, N, K) in [(40, 96, 512), (300, 200, 640), (130, 264, 4096), (8, 64, 1152)]:
        G = K // 128
        x = rng.integers(lo_x, hi_x, (M, K)).astype(np.int32)
        w = rng.integers(lo_w, hi_w, (N, K)).astype(np.int32)
        xs = rng.uniform(0.01, 0.05, M)
        xz = rng.integers(lo_x // 2, hi_x // 2 + 1, M).astype(np.float64)
        wsc = rng.uniform(0.001, 0.02, (N, G))
        wz = rng.integers(lo_w, hi_w + (0 if signed_codes else 1), (N, G)).astype(np.float64)
        want = Q.dequant_matmul(x, xs, xz, w, wsc, wz, 128)
        wp, xp = planes_dev(oracle.pack_i32(w, p)), planes_dev(oracle.pack_i32(x, q))
        term = abq.weight_zero_term(wp, signed_codes, fdev(wsc), fdev(wz), 128)
        wf = abq.relayout_planes_fp6_folded(wp, fdev(wz), 128, signed_codes)
        g = abq.Gemm(abq.relayout_planes_fp6(xp, signed_codes), wf, True, out_kind=abq.OUT_F16_SCALED, x_fp6=q, w_fp6=p,
                     x_scale=fdev(xs), w_scale=fdev(wsc), group_size=128, x_zero=fdev(xz), w_zero_term=term)
        assert g.strategy == "fp6"
        assert_close_rel(g.run().float().cpu().numpy(), want)
    wz_bad = wz.copy()
    wz_bad[2, 0] = lo_w - 17.0  # code - zero point reaches 17
    with pytest.raises(ValueError):
        abq.relayout_planes_fp6_folded(wp, fdev(wz_bad), 128, signed_codes)


@pytest.mark.parametrize("q,p,fp6", [(8, 2, False), (8, 3, False), (8, 4, False), (8, 7, False), (4, 4, True), (4, 2, True), (3, 3, True)])
@pytest.mark.parametrize("signed_codes", [True, False])
def test_folded_records_accept_exactly_what_they_can_hold(abq, oracle, q, p, fp6, signed_codes):
    """Zero points chosen from the weights so that the largest or the smallest difference of a group lands on the
    last value the records hold (two's complement of the folded width; magnitude 16 on the FP6 records): accepted, and
    the GEMM agrees with the dequantised reference.  One group moved one step further, at either end: reported."""
    from oracle import quantizer as Q
    rng = np.random.default_rng(5200 + 10 * q + p + 2 * fp6 + signed_codes)
    M, N, K, gs = 24, 72, 640, 128
    G = K // gs
    lo_w, hi_w = (-(1 << (p - 1)), 1 << (p - 1)) if signed_codes else (0, 1 << p)
    lo_x, hi_x = (-(1 << (q - 1)), 1 << (q - 1)) if signed_codes or not fp6 else (0, 1 << q)
    rb = abq.lib().abq_folded_bits(p)
    lim_lo, lim_hi = (-16, 16) if fp6 else (-(1 << (rb - 1)), (1 << (rb - 1)) - 1)
    x = rng.integers(lo_x, hi_x, (M, K)).astype(np.int32)
    w = rng.integers(lo_w, hi_w, (N, K)).astype(np.int32)
    wg = w.reshape(N, G, gs)
    z_least, z_most = wg.max(axis=2) - lim_hi, wg.min(axis=2) - lim_lo  # the zero points a group can take
    wz = np.where(rng.integers(0, 2, (N, G)) == 0, z_least, z_most).astype(np.float64)
    xs, wsc = rng.uniform(0.01, 0.05, M), rng.uniform(0.001, 0.02, (N, G))
    xz = rng.integers(lo_x // 2, hi_x // 2 + 1, M).astype(np.float64)
    wp, xp = planes_dev(oracle.pack_i32(w, p)), planes_dev(oracle.pack_i32(x, q))
    fold = abq.relayout_planes_fp6_folded if fp6 else abq.relayout_planes_folded
    wf = fold(wp, fdev(wz), gs, signed_codes)
    kw = dict(out_kind=abq.OUT_F16_SCALED, x_scale=fdev(xs), w_scale=fdev(wsc), group_size=gs, x_zero=fdev(xz),
              w_zero_term=abq.weight_zero_term(wp, signed_codes, fdev(wsc), fdev(wz), gs))
    if fp6:
        g = abq.Gemm(abq.relayout_planes_fp6(xp, signed_codes), wf, True, x_fp6=q, w_fp6=p, **kw)
    else:
        g = abq.Gemm(abq.relayout_planes(xp), wf, True, x_tiled=True, w_tiled=True, **kw)
    assert_close_rel(g.run().float().cpu().numpy(), Q.dequant_matmul(x, xs, xz, w, wsc, wz, gs))
    for (i, j, beyond) in [(3, 1, z_least[3, 1] - 1), (70, 4, z_most[70, 4] + 1)]:
        wz_bad = wz.copy()
        wz_bad[i, j] = beyond
        with pytest.raises(ValueError):
            fold(wp, fdev(wz_bad), gs, signed_codes)


@pytest.mark.parametrize("M,K", [(200, 4096), (130, 4608), (136, 8192)])
@pytest.mark.parametrize("q,p,fp6", [(8, 2, False), (4, 4, False), (4, 4, True)])
def test_zero_points_over_whole_chunks_of_groups(abq, oracle, M, K, q, p, fp6):
    """The weight zero points on the prefill kernels when the groups of a row come in whole chunks of 32 that start
    on 16-byte boundaries (32, 36 = 32 + 4 and 64 groups; token counts that are and are not multiples of 4):
    the 16-byte loads of the group sums, scales and zero points, and the row scales as 16-byte loads."""
    from oracle import quantizer as Q
    rng = np.random.default_rng(M + K + q)
    N, G = 264, K // 128
    lo_x, hi_x, lo_w, hi_w = -(1 << (q - 1)), 1 << (q - 1), -(1 << (p - 1)), 1 << (p - 1)
    x = rng.integers(lo_x, hi_x, (M, K)).astype(np.int32) + (rng.integers(0, hi_x // 2, (M, 1)) if q == 8 else 0)
    x = np.clip(x, lo_x, hi_x - 1).astype(np.int32)  # rows with a mean: group sums of several thousand
    w = rng.integers(lo_w, hi_w, (N, K)).astype(np.int32)
    xs = rng.uniform(0.01, 0.05, M)
    xz = rng.integers(lo_x // 2, hi_x // 2 + 1, M).astype(np.float64)
    wsc = rng.uniform(0.001, 0.02, (N, G))
    wz = rng.integers(lo_w, hi_w, (N, G)).astype(np.float64) + rng.uniform(-0.5, 0.5, (N, G))  # not whole numbers
    want = Q.dequant_matmul(x, xs, xz, w, wsc, wz, 128)
    wp, xp = planes_dev(oracle.pack_i32(w, p)), planes_dev(oracle.pack_i32(x, q))
    kw = dict(x_scale=fdev(xs), w_scale=fdev(wsc), group_size=128, w_zero=fdev(wz), x_zero=fdev(xz),
              x_group_sums=torch.from_numpy(x.reshape(M, G, 128).sum(axis=2).astype(np.int32)).cuda())
    kw["w_zero_term"] = abq.weight_zero_term(wp, True, kw["w_scale"], kw["w_zero"], 128)
    if fp6:
        g = abq.Gemm(abq.relayout_planes_fp6(xp, True), abq.relayout_planes_fp6(wp, True), True, out_kind=abq.OUT_F16_SCALED,
                     x_fp6=q, w_fp6=p, **kw)
    else:
        g = abq.Gemm(abq.relayout_planes(xp), abq.relayout_planes(wp), True, out_kind=abq.OUT_F16_SCALED, x_tiled=True,
                     w_tiled=True, **kw)
    got = g.run()
    torch.cuda.synchronize()
    assert g.strategy in ("tiled", "fp6"), g.strategy
    assert_close_rel(got.cpu().numpy(), want)


@pytest.mark.parametrize("q,p,signed", [(4, 4, True), (4, 4, False), (5, 5, True), (4, 2, True), (3, 3, False)])
def test_group_scales_on_the_fp6_route(abq, oracle, q, p, signed):
    """Groups of 128 with zero points on both sides through the FP6 matrix-core kernel: the library's own
    tile choice and every tile it is built for, operands as FP6 records or converted from planes."""
    from oracle import quantizer as Q
    rng = np.random.default_rng(300 + 10 * q + p + signed)
    tiles = [None] + [c for c in abq.native_configs(q, p, signed)
                      if c.nstage == 5 and (c.block_m, c.block_n, c.warp_m) in ((256, 128, 64), (128, 128, 64), (128, 64, 64))]
    assert len(tiles) == 4
    lo_x, hi_x = (-(1 << (q - 1)), 1 << (q - 1)) if signed else (0, 1 << q)
    lo_w, hi_w = (-(1 << (p - 1)), 1 << (p - 1)) if signed else (0, 1 << p)
    for (M, N, K) in [(300, 200, 640), (70, 330, 256), (129, 72, 128)]:
        G = K // 128
        x = rng.integers(lo_x, hi_x, (M, K)).astype(np.int32)
        w = rng.integers(lo_w, hi_w, (N, K)).astype(np.int32)
        xs = rng.uniform(0.01, 0.05, M)
        xz = rng.integers(lo_x // 2, hi_x // 2 + 1, M).astype(np.float64)
        wsc = rng.uniform(0.001, 0.02, (N, G))
        wz = rng.integers(lo_w, hi_w, (N, G)).astype(np.float64)
        want = Q.dequant_matmul(x, xs, xz, w, wsc, wz, 128)
        xp, wp = planes_dev(oracle.pack_i32(x, q)), planes_dev(oracle.pack_i32(w, p))
        kw = dict(x_scale=fdev(xs), w_scale=fdev(wsc), group_size=128, w_zero=fdev(wz), x_zero=fdev(xz),
                  x_group_sums=torch.from_numpy(x.reshape(M, G, 128).sum(axis=2).astype(np.int32)).cuda())
        kw["w_zero_term"] = abq.weight_zero_term(wp, signed, kw["w_scale"], kw["w_zero"], 128)
        xf, wf = abq.relayout_planes_fp6(xp, signed), abq.relayout_planes_fp6(wp, signed)
        for cfg in tiles:
            g = abq.Gemm(xf, wf, signed, cfg=cfg, out_kind=abq.OUT_F16_SCALED, x_fp6=q, w_fp6=p, **kw)
            assert g.strategy == "fp6" and g.state.group_size == 128
            got = g.run()
            torch.cuda.synchronize()
            assert_close_rel(got.cpu().numpy(), want)
        # activations still as planes: converted into the caller's workspace inside the call
        ws = torch.empty((K // 128) * M * 96, dtype=torch.uint8, device="cuda")
        g = abq.Gemm(xp, wf, signed, out_kind=abq.OUT_F16_SCALED, w_fp6=p, workspace=ws, **kw)
        assert g.strategy == "fp6"
        assert_close_rel(g.run().cpu().numpy(), want)
    # groups of 64 have no FP6 build
    with pytest.raises(abq.AbqError):
        abq.Gemm(xf, wf, signed, out_kind=abq.OUT_F16_SCALED, x_fp6=q, w_fp6=p, x_scale=kw["x_scale"],
                 w_scale=fdev(rng.uniform(0.001, 0.02, (N, 2 * G))), group_size=64)


# ------------------------------------------------------------------ BASELINE.json configs[4]

LAYER_LINEARS = [("qkv", 12288, 4096), ("o", 4096, 4096), ("gate_up", 2 * 11008, 4096), ("down", 4096, 11008)]


def _layer_linear(abq, oracle, name, N, K, tokens, x_symmetric, seed, sample_rows, bit_balance=False, full_check=False):
    """One W2A8 linear: fp16 weights N(0, 0.02) quantised to 2 bits per (channel, group of 128),
    fp16 activations quantised per token on the device; checks `sample_rows` output rows.
    bit_balance: the reference's default 2-bit weight quantiser (five levels, quantizer.py:66-68,169-171),
    whose codes take three planes."""
    from oracle import quantizer as Q
    rng = np.random.default_rng(seed)
    w = rng.normal(0, 0.02, (N, K)).astype(np.float16)
    if bit_balance:
        w_codes, w_scale, w_zero, w_planes = Q.group_affine_codes_bit_balance(w, 2, 128)
    else:
        (w_codes, w_scale, w_zero), w_planes = Q.group_affine_codes(w, 2, 128), 2
    wp = planes_dev(oracle.pack_i32(w_codes, w_planes))
    wt = abq.relayout_planes(wp)
    ws_d, wz_d = fdev(w_scale), fdev(w_zero)

    xg = torch.Generator(device="cuda").manual_seed(seed)
    x = torch.randn((tokens, K), generator=xg, device="cuda", dtype=torch.float32)
    x[:, ::97] *= 8.0  # a few outlier channels, as LLM activations have
    x = x.to(torch.float16)
    xt, xs, xz, sums = abq.quant_pack_f16(x, 8, symmetric=x_symmetric, tiled=True, group_size=128)
    kw = dict(x_scale=xs, w_scale=ws_d, group_size=128, w_zero=wz_d, x_group_sums=sums, x_tiled=True, w_tiled=True)
    if not x_symmetric:
        kw.update(x_zero=xz, w_zero_term=abq.weight_zero_term(wp, True, ws_d, wz_d, 128))
    got = run_grouped(abq, xt, wt, True, **kw)
    got2 = None
    if tokens <= 16:  # decode-sized: also the decode kernel's group-scale variant on plane operands
        xp, xs2, xz2, sums2 = abq.quant_pack_f16(x, 8, symmetric=x_symmetric, tiled=False, group_size=128)
        kw2 = dict(kw, x_scale=xs2, x_group_sums=sums2, x_tiled=False, w_tiled=False)
        if not x_symmetric:
            kw2.update(x_zero=xz2)
        got2 = run_grouped(abq, xp, wp, True, strategy="decode", **kw2)

    rows = np.sort(rng.choice(tokens, size=min(sample_rows, tokens), replace=False))
    x_rows = x[torch.from_numpy(rows).cuda()].cpu().numpy()
    codes, scale, zero = Q.per_token_codes_f32(x_rows, 8, x_symmetric)
    assert np.array_equal(xs.cpu().numpy()[rows], scale)
    want = Q.dequant_matmul(codes, scale, zero, w_codes, w_scale, w_zero, 128)
    assert_close_rel(got[rows], want)
    if got2 is not None:
        assert_close_rel(got2[rows], want)
    if full_check:
        # every row, on the GPU in fp64: the codes the kernel itself packed (read back from its planes, which hold the
        # same codes as the K-tiled records: the sampled rows above pin them to the restated quantiser), dequantised,
        # times the dequantised weights; every product and partial sum is far inside fp64's exact range
        xp_d, xs_p, xz_p, _ = abq.quant_pack_f16(x, 8, symmetric=x_symmetric, tiled=False, group_size=128)
        assert torch.equal(xs_p, xs)
        shifts = torch.arange(31, -1, -1, device="cuda", dtype=torch.int32)
        codes_d = torch.zeros((tokens, K), dtype=torch.int32, device="cuda")
        for b in range(8):
            bits = ((xp_d[b].unsqueeze(-1) >> shifts) & 1).reshape(tokens, K)
            codes_d += bits * (-(1 << b) if b == 7 else (1 << b))  # two's complement: the top plane is negative
        zero_d = xz_p.double().unsqueeze(1) if xz_p is not None else 0.0
        x_dq = (codes_d.double() - zero_d) * xs.double().unsqueeze(1)
        w_dq = ((torch.from_numpy(w_codes).cuda().double().reshape(N, K // 128, 128) - wz_d.double().unsqueeze(2)) *
                ws_d.double().unsqueeze(2)).reshape(N, K)
        want_d = x_dq @ w_dq.T
        got_d = torch.from_numpy(got).cuda().double()
        rms = torch.sqrt(torch.mean(want_d ** 2))
        err = torch.abs(got_d - want_d)
        assert bool(torch.all(torch.isfinite(got_d)))
        assert bool(torch.all(err <= REL_TOL * torch.abs(want_d) + 1e-3 * rms)), float((err / (torch.abs(want_d) + 1e-1 * rms)).max())
        assert float(torch.linalg.norm(got_d - want_d)) <= 2e-3 * float(torch.linalg.norm(want_d))
        del x_dq, w_dq, want_d, got_d, err, codes_d
    # and the quantised result tracks the unquantised fp16 linear as 2-bit weights allow: the
    # dequantised weights are within scale/2 of the originals, so this is only a sanity bound
    full = x_rows.astype(np.float64) @ w.astype(np.float64).T
    assert np.linalg.norm(want - full) < 0.7 * np.linalg.norm(full)


@pytest.mark.parametrize("name,N,K", LAYER_LINEARS)
@pytest.mark.parametrize("x_symmetric", [True, False])
def test_config4_decoder_layer_linears_batch1(abq, oracle, name, N, K, x_symmetric):
    _layer_linear(abq, oracle, name, N, K, 1024, x_symmetric, seed=len(name) + N % 97, sample_rows=48)


@pytest.mark.parametrize("tokens", [8, 1024])
@pytest.mark.parametrize("x_symmetric", [True, False])
def test_config4_linear_with_bit_balanced_2bit_weights(abq, oracle, tokens, x_symmetric):
    """The O projection with the reference's default 2-bit weight quantiser (bit balance: five levels, three planes):
    W3A8 with group-128 scales and zero points against the fp64 matmul of the dequantised operands."""
    _layer_linear(abq, oracle, "o", 4096, 4096, tokens, x_symmetric, seed=91 + tokens, sample_rows=48, bit_balance=True)


@pytest.mark.parametrize("name,N,K", LAYER_LINEARS)
def test_config4_decoder_layer_linears_batch16(abq, oracle, name, N, K):
    _layer_linear(abq, oracle, name, N, K, 16 * 1024, True, seed=7 + len(name), sample_rows=32, full_check=True)
