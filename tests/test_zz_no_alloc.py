"""abq_gemm_exec_static: the entry point that allocates nothing (operand conversions go into a static device
array inside the library) against abq_gemm_exec with a caller workspace, through the C ABI."""
import ctypes

import numpy as np
import pytest

torch = pytest.importorskip("torch")

pytestmark = pytest.mark.gpu


def _planes(torch_, shape, seed):
    g = torch_.Generator(device="cuda").manual_seed(seed)
    lo = torch_.randint(0, 1 << 16, shape, dtype=torch_.int32, device="cuda", generator=g)
    hi = torch_.randint(0, 1 << 16, shape, dtype=torch_.int32, device="cuda", generator=g)
    return lo | (hi << 16)


def test_exec_static_matches_exec_with_workspace(abq):
    if not torch.cuda.is_available():
        pytest.fail("marked gpu but no GPU is visible")
    limit = 32 << 20
    # two calls in a row, the second with a smaller input; then the FP6 route (other conversion kernels)
    cases = [(8, 2, True, 1024, 768, 2048, False), (8, 2, True, 40, 200, 384, False), (4, 4, True, 300, 256, 1024, True)]
    for (q, p, signed, M, N, K, fp6) in cases:
        xd = _planes(torch, (q, M, K // 32), 10 * M + q)
        wd = _planes(torch, (p, N, K // 32), 10 * N + p)
        if fp6:
            wprep, kw = abq.relayout_planes_fp6(wd, signed), dict(w_fp6=p)
        else:
            wprep, kw = abq.relayout_planes(wd), dict(w_tiled=True)
        probe = abq.Gemm(xd, wprep, signed, **kw)
        need = probe.workspace_bytes
        assert 0 < need <= limit
        ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        want = abq.Gemm(xd, wprep, signed, workspace=ws, **kw).run().clone()
        out = torch.full((M, N), -7, dtype=torch.int32, device="cuda")
        g = abq.Gemm(xd, wprep, signed, out=out, **kw)  # no workspace attached
        with pytest.raises(abq.AbqError):
            g.run()  # abq_gemm_exec needs one
        got = g.run_static()
        torch.cuda.synchronize()
        assert torch.equal(got, want), (q, p, M, N, K, fp6)
    # a state that needs no conversion runs as abq_gemm_exec does
    xd, wd = _planes(torch, (8, 4, 32), 1), _planes(torch, (2, 64, 32), 2)
    g = abq.Gemm(xd, wd, True)
    assert g.strategy == "decode"
    assert torch.equal(g.run().clone(), g.run_static())
    # beyond the static array's size: refused, nothing launched
    M, K = 4096, 11008
    xd = _planes(torch, (8, M, K // 32), 3)
    wt = abq.relayout_planes(_planes(torch, (2, 128, K // 32), 4))
    g = abq.Gemm(xd, wt, True, w_tiled=True)
    assert g.workspace_bytes > limit
    with pytest.raises(abq.AbqError) as ei:
        g.run_static()
    assert ei.value.status == abq.ABQ_ERR_TOO_LARGE
