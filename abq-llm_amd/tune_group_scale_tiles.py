#!/usr/bin/env python3
"""Times every tile of the group-scale prefill kernels on one shape grid: the counterpart, for GEMMs with
group scales and zero points (fp16 out), of what engine/test_any_mma does for the int32 GEMMs.

    python3 tune_group_scale_tiles.py X_BITS W_BITS [--group 128] [--m 256,512,...] [--nk 4096x4096,...] [--fp6]

Operands are random bit patterns in the prepared (K-tiled) layout, scales and zero points random; each
tile is picked by its tuple, run five times after a warm-up and timed with HIP events.  One line per
(shape, tile): BM BN warp_M warp_N us TOPS lds.  --fp6: the operands are FP6 records and the tiles those
of the FP6 route (pairs of at most 5 bits).
"""
import argparse
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import abq_gemm as abq  # noqa: E402


def random_planes(shape):
    return torch.randint(-2 ** 31, 2 ** 31 - 1, shape, dtype=torch.int64, device="cuda").to(torch.int32)


def time_us(gemm, reps=5):
    gemm.run()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        gemm.run()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / reps


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("x_bits", type=int)
    ap.add_argument("w_bits", type=int)
    ap.add_argument("--group", type=int, default=128)
    ap.add_argument("--m", default="256,512,1024,2048,4096,16384")
    ap.add_argument("--nk", default="4096x4096,11008x4096,4096x11008,12288x4096,22016x4096")
    ap.add_argument("--fp6", action="store_true")
    args = ap.parse_args()
    q, p, gs = args.x_bits, args.w_bits, args.group
    torch.cuda.set_device(0)
    tiles = [c for c in abq.native_configs(q, p, True) if c.nstage == (5 if args.fp6 else 4) and c.warp_k == 128]
    if args.fp6:
        prepare, layout = (lambda planes: abq.relayout_planes_fp6(planes, True)), (lambda bits: dict(x_fp6=q, w_fp6=p))
    else:
        prepare, layout = abq.relayout_planes, (lambda bits: dict(x_tiled=True, w_tiled=True))
    for nk in args.nk.split(","):
        N, K = (int(v) for v in nk.split("x"))
        G = K // gs
        wt = prepare(random_planes((p, N, K // 32)))
        w_scale = torch.rand((N, G), device="cuda") * 0.01 + 0.001
        w_zero = torch.randint(-2, 2, (N, G), device="cuda").float()
        for M in (int(v) for v in args.m.split(",")):
            xt = prepare(random_planes((q, M, K // 32)))
            x_scale = torch.rand(M, device="cuda") * 0.01 + 0.001
            sums = torch.randint(-1000, 1000, (M, G), device="cuda", dtype=torch.int32)
            out = torch.empty((M, N), dtype=torch.float16, device="cuda")
            print("== M=%d N=%d K=%d W%dA%d group %d%s" % (M, N, K, p, q, gs, " FP6" if args.fp6 else ""), flush=True)
            seen = set()
            for cfg in tiles:
                try:
                    g = abq.Gemm(xt, wt, True, cfg=cfg, out=out, out_kind=abq.OUT_F16_SCALED, x_scale=x_scale,
                                 w_scale=w_scale, group_size=gs, w_zero=w_zero, x_group_sums=sums, **layout(q))
                except abq.AbqError:
                    continue  # no group-scale build of this tile
                c = g.state.cfg
                key = (c.block_m, c.block_n, c.warp_m, c.warp_n, g.state.shared_mem_size)
                if key in seen:
                    continue
                seen.add(key)
                us = time_us(g)
                print("%d %d %d %d %.1f us %.0f TOPS lds=%d" % (c.block_m, c.block_n, c.warp_m, c.warp_n, us,
                                                               2.0 * M * N * K / us / 1e6, g.state.shared_mem_size), flush=True)
            del xt, out


if __name__ == "__main__":
    main()
