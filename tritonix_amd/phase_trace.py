"""Where one launch of the 256x256 tile kernels spends its time, workgroup by workgroup.

    python -m tritonix_amd.build -D TNX_PHASE_TRACE --only bf16:256:256:64:4:2,bf16:256:256:64:8:2,i8:256:256:128:4:2 \\
        --out /tmp/libtritonix_phase.so
    python -m tritonix_amd.phase_trace /tmp/libtritonix_phase.so

A library built with ``TNX_PHASE_TRACE`` makes wave 0 of every workgroup write four 100 MHz timestamps (start,
first slab landed, last MFMA issued, last store issued) and its CU's hardware ids into the workspace of an uncut
launch.  This script launches the three MFMA-bound benchmark problems (8192^3 bf16, 8192^3 int8, the gated
4096x28672x4096) through the C ABI of that library, on the benchmark's operands and on all-zero ones, and prints per
round of workgroups on a CU the mean time of each phase and the gap between one workgroup's last store and its
successor's first instruction.  The ordinary library carries none of this.
"""
import collections
import ctypes
import sys

import torch

from . import _C

CASES = [("C2 bf16 8192^3", torch.bfloat16, _C.BF16, _C.BF16, 8192, 8192, 8192, _C.EPI_NONE, (256, 256, 64, 4, 2)),
         ("C5 int8 8192^3", torch.int8, _C.I8, _C.I32, 8192, 8192, 8192, _C.EPI_NONE, (256, 256, 128, 4, 2)),
         ("C4 GLU 4096x28672x4096", torch.bfloat16, _C.BF16, _C.BF16, 4096, 28672, 4096, _C.EPI_GLU_SILU, (256, 256, 64, 8, 2))]


def operands(tdt, m, n, k, zeros, dev):
    g = torch.Generator("cpu").manual_seed(1)
    if tdt == torch.int8:
        a = torch.randint(-127, 128, (m, k), generator=g, dtype=torch.int8)
        b = torch.randint(-127, 128, (k, n), generator=g, dtype=torch.int8)
    else:
        a = (torch.randn(m, k, generator=g) / k ** 0.5).to(tdt)
        b = (torch.randn(k, n, generator=g) * 0.02).to(tdt)
    if zeros:
        a.zero_(), b.zero_()
    return a.to(dev), b.to(dev)


def main(path):
    lib = ctypes.CDLL(path)
    lib.tnx_gemm.argtypes = [ctypes.POINTER(_C.GemmArgs)]
    lib.tnx_gemm.restype = ctypes.c_int
    dev = torch.device("cuda", 0)
    mean = lambda v: sum(v) / max(1, len(v))
    for name, tdt, idt, odt, m, n, k, epi, (bm, bn, bk, nw, st) in CASES:
        for zeros in (False, True):
            a, b = operands(tdt, m, n, k, zeros, dev)
            nc = n // 2 if epi != _C.EPI_NONE else n
            c = torch.zeros((m, nc), dtype=torch.int32 if tdt == torch.int8 else tdt, device=dev)
            ntile = (m // bm) * (n // bn)
            ws = torch.zeros((ntile * 8,), dtype=torch.int64, device=dev)
            g = _C.GemmArgs()
            g.a, g.b, g.c = a.data_ptr(), b.data_ptr(), c.data_ptr()
            g.m, g.n, g.k = m, n, k
            g.stride_am, g.stride_ak, g.stride_bk, g.stride_bn, g.stride_cm, g.stride_cn = k, 1, n, 1, nc, 1
            g.in_dtype, g.out_dtype = idt, odt
            g.block_m, g.block_n, g.block_k, g.num_warps, g.num_stages, g.group_m = bm, bn, bk, nw, st, 8
            g.split_k, g.epilogue, g.schedule = 1, epi, _C.SCHED_SUPERBLOCK
            g.stream = torch.cuda.current_stream().cuda_stream
            for _ in range(60):                                  # untraced: clocks and caches as in a steady run
                _C.raise_for_status(lib.tnx_gemm(ctypes.byref(g)), g)
            g.workspace, g.workspace_bytes = ws.data_ptr(), ws.numel() * 8
            _C.raise_for_status(lib.tnx_gemm(ctypes.byref(g)), g)
            torch.cuda.synchronize()
            t = ws.cpu().view(ntile, 8)
            if int(t[:, 0].min()) == 0:
                raise SystemExit(f"{path} was not built with -D TNX_PHASE_TRACE")
            t0 = int(t[:, 0].min())
            per_cu = collections.defaultdict(list)
            for i in range(ntile):
                hw, xcc = int(t[i, 4]), int(t[i, 5]) & 0xF
                cu = (xcc, (hw >> 13) & 7, (hw >> 8) & 15)          # XCC, shader engine, CU
                per_cu[cu].append([(int(t[i, x]) - t0) / 100.0 for x in range(4)])
            rounds, gaps = collections.defaultdict(list), []
            for lst in per_cu.values():
                lst.sort()
                for j, r in enumerate(lst):
                    rounds[j].append(r)
                    if j:
                        gaps.append(r[0] - lst[j - 1][3])
            every = [r for lst in per_cu.values() for r in lst]
            print(f"{name}, {'zero' if zeros else 'benchmark'} operands: {len(per_cu)} CUs, {ntile} workgroups, "
                  f"last store at {max(r[3] for r in every):.1f} us")
            print(f"   all rounds: first slab {mean([r[1] - r[0] for r in every]):.2f} us | K loop "
                  f"{mean([r[2] - r[1] for r in every]):.2f} (min {min(r[2] - r[1] for r in every):.2f}, max "
                  f"{max(r[2] - r[1] for r in every):.2f}) | epilogue {mean([r[3] - r[2] for r in every]):.2f} | "
                  f"gap to the next workgroup {mean(gaps):.2f} (max {max(gaps):.2f})")
            for j in sorted(rounds):
                rs = rounds[j]
                print(f"   round {j}: starts {min(r[0] for r in rs):.1f}..{max(r[0] for r in rs):.1f}  first slab "
                      f"{mean([r[1] - r[0] for r in rs]):.2f}  K loop {mean([r[2] - r[1] for r in rs]):.2f}  epilogue "
                      f"{mean([r[3] - r[2] for r in rs]):.2f}  ends {min(r[3] for r in rs):.1f}..{max(r[3] for r in rs):.1f}",
                      flush=True)


if __name__ == "__main__":
    if len(sys.argv) != 2:
        raise SystemExit(__doc__)
    main(sys.argv[1])
