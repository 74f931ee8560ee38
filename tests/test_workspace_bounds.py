"""Host-side bounds of the split-K scratch, for every built tile kernel and a grid of problems.

The device code addresses the workspace as
    counters:  word  ctile                                     (ctile = index of a cut tile, < cut tiles)
    slices:    WS_COUNTER_BYTES + split * slice_stride + (ctile * waves + wave) * wave_bytes
                                + (row_block * groups + group) * 1024 + lane * 16 .. + 16
with slice_stride = cut_tiles * block_m * block_n * 4 and wave_bytes = wave_tile_m * wave_tile_n * 4
(gemm_tile.h, end of gemm_tile_kernel and splitk_arrive).  This test recomputes the largest byte and the
largest counter index the kernel can touch from those formulas, independently of capi.hip, and requires
them to lie inside what tnx_gemm_workspace_bytes asks the caller for; it also restates the grid size.
No launch, no GPU."""
import ctypes
import itertools

import pytest

from tritonix_amd import _C

COUNTER_BYTES = 65536
DT = {"f16": _C.F16, "bf16": _C.BF16, "i8": _C.I8}


def built_tiles():
    out = []
    for name in _C.kernel_names():
        parts = name.split()
        out.append((parts[0], *(int(v) for v in parts[1:6])))
    return out


def wave_tile(bm, bn, nw):
    wgm = 2 if nw == 4 else (4 if bm > bn else 2)
    return bm // wgm, bn // (nw // wgm)


def cdiv(a, b):
    return -(-a // b)


def make(dt, bm, bn, bk, nw, st, m, n, k, split_k, tail):
    g = _C.GemmArgs()
    g.m, g.n, g.k = m, n, k
    g.stride_am, g.stride_ak, g.stride_bk, g.stride_bn, g.stride_cm, g.stride_cn = k, 1, n, 1, n, 1
    g.in_dtype = DT[dt]
    g.out_dtype = _C.I32 if dt == "i8" else DT[dt]
    g.block_m, g.block_n, g.block_k, g.group_m = bm, bn, bk, 8
    g.split_k, g.tail_tiles, g.num_stages, g.num_warps = split_k, tail, st, nw
    return g


PROBLEMS = [(1, 8, 64), (16, 4096, 14336), (100, 264, 200), (512, 2048, 8192), (6144, 6144, 6144), (8192, 8192, 8192),
            (4096, 28672, 4096), (300, 40000, 128)]


def test_every_built_tile_stays_inside_its_workspace():
    lib = _C.load()
    tiles = built_tiles()
    assert len(tiles) == lib.tnx_kernel_count() and len(tiles) > 100
    checked = 0
    for (dt, bm, bn, bk, nw, st), (m, n, k), split_k, tail in itertools.product(tiles, PROBLEMS, (2, 3, 8, 16),
                                                                                (0, 1, 64, 10 ** 6)):
        g = make(dt, bm, bn, bk, nw, st, m, n, k, split_k, tail)
        status = lib.tnx_gemm_supported(ctypes.byref(g))
        tiles_total = cdiv(m, bm) * cdiv(n, bn)
        ncut = tail if 0 < tail < tiles_total else tiles_total
        if status != _C.OK:
            # the only size-related refusals: more cut tiles than counters, or slices past 32-bit offsets
            if status == _C.E_UNSUPPORTED and (ncut > COUNTER_BYTES // 4 or
                                               COUNTER_BYTES + split_k * ncut * bm * bn * 4 >= 1 << 32):
                continue
            # anything else must be a layout refusal (DMA-only tile, ragged K): not a workspace matter
            assert status == _C.E_UNSUPPORTED, (dt, bm, bn, bk, nw, st, m, n, k, split_k, tail, status)
            continue
        need = lib.tnx_gemm_workspace_bytes(ctypes.byref(g))
        wtm, wtn = wave_tile(bm, bn, nw)
        wave_bytes = wtm * wtn * 4
        slice_stride = ncut * bm * bn * 4
        # largest values of every index the kernel forms
        ctile, wave, split = ncut - 1, nw - 1, split_k - 1
        last_byte = COUNTER_BYTES + split * slice_stride + (ctile * nw + wave) * wave_bytes + wave_bytes
        assert last_byte <= need, (dt, bm, bn, bk, nw, st, m, n, k, split_k, tail)
        assert last_byte == need                               # and nothing is asked for beyond it
        assert ctile < COUNTER_BYTES // 4 and (ctile + 1) * 4 <= COUNTER_BYTES
        assert split_k * slice_stride + COUNTER_BYTES < 1 << 32  # 32-bit slice offsets cannot wrap
        # grid: whole tiles once, cut tiles split_k times
        assert (tiles_total - ncut) + ncut * split_k < 1 << 31
        checked += 1
    assert checked > 1000


def test_workspace_is_refused_when_missing_small_or_misaligned():
    lib = _C.load()
    g = make("bf16", 128, 128, 64, 4, 2, 512, 512, 512, 4, 0)
    g.a = g.b = g.c = 4096                                    # never dereferenced: the call is refused before any launch
    need = lib.tnx_gemm_workspace_bytes(ctypes.byref(g))
    assert need == COUNTER_BYTES + 4 * 16 * 128 * 128 * 4
    assert lib.tnx_gemm(ctypes.byref(g)) == _C.E_WORKSPACE      # null workspace
    g.workspace, g.workspace_bytes = 1 << 20, need - 1
    assert lib.tnx_gemm(ctypes.byref(g)) == _C.E_WORKSPACE      # one byte short
    g.workspace, g.workspace_bytes = (1 << 20) + 16, need
    assert lib.tnx_gemm(ctypes.byref(g)) == _C.E_WORKSPACE      # not 256-byte aligned
    with pytest.raises(RuntimeError):
        _C.raise_for_status(_C.E_WORKSPACE, g)
