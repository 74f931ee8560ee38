"""The C-ABI library loads, exports every symbol include/tritonix_hip.h declares, and its host-only entry points
answer without a GPU."""
import ctypes
import os
import re

import pytest

from tritonix_amd import _C
from tritonix_amd.testing import LDS_LIMIT_BYTES, OutOfResources

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def args(**kw):
    g = _C.GemmArgs()
    base = dict(m=512, n=512, k=512, stride_am=512, stride_ak=1, stride_bk=512, stride_bn=1, stride_cm=512,
                stride_cn=1, in_dtype=_C.BF16, out_dtype=_C.BF16, block_m=128, block_n=128, block_k=64, group_m=8,
                split_k=1, num_stages=2, num_warps=4, epilogue=_C.EPI_NONE)
    base.update(kw)
    for k, v in base.items():
        setattr(g, k, v)
    return g


def test_library_is_built_and_exports_the_header():
    lib = _C.load()
    header = open(os.path.join(ROOT, "include", "tritonix_hip.h")).read()
    declared = set(re.findall(r"\b(tnx_[a-z_0-9]+)\s*\(", header)) - {"tnx_gemm_args"}
    assert declared == set(_C.EXPORTS)
    for name in declared:
        assert hasattr(lib, name), name
    assert lib.tnx_version() == int(re.search(r"#define TNX_VERSION (\d+)", header).group(1))
    assert int(re.search(r"#define TNX_LDS_LIMIT_BYTES (\d+)", header).group(1)) == LDS_LIMIT_BYTES


def test_struct_layout_matches_the_header_field_order():
    header = open(os.path.join(ROOT, "include", "tritonix_hip.h")).read()
    start = header.index("typedef struct tnx_gemm_args {") + len("typedef struct tnx_gemm_args {")
    body = header[start:header.index("} tnx_gemm_args;")]
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    names = []
    for decl in body.split(";"):
        decl = decl.strip()
        if not decl or decl.startswith("typedef"):
            continue
        decl = re.sub(r"^(const\s+)?(void|int64_t|int32_t|size_t)\s*\*?", "", decl)
        names += [n.strip(" *") for n in decl.split(",")]
    assert names == [f[0] for f in _C.GemmArgs._fields_]
    assert ctypes.sizeof(_C.GemmArgs) == 3 * 8 + 9 * 8 + 12 * 4 + 8 + 8 + 8


def test_lds_bytes_is_host_arithmetic():
    lib = _C.load()
    assert lib.tnx_gemm_lds_bytes(ctypes.byref(args())) == 2 * (128 * 64 + 64 * 128) * 2
    assert lib.tnx_gemm_lds_bytes(ctypes.byref(args(block_m=256, block_n=256, num_stages=2))) == 131072
    assert lib.tnx_gemm_lds_bytes(ctypes.byref(args(in_dtype=_C.I8, out_dtype=_C.I32, block_k=128))) == 65536
    assert lib.tnx_gemm_lds_bytes(ctypes.byref(args(block_m=0))) == -1


def test_supported_status_codes_and_python_exceptions():
    lib = _C.load()
    ok = args()
    assert lib.tnx_gemm_supported(ctypes.byref(ok)) == _C.OK
    too_big = args(block_m=256, block_n=256, num_stages=3)             # 196608 bytes of LDS
    assert lib.tnx_gemm_supported(ctypes.byref(too_big)) == _C.E_LDS
    with pytest.raises(OutOfResources) as ei:
        _C.raise_for_status(_C.E_LDS, too_big)
    assert (ei.value.required, ei.value.limit, ei.value.name) == (196608, 163840, "shared memory")
    assert "Required: 196608" in str(ei.value)
    odd = args(block_m=96)
    assert lib.tnx_gemm_supported(ctypes.byref(odd)) == _C.E_UNSUPPORTED
    with pytest.raises(ValueError):
        _C.raise_for_status(_C.E_UNSUPPORTED, odd)
    assert lib.tnx_gemm_supported(ctypes.byref(args(out_dtype=_C.F16))) == _C.E_UNSUPPORTED   # bf16 in, f16 out
    assert lib.tnx_gemm_supported(ctypes.byref(args(epilogue=_C.EPI_GLU_SILU, n=511))) == _C.E_UNSUPPORTED
    assert lib.tnx_gemm_supported(ctypes.byref(args(m=-1))) == _C.E_INVALID
    assert lib.tnx_gemm_supported(ctypes.byref(args(in_dtype=9))) == _C.E_INVALID
    assert lib.tnx_gemm_supported(None) == _C.E_INVALID
    with pytest.raises(RuntimeError):
        _C.raise_for_status(_C.E_HIP, ok)
    assert _C.strerror(_C.OK) == "ok" and "LDS" in _C.strerror(_C.E_LDS)


def test_ragged_layouts_need_a_generic_kernel():
    lib = _C.load()
    # row-major 16-bit operands with a ragged K, rows that are not 16-byte aligned or a ragged N: every tile takes
    # them (DMA loader, last K slab chunk by chunk), int8 included; the persistent schedule does not
    assert lib.tnx_gemm_supported(ctypes.byref(args(k=500, stride_am=500))) == _C.OK          # 128x128x64 w4 s2
    assert lib.tnx_gemm_supported(ctypes.byref(args(k=500, stride_am=500, num_stages=3))) == _C.OK
    assert lib.tnx_gemm_supported(ctypes.byref(args(n=509, stride_bk=509, stride_cm=509, num_stages=3))) == _C.OK
    assert lib.tnx_gemm_supported(ctypes.byref(args(k=500, stride_am=500, num_stages=3,
                                                    schedule=_C.SCHED_PERSISTENT))) == _C.E_UNSUPPORTED
    i8 = dict(in_dtype=_C.I8, out_dtype=_C.I32, block_k=128, num_stages=3)
    assert lib.tnx_gemm_supported(ctypes.byref(args(k=528, stride_am=528, **i8))) == _C.OK       # ragged K, aligned rows
    assert lib.tnx_gemm_supported(ctypes.byref(args(k=500, stride_am=500, **i8))) == _C.OK
    assert lib.tnx_gemm_supported(ctypes.byref(args(k=500, stride_am=400, num_stages=3))) == _C.E_UNSUPPORTED   # rows overlap
    # k-contiguous B (w.t() of a row-major weight) has a DMA loader of its own in every tile whose K slab is 128 bytes
    # per row, 16-bit rows at any alignment included
    assert lib.tnx_gemm_supported(ctypes.byref(args(stride_bk=1, stride_bn=512))) == _C.OK
    assert lib.tnx_gemm_supported(ctypes.byref(args(stride_bk=1, stride_bn=512, num_warps=8))) == _C.OK
    assert lib.tnx_gemm_supported(ctypes.byref(args(stride_bk=1, stride_bn=512, block_k=32, num_stages=3))) == _C.E_UNSUPPORTED
    assert lib.tnx_gemm_supported(ctypes.byref(args(stride_bk=1, stride_bn=516))) == _C.OK
    assert lib.tnx_gemm_supported(ctypes.byref(args(stride_bk=1, stride_bn=516, num_warps=8))) == _C.OK
    assert lib.tnx_gemm_supported(ctypes.byref(args(stride_bk=1, stride_bn=500, num_warps=8))) == _C.E_UNSUPPORTED   # rows of w overlap
    # strided A: element-wise loader only
    assert lib.tnx_gemm_supported(ctypes.byref(args(stride_am=1, stride_ak=512, num_warps=8))) == _C.E_UNSUPPORTED


def test_workspace_bytes_and_default_config():
    lib = _C.load()
    assert lib.tnx_gemm_workspace_bytes(ctypes.byref(args())) == 0
    assert lib.tnx_gemm_workspace_bytes(ctypes.byref(args(m=16, n=4096, k=14336, split_k=8))) == 65536 + 8 * 32 * 128 * 128 * 4  # 32 tiles of 128x128, eight slices each
    # only the last 10 of the 6 x 6 tiles are cut: the workspace holds their slices and nothing else
    assert lib.tnx_gemm_workspace_bytes(ctypes.byref(args(m=768, n=768, split_k=4, tail_tiles=10))) == \
        65536 + 4 * 10 * 128 * 128 * 4
    assert lib.tnx_gemm_workspace_bytes(ctypes.byref(args(m=768, n=768, split_k=4, tail_tiles=99))) == \
        65536 + 4 * 36 * 128 * 128 * 4
    assert lib.tnx_gemm_supported(ctypes.byref(args(tail_tiles=-1))) == _C.E_INVALID
    g = args(m=8192, n=8192, k=8192)
    assert lib.tnx_gemm_default_config(ctypes.byref(g)) == _C.OK
    assert lib.tnx_gemm_supported(ctypes.byref(g)) == _C.OK
    g = args(m=16, n=4096, k=14336)
    lib.tnx_gemm_default_config(ctypes.byref(g))
    assert g.split_k >= 4 and lib.tnx_gemm_supported(ctypes.byref(g)) == _C.OK
    g = args(in_dtype=_C.I8, out_dtype=_C.I32, m=8192, n=8192, k=8192)
    lib.tnx_gemm_default_config(ctypes.byref(g))
    assert lib.tnx_gemm_supported(ctypes.byref(g)) == _C.OK


def test_kernel_table_lists_every_dtype():
    names = _C.kernel_names()
    assert len(names) == _C.load().tnx_kernel_count() > 0
    assert {n.split()[0] for n in names} == {"bf16", "f16", "i8"}
    assert _C.load().tnx_kernel_name(len(names)) is None


def test_default_config_is_always_launchable():
    """Whatever shape and dtype: the built-in choice names a kernel that exists, and its K cut fits one wave of CUs."""
    lib = _C.load()
    shapes = [(8192, 8192, 8192), (1024, 768, 512), (4096, 28672, 4096), (16, 4096, 14336), (6144, 6144, 6144),
              (5120, 5120, 8192), (4096, 5120, 4096), (2048, 2048, 8192), (512, 2048, 8192), (512, 512, 512),
              (128, 128, 128), (1, 8, 64), (64, 64, 64), (300, 200, 100), (4097, 4095, 4096), (256, 8192, 8192),
              (33, 1024, 8192), (65, 12288, 4096), (10000, 10000, 1000), (2048, 2048, 64)]
    for dt, out in ((_C.BF16, _C.BF16), (_C.F16, _C.F16), (_C.I8, _C.I32)):
        for m, n, k in shapes:
            g = args(m=m, n=n, k=k, stride_am=k, stride_bk=n, stride_cm=n, in_dtype=dt, out_dtype=out)
            assert lib.tnx_gemm_default_config(ctypes.byref(g)) == _C.OK
            assert lib.tnx_gemm_supported(ctypes.byref(g)) == _C.OK, (dt, m, n, k, g.block_m, g.block_n, g.block_k)
            tiles = -(-m // g.block_m) * -(-n // g.block_n)
            assert 1 <= g.split_k <= 16 and 0 <= g.tail_tiles < max(tiles, 1)
            if g.split_k > 1:
                cut = g.tail_tiles or tiles
                assert cut * g.split_k <= 256 + (0 if m > 64 else 256)      # one wave of workgroups (skinny: up to two)
                assert -(-k // g.block_k) // g.split_k >= 4                    # slices keep a useful number of K slabs
                assert lib.tnx_gemm_workspace_bytes(ctypes.byref(g)) == 65536 + g.split_k * cut * g.block_m * g.block_n * 4
            else:
                assert g.tail_tiles == 0 and lib.tnx_gemm_workspace_bytes(ctypes.byref(g)) == 0


def test_default_config_on_random_problems_is_launchable_for_every_output_type():
    """600 problems from a fixed seed, all three input types and, for the 16-bit floats, both output types (the input's
    own and binary32, the output of a split float32 product): the built-in choice always names a built kernel that
    takes these operands, within the LDS budget, and a float32 result never lands on a tile without that epilogue."""
    import random

    lib = _C.load()
    rng = random.Random(20251)
    for _ in range(600):
        m = rng.choice([1, 7, 16, 33, 64, 100, 128, 257, 512, 1000, 2048, 4096, 8192, 12288])
        n = rng.choice([8, 24, 64, 136, 256, 520, 1024, 3072, 4096, 14336, 28672])
        k = rng.choice([8, 64, 72, 200, 512, 1032, 4096, 8192, 14336])
        dt, out = rng.choice([(_C.BF16, _C.BF16), (_C.F16, _C.F16), (_C.I8, _C.I32), (_C.BF16, _C.F32), (_C.F16, _C.F32)])
        if dt == _C.I8:
            n, k = -(-n // 16) * 16, -(-k // 16) * 16          # int8 rows of A and B as the DMA loader takes them
        g = args(m=m, n=n, k=k, stride_am=k, stride_bk=n, stride_cm=n, in_dtype=dt, out_dtype=out)
        assert lib.tnx_gemm_default_config(ctypes.byref(g)) == _C.OK
        assert lib.tnx_gemm_supported(ctypes.byref(g)) == _C.OK, (dt, out, m, n, k, g.block_m, g.block_n, g.block_k, g.num_warps, g.num_stages)
        assert 0 < lib.tnx_gemm_lds_bytes(ctypes.byref(g)) <= _C.LDS_LIMIT_BYTES
        if out == _C.F32:
            assert g.block_m * g.block_n <= 128 * 128


def test_default_config_of_the_benchmark_shapes():
    lib = _C.load()

    def pick(dt, out, m, n, k):
        g = args(m=m, n=n, k=k, stride_am=k, stride_bk=n, stride_cm=n, in_dtype=dt, out_dtype=out)
        lib.tnx_gemm_default_config(ctypes.byref(g))
        picked.append(g.schedule)
        return (g.block_m, g.block_n, g.block_k, g.num_warps, g.num_stages, g.split_k, g.tail_tiles)

    picked = []
    assert pick(_C.BF16, _C.BF16, 8192, 8192, 8192) == (256, 256, 64, 4, 2, 1, 0)
    assert pick(_C.BF16, _C.BF16, 4096, 28672, 4096) == (256, 256, 64, 8, 2, 1, 0)     # short K loop: two waves per SIMD
    assert pick(_C.I8, _C.I32, 8192, 8192, 8192) == (256, 256, 128, 4, 2, 1, 0)
    assert pick(_C.F16, _C.F16, 1024, 768, 512) == (64, 64, 64, 4, 4, 1, 0)
    assert pick(_C.BF16, _C.BF16, 16, 4096, 14336) == (64, 128, 64, 8, 3, 8, 0)
    # 576 tiles of 256x256 are 2.25 waves of 256 CUs: the last 64 tiles are cut four ways
    assert pick(_C.BF16, _C.BF16, 6144, 6144, 6144) == (256, 256, 64, 4, 2, 4, 64)
    # 400 tiles of 256x256 are 1.56 waves and the 144 trailing ones cannot be cut without spilling into another wave;
    # 729 tiles of 192x192 are 2.85 (measured 326-331 us against 348-353)
    assert pick(_C.BF16, _C.BF16, 5120, 5120, 8192) == (192, 192, 64, 8, 3, 1, 0)
    assert pick(_C.I8, _C.I32, 5120, 5120, 8192) == (192, 192, 128, 8, 3, 1, 0)            # int8 has the 192 tiles too
    picked.pop()
    # 144 tiles of 256x256 leave 112 CUs idle; 256 tiles of 192x192 are one full wave
    assert pick(_C.BF16, _C.BF16, 3072, 3072, 3072) == (192, 192, 64, 8, 3, 1, 0)
    picked.pop()
    # grids of at least 16 x 16 uncut tiles are walked in super-block order; nothing is made persistent by default
    assert picked == [_C.SCHED_SUPERBLOCK, _C.SCHED_SUPERBLOCK, _C.SCHED_SUPERBLOCK, 0, 0, 0, _C.SCHED_SUPERBLOCK]


