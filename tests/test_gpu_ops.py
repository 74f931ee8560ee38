"""The reference's own GPU tests (tests/test_matmul.py: correctness, forced backends, cached winner) on the
HIP path, plus the ops it never tested: split-K, GLU, int8."""
import pytest
import torch

import oracle
import tritonix_amd
import importlib

mm = importlib.import_module("tritonix_amd.ops.matmul")   # the module; `tritonix_amd.ops.matmul` the attribute is the dispatcher

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def short_tuning(monkeypatch):
    monkeypatch.setitem(mm.TUNE_OPTIONS, "warmup", 1)
    monkeypatch.setitem(mm.TUNE_OPTIONS, "rep", 3)


def close(ref, out):
    # the reference's own bar (tests/test_matmul.py:18-20)
    return torch.allclose(ref.float(), out.float(), atol=1.0, rtol=1e-2)


@pytest.mark.parametrize("M,N,K", [(512, 512, 512), (1024, 2048, 512), (2048, 2048, 2048)])
def test_matmul_correctness(device, M, N, K):
    g = torch.Generator("cpu").manual_seed(M + N + K)
    a = torch.randn(M, K, generator=g).half().to(device)
    b = torch.randn(K, N, generator=g).half().to(device)
    out = tritonix_amd.triton_matmul(a, b)
    assert close(torch.matmul(a, b), out), f"max diff: {(torch.matmul(a, b) - out).abs().max()}"
    ok, _, rel = oracle.within_tolerance(out, oracle.reference_matmul(a, b))
    assert ok and rel <= 1e-2
    assert (M, N, K, torch.float16, 1) in mm._matmul_cfg


@pytest.mark.parametrize("M,N,K", [(512, 512, 512), (2048, 2048, 2048)])
def test_dispatch_correctness(device, M, N, K):
    a = torch.randn(M, K, device=device, dtype=torch.float16)
    b = torch.randn(K, N, device=device, dtype=torch.float16)
    ref = torch.matmul(a, b)
    with tritonix_amd.matmul.force_backend("triton"):
        tri = tritonix_amd.matmul(a, b)
    with tritonix_amd.matmul.force_backend("pytorch"):
        pt = tritonix_amd.matmul(a, b)
    assert close(ref, tri) and close(ref, pt)


def test_dispatch_caches_winner(device):
    matmul = tritonix_amd.matmul
    matmul.clear_cache()
    a = torch.randn(1024, 1024, device=device, dtype=torch.float16)
    b = torch.randn(1024, 1024, device=device, dtype=torch.float16)
    out1 = matmul(a, b)
    assert len(matmul.cache) == 1
    assert list(matmul.cache.values())[0] in ("triton", "pytorch")          # the reference's own assertion (tests/test_matmul.py:47)
    assert list(matmul.cache)[0] == (1024, 1024, "torch.float16", 1024, 1024, "torch.float16")
    out2 = matmul(a, b)
    assert torch.allclose(out1.float(), out2.float(), atol=1.0, rtol=1e-2)


def test_tune_entry_point_with_a_user_launcher(device):
    # the flow of examples/tune_matmul.py: the caller writes the launcher and gets a config dict back
    a = torch.randn(512, 1024, device=device, dtype=torch.bfloat16)
    b = torch.randn(1024, 768, device=device, dtype=torch.bfloat16)
    kernel = tritonix_amd.matmul_kernel

    def launcher(cfg):
        c = torch.empty((512, 768), device=device, dtype=a.dtype)
        grid = ((512 + cfg["block_m"] - 1) // cfg["block_m"], (768 + cfg["block_n"] - 1) // cfg["block_n"])
        kernel[grid](a, b, c, 512, 768, 1024, a.stride(0), a.stride(1), b.stride(0), b.stride(1), c.stride(0),
                     c.stride(1), **cfg)
        return c

    best = kernel.tune(launcher, method="grid", warmup=1, rep=3, max_configs=12)
    assert set(best) == set(kernel.space)
    ok, _, _ = oracle.within_tolerance(launcher(best), oracle.reference_matmul(a, b))
    assert ok


def test_matmul_splitk(device):
    a, b = oracle.make_inputs("C3", scale_down=2)
    out = tritonix_amd.matmul_splitk(a.to(device), b.to(device))
    ok, _, rel = oracle.within_tolerance(out, oracle.reference_matmul(a, b))
    assert ok and rel <= 1e-2
    assert mm._splitk_cfg[(16, 2048, 7168, 4, torch.bfloat16, 1)]["split_k"] >= 2


def test_glu_and_swiglu_wrappers(device):
    x, w12 = oracle.make_inputs("C4", scale_down=16)
    xd, wd = x.to(device), w12.to(device)
    z = tritonix_amd.swiglu(xd, wd)
    assert z.shape == (x.shape[0], w12.shape[1] // 2) and z.dtype == torch.bfloat16
    assert oracle.within_tolerance(z, oracle.reference_glu(x, w12, "silu"))[0]
    assert oracle.within_tolerance(tritonix_amd.glu(xd, wd, activation="sigmoid"),
                                   oracle.reference_glu(x, w12, "sigmoid"))[0]
    assert torch.equal(tritonix_amd.fused_glu(xd, wd), z)
    from tritonix_amd.ops.swiglu import interleave_weights

    w1, w2 = w12[:, 0::2].contiguous(), w12[:, 1::2].contiguous()
    assert torch.equal(interleave_weights(w1, w2), w12)
    with pytest.raises(ValueError):
        tritonix_amd.glu(xd, wd[:, :-1])


def test_int8_through_the_dispatcher(device):
    a, b = oracle.make_inputs("C5", scale_down=16)
    out = tritonix_amd.matmul(a.to(device), b.to(device))
    assert out.dtype == torch.int32
    assert torch.equal(out.cpu(), oracle.reference_matmul(a, b))


def test_default_config_path(device, monkeypatch):
    monkeypatch.setenv("TRITONIX_AUTOTUNE", "0")
    mm._matmul_cfg.clear()
    a, b = oracle.make_inputs("C2", scale_down=4)
    out = tritonix_amd.triton_matmul(a.to(device), b.to(device))
    assert oracle.within_tolerance(out, oracle.reference_matmul(a, b))[0]


def test_do_bench_returns_sane_numbers(device):
    from tritonix_amd.testing import do_bench

    a = torch.randn(2048, 2048, device=device, dtype=torch.bfloat16)
    ms = do_bench(lambda: torch.matmul(a, a), warmup=2, rep=10)
    tflops = 2 * 2048 ** 3 / ms / 1e9
    assert 0 < tflops < 1e4
    q = do_bench(lambda: torch.matmul(a, a), warmup=2, rep=10, quantiles=[0.5, 0.2, 0.8])
    assert len(q) == 3 and q[1] <= q[0] <= q[2]


def test_prepared_launch_repeats_one_c_abi_call(device):
    a, b = oracle.make_inputs("C3", scale_down=4)
    ad, bd = a.to(device), b.to(device)
    m, k = ad.shape
    n = bd.shape[1]
    c = torch.zeros((m, n), device=device, dtype=torch.bfloat16)
    cfg = mm.default_config(ad, bd, split=True)
    launch = tritonix_amd.gemm_splitk_kernel.prepare(ad, bd, c, m, n, k, k, 1, n, 1, n, 1, **cfg)
    launch()
    first = c.clone()
    for _ in range(5):                     # the counters of the workspace are re-armed by every launch
        c.zero_()
        launch()
    assert torch.equal(c, first)
    assert oracle.within_tolerance(c, oracle.reference_matmul(a, b))[0]
    with pytest.raises(ValueError):
        tritonix_amd.matmul_kernel.prepare(ad, bd, c, m, n, k, k, 1, n, 1, n, 1, block_m=96, block_n=128, block_k=64,
                                           group_m=8, num_stages=2, num_warps=4)


@pytest.mark.parametrize("shape", [(1024, 768, 512), (300, 200, 128), (4096, 4096, 1024), (64, 8192, 2048)])
def test_default_configs_are_valid_and_correct(device, shape):
    m, n, k = shape
    g = torch.Generator("cpu").manual_seed(m + n)
    for dt in (torch.float16, torch.int8):
        if dt == torch.int8:
            a = torch.randint(-127, 128, (m, k), generator=g, dtype=dt)
            b = torch.randint(-127, 128, (k, n), generator=g, dtype=dt)
        else:
            a, b = torch.randn(m, k, generator=g).to(dt), torch.randn(k, n, generator=g).to(dt)
        cfg = mm.default_config(a, b)
        out = mm._launch_matmul(a.to(device), b.to(device), cfg)
        ref = oracle.reference_matmul(a, b)
        if dt == torch.int8:
            assert torch.equal(out.cpu(), ref)
        else:
            assert oracle.within_tolerance(out, ref)[0]


def test_swiglu_ffn(device):
    from tritonix_amd.ops.swiglu import swiglu_ffn

    x, w12 = oracle.make_inputs("C4", scale_down=16)          # x[256,256], w12[256,1792]
    g = torch.Generator("cpu").manual_seed(44)
    w3 = (0.05 * torch.randn(w12.shape[1] // 2, 320, generator=g)).bfloat16()
    out = swiglu_ffn(x.to(device), w12.to(device), w3.to(device))
    hidden = oracle.reference_glu(x, w12, "silu").bfloat16().float()   # the intermediate is stored in bf16
    ok, _, rel = oracle.within_tolerance(out, hidden @ w3.float())
    assert ok and rel <= 1e-2 and out.shape == (256, 320)
    with pytest.raises(ValueError):
        swiglu_ffn(x.to(device), w12.to(device), w3[:-1].to(device))


@pytest.mark.parametrize("activation", ["silu", "sigmoid", "none"])
def test_swiglu_kernel_launch_object(device, activation):
    """The reference's calling convention (tritonix/ops/swiglu.py:127-152) against ``reference_glu(...) @ w3``."""
    from tritonix.ops.swiglu import swiglu_kernel

    x, w12 = oracle.make_inputs("C4", scale_down=16)          # x[256,256], w12[256,1792]
    g = torch.Generator("cpu").manual_seed(45)
    w3 = (0.05 * torch.randn(w12.shape[1] // 2, 320, generator=g)).bfloat16()
    xd, wd, w3d = x.to(device), w12.to(device), w3.to(device)
    m, k = x.shape
    n, f = w12.shape[1], w3.shape[1]
    z = torch.full((m, f), float("nan"), device=device, dtype=torch.bfloat16)   # written, never accumulated into
    swiglu_kernel[(2, 14)](xd, wd, w3d, z, m, n, k, f, xd.stride(0), xd.stride(1), wd.stride(0), wd.stride(1),
                           w3d.stride(0), w3d.stride(1), z.stride(0), z.stride(1),
                           block_m=128, block_n=128, block_k=64, group_m=8, block_l=64, activation=activation,
                           num_stages=2, num_warps=4)
    hidden = oracle.reference_glu(x, w12, activation).bfloat16().float()          # the intermediate is stored in bf16
    ok, _, rel = oracle.within_tolerance(z, hidden @ w3.float())
    assert ok and rel <= 1e-2
    # the same through a k-contiguous w3 (strides of a transposed view) and a tile pair the tuner would propose
    w3t = w3.t().contiguous().to(device).t()
    z2 = torch.empty_like(z)
    swiglu_kernel[(1, 7)](xd, wd, w3t, z2, m, n, k, f, xd.stride(0), xd.stride(1), wd.stride(0), wd.stride(1),
                          w3t.stride(0), w3t.stride(1), z2.stride(0), z2.stride(1),
                          block_m=256, block_n=256, block_k=64, group_m=4, block_l=128, activation=activation,
                          num_stages=2, num_warps=4)
    assert oracle.within_tolerance(z2, hidden @ w3.float())[0]
    with pytest.raises(ValueError):                                               # a tile that is not built
        swiglu_kernel[(1, 7)](xd, wd, w3d, z, m, n, k, f, xd.stride(0), 1, wd.stride(0), 1, w3d.stride(0), 1, z.stride(0), 1,
                              block_m=128, block_n=128, block_k=64, group_m=8, block_l=16, num_stages=2, num_warps=4)


def test_swiglu_kernel_tunes_like_the_other_kernels(device):
    from tritonix_amd.ops.swiglu import swiglu_kernel

    x, w12 = oracle.make_inputs("C4", scale_down=16)
    w3 = (0.05 * torch.randn(w12.shape[1] // 2, 256)).bfloat16()
    xd, wd, w3d = x.to(device), w12.to(device), w3.to(device)
    m, k = x.shape
    n, f = w12.shape[1], w3.shape[1]
    z = torch.empty((m, f), device=device, dtype=torch.bfloat16)

    def launcher(cfg):
        swiglu_kernel[(1,)](xd, wd, w3d, z, m, n, k, f, k, 1, n, 1, f, 1, f, 1, **cfg)

    cfg = swiglu_kernel.tune(launcher, max_configs=6, warmup=2, rep=5)
    assert cfg is not None and set(cfg) == set(swiglu_kernel.space)
    launcher(cfg)
    hidden = oracle.reference_glu(x, w12, "silu").bfloat16().float()
    assert oracle.within_tolerance(z, hidden @ w3.float())[0]


def test_thin_problems_settle_tile_against_k_split_inside_the_triton_backend(device, tmp_path, monkeypatch):
    """A problem whose output tiles leave CUs idle is timed with its tuned tile and its tuned K split by
    ``triton_matmul`` itself; the dispatcher only ever sees the reference's backend names."""
    monkeypatch.setenv("TRITONIX_CACHE_DIR", str(tmp_path))
    g = torch.Generator("cpu").manual_seed(77)
    a = torch.randn(128, 4096, generator=g).bfloat16().to(device)
    b = (0.02 * torch.randn(4096, 1536, generator=g)).bfloat16().to(device)
    uncut = {k_: v for k_, v in mm.default_config(a, b).items() if k_ not in ("split_k", "tail_tiles")}
    cut = mm.default_config(a, b, split=True)
    timed = []
    # stand-ins for the two grid searches (minutes each); the choice between their results is what is under test
    monkeypatch.setattr(mm.matmul_kernel, "tune", lambda launcher, **kw: (launcher(uncut), timed.append("tile"), dict(uncut))[2])
    monkeypatch.setattr(mm.gemm_splitk_kernel, "tune", lambda launcher, **kw: (launcher(cut), timed.append("cut"), dict(cut))[2])
    mm._matmul_cfg.clear()
    matmul = tritonix_amd.matmul
    matmul.clear_cache()
    out = matmul(a, b)
    key = (128, 1536, 4096, torch.bfloat16, 1)
    assert timed == ["tile", "cut"]
    assert mm._matmul_cfg[key] in (uncut, cut) and set(matmul.cache.values()) == {"triton"}
    assert set(matmul.timings[next(iter(matmul.cache))]) == {"triton"}
    assert oracle.within_tolerance(out, oracle.reference_matmul(a.cpu(), b.cpu()))[0]
    assert torch.equal(tritonix_amd.triton_matmul(a, b), out) and timed == ["tile", "cut"]
    # what was chosen is what the disk record holds for the next process
    assert mm.load_tuned("matmul", key) == mm._matmul_cfg[key]
    mm._matmul_cfg.clear()
    matmul.clear_cache()


def _split_reference(x):
    """bf16 head and tail of a float32 tensor, as tnx_split_f32 is specified (round to nearest even twice)."""
    hi = x.bfloat16()
    return hi, (x - hi.float()).bfloat16()


def test_split_f32_lays_out_head_and_tail(device):
    import ctypes

    from tritonix_amd import _C

    g = torch.Generator("cpu").manual_seed(5)
    x = torch.randn(37, 53, generator=g) * torch.logspace(-6, 6, 53)
    x[3, 4], x[5, 6], x[7, 8] = float("inf"), float("-inf"), 0.0
    hi, lo = _split_reference(x)
    lo[3, 4] = lo[5, 6] = 0                                            # non-finite elements keep their head only,
    hi2 = hi.clone()
    hi2[3, 4] = hi2[5, 6] = 0                                          # and only in its first copy
    xd = x.to(device)
    lib, stream = _C.load(), torch.cuda.current_stream().cuda_stream
    a3 = torch.empty(37, 3 * 53, dtype=torch.bfloat16, device=device)
    b3 = torch.empty(3 * 37, 53, dtype=torch.bfloat16, device=device)
    assert lib.tnx_split_f32(xd.data_ptr(), 37, 53, 53, 1, a3.data_ptr(), 0, stream) == _C.OK
    assert lib.tnx_split_f32(xd.data_ptr(), 37, 53, 53, 1, b3.data_ptr(), 1, stream) == _C.OK
    assert torch.equal(a3.cpu().view(torch.int16), torch.cat([hi, hi2, lo], dim=1).view(torch.int16))
    assert torch.equal(b3.cpu().view(torch.int16), torch.cat([hi, lo, hi2], dim=0).view(torch.int16))
    w3 = torch.empty(37, 3 * 53, dtype=torch.bfloat16, device=device)
    assert lib.tnx_split_f32(xd.data_ptr(), 37, 53, 53, 1, w3.data_ptr(), 2, stream) == _C.OK
    assert torch.equal(w3.cpu().view(torch.int16), torch.cat([hi, lo, hi2], dim=1).view(torch.int16))
    # a transposed view: strides (1, 53) of the same storage
    t3 = torch.empty(53, 3 * 37, dtype=torch.bfloat16, device=device)
    assert lib.tnx_split_f32(xd.data_ptr(), 53, 37, 1, 53, t3.data_ptr(), 0, stream) == _C.OK
    assert torch.equal(t3.cpu().view(torch.int16), torch.cat([hi.t(), hi2.t(), lo.t()], dim=1).contiguous().view(torch.int16))


def test_float32_matmul_keeps_infinities_and_nans_where_fp32_has_them(device, monkeypatch):
    """inf * finite is inf and inf * 0 is NaN in the fp32 product; the three-term split must not add an inf * 0 of its
    own (the tail of a value bf16 holds exactly is 0).  Same pattern of inf / -inf / NaN as the CPU fp32 matmul, and
    the finite entries within the float32 tolerance."""
    monkeypatch.setenv("TRITONIX_AUTOTUNE", "0")
    g = torch.Generator("cpu").manual_seed(77)
    a, b = torch.randn(128, 256, generator=g), torch.randn(256, 192, generator=g) / 16
    b[:, :8] = b[:, :8].bfloat16().float()                            # columns whose tails are exactly zero
    b[5, 3] = 1.0
    a[2, 5], a[9, 100], a[40, 7] = float("inf"), float("-inf"), float("nan")
    b[17, 150], b[200, 20] = float("inf"), 0.0
    a[70, 200] = float("inf")                                          # meets b[200, 20] == 0: NaN in fp32 too
    ref = a @ b
    out = tritonix_amd.triton_matmul(a.to(device), b.to(device)).cpu()
    assert torch.equal(torch.isnan(out), torch.isnan(ref))
    assert torch.equal(torch.isposinf(out), torch.isposinf(ref)) and torch.equal(torch.isneginf(out), torch.isneginf(ref))
    fin = torch.isfinite(ref)
    assert ((out[fin] - ref[fin]).abs().max() / ref[fin].abs().max()).item() < 2e-4


@pytest.mark.parametrize("m,n,k", [(256, 384, 512), (300, 520, 200), (16, 1024, 4096), (1000, 72, 1003)])
def test_float32_matmul(device, m, n, k, monkeypatch):
    """float32 in, float32 out (the reference serves such calls through tl.dot in TF32, tritonix/ops/matmul.py:98):
    three bf16 terms with fp32 accumulation.  Bar: the GEMM tolerance of the other dtypes against the fp32 CPU matmul,
    and -- what the split buys -- an error at least 30 times below a plain bf16 product's."""
    monkeypatch.setenv("TRITONIX_AUTOTUNE", "0")
    g = torch.Generator("cpu").manual_seed(m + n + k)
    a, b = torch.randn(m, k, generator=g), torch.randn(k, n, generator=g) / k ** 0.5
    out = tritonix_amd.triton_matmul(a.to(device), b.to(device))
    assert out.dtype == torch.float32 and out.shape == (m, n)
    ref = a.double() @ b.double()
    ok, _, rel = oracle.within_tolerance(out, oracle.reference_matmul(a, b))
    assert ok and rel <= 1e-2
    err = (out.cpu().double() - ref).abs().max().item() / ref.abs().max().item()
    bf16 = ((a.bfloat16().double() @ b.bfloat16().double()) - ref).abs().max().item() / ref.abs().max().item()
    assert err < 2e-4 and err * 30 < bf16, (err, bf16)
    # transposed views go through the same path (the splitter reads any strides)
    out_t = tritonix_amd.triton_matmul(a.t().contiguous().to(device).t(), b.t().contiguous().to(device).t())
    assert torch.equal(out_t, out)
    with tritonix_amd.matmul.force_backend("triton"):
        assert torch.equal(tritonix_amd.matmul(a.to(device), b.to(device)), out)


def test_float32_splitk_and_glu(device, monkeypatch):
    monkeypatch.setenv("TRITONIX_AUTOTUNE", "0")
    g = torch.Generator("cpu").manual_seed(91)
    a, b = torch.randn(16, 4096, generator=g), 0.02 * torch.randn(4096, 1024, generator=g)
    out = tritonix_amd.matmul_splitk(a.to(device), b.to(device))
    ref = a.double() @ b.double()
    assert out.dtype == torch.float32 and (out.cpu().double() - ref).abs().max() / ref.abs().max() < 2e-4
    x, w12 = torch.randn(256, 512, generator=g), 0.05 * torch.randn(512, 768, generator=g)
    for act in ("silu", "sigmoid", "none"):
        z = tritonix_amd.glu(x.to(device), w12.to(device), activation=act)
        zr = oracle.reference_glu(x, w12, act)
        assert z.dtype == torch.float32 and z.shape == (256, 384)
        assert (z.cpu() - zr).abs().max() / zr.abs().max() < 5e-4, act
    with pytest.raises(ValueError):                                    # the result of a float32 call is float32
        c = torch.empty(16, 1024, device=device, dtype=torch.bfloat16)
        tritonix_amd.matmul_kernel[(1, 8)](a.to(device), b.to(device), c, 16, 1024, 4096, 4096, 1, 1024, 1, 1024, 1,
                                            block_m=64, block_n=128, block_k=64, group_m=8, num_stages=3, num_warps=8)


def test_tuned_config_is_reused_from_disk(device, tmp_path, monkeypatch):
    monkeypatch.setenv("TRITONIX_CACHE_DIR", str(tmp_path))
    a = torch.randn(384, 256, device=device, dtype=torch.float16)
    b = torch.randn(256, 512, device=device, dtype=torch.float16)
    mm._matmul_cfg.clear()
    out1 = tritonix_amd.triton_matmul(a, b)
    picked = mm._matmul_cfg[(384, 512, 256, torch.float16, 1)]
    assert mm.load_tuned("matmul", (384, 512, 256, torch.float16, 1)) == picked
    mm._matmul_cfg.clear()
    monkeypatch.setattr(mm.matmul_kernel, "tune", lambda *a, **k: pytest.fail("tuned again despite the disk record"))
    assert torch.equal(tritonix_amd.triton_matmul(a, b), out1)


def test_memoised_config_follows_the_operand_layout(device, monkeypatch):
    """A tile remembered for row-major operands must not be handed to a transposed view of the same shape
    (most tiles exist with the direct-to-LDS loader only), and the other way round."""
    monkeypatch.setenv("TRITONIX_AUTOTUNE", "0")
    mm._matmul_cfg.clear()
    g = torch.Generator("cpu").manual_seed(9)
    a = torch.randn(512, 256, generator=g).half()
    w = torch.randn(384, 256, generator=g).half()            # w.t() is [256, 384] with stride_bn != 1
    ref = oracle.reference_matmul(a, w.t())
    ad, wd = a.to(device), w.to(device)
    b_contig = wd.t().contiguous()
    out1 = tritonix_amd.triton_matmul(ad, b_contig)
    out2 = tritonix_amd.triton_matmul(ad, wd.t())
    out3 = tritonix_amd.triton_matmul(ad, b_contig)
    for out in (out1, out2, out3):
        assert oracle.within_tolerance(out, ref)[0]
    assert torch.equal(out1, out3)
    # row-major B (class 1) and k-contiguous B (class 2) are remembered apart
    assert (512, 384, 256, torch.float16, 1) in mm._matmul_cfg and (512, 384, 256, torch.float16, 2) in mm._matmul_cfg
    # a misaligned base pointer is a class of its own: the DMA loader with an element-wise last K slab
    flat = torch.zeros(512 * 256 + 8, dtype=torch.float16, device=device)
    a_off = flat[1:1 + 512 * 256].view(512, 256)
    a_off.copy_(ad)
    assert mm.dma_layout(a_off, b_contig) == 3 and mm.dma_layout(ad, b_contig) == 1 and mm.dma_layout(ad, wd.t()) == 2
    assert torch.equal(tritonix_amd.triton_matmul(a_off, b_contig), out1)
    # a column-major A is none of the DMA layouts: the wrapper hands the kernel a row-major copy (same bits as out1),
    # the kernel object itself takes the strides as they are (one of the two tiles built with the chunk-wise loader)
    a_cm = ad.t().contiguous().t()
    assert a_cm.stride() == (1, 512) and mm.dma_layout(a_cm, b_contig) == 0
    assert torch.equal(tritonix_amd.triton_matmul(a_cm, b_contig), out1)
    assert mm.dma_operands(a_cm, b_contig)[0].stride() == (256, 1)
    raw = mm._launch_matmul(a_cm, b_contig, dict(block_m=128, block_n=128, block_k=64, group_m=8, num_stages=2, num_warps=4))
    assert oracle.within_tolerance(raw, ref)[0]
    # a memo entry the engine refuses for these operands is replaced, not raised: the persistent schedule does not
    # take operands off 16 bytes
    mm._matmul_cfg[(512, 384, 256, torch.float16, 3)] = dict(mm._matmul_cfg[(512, 384, 256, torch.float16, 3)],
                                                             block_m=128, block_n=128, num_stages=3, num_warps=4, persistent=1)
    assert torch.equal(tritonix_amd.triton_matmul(a_off, b_contig), out1)
    assert "persistent" not in mm._matmul_cfg[(512, 384, 256, torch.float16, 3)]      # replaced by the built-in choice
    mm._matmul_cfg.clear()


@pytest.mark.parametrize("name,scale", [("C1", 1), ("C2", 4), ("C3", 2), ("C5", 8)])
def test_unforced_dispatch_never_selects_the_vendor_library(device, name, scale, tmp_path, monkeypatch):
    monkeypatch.setenv("TRITONIX_CACHE_DIR", str(tmp_path))
    monkeypatch.setenv("TRITONIX_AUTOTUNE", "0")
    matmul = tritonix_amd.matmul
    matmul.clear_cache()
    a, b = oracle.make_inputs(name, scale_down=scale)
    out = matmul(a.to(device), b.to(device))
    (key, winner), = matmul.cache.items()
    assert winner == "triton" and set(matmul.timings[key]) == {"triton"}
    ref = oracle.reference_matmul(a, b)
    if a.dtype == torch.int8:
        assert torch.equal(out.cpu(), ref)
    else:
        assert oracle.within_tolerance(out, ref)[0]
    matmul.clear_cache()


def test_built_in_choice_on_seeded_random_problems(device, monkeypatch):
    """150 problems from a fixed seed (round sizes, ragged sizes, thin and wide, all three types, every fifth with a
    k-contiguous B) through ``triton_matmul`` with the library's own tile choice: whatever tile, K cut or tail cut it
    names must give the right product (int8 exactly)."""
    import random

    monkeypatch.setenv("TRITONIX_AUTOTUNE", "0")
    mm._matmul_cfg.clear()
    rnd = random.Random(5)
    picked = set()
    for case in range(150):
        kind = case % 4
        if kind == 0:
            m, n, k = (rnd.choice([128, 192, 256, 384, 512, 768, 1024, 1536, 2048, 2560, 3072]) for _ in range(3))
        elif kind == 1:
            m, n, k = rnd.randint(1, 700), rnd.randint(1, 3000), rnd.randint(1, 3000)
        elif kind == 2:
            m, n, k = rnd.randint(100, 3000), rnd.randint(100, 3000), 64 * rnd.randint(1, 64)
        else:
            m, n, k = 8 * rnd.randint(1, 400), 8 * rnd.randint(1, 400), 8 * rnd.randint(1, 600)
        dt = [torch.bfloat16, torch.float16, torch.int8][case % 3]
        g = torch.Generator(device=device).manual_seed(case)
        if dt == torch.int8:
            a = torch.randint(-127, 128, (m, k), dtype=torch.int8, device=device, generator=g)
            b = torch.randint(-127, 128, (k, n), dtype=torch.int8, device=device, generator=g)
        else:
            a = torch.randn(m, k, device=device, generator=g).to(dt)
            b = (torch.randn(k, n, device=device, generator=g) / k ** 0.5).to(dt)
        if case % 5 == 4:
            b = b.t().contiguous().t()
        cfg = mm.default_config(a, b)
        picked.add((cfg["block_m"], cfg["block_n"], cfg.get("split_k", 1) > 1))
        out = tritonix_amd.triton_matmul(a, b)
        what = (case, m, n, k, dt, cfg)
        if dt == torch.int8:
            assert torch.equal(out.double(), a.double() @ b.double()), what
        else:
            assert oracle.within_tolerance(out, a.float() @ b.float())[0], what
    assert len(picked) >= 6, picked
