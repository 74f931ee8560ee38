"""Tuned tile configs persist across processes (host logic only: fake kernels, temporary cache directory)."""
import importlib
import json

import pytest
import torch

mm = importlib.import_module("tritonix_amd.ops.matmul")


@pytest.fixture
def cache(tmp_path, monkeypatch):
    monkeypatch.setenv("TRITONIX_CACHE_DIR", str(tmp_path))
    monkeypatch.delenv("TRITONIX_TUNE_CACHE", raising=False)
    monkeypatch.delenv("TRITONIX_AUTOTUNE", raising=False)
    return tmp_path


class FakeKernel:
    def __init__(self, best):
        self.best, self.tunes = best, 0

    def tune(self, launcher, **kw):
        self.tunes += 1
        return self.best


def test_round_trip_and_key_separation(cache):
    key = (16, 4096, 14336, torch.bfloat16)
    cfg = {"block_m": 64, "block_n": 128, "block_k": 64, "group_m": 8, "num_stages": 3, "num_warps": 8, "split_k": 8}
    assert mm.load_tuned("matmul_splitk", key) is None
    mm.save_tuned("matmul_splitk", key, cfg)
    assert mm.load_tuned("matmul_splitk", key) == cfg
    assert mm.load_tuned("matmul", key) is None                              # other op
    assert mm.load_tuned("matmul_splitk", (16, 4096, 14336, torch.float16)) is None   # other dtype
    files = list((cache / "tuned").glob("*.json"))
    assert len(files) == 1 and json.loads(files[0].read_text())["config"] == cfg


def test_tune_once_then_read_from_disk(cache):
    best = {"block_m": 128, "block_n": 128, "block_k": 64, "group_m": 8, "num_stages": 3, "num_warps": 4}
    calls = []
    k1 = FakeKernel(best)
    got = mm._tuned_or_tune("matmul", (1, 2, 3, torch.float16), k1, calls.append, lambda: {"fallback": 1})
    assert got == best and k1.tunes == 1
    k2 = FakeKernel({"other": 1})
    got = mm._tuned_or_tune("matmul", (1, 2, 3, torch.float16), k2, calls.append, lambda: {"fallback": 1})
    assert got == best and k2.tunes == 0 and calls == [best]               # the stored config was re-validated by one launch


def test_stale_record_falls_back_to_tuning(cache):
    key = (4, 4, 4, torch.int8)
    mm.save_tuned("matmul", key, {"block_m": 96})

    def launcher(cfg):
        if cfg.get("block_m") == 96:
            raise ValueError("no such tile")

    k = FakeKernel({"block_m": 128})
    assert mm._tuned_or_tune("matmul", key, k, launcher, dict) == {"block_m": 128} and k.tunes == 1
    assert mm.load_tuned("matmul", key) == {"block_m": 128}


def test_switches(cache, monkeypatch):
    key = (8, 8, 8, torch.float16)
    monkeypatch.setenv("TRITONIX_TUNE_CACHE", "0")
    mm.save_tuned("matmul", key, {"block_m": 64})
    assert list(cache.rglob("*.json")) == [] and mm.load_tuned("matmul", key) is None
    monkeypatch.setenv("TRITONIX_AUTOTUNE", "0")
    k = FakeKernel({"block_m": 1})
    assert mm._tuned_or_tune("matmul", key, k, print, lambda: {"fallback": 1}) == {"fallback": 1} and k.tunes == 0
    k = FakeKernel(None)
    monkeypatch.setenv("TRITONIX_AUTOTUNE", "1")
    with pytest.raises(RuntimeError):
        mm._tuned_or_tune("matmul", key, k, print, dict)
