"""Lifetime rules of the split-K workspaces (host logic, no GPU): a buffer that was handed out is never
freed, and nothing is allocated while the stream is capturing."""

import importlib

import pytest
import torch


@pytest.fixture()
def pool_mod(ta):
    return importlib.import_module(ta.__name__ + "._workspace")


def test_same_stream_reuses_and_growth_retires(pool_mod, monkeypatch):
    monkeypatch.setattr(torch.cuda, "is_current_stream_capturing", lambda: False)
    pool = pool_mod.WorkspacePool(1024, "test")
    cpu = torch.device("cpu")
    a = pool.get(cpu, 10, stream=7)
    assert a.numel() == 1024 and a.dtype == torch.uint8 and not a.any()
    assert pool.get(cpu, 1024, stream=7) is a            # fits: same buffer
    assert pool.get(cpu, 10, stream=8) is not a          # another stream: its own buffer
    b = pool.get(cpu, 5000, stream=7)                    # outgrown
    assert b.numel() == 5000 and b is not a
    assert any(t is a for t in pool._retired), "an outgrown workspace must stay alive: graphs may hold its address"
    assert pool.get(cpu, 2000, stream=7) is b
    assert pool.stats() == {"live": 2, "retired": 1, "bytes": 1024 + 1024 + 5000}


def test_no_allocation_while_capturing(pool_mod, monkeypatch):
    capturing = {"on": False}
    monkeypatch.setattr(torch.cuda, "is_current_stream_capturing", lambda: capturing["on"])
    pool = pool_mod.WorkspacePool(1024, "NF4 matmul")
    cpu = torch.device("cpu")
    capturing["on"] = True
    with pytest.raises(RuntimeError, match="capturing"):
        pool.get(cpu, 10, stream=1)                      # first use of the stream inside a capture
    capturing["on"] = False
    assert pool.reserve(cpu, None, stream=1) == 1024     # reserved before the capture
    capturing["on"] = True
    ws = pool.get(cpu, 512, stream=1)                    # fits: served during capture
    with pytest.raises(RuntimeError, match="one of 1024 bytes"):
        pool.get(cpu, 4096, stream=1)                    # growth during capture is refused ...
    assert pool.get(cpu, 512, stream=1) is ws            # ... and the existing buffer is untouched
    assert pool.stats()["retired"] == 0


def test_functional_pool_covers_llama_shapes(ta):
    lib = ta._lib.load()
    floor = ta.functional._workspace_pool.floor_bytes
    shapes = [(4096, 4096), (1024, 4096), (6144, 4096), (14336, 4096), (28672, 4096), (4096, 14336), (128256, 4096),
              (8192, 8192), (1024, 8192), (10240, 8192), (28672, 8192), (57344, 8192), (8192, 28672), (16384, 8192)]
    for N, K in shapes:
        for M in (1, 2, 4, 8, 16):
            assert lib.nf4hip_gemv_workspace_bytes(M, N, K) <= floor
        for M in (17, 32, 64, 128, 512, 2048, 8192):
            assert lib.nf4hip_gemm_workspace_bytes(M, N, K) <= floor, (M, N, K)
