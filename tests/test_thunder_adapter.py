"""thunder_adapter.install() against a minimal stand-in `thunder` package (tests/fake_thunder): host logic only.

What a real Thunder would exercise and this cannot: tracing, the dispatch pass keeping the bound symbol, execution
of a compiled module.  What it does check: the executor and operator are registered once and found again, the
operator's meta function infers the output shape the way the reference's does (quantization.py:29-32), the
transform subclass never runs the reference's bitsandbytes-importing __init__, quantize_weight follows the
reference's device policy and returns the (qweight, state) pair the class reads, and the trace hook runs with the
module global pointing at the HIP symbol and restores whatever was there -- also when the hook raises, and also
when the global did not exist."""

import importlib
import os
import sys
import types

import pytest
import torch

import fake_backend

FAKE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "fake_thunder")


@pytest.fixture
def fake_thunder():
    saved = {k: v for k, v in sys.modules.items() if k == "thunder" or k.startswith("thunder.")}
    for k in saved:
        del sys.modules[k]
    sys.path.insert(0, FAKE)
    try:
        yield importlib.import_module("thunder")
    finally:
        sys.path.remove(FAKE)
        for k in [k for k in sys.modules if k == "thunder" or k.startswith("thunder.")]:
            del sys.modules[k]
        sys.modules.update(saved)


def test_install_without_thunder_says_so(ta):
    if importlib.util.find_spec("thunder") is not None:
        pytest.skip("a thunder package is importable here")
    adapter = importlib.import_module("lightning-thunder_amd.thunder_adapter")
    with pytest.raises(ImportError, match="lightning-thunder"):
        adapter.install()


def test_install_on_a_stand_in_thunder(ta, fake_thunder):
    adapter = importlib.import_module("lightning-thunder_amd.thunder_adapter")
    ref = importlib.import_module("thunder.transforms.quantization")
    T = adapter.install()
    ex = fake_thunder.extend.get_executor("quant_hip_nf4")
    assert ex is T.executor and set(ex.opmap) == {"hip_matmul_nf4"}
    assert adapter.install().executor is ex  # a second install finds the executor, registers nothing twice
    sym = ex.opmap["hip_matmul_nf4"]

    # meta: [..., K] x weight [N, K] -> [..., N]; a wrong K is refused
    x = types.SimpleNamespace(shape=(2, 5, 64), dtype=torch.bfloat16, device="cuda")
    out = sym.meta(x, None, None, None, None, 64, torch.bfloat16, (48, 64))
    assert out.shape == (2, 5, 48)
    with pytest.raises(AssertionError):
        sym.meta(x, None, None, None, None, 64, torch.bfloat16, (48, 32))

    t = T(blocksize=128)  # must not reach the reference's __init__
    assert issubclass(T, ref.BitsAndBytesLinearQuant4bit)
    assert t.quant_states == {} and t.quantized_submodule_names == set() and t.blocksize == 128

    with fake_backend.installed(ta):
        w = (torch.randn(48, 256, generator=torch.Generator().manual_seed(1)) * 0.02).to(torch.bfloat16)
        qw, state = t.quantize_weight(w)
        assert qw.dtype == torch.uint8 and qw.numel() == 48 * 256 // 2
        assert state.shape == (48, 256) and state.dtype == torch.bfloat16 and state.blocksize == 128
        assert state.absmax.numel() == 48 * 256 // 128 and state.code.numel() == 16
        qz, sz = t.quantize_weight(torch.empty(48, 256, dtype=torch.bfloat16, device="meta"))  # meta stands for zeros
        assert qz.device.type == "cpu" and not bool(sz.absmax.any())
        # the registered implementation is the package's matmul (here: its CPU stand-in)
        xr = torch.randn(3, 256, generator=torch.Generator().manual_seed(2)).to(torch.bfloat16)
        y = sym(xr, qw, None, state.absmax, state.code, 128, torch.bfloat16, (48, 256))
        assert y.shape == (3, 48)
        deq = ta.functional.dequantize_nf4(qw, state.absmax, state.code, 128, torch.bfloat16, (48, 256))
        torch.testing.assert_close(y.float(), (xr.float() @ deq.float().t()), rtol=2e-2, atol=2e-2)

    # the trace hook sees the HIP symbol under the reference's global name, and the name is restored afterwards
    assert not hasattr(ref, "bnb_matmul_nf4")
    _, (comp, bound), _ = t.transform_traces_pre_prologue("p", "c", "e")
    assert comp == "c" and bound is sym and not hasattr(ref, "bnb_matmul_nf4")
    ref.bnb_matmul_nf4 = "theirs"
    _, (_, bound), _ = t.transform_traces_pre_prologue("p", "c", "e")
    assert bound is sym and ref.bnb_matmul_nf4 == "theirs"
    with pytest.raises(RuntimeError, match="trace rewrite failed"):
        t.transform_traces_pre_prologue("p", "c", "e", fail=True)
    assert ref.bnb_matmul_nf4 == "theirs"


@pytest.mark.gpu
@pytest.mark.parametrize("M", [1, 16, 512])
def test_installed_operator_runs_the_hip_kernels(ta, oracle, fake_thunder, M):
    """``install()`` on the stand-in ``thunder`` with the real libnf4hip.so behind it (no CPU stand-in installed): the
    subclass's ``quantize_weight`` on a GPU tensor gives the oracle's codes and absmax bit for bit, keeps the
    reference's device policy for CPU and meta weights (thunder/transforms/quantization.py:53-63), and the operator
    registered on the executor (thunder/extend/__init__.py:146-198) multiplies GPU tensors within rtol = atol = 2e-2
    of the oracle's float64 dequantize-then-matmul -- one row of x (row kernel), sixteen (tile kernel), 512 (GEMM)."""
    print(f"thunder adapter on the HIP kernels M={M}", flush=True)
    adapter = importlib.import_module("lightning-thunder_amd.thunder_adapter")
    T = adapter.install()
    ex = fake_thunder.extend.get_executor("quant_hip_nf4")
    sym = ex.opmap["hip_matmul_nf4"]
    assert ex is T.executor
    N, K = 1536, 4096
    dev = torch.device("cuda:0")
    w = (torch.randn(N, K, generator=torch.Generator().manual_seed(11)) * 0.02).to(torch.bfloat16)
    t = T()
    qw, state = t.quantize_weight(w.to(dev))
    qw_o, absmax_o = oracle.C().quantize(w, 64)
    assert qw.is_cuda and state.absmax.is_cuda and state.code.is_cuda
    assert torch.equal(qw.cpu(), qw_o) and torch.equal(state.absmax.cpu().view(torch.int32), absmax_o.view(torch.int32))
    assert torch.equal(state.code.cpu(), oracle.nf4_lut()) and state.shape == (N, K) and state.dtype == torch.bfloat16
    # a CPU weight is quantised on the GPU (the reference moves it there), a meta weight stands for zeros
    qc, sc = t.quantize_weight(w)
    assert qc.is_cuda and torch.equal(qc.cpu(), qw_o)
    qz, sz = t.quantize_weight(torch.empty(N, K, dtype=torch.bfloat16, device="meta"))
    assert qz.is_cuda and not bool(sz.absmax.any())

    x = torch.randn(M, K, generator=torch.Generator().manual_seed(12 + M)).to(torch.bfloat16)
    bias = (torch.randn(N, generator=torch.Generator().manual_seed(13)) * 0.5).to(torch.bfloat16)
    for b in (None, bias):
        y = sym(x.to(dev), qw, None if b is None else b.to(dev), state.absmax, state.code, 64, torch.bfloat16, (N, K))
        assert y.is_cuda and y.shape == (M, N) and y.dtype == torch.bfloat16
        ref = oracle.matmul_4bit_f64(x, qw_o, b, absmax_o, oracle.nf4_lut(), 64, torch.bfloat16, (N, K))
        torch.testing.assert_close(y.cpu().float(), ref.float(), rtol=2e-2, atol=2e-2)
    # leading dimensions pass through, as the meta function promises
    y3 = sym(x.to(dev).reshape(1, M, K), qw, None, state.absmax, state.code, 64, torch.bfloat16, (N, K))
    assert y3.shape == sym.meta(types.SimpleNamespace(shape=(1, M, K), dtype=torch.bfloat16, device="cuda"), None, None, None, None,
                                64, torch.bfloat16, (N, K)).shape
