"""The choice between the fused GEMM and dequantize + dense GEMM (the hand-written kernel, or the vendor library's when
it wins by more than 3 %) for many rows of x, made by timing the routes once per shape and device
(functional._measure_route): whatever it picks must be one of the routes, must be what ``fused_route`` then reports,
must give the oracle's result, and must not be attempted under stream capture."""

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda"


def _case(ta, oracle, M, N, K, seed):
    g = torch.Generator().manual_seed(seed)
    w = (torch.randn(N, K, generator=g) * 0.02).to(torch.bfloat16)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    qw, absmax, code = ta.quantize_nf4(w.to(DEV))
    ref = oracle.matmul_4bit_f64(x, qw.cpu(), None, absmax.cpu(), oracle.nf4_lut(), 64, torch.bfloat16, (N, K))
    return x.to(DEV), qw, absmax, code, ref


@pytest.mark.parametrize("M,N,K", [(512, 4096, 4096), (2048, 6144, 4096), (4096, 1024, 4096)])
def test_first_call_times_both_routes_and_later_calls_follow(ta, oracle, monkeypatch, M, N, K):
    print(f"route calibration M={M} N={N} K={K}", flush=True)
    F = ta.functional
    monkeypatch.setenv("NF4HIP_CALIBRATE", "1")
    monkeypatch.setattr(F, "_route_measured", {})
    x, qw, absmax, code, ref = _case(ta, oracle, M, N, K, seed=M + N)
    key = F._route_key(x.device, M, N, K, 64, False, False)
    model = F.fused_route(x, None, 64, torch.bfloat16, (N, K))
    assert model in ("gemm", "dequant+gemm") and key not in F._route_measured
    ran = []
    real = F._matmul_nf4_on
    monkeypatch.setattr(F, "_matmul_nf4_on", lambda *a: (ran.append(a[-1]), real(*a))[1])
    y = F.matmul_nf4(x, qw, None, absmax, code, 64, torch.bfloat16, (N, K))
    picked = F._route_measured[key]
    assert picked in ("gemm", "dequant+gemm", "dequant+libgemm") and F.fused_route(x, None, 64, torch.bfloat16, (N, K)) == picked
    # all three timed, the winner ran last
    assert ran.count("gemm") >= 4 and ran.count("dequant+gemm") >= 4 and ran.count("dequant+libgemm") >= 4 and ran[-1] == picked
    torch.testing.assert_close(y.cpu().float(), ref.float(), rtol=2e-2, atol=2e-2)
    ran.clear()
    y2 = F.matmul_nf4(x, qw, None, absmax, code, 64, torch.bfloat16, (N, K))
    assert ran == [picked]  # no second measurement
    assert torch.equal(y2, y)
    # every route gives the oracle's result, whichever was picked
    for route in ("gemm", "dequant+gemm", "dequant+libgemm"):
        torch.testing.assert_close(real(x, qw, None, absmax, code, 64, torch.bfloat16, (N, K), route).cpu().float(), ref.float(),
                                   rtol=2e-2, atol=2e-2)


def test_library_gemm_can_be_kept_out_and_needs_a_margin(ta, oracle, monkeypatch):
    print("route calibration: library GEMM switched off / handicap", flush=True)
    F = ta.functional
    M, N, K = 512, 2048, 1024
    x, qw, absmax, code, ref = _case(ta, oracle, M, N, K, seed=9)
    monkeypatch.setenv("NF4HIP_CALIBRATE", "1")
    monkeypatch.setenv("NF4HIP_LIBRARY_GEMM", "0")
    monkeypatch.setattr(F, "_route_measured", {})
    ran = []
    real = F._matmul_nf4_on
    monkeypatch.setattr(F, "_matmul_nf4_on", lambda *a: (ran.append(a[-1]), real(*a))[1])
    y = F.matmul_nf4(x, qw, None, absmax, code, 64, torch.bfloat16, (N, K))
    assert "dequant+libgemm" not in ran and set(ran) == {"gemm", "dequant+gemm"}
    torch.testing.assert_close(y.cpu().float(), ref.float(), rtol=2e-2, atol=2e-2)
    # the choice itself, on made-up times: the library has to win by more than 3 %; the fused kernel takes a 2 % tie
    import types

    def pick(times):
        clock = iter(times.values())
        fake_event = lambda **k: types.SimpleNamespace(record=lambda: None, synchronize=lambda: None, elapsed_time=lambda other: next(clock))
        monkeypatch.setattr(torch.cuda, "Event", fake_event)
        return F._measure_route(("made-up",), {name: (lambda: None) for name in times})

    assert pick({"gemm": 1.10, "dequant+gemm": 1.02, "dequant+libgemm": 1.00}) == "dequant+gemm"
    assert pick({"gemm": 1.10, "dequant+gemm": 1.05, "dequant+libgemm": 1.00}) == "dequant+libgemm"
    assert pick({"gemm": 1.03, "dequant+gemm": 1.02, "dequant+libgemm": 1.00}) == "gemm"
    assert pick({"gemm": 1.00, "dequant+gemm": 1.01}) == "gemm"


def test_no_measurement_under_stream_capture_or_when_switched_off(ta, oracle, monkeypatch):
    print("route calibration: capture / switched off", flush=True)
    F = ta.functional
    M, N, K = 256, 2048, 1024
    x, qw, absmax, code, ref = _case(ta, oracle, M, N, K, seed=5)
    monkeypatch.setattr(F, "_route_measured", {})
    monkeypatch.setenv("NF4HIP_CALIBRATE", "0")
    F.matmul_nf4(x, qw, None, absmax, code, 64, torch.bfloat16, (N, K))
    assert not F._route_measured
    monkeypatch.setenv("NF4HIP_CALIBRATE", "1")
    F.reserve_workspace(x.device)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        F.reserve_workspace(x.device)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            y = F.matmul_nf4(x, qw, None, absmax, code, 64, torch.bfloat16, (N, K))
    torch.cuda.current_stream().wait_stream(side)
    assert not F._route_measured  # a capture records, it cannot time: the model's route was taken
    for _ in range(3):
        graph.replay()
        torch.cuda.synchronize()
        torch.testing.assert_close(y.cpu().float(), ref.float(), rtol=2e-2, atol=2e-2)
