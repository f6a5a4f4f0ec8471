"""Pins the CPU oracle (oracle/nf4_oracle.c and oracle/nf4_oracle.py) WITHOUT using its own
formulas: closed forms, brute force in float64, torch's own casts, and the committed golden
vectors.  The reference's tests hold no golden vectors or known answers for this path
(thunder/tests/test_transforms.py:116-230,293-344 only compare bitsandbytes with itself), so these
checks are what the oracle stands on.
"""

import os

import numpy as np
import pytest
import torch

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "nf4_golden.npz")


def _from_bits(arr, dtype):
    t = torch.from_numpy(np.ascontiguousarray(arr))
    return t.view(dtype) if dtype in (torch.bfloat16, torch.float16, torch.float32) else t


# ---- constants --------------------------------------------------------------------------------------


def test_codebook_is_the_qlora_closed_form(oracle):
    """16 values = normalised quantiles of N(0,1): 8 positive from linspace(offset, 0.5, 9)[:-1],
    zero, 7 negative from linspace(offset, 0.5, 8)[:-1], offset = 0.9677083 (QLoRA, appendix E)."""
    from scipy.stats import norm

    offset = 0.9677083
    pos = norm.ppf(np.linspace(offset, 0.5, 9)[:-1])
    neg = -norm.ppf(np.linspace(offset, 0.5, 8)[:-1])
    v = np.sort(np.concatenate([pos, [0.0], neg]))
    v = (v / v.max()).astype(np.float32)
    c = oracle.C().lut16().numpy()
    assert np.allclose(c, v, rtol=0, atol=2e-7)  # linspace in double vs torch's float: last-bit slack
    assert (np.diff(c) > 0).all() and c[0] == -1 and c[7] == 0 and c[15] == 1
    assert torch.equal(oracle.C().lut16(), oracle.nf4_lut())
    assert torch.equal(oracle.C().lut16(), oracle.create_normal_map_closed_form())


def test_thresholds_are_midpoints(oracle):
    lut = oracle.C().lut16().double()
    mid = (lut[1:] + lut[:-1]) / 2
    thr = oracle.C().thresholds()
    # fp32 value nearest to the decimal literal: within one ulp of the double midpoint, and four of
    # the midpoints are exact ties between two floats
    assert ((thr.double() - mid).abs() <= mid.abs() * 2.0**-24).all()
    assert torch.equal(thr, oracle.nf4_thresholds_f32())
    for j in range(15):  # strict '>' : a value equal to the threshold stays in the lower code
        assert oracle.C().L.nf4o_code_of(float(thr[j])) == j
        up = np.nextafter(np.float32(thr[j]), np.float32(2))
        assert oracle.C().L.nf4o_code_of(float(up)) == j + 1
    assert oracle.C().L.nf4o_code_of(float("nan")) == 0


def test_float_conversions_match_torch(oracle):
    g = torch.Generator().manual_seed(0)
    bits = torch.randint(-(2**31), 2**31 - 1, (200000,), generator=g, dtype=torch.int64).to(torch.int32)
    f = bits.view(torch.float32)
    f = f[torch.isfinite(f)]
    f = torch.cat([f, torch.tensor([0.0, -0.0, 65504.0, 65520.0, 65519.99, 6e-8, 2.98e-8, 2.99e-8, 6.1e-5, 1e-45, 3.4e38])])
    L = oracle.C().L
    for dtype, fn in ((torch.bfloat16, L.nf4o_f32_to_bf16), (torch.float16, L.nf4o_f32_to_f16)):
        want = f.to(dtype).view(torch.int16).numpy().astype(np.uint16)
        got = np.array([fn(float(v)) for v in f[:20000].tolist()] + [fn(float(v)) for v in f[-11:].tolist()], dtype=np.uint16)
        assert np.array_equal(got, np.concatenate([want[:20000], want[-11:]])), dtype
    h = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16)
    hv = h.view(torch.float16).float()
    ok = torch.isfinite(hv)
    got = torch.tensor([L.nf4o_f16_to_f32(int(v) & 0xFFFF) for v in h.tolist()])
    assert torch.equal(got[ok], hv[ok])


# ---- quantize ---------------------------------------------------------------------------------------


def _nearest_code_f64(w: torch.Tensor, absmax: float, lut: torch.Tensor) -> torch.Tensor:
    s = w.double() / absmax
    return (s.unsqueeze(-1) - lut.double()).abs().argmin(dim=-1)


@pytest.mark.parametrize("amax", [2.0**-7, 0.025146484375, 0.0517578125, 0.10595703125, 1.0, 3.5, 0.0201416015625, 7.62939453125e-06, 65280.0, 0.0703125, 11.5])
def test_quantize_exhaustive_bf16_is_nearest_neighbour(oracle, amax):
    """Every finite bf16 value |x| <= absmax: the threshold rule on x * (1/absmax) picks the nearest
    code value (float64 brute force); no value lands on a tie."""
    bits = torch.arange(0, 1 << 16, dtype=torch.int32).to(torch.int16)
    vals = bits.view(torch.bfloat16)
    vals = vals[torch.isfinite(vals.float()) & (vals.float().abs() <= amax)]
    pad = (-vals.numel()) % 63
    v = torch.cat([vals, torch.zeros(pad, dtype=torch.bfloat16)]).view(-1, 63)
    w = torch.cat([torch.full((v.shape[0], 1), amax, dtype=torch.bfloat16), v], dim=1).contiguous()
    qw, absmax = oracle.C().quantize(w, 64)
    assert (absmax == amax).all()
    codes = oracle.unpack_codes(qw, w.numel()).view(w.shape)
    lut = oracle.C().lut16()
    want = _nearest_code_f64(w.float(), amax, lut)
    d = (w.double() / amax).unsqueeze(-1) - lut.double()
    two_best = d.abs().topk(2, dim=-1, largest=False).values
    assert (two_best[..., 0] < two_best[..., 1]).all(), "a tie: nearest neighbour is ambiguous"
    assert torch.equal(codes, want)
    # both restatements and both rules agree
    for rule in ("threshold", "argmin"):
        qw2, absmax2 = oracle.quantize_4bit_eager(w, 64, rule=rule)
        assert torch.equal(qw2, qw) and torch.equal(absmax2, absmax)


def test_quantize_known_answers(oracle):
    w = torch.zeros(5, 64, dtype=torch.bfloat16)
    w[1, 5] = 0.5                       # single non-zero: code 15 there, code 7 (0.0) elsewhere
    w[2, 0], w[2, 1] = -2.0, 2.0        # -absmax -> 0, +absmax -> 15
    w[3] = 0.25
    w[3, 7] = -0.25 * 0.6961928009986877 * 1.0001  # just past code 1's value, still code 1
    w[4, ::2] = 1.0
    w[4, 1::2] = 1.0 * 0.07958029955625534  # ~ code 8
    qw, absmax = oracle.C().quantize(w, 64)
    codes = oracle.unpack_codes(qw, w.numel()).view(5, 64)
    assert absmax.tolist() == [0.0, 0.5, 2.0, 0.25, 1.0]
    assert (codes[0] == 0).all()  # 0 * (1/0) = NaN: every comparison false
    assert codes[1, 5] == 15 and (codes[1, torch.arange(64) != 5] == 7).all()
    assert codes[2, 0] == 0 and codes[2, 1] == 15 and (codes[2, 2:] == 7).all()
    assert codes[3, 7] == 1 and (codes[3, torch.arange(64) != 7] == 15).all()
    assert (codes[4, ::2] == 15).all() and (codes[4, 1::2] == 8).all()
    # packing: first element in the HIGH nibble
    assert qw[32 + 2, 0].item() == (7 << 4) | 15  # row 1, elements 4 and 5
    assert qw.shape == (5 * 32, 1) and qw.dtype == torch.uint8


def test_quantize_shapes_absmax_and_padding(oracle):
    g = torch.Generator().manual_seed(5)
    for shape, bs in [((2, 2), 64), ((1, 1), 64), ((3, 21), 64), ((64, 1376), 64), ((7, 999), 256), ((5, 4096), 4096), ((1, 130), 128)]:
        w = (torch.randn(*shape, generator=g) * 0.02).to(torch.bfloat16)
        n = w.numel()
        qw, absmax = oracle.C().quantize(w, bs)
        assert qw.shape == ((n + 1) // 2, 1) and absmax.shape == ((n + bs - 1) // bs,)
        flat = w.float().reshape(-1)
        for b in range(absmax.numel()):
            assert absmax[b] == flat[b * bs:(b + 1) * bs].abs().max()  # brute force, order-free
        if n % 2:
            assert qw[-1, 0].item() & 15 == 7  # pad element 0.0 -> code of 0.0
        qw2, absmax2 = oracle.quantize_4bit_eager(w, bs)
        assert torch.equal(qw, qw2) and torch.equal(absmax, absmax2)


def test_roundtrip_is_ordered_and_bounded(oracle):
    """dequant(quant(w)) stays within half the largest code gap of w, ELEMENT BY ELEMENT: a swapped
    nibble order or a transposed block index would break it."""
    g = torch.Generator().manual_seed(9)
    w = (torch.randn(33, 192, generator=g) * torch.logspace(-3, 1, 33).unsqueeze(1)).to(torch.bfloat16)
    qw, absmax = oracle.C().quantize(w, 64)
    deq = oracle.C().dequantize(qw, absmax, oracle.C().lut16(), 64, torch.float32, w.shape)
    gap = oracle.C().lut16().diff().max().item()  # 0.3038 between -1 and -0.696
    scale = absmax.repeat_interleave(64).view(w.shape)
    assert ((deq - w.float()).abs() <= scale * gap / 2 * (1 + 1e-6)).all()
    assert (deq.sign() * w.float().sign() >= 0).all()


# ---- dequantize -------------------------------------------------------------------------------------


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_dequantize_exhaustive_against_float64(oracle, dtype):
    """16 codes x every non-negative finite bf16 absmax.  A 24-bit x 8-bit significand product is
    exact in float64, so float64 -> fp32 -> dtype reproduces 'one fp32 multiply, one rounding'."""
    bits = torch.arange(0, 0x7F80, dtype=torch.int32).to(torch.int16)
    amax = bits.view(torch.bfloat16).float()
    nb = amax.numel()
    codes = (torch.arange(64) % 16).to(torch.uint8).repeat(nb, 1)
    packed = ((codes[:, 0::2] << 4) | codes[:, 1::2]).reshape(-1, 1).contiguous()
    lut = oracle.C().lut16()
    got = oracle.C().dequantize(packed, amax, lut, 64, dtype, (nb, 64))
    want = (lut.double()[codes.long()] * amax.double().unsqueeze(1)).to(torch.float32).to(dtype)
    view = torch.int32 if dtype == torch.float32 else torch.int16
    assert torch.equal(got.view(view), want.view(view))
    assert torch.equal(oracle.dequantize_4bit_eager(packed, amax, lut, 64, dtype, (nb, 64)).view(view), want.view(view))


def test_dequantize_lut_rounding_modes_differ_where_expected(oracle):
    """Pre-rounding the table to bf16 (bitsandbytes' eager backend) changes many outputs but never
    codes 0, 7, 15, whose values are exact in bf16."""
    g = torch.Generator().manual_seed(3)
    amax = (torch.rand(4096, generator=g) * 0.1).to(torch.bfloat16).float()
    codes = (torch.arange(64) % 16).to(torch.uint8).repeat(4096, 1)
    packed = ((codes[:, 0::2] << 4) | codes[:, 1::2]).reshape(-1, 1).contiguous()
    lut = oracle.C().lut16()
    a = oracle.C().dequantize(packed, amax, lut, 64, torch.bfloat16, (4096, 64))
    b = oracle.C().dequantize(packed, amax, lut.to(torch.bfloat16).float(), 64, torch.bfloat16, (4096, 64))
    diff = (a.view(torch.int16) != b.view(torch.int16)).view(4096, 4, 16).float().mean(dim=(0, 1))
    assert diff[0] == 0 and diff[7] == 0 and diff[15] == 0
    assert 0.1 < diff.mean() < 0.35


# ---- matmul -----------------------------------------------------------------------------------------


def test_matmul_reduces_to_textbook(oracle):
    g = torch.Generator().manual_seed(21)
    for (M, N, K, bs, bias) in [(1, 8, 64, 64, False), (3, 20, 192, 64, True), (2, 6, 1376, 64, True), (5, 3, 256, 128, False)]:
        w = (torch.randn(N, K, generator=g) * 0.05).to(torch.bfloat16)
        x = torch.randn(M, K, generator=g).to(torch.bfloat16)
        b = torch.randn(N, generator=g).to(torch.bfloat16) if bias else None
        qw, absmax = oracle.C().quantize(w, bs)
        deq = oracle.C().dequantize(qw, absmax, oracle.C().lut16(), bs, torch.bfloat16, (N, K))
        want = x.double() @ deq.double().t() + (b.double() if bias else 0)
        got = oracle.C().matmul(x, qw, b, absmax, oracle.C().lut16(), bs, torch.bfloat16, (N, K))
        assert torch.equal(got.view(torch.int16), want.to(torch.bfloat16).view(torch.int16))
        eager = oracle.matmul_4bit_eager(x, qw, b, absmax, oracle.C().lut16(), bs, torch.bfloat16, (N, K))
        torch.testing.assert_close(eager.float(), want.float(), rtol=2e-2, atol=2e-2)
    # brute force, tiny
    x = torch.tensor([[1.0, -2.0] + [0.0] * 62], dtype=torch.bfloat16)
    w = torch.zeros(2, 64, dtype=torch.bfloat16)
    w[0, 0], w[0, 1], w[1, 0] = 1.0, 1.0, -0.5
    qw, absmax = oracle.C().quantize(w, 64)
    y = oracle.C().matmul(x, qw, None, absmax, oracle.C().lut16(), 64, torch.bfloat16, (2, 64))
    assert y.tolist() == [[-1.0, -0.5]]


# ---- nested absmax ----------------------------------------------------------------------------------


def test_dynamic_map_closed_form(oracle):
    D = oracle.create_dynamic_map()
    assert D.shape == (256,) and D.unique().numel() == 256 and (D.diff() > 0).all()
    assert D[0].item() == pytest.approx(-0.99296875, abs=1e-7) and D[127] == 0 and D[255] == 1
    pos, neg = D[128:255], D[:127].flip(0)
    assert torch.equal(pos, -neg)  # symmetric except for the lone 1.0
    # decade i holds 2^i values: means of linspace(0.1, 1, 2^i + 1) scaled by 10^(i-6)
    idx = 0
    for i in range(7):
        cnt = 2**i
        seg = pos[idx:idx + cnt].double() / 10.0 ** (i - 6)
        edges = np.linspace(0.1, 1, cnt + 1)
        assert np.allclose(seg.numpy(), (edges[:-1] + edges[1:]) / 2, rtol=1e-6)
        idx += cnt


def test_nested_absmax_invariants(oracle):
    g = torch.Generator().manual_seed(13)
    absmax = (torch.rand(1000, generator=g) * 0.08 + 0.01).float()
    D = oracle.create_dynamic_map()
    off = oracle.C().dq_offset(absmax)
    assert off == float(absmax.double().mean().float())
    q, a2 = oracle.C().dq_compress(absmax, D, off)
    r = absmax - torch.tensor(off)
    for c in range(4):
        blk = r[c * 256:(c + 1) * 256]
        assert a2[c] == blk.abs().max()
        s = blk * (1.0 / a2[c])
        want = (s.unsqueeze(-1) - D).abs().argmin(dim=-1)  # nearest neighbour, lowest index on ties
        assert torch.equal(q[c * 256:(c + 1) * 256].long(), want)
    rec = oracle.C().dq_reconstruct(q, a2, D, off)
    assert torch.equal(rec, D[q.long()] * a2.repeat_interleave(256)[:1000] + torch.tensor(off))
    # 8-bit nested code: relative error of the reconstruction is small and bounded by the map's spacing
    assert ((rec - absmax).abs() <= a2.repeat_interleave(256)[:1000] * D.diff().max() / 2 + 1e-9).all()
    q2, a22, off2 = oracle.dq_compress_eager(absmax, D)
    assert torch.equal(q, q2) and torch.equal(a2, a22) and off == off2
    # all-zero statistics: code of 0.0, reconstruction = offset = 0
    z = torch.zeros(300)
    qz, az = oracle.C().dq_compress(z, D, 0.0)
    assert (qz == 127).all() and (az == 0).all() and (oracle.C().dq_reconstruct(qz, az, D, 0.0) == 0).all()


# ---- nested absmax, pinned by mathematics -----------------------------------------------------------
#
# No file of the reference uses compress_statistics, so there is no call site, test or fixture to pin these
# against; what follows checks the oracle's nested functions against exact rational arithmetic
# (fractions.Fraction), math.fsum and closed forms -- none of them a restatement of the oracle's own fp32
# formulas -- with inputs chosen so that a dropped offset, a fused multiply-add, fp32 accumulation of the
# mean, a wrong nested block index or a wrong tie rule each fail at least one check.

from fractions import Fraction
import math


def _f32(x: float) -> float:
    return float(np.float32(x))


def _round_fraction_to_f32(v: Fraction) -> float:
    """Round-to-nearest-even of an exact rational to binary32 (normal range), by integer arithmetic."""
    if v == 0:
        return 0.0
    sign = -1 if v < 0 else 1
    a = abs(v)
    e = a.numerator.bit_length() - a.denominator.bit_length()  # 2^(e-1) <= a < 2^(e+1)
    if a < Fraction(2) ** e:
        e -= 1
    assert Fraction(2) ** e <= a < Fraction(2) ** (e + 1)
    assert -126 <= e <= 127
    scaled = a / Fraction(2) ** (e - 23)  # in [2^23, 2^24)
    m = scaled.numerator // scaled.denominator
    rem = scaled - m
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and m % 2 == 1):
        m += 1
    return sign * float(m) * 2.0 ** (e - 23)  # m <= 2^24 and the power of two are exact in double


def test_round_fraction_helper_agrees_with_numpy_casts():
    g = np.random.default_rng(5)
    for x in np.concatenate([g.standard_normal(2000) * 0.05, g.standard_normal(2000) * 1e-4, [1.0, 0.1, 1 / 3, 2**-20 * (2**24 + 1)]]):
        assert _round_fraction_to_f32(Fraction(float(x))) == _f32(float(x))
    # an exact tie goes to the even significand: 2^24 + 1 is halfway between 2^24 and 2^24 + 2
    assert _round_fraction_to_f32(Fraction(2**24 + 1)) == float(2**24)
    assert _round_fraction_to_f32(Fraction(2**24 + 3)) == float(2**24 + 4)


def test_dynamic_map_closed_form_by_rationals(oracle):
    """256 distinct values; 0 and 1; for decade i = 0..6, 2^i positive values, equally spaced by 0.9 * 10^(i-6) / 2^i,
    the first at (0.1 + 0.45 / 2^i) * 10^(i-6) -- all inside (0.1 * 10^(i-6), 10^(i-6)) -- and their mirror images."""
    D = oracle.create_dynamic_map()
    vals = [float(v) for v in D]
    assert len(set(vals)) == 256 and vals == sorted(vals)
    # the minimum is -(0.1 + 0.9 * 127 / 128) = -0.99296875 up to the fp32 linspace's last bit (-0.99296874 as published)
    assert vals[127] == 0.0 and vals[255] == 1.0 and abs(vals[0] + 0.99296875) <= 2.0**-23
    pos = vals[128:255]
    assert [-v for v in reversed(vals[:127])] == pos, "the map is symmetric except for the lone 1.0"
    k = 0
    for i in range(7):
        cnt = 2**i
        scale = Fraction(10) ** (i - 6)
        lo, hi = Fraction(1, 10) * scale, scale
        seg = pos[k:k + cnt]
        assert all(lo < Fraction(v) < hi for v in seg), f"decade {i} out of its edges"
        for j, v in enumerate(seg):
            exact = (Fraction(1, 10) + Fraction(9, 10) * Fraction(2 * j + 1, 2 * cnt)) * scale
            # the published construction goes through fp32 linspace and a double product: allow 2 ulp of fp32
            assert abs(Fraction(v) - exact) <= exact * Fraction(2, 2**23), (i, j, v, float(exact))
        k += cnt
    assert k == 127


def test_offset_is_the_correctly_rounded_mean(oracle):
    g = torch.Generator().manual_seed(99)
    cases = [
        (torch.rand(100000, generator=g) * 0.08 + 0.01).float(),
        torch.cat([torch.full((1,), 1000.0), torch.rand(70000, generator=g) * 1e-4]).float(),  # fp32 accumulation loses the tail
        torch.tensor([0.1, 0.2, 0.30000001, 1e-8], dtype=torch.float32),
        torch.full((3,), 0.1, dtype=torch.float32),
    ]
    for a in cases:
        exact = Fraction(0)
        for v in a.tolist():
            exact += Fraction(v)
        want = _round_fraction_to_f32(exact / len(a))
        assert oracle.C().dq_offset(a) == want
        assert want == _f32(math.fsum(a.tolist()) / len(a))
    # the case with one large value must tell a float32 running sum from the exact mean
    a = cases[1]
    running = np.float32(0)
    for v in a.numpy():
        running = np.float32(running + v)
    assert _f32(float(running) / len(a)) != oracle.C().dq_offset(a)


def test_nested_codes_are_exact_nearest_neighbours(oracle):
    """absmax2 = max |absmax - offset| (each difference rounded to fp32, as the format stores fp32 statistics), code =
    the map entry nearest to r / absmax2 in EXACT arithmetic.  The oracle works in fp32 (r * (1 / absmax2)), so it may
    differ from the exact rule only where r / absmax2 lies within fp32 rounding distance of the midpoint of two map
    entries; every such case found by the sweep is counted and its distance from the midpoint checked."""
    D = oracle.create_dynamic_map()
    Dq = [Fraction(float(v)) for v in D]
    mids = [(Dq[j] + Dq[j + 1]) / 2 for j in range(255)]
    g = torch.Generator().manual_seed(7)
    # two nested blocks of ordinary statistics, plus a block built to land near every midpoint
    ordinary = (torch.rand(512, generator=g) * 0.08 + 0.01).float()
    probe = torch.tensor([float(m) for m in mids] + [1.0], dtype=torch.float32)  # absmax2 = 1, offset = 0 below
    near_ties = {}
    for name, absmax, offset in (("ordinary", ordinary, oracle.C().dq_offset(ordinary)), ("probe", probe, 0.0)):
        near_ties[name] = 0
        q, a2 = oracle.C().dq_compress(absmax, D, offset)
        nb = absmax.numel()
        for c in range((nb + 255) // 256):
            blk = absmax[c * 256:(c + 1) * 256].tolist()
            r = [Fraction(float(np.float32(v) - np.float32(offset))) for v in blk]  # fp32 subtraction, exact afterwards
            m = max(abs(x) for x in r)
            assert Fraction(float(a2[c])) == m, "absmax2 is the exact maximum of the fp32 differences"
            for i, x in enumerate(r):
                s = x / m
                dist = [abs(s - d) for d in Dq]
                best = min(dist)
                winners = [j for j, d in enumerate(dist) if d == best]
                got = int(q[c * 256 + i])
                if got in winners:
                    if len(winners) > 1:
                        assert got == winners[0], "exact tie: the lowest index wins"
                    continue
                # not the exact nearest neighbour: only legitimate within fp32 rounding of a midpoint
                near_ties[name] += 1
                j = min(got, winners[0])
                assert abs(got - winners[0]) == 1 and abs(s - mids[j]) <= abs(mids[j]) * Fraction(4, 2**24) + Fraction(1, 2**40), (i, got, winners)
    # ordinary statistics never land that close; the probe block may, for some of its 255 midpoints
    assert near_ties["ordinary"] == 0 and near_ties["probe"] <= 255, near_ties
    print("nested codes: near-midpoint cases where fp32 and exact arithmetic pick neighbouring entries:", near_ties)
    q, _ = oracle.C().dq_compress(ordinary, D, oracle.C().dq_offset(ordinary))
    assert len(set(q.tolist())) > 100  # the sweep really exercises the map, not a handful of codes


def test_nested_block_indexing_and_partial_last_block(oracle):
    """Statistics of different magnitude per nested block: a wrong block index or a maximum taken over the wrong range
    changes absmax2; 600 entries = two full nested blocks and one of 88."""
    D = oracle.create_dynamic_map()
    a = torch.cat([torch.linspace(0.01, 0.02, 256), torch.linspace(1.0, 3.0, 256), torch.linspace(10.0, 10.5, 88)]).float()
    off = oracle.C().dq_offset(a)
    q, a2 = oracle.C().dq_compress(a, D, off)
    assert a2.numel() == 3 and q.numel() == 600
    for c, (lo, hi) in enumerate(((0, 256), (256, 512), (512, 600))):
        want = max(abs(float(np.float32(v) - np.float32(off))) for v in a[lo:hi].tolist())
        assert float(a2[c]) == want
    # the element that attains the maximum gets code 255 (+1.0) or 0 (the most negative entry's neighbour -1 is absent:
    # the map's minimum is -0.99296875, so a value of exactly -absmax2 maps to index 0)
    r = a.numpy() - np.float32(off)
    for c, (lo, hi) in enumerate(((0, 256), (256, 512), (512, 600))):
        i = lo + int(np.abs(r[lo:hi]).argmax())
        assert int(q[i]) == (255 if r[i] > 0 else 0)


def test_reconstruction_is_multiply_then_add_rounded_twice(oracle):
    D = oracle.create_dynamic_map()
    g = torch.Generator().manual_seed(21)
    q = torch.randint(0, 256, (4000,), generator=g, dtype=torch.int64).to(torch.uint8)
    a2 = (torch.rand(16, generator=g) * 0.05 + 1e-3).float()
    off = _f32(0.0423)
    rec = oracle.C().dq_reconstruct(q, a2, D, off)
    fused_differs = 0
    for i in range(q.numel()):
        d, s = Fraction(float(D[int(q[i])])), Fraction(float(a2[i // 256]))
        p = _round_fraction_to_f32(d * s)
        want = _round_fraction_to_f32(Fraction(p) + Fraction(off))
        assert float(rec[i]) == want, i
        fused_differs += want != _round_fraction_to_f32(d * s + Fraction(off))
    # the sample tells two roundings from one (a fused multiply-add) ...
    assert fused_differs > 50
    # ... a dropped offset, and swapped nested blocks
    assert not torch.equal(rec, oracle.C().dq_reconstruct(q, a2, D, 0.0))
    assert not torch.equal(rec, oracle.C().dq_reconstruct(q, a2.flip(0), D, off))
    # round trip: compress then reconstruct stays within half the widest map gap of each nested block's scale
    absmax = (torch.rand(1000, generator=g) * 0.08 + 0.01).float()
    o = oracle.C().dq_offset(absmax)
    qq, aa = oracle.C().dq_compress(absmax, D, o)
    back = oracle.C().dq_reconstruct(qq, aa, D, o)
    gap = float(D.diff().max())
    assert ((back - absmax).abs() <= aa.repeat_interleave(256)[:1000] * (gap / 2) + 1e-7).all()


# ---- golden vectors ---------------------------------------------------------------------------------


def test_golden_vectors(oracle):
    G = np.load(GOLDEN)
    cases = {"bf16_4x130": ((4, 130), torch.bfloat16, 64), "bf16_2x2": ((2, 2), torch.bfloat16, 64),
             "f16_3x21": ((3, 21), torch.float16, 64), "f32_8x64": ((8, 64), torch.float32, 64),
             "bf16_16x256_b128": ((16, 256), torch.bfloat16, 128)}
    assert torch.equal(_from_bits(G["lut16"], torch.float32), oracle.C().lut16())
    assert torch.equal(_from_bits(G["thresholds"], torch.float32), oracle.C().thresholds())
    for name, (shape, dtype, bs) in cases.items():
        w = _from_bits(G[f"{name}.w"], dtype).reshape(shape)
        packed = torch.from_numpy(G[f"{name}.packed"])
        absmax = _from_bits(G[f"{name}.absmax"], torch.float32)
        for impl in (oracle.C().quantize, oracle.quantize_4bit_eager):
            qw, am = impl(w, bs)
            assert torch.equal(qw, packed) and torch.equal(am, absmax), name
        for mode in ("f32", "rounded"):
            lut = oracle.nf4_lut() if mode == "f32" else oracle.nf4_lut().to(dtype).float()
            want = torch.from_numpy(G[f"{name}.deq_{mode}"]).reshape(shape)
            got = oracle.C().dequantize(packed, absmax, lut, bs, dtype, shape)
            view = torch.int32 if dtype == torch.float32 else torch.int16
            assert torch.equal(got.view(view), want), (name, mode)
    x = _from_bits(G["mm.x"], torch.bfloat16)
    b = _from_bits(G["mm.bias"], torch.bfloat16)
    y = oracle.C().matmul(x, torch.from_numpy(G["mm.packed"]), b, _from_bits(G["mm.absmax"], torch.float32),
                          oracle.nf4_lut(), 64, torch.bfloat16, (48, 256))
    assert torch.equal(y.view(torch.int16), torch.from_numpy(G["mm.y"]))
    D = _from_bits(G["dq.map256"], torch.float32)
    assert torch.equal(D, oracle.create_dynamic_map())
    q, a2 = oracle.C().dq_compress(_from_bits(G["mm.absmax"], torch.float32), D, float(G["dq.offset"][0]))
    assert torch.equal(q, torch.from_numpy(G["dq.q"])) and torch.equal(a2, _from_bits(G["dq.absmax2"], torch.float32))
