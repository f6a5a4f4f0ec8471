"""Writes tests/golden/nf4_golden.npz: small seeded inputs with the outputs of the CPU oracle
(C restatement; the torch-eager restatement must agree before anything is written).

The reference holds no golden vectors for this path (its tests compare bitsandbytes with itself)
and neither thunder nor bitsandbytes can be imported here, so these vectors pin the oracle against
regressions and tie the three implementations (C, torch-eager, HIP) to one set of numbers; the
oracle itself is pinned by the closed forms and brute-force checks in tests/test_oracle.py.

Run from the repo root:  python tests/golden/make_golden.py
"""

import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import nf4_oracle as O  # noqa: E402


def bits(t: torch.Tensor) -> np.ndarray:
    if t.dtype in (torch.bfloat16, torch.float16):
        return t.contiguous().view(torch.int16).numpy().copy()
    if t.dtype == torch.float32:
        return t.contiguous().view(torch.int32).numpy().copy()
    return t.contiguous().numpy().copy()


def main():
    out = {}
    g = torch.Generator().manual_seed(20240607)
    cases = {
        "bf16_4x130": ((4, 130), torch.bfloat16, 64),      # partial last block, blocks straddle rows
        "bf16_2x2": ((2, 2), torch.bfloat16, 64),          # n < blocksize (Linear(2,2) of the reference's test)
        "f16_3x21": ((3, 21), torch.float16, 64),          # odd n: pad nibble
        "f32_8x64": ((8, 64), torch.float32, 64),
        "bf16_16x256_b128": ((16, 256), torch.bfloat16, 128),
    }
    for name, (shape, dtype, bs) in cases.items():
        w = (torch.randn(*shape, generator=g) * 0.02).to(dtype)
        if name == "bf16_4x130":
            w[1, :64] = 0  # a zero region
            w[2, 5] = 1.5  # an outlier
        qw, absmax = O.C().quantize(w, bs)
        qw2, absmax2 = O.quantize_4bit_eager(w, bs)
        assert torch.equal(qw, qw2) and torch.equal(absmax, absmax2), name
        out[f"{name}.w"] = bits(w)
        out[f"{name}.packed"] = bits(qw)
        out[f"{name}.absmax"] = bits(absmax)
        for mode in ("f32", "rounded"):
            lut = O.nf4_lut() if mode == "f32" else O.nf4_lut().to(dtype).float()
            d = O.C().dequantize(qw, absmax, lut, bs, dtype, shape)
            d2 = O.dequantize_4bit_eager(qw, absmax, lut, bs, dtype, shape)
            assert torch.equal(bits_t(d), bits_t(d2)), (name, mode)
            out[f"{name}.deq_{mode}"] = bits(d)
    # matmul + nested absmax on one case
    N, K, M = 48, 256, 3
    w = (torch.randn(N, K, generator=g) * 0.02).to(torch.bfloat16)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    b = torch.randn(N, generator=g).to(torch.bfloat16)
    qw, absmax = O.C().quantize(w, 64)
    y = O.C().matmul(x, qw, b, absmax, O.nf4_lut(), 64, torch.bfloat16, (N, K))
    y2 = O.matmul_4bit_f64(x, qw, b, absmax, O.nf4_lut(), 64, torch.bfloat16, (N, K))
    assert torch.equal(bits_t(y), bits_t(y2))
    D = O.create_dynamic_map()
    off = O.C().dq_offset(absmax)
    q, a2 = O.C().dq_compress(absmax, D, off)
    q2, a22, off2 = O.dq_compress_eager(absmax, D)
    assert torch.equal(q, q2) and torch.equal(a2, a22) and off == off2
    rec = O.C().dq_reconstruct(q, a2, D, off)
    assert torch.equal(rec, O.dq_reconstruct_eager(q, a2, D, off))
    out.update({"mm.w": bits(w), "mm.x": bits(x), "mm.bias": bits(b), "mm.packed": bits(qw), "mm.absmax": bits(absmax),
                "mm.y": bits(y), "dq.map256": bits(D), "dq.offset": np.array([off], dtype=np.float32),
                "dq.q": bits(q), "dq.absmax2": bits(a2), "dq.reconstructed": bits(rec)})
    out["lut16"] = bits(O.nf4_lut())
    out["thresholds"] = bits(O.nf4_thresholds_f32())
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "nf4_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes,", len(out), "arrays")


def bits_t(t):
    return torch.from_numpy(bits(t))


if __name__ == "__main__":
    main()
