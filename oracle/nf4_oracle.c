/*
 * nf4_oracle.c -- scalar CPU restatement of the NF4 weight-only linear arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker that the HIP kernels are
 * compared against.  Nothing in the shipped package may link, load or call it;
 * only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg do.
 *
 * What it restates.  Thunder's 4-bit path (thunder/transforms/quantization.py)
 * has no arithmetic of its own: every number comes from the third-party package
 * bitsandbytes==0.48.0 (pinned in requirements/test.txt:20), which is not
 * vendored under the reference tree.  The call sites that fix the contract are
 *   quantize : thunder/transforms/quantization.py:63
 *              bitsandbytes.functional.quantize_4bit(w, quant_type="nf4")
 *   matmul   : thunder/transforms/quantization.py:34-39
 *              bitsandbytes.matmul_4bit(x, qweight.t(), bias, quant_state)
 *              which dequantizes (dequantize_4bit) and calls F.linear, or runs
 *              the fused gemv when x is a single row.
 * The published bitsandbytes algorithm (QLoRA NF4, blockwise absmax scaling) is
 * restated here function by function.
 *
 * Pinning status (what independent check each function has; see tests/):
 *   nf4o_lut16, thresholds   : closed form (normal quantiles via scipy), midpoints
 *   nf4o_quantize            : exhaustive bf16 sweep vs float64 nearest neighbour,
 *                              absmax by brute force, nibble order by round trip
 *   nf4o_dequantize          : exhaustive 16 codes x all bf16 absmax vs float64 product
 *                              rounded once (torch), for bf16/f16/f32 outputs
 *   nf4o_matmul              : torch float64 matmul on the dequantized weight
 *   nf4o_dq_*                : nearest-neighbour invariant, reconstruction bound;
 *                              PARITY UNPINNED against bitsandbytes itself (no call
 *                              site or test in the reference uses compress_statistics)
 *   corner cases that only an import of bitsandbytes could pin (exact threshold
 *   ties, the pad nibble for odd n, NaN/Inf inputs): PARITY UNPINNED, behaviour
 *   defined below and documented.
 *
 * dtype codes: 0 = bf16, 1 = f16, 2 = f32.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define NF4O_BF16 0
#define NF4O_F16 1
#define NF4O_F32 2

/* The 16 NF4 code values (QLoRA: quantiles of N(0,1) normalised to [-1,1]). */
static const float NF4_LUT[16] = {
    -1.0f,
    -0.6961928009986877f,
    -0.5250730514526367f,
    -0.39491748809814453f,
    -0.28444138169288635f,
    -0.18477343022823334f,
    -0.09105003625154495f,
    0.0f,
    0.07958029955625534f,
    0.16093020141124725f,
    0.24611230194568634f,
    0.33791524171829224f,
    0.44070982933044434f,
    0.5626170039176941f,
    0.7229568362236023f,
    1.0f,
};

/* Decision thresholds: midpoints of adjacent code values, used as fp32. */
static const float NF4_THRESH[15] = {
    -0.8480964004993439f, -0.6106329262256622f, -0.4599952697753906f, -0.33967943489551544f,
    -0.23460740596055984f, -0.13791173323988914f, -0.045525018125772476f, 0.03979014977812767f,
    0.1202552504837513f, 0.2035212516784668f, 0.2920137718319893f, 0.3893125355243683f,
    0.5016634166240692f, 0.6427869200706482f, 0.8614784181118011f,
};

/* ---------- scalar format conversions (round to nearest even) ---------- */

static inline uint32_t f2u(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}
static inline float u2f(uint32_t u) {
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static inline float bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

static inline uint16_t f32_to_bf16(float f) {
    uint32_t u = f2u(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u); /* quiet NaN */
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

static inline float f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    if (exp == 0) {
        if (man == 0) return u2f(sign);
        /* subnormal: value = man * 2^-24 */
        float v = (float)man * 5.9604644775390625e-08f;
        return sign ? -v : v;
    }
    if (exp == 31) return u2f(sign | 0x7f800000u | (man << 13));
    return u2f(sign | ((exp + 112u) << 23) | (man << 13));
}

static inline uint16_t f32_to_f16(float f) {
    uint32_t u = f2u(f);
    uint32_t sign = (u >> 16) & 0x8000u;
    uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);  /* NaN */
    if (a >= 0x47800000u) {                                  /* >= 65536: overflow (also inf) */
        return (uint16_t)(sign | 0x7c00u);
    }
    if (a >= 0x38800000u) { /* normal half range: exponent >= -14 */
        uint32_t m = a - 0x38000000u; /* rebias 127 -> 15 */
        uint32_t r = m + 0xfffu + ((m >> 13) & 1u);
        return (uint16_t)(sign | (r >> 13)); /* carry into exponent, up to inf, is correct */
    }
    if (a < 0x33000000u) return (uint16_t)sign; /* < 2^-25 rounds to zero */
    /* subnormal half: value = mant * 2^-24, round to nearest even */
    {
        int e = (int)(a >> 23);                 /* biased exponent, 102..112 */
        uint32_t m = (a & 0x7fffffu) | 0x800000u; /* 24-bit significand */
        int shift = 126 - e;                    /* 14..24 : m * 2^(e-150) / 2^-24 = m >> (126-e) */
        uint32_t q = m >> shift;
        uint32_t rem = m & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1);
        if (rem > half || (rem == half && (q & 1u))) q++;
        return (uint16_t)(sign | q);
    }
}

static inline float load_as_f32(const void* p, int dtype, int64_t i) {
    switch (dtype) {
        case NF4O_BF16: return bf16_to_f32(((const uint16_t*)p)[i]);
        case NF4O_F16: return f16_to_f32(((const uint16_t*)p)[i]);
        default: return ((const float*)p)[i];
    }
}

/* Round an fp32 value once (nearest even) to `dtype` and return it widened again. */
static inline float round_to_dtype(float v, int dtype) {
    switch (dtype) {
        case NF4O_BF16: return bf16_to_f32(f32_to_bf16(v));
        case NF4O_F16: return f16_to_f32(f32_to_f16(v));
        default: return v;
    }
}

static inline void store_from_f32(void* p, int dtype, int64_t i, float v) {
    switch (dtype) {
        case NF4O_BF16: ((uint16_t*)p)[i] = f32_to_bf16(v); break;
        case NF4O_F16: ((uint16_t*)p)[i] = f32_to_f16(v); break;
        default: ((float*)p)[i] = v; break;
    }
}

/* ---------- constants ---------- */

void nf4o_lut16(float* out16) { memcpy(out16, NF4_LUT, sizeof(NF4_LUT)); }
void nf4o_thresholds(float* out15) { memcpy(out15, NF4_THRESH, sizeof(NF4_THRESH)); }

/*
 * code = number of thresholds strictly below s.  Equivalent to the if/else tree of
 * bitsandbytes' dQuantizeNF4 (csrc/kernels.cu), which compares with '>' throughout.
 * NaN compares false everywhere and yields code 0.
 */
static inline int nf4_code(float s) {
    int c = 0;
    for (int j = 0; j < 15; ++j) c += (s > NF4_THRESH[j]);
    return c;
}

int nf4o_code_of(float s) { return nf4_code(s); }

/* ---------- quantize (bitsandbytes.functional.quantize_4bit, quant_type="nf4") ---------- */
/*
 * Flattened row-major input of n elements, blocks of `blocksize` consecutive elements.
 *   absmax[b] = max |w_i| over the valid elements of block b            (fp32, exact)
 *   inv       = 1.0f / absmax[b]                                        (IEEE division)
 *   code_i    = nf4_code(w_i * inv)                                     (one fp32 multiply)
 *   packed[j] = code_{2j} << 4 | code_{2j+1}        first element in the HIGH nibble
 * Odd n: the missing last element is treated as 0.0f run through the same arithmetic
 * (the CUDA kernel loads out-of-range items as 0.0f), so the pad nibble is 7 unless the
 * last block is all zero (0*inf = NaN -> code 0).
 * packed has (n+1)/2 bytes; absmax has ceil(n/blocksize) entries.
 */
int nf4o_quantize(const void* w, int dtype, int64_t n, int blocksize, uint8_t* packed, float* absmax) {
    if (!w || !packed || !absmax) return -1;
    if (dtype < 0 || dtype > 2) return -2;
    if (blocksize < 2 || (blocksize & 1)) return -3;
    int64_t nblocks = (n + blocksize - 1) / blocksize;
    for (int64_t b = 0; b < nblocks; ++b) {
        int64_t lo = b * blocksize;
        int64_t hi = lo + blocksize < n ? lo + blocksize : n;
        float m = 0.0f;
        for (int64_t i = lo; i < hi; ++i) {
            float a = fabsf(load_as_f32(w, dtype, i));
            if (a > m) m = a;
        }
        absmax[b] = m;
        volatile float inv = 1.0f / m; /* volatile: keep the division, forbid reassociation */
        int64_t hi_even = (hi + 1) & ~(int64_t)1;
        for (int64_t i = lo; i < hi_even; i += 2) {
            float v0 = load_as_f32(w, dtype, i);
            float v1 = (i + 1 < n) ? load_as_f32(w, dtype, i + 1) : 0.0f;
            volatile float s0 = v0 * inv;
            volatile float s1 = v1 * inv;
            packed[i >> 1] = (uint8_t)((nf4_code(s0) << 4) | nf4_code(s1));
        }
    }
    return 0;
}

/* ---------- dequantize (bitsandbytes.functional.dequantize_4bit) ---------- */
/*
 * out_i = round_to(out_dtype, lut16[code_i] * absmax[i / blocksize])
 * one fp32 multiply, one rounding.  The 16-entry table is an INPUT: the reference op
 * receives it as its `quant_map` argument (thunder/transforms/quantization.py:34), and
 * bitsandbytes' eager backend pre-rounds the table to the output dtype while its CUDA
 * kernel does not -- the caller selects either by what it passes.
 */
int nf4o_dequantize(const uint8_t* packed, const float* absmax, const float* lut16, int64_t n, int blocksize,
                    void* out, int out_dtype) {
    if (!packed || !absmax || !lut16 || !out) return -1;
    if (out_dtype < 0 || out_dtype > 2) return -2;
    if (blocksize < 2 || (blocksize & 1)) return -3;
    for (int64_t i = 0; i < n; ++i) {
        uint8_t byte = packed[i >> 1];
        int code = (i & 1) ? (byte & 15) : (byte >> 4);
        volatile float v = lut16[code] * absmax[i / blocksize];
        store_from_f32(out, out_dtype, i, v);
    }
    return 0;
}

/* ---------- matmul (bitsandbytes.matmul_4bit, MatMul4Bit route) ---------- */
/*
 * W_deq = dequantize(...) rounded to w_dtype (the dtype recorded at quantisation time),
 * then converted to x's dtype (MatMul4Bit: dequantize_4bit(...).to(A.dtype)), then
 *   y[m][n] = round_to(x_dtype, sum_k x[m][k] * W_deq[n][k] + bias[n])
 * The reference accumulates in fp32 in a library-defined order; the oracle accumulates in
 * double so that it sits at the centre of every legal ordering (tolerance 2e-2).
 * Blocks run over the flattened [N*K] weight, so they may straddle rows when K % blocksize != 0.
 */
int nf4o_matmul(const void* x, int x_dtype, int64_t M, const uint8_t* packed, const float* absmax,
                const float* lut16, const void* bias, int64_t N, int64_t K, int blocksize, int w_dtype,
                void* out) {
    if (!x || !packed || !absmax || !lut16 || !out) return -1;
    if (x_dtype < 0 || x_dtype > 2 || w_dtype < 0 || w_dtype > 2) return -2;
    if (blocksize < 2 || (blocksize & 1)) return -3;
    float* wrow = (float*)malloc((size_t)K * sizeof(float));
    float* xf = (float*)malloc((size_t)M * (size_t)K * sizeof(float));
    if (!wrow || !xf) {
        free(wrow);
        free(xf);
        return -4;
    }
    for (int64_t i = 0; i < M * K; ++i) xf[i] = load_as_f32(x, x_dtype, i);
    for (int64_t nn = 0; nn < N; ++nn) {
        for (int64_t k = 0; k < K; ++k) {
            int64_t i = nn * K + k;
            uint8_t byte = packed[i >> 1];
            int code = (i & 1) ? (byte & 15) : (byte >> 4);
            volatile float v = lut16[code] * absmax[i / blocksize];
            wrow[k] = round_to_dtype(round_to_dtype(v, w_dtype), x_dtype);
        }
        float b = bias ? load_as_f32(bias, x_dtype, nn) : 0.0f;
        for (int64_t m = 0; m < M; ++m) {
            double acc = 0.0;
            const float* xr = xf + m * K;
            for (int64_t k = 0; k < K; ++k) acc += (double)xr[k] * (double)wrow[k];
            acc += (double)b;
            store_from_f32(out, x_dtype, m * N + nn, (float)acc);
        }
    }
    free(wrow);
    free(xf);
    return 0;
}

/* ---------- nested ("double") quantisation of absmax ---------- */
/*
 * bitsandbytes quantize_4bit(..., compress_statistics=True):
 *   offset = absmax.mean();  r = absmax - offset
 *   8-bit blockwise quantisation of r (nested blocksize 256) against the 256-entry
 *   dynamic map D (an input, like lut16):
 *     absmax2[c] = max |r| over nested block c;  q_b = argmin_j |r_b * (1/absmax2[c]) - D_j|
 *   reconstruction:  absmax_b = D[q_b] * absmax2[b / 256] + offset    (mul, then add; no fma)
 * Build-defined where bitsandbytes is not reproducible: offset is the float64 mean rounded
 * to fp32; ties go to the lowest index; an all-zero nested block stores the code of 0.0.
 * PARITY UNPINNED against bitsandbytes (see file header).
 */
float nf4o_dq_offset(const float* absmax, int64_t nblocks) {
    double s = 0.0;
    for (int64_t i = 0; i < nblocks; ++i) s += (double)absmax[i];
    return nblocks > 0 ? (float)(s / (double)nblocks) : 0.0f;
}

int nf4o_dq_compress(const float* absmax, int64_t nblocks, int nested_blocksize, const float* map256, float offset,
                     uint8_t* q, float* absmax2) {
    if (!absmax || !map256 || !q || !absmax2) return -1;
    if (nested_blocksize < 1) return -3;
    int zero_code = 0;
    for (int j = 0; j < 256; ++j)
        if (map256[j] == 0.0f) {
            zero_code = j;
            break;
        }
    int64_t nnb = (nblocks + nested_blocksize - 1) / nested_blocksize;
    for (int64_t c = 0; c < nnb; ++c) {
        int64_t lo = c * nested_blocksize;
        int64_t hi = lo + nested_blocksize < nblocks ? lo + nested_blocksize : nblocks;
        float m = 0.0f;
        for (int64_t i = lo; i < hi; ++i) {
            volatile float r = absmax[i] - offset;
            float a = fabsf(r);
            if (a > m) m = a;
        }
        absmax2[c] = m;
        if (m == 0.0f) {
            for (int64_t i = lo; i < hi; ++i) q[i] = (uint8_t)zero_code;
            continue;
        }
        volatile float inv = 1.0f / m;
        for (int64_t i = lo; i < hi; ++i) {
            volatile float r = absmax[i] - offset;
            volatile float s = r * inv;
            int best = 0;
            float bestd = INFINITY;
            for (int j = 0; j < 256; ++j) {
                volatile float d = fabsf(s - map256[j]);
                if (d < bestd) {
                    bestd = d;
                    best = j;
                }
            }
            q[i] = (uint8_t)best;
        }
    }
    return 0;
}

int nf4o_dq_reconstruct(const uint8_t* q, const float* absmax2, const float* map256, float offset, int64_t nblocks,
                        int nested_blocksize, float* absmax_out) {
    if (!q || !absmax2 || !map256 || !absmax_out) return -1;
    if (nested_blocksize < 1) return -3;
    for (int64_t i = 0; i < nblocks; ++i) {
        volatile float p = map256[q[i]] * absmax2[i / nested_blocksize];
        volatile float v = p + offset;
        absmax_out[i] = v;
    }
    return 0;
}

/* conversions exported so the tests can pin them against torch's casts */
uint16_t nf4o_f32_to_bf16(float f) { return f32_to_bf16(f); }
uint16_t nf4o_f32_to_f16(float f) { return f32_to_f16(f); }
float nf4o_f16_to_f32(uint16_t h) { return f16_to_f32(h); }
float nf4o_bf16_to_f32(uint16_t h) { return bf16_to_f32(h); }
