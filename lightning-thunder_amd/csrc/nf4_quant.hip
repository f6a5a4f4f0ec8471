// NF4 blockwise quantize / dequantize kernels for gfx950 (bit-exact contract, HBM-bound).
//
// quantize  : bitsandbytes.functional.quantize_4bit(w, quant_type="nf4"), the call made at
//             thunder/transforms/quantization.py:63
// dequantize: bitsandbytes.functional.dequantize_4bit, reached through matmul_4bit from
//             thunder/transforms/quantization.py:39
//
// Data layout.  The weight is a flat row-major array of n elements.  Every lane owns 8
// consecutive elements: one 128-bit load of bf16/f16 input (two for fp32), one 32-bit word of
// packed codes, one 128-bit store of bf16/f16 output.  A quantisation block of B elements is
// therefore B/8 adjacent lanes, and the block maximum is a butterfly over those lanes.
//
// This file is compiled with -ffp-contract=off: every product and sum below is rounded once.
#include <hip/hip_fp16.h>

#include "nf4_common.h"

namespace nf4 {
namespace {

// The decision thresholds of the NF4 code (midpoints of adjacent code values) appear below as the
// exact fp32 bit patterns a C compiler produces for the literals -0.8480964004993439f ...
// 0.8614784181118011f (four of the midpoints are exact ties in fp32).
// code = number of thresholds strictly below s (NaN -> 0).
//
// [-1, 1] is cut into 32 cells of width 1/16; adjacent thresholds are at least 0.08 apart, so a cell
// holds at most one of them, and code = (thresholds below the cell) + (s > the cell's threshold).
// Lane c of a wave keeps cell c & 31 in two registers and every lane fetches its cell with
// ds_bpermute: 6 VALU operations per element instead of a 4-level tree of compares and selects.
// The cell index comes from fma(s, 16, 16) rounded to fp32; a value within rounding distance of a
// cell boundary may land in the neighbouring cell, which gives the same code because no threshold
// is closer than 1.6e-3 to a boundary.
__device__ __constant__ const uint32_t CELL_THR[32] = {
    0x7F800000u, 0x7F800000u, 0xBF591CD9u, 0x7F800000u, 0x7F800000u, 0x7F800000u, 0xBF1C5270u, 0x7F800000u,
    0xBEEB8480u, 0x7F800000u, 0xBEADEA76u, 0x7F800000u, 0xBE703CECu, 0xBE0D38BCu, 0x7F800000u, 0xBD3A7871u,
    0x3D22FAFFu, 0x3DF64863u, 0x7F800000u, 0x3E5067E0u, 0x3E9582D4u, 0x7F800000u, 0x3EC753F9u, 0x7F800000u,
    0x3F006D03u, 0x7F800000u, 0x3F248DAFu, 0x7F800000u, 0x7F800000u, 0x3F5C89D9u, 0x7F800000u, 0x7F800000u};
__device__ __constant__ const uint32_t CELL_BASE[32] = {0, 0, 0,  1,  1,  1,  1,  2,  2,  3,  3,  4,  4,  5,  6,  6,
                                                        7, 8, 9,  9,  10, 11, 11, 12, 12, 13, 13, 14, 14, 14, 15, 15};

struct CodeCells {
    uint32_t thr;   // CELL_THR[lane & 31]
    uint32_t base;  // CELL_BASE[lane & 31]
};

__device__ __forceinline__ uint32_t nf4_code(float s, const CodeCells& cc) {
    // NaN and negatives convert to 0, values above 31 are clamped
    const uint32_t cell = min((uint32_t)__builtin_fmaf(s, 16.0f, 16.0f), 31u);
    const float t = __uint_as_float((uint32_t)__builtin_amdgcn_ds_bpermute((int)(cell << 2), (int)cc.thr));
    const uint32_t b = (uint32_t)__builtin_amdgcn_ds_bpermute((int)(cell << 2), (int)cc.base);
    return b + (s > t ? 1u : 0u);
}

__device__ __forceinline__ float load_elem(const void* w, int dtype, int64_t i) {
    if (dtype == BF16) return bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(w)[i]);
    if (dtype == F16) return __half2float(reinterpret_cast<const __half*>(w)[i]);
    return reinterpret_cast<const float*>(w)[i];
}

// Load the 8 elements [e0, e0+8) as fp32; elements at or beyond n read as 0.
__device__ __forceinline__ void load8(const void* w, int dtype, int64_t e0, int64_t n, float v[8]) {
    if (e0 + 8 <= n) {
        if (dtype == F32) {
            const float4 a = reinterpret_cast<const float4*>(w)[e0 / 4];
            const float4 b = reinterpret_cast<const float4*>(w)[e0 / 4 + 1];
            v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
            v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
        } else {
            const uint4 q = reinterpret_cast<const uint4*>(w)[e0 / 8];
            const uint32_t d[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (dtype == BF16) {
                    v[2 * j] = __uint_as_float(d[j] << 16);
                    v[2 * j + 1] = __uint_as_float(d[j] & 0xffff0000u);
                } else {
                    v[2 * j] = __half2float(__ushort_as_half((unsigned short)(d[j] & 0xffffu)));
                    v[2 * j + 1] = __half2float(__ushort_as_half((unsigned short)(d[j] >> 16)));
                }
            }
        }
    } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = (e0 + j < n) ? load_elem(w, dtype, e0 + j) : 0.0f;
    }
}

// A workgroup covers Q_SLOTS consecutive spans of THREADS * 8 elements (a span holds whole
// quantisation blocks); a thread owns 8 consecutive elements of each span.  The loads of all spans
// are in flight before the first reduction.
constexpr int Q_SLOTS = 4;

template <int THREADS>
__global__ __launch_bounds__(THREADS) void quantize_kernel(const void* __restrict__ w, int dtype, int64_t n,
                                                           int block_log2, uint8_t* __restrict__ packed,
                                                           float* __restrict__ absmax) {
    __shared__ float wave_max[Q_SLOTS][THREADS / 64];
    const int tid = threadIdx.x;
    const int group = 1 << (block_log2 - 3);  // lanes per quantisation block
    const CodeCells cc = {CELL_THR[tid & 31], CELL_BASE[tid & 31]};
    float v[Q_SLOTS][8];
    float m[Q_SLOTS];
#pragma unroll
    for (int c = 0; c < Q_SLOTS; ++c) {
        const int64_t e0 = (((int64_t)blockIdx.x * Q_SLOTS + c) * THREADS + tid) * 8;
        load8(w, dtype, e0, n, v[c]);
    }
    const int in_wave = group < 64 ? group : 64;
#pragma unroll
    for (int c = 0; c < Q_SLOTS; ++c) {
        float mm = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) mm = fmaxf(mm, fabsf(v[c][j]));
        // max over the lanes of one quantisation block
        for (int off = 1; off < in_wave; off <<= 1) mm = fmaxf(mm, __shfl_xor(mm, off, 64));
        m[c] = mm;
    }
    if (group > 64) {  // uniform branch: blocks of 1024, 2048 or 4096 elements span several waves
#pragma unroll
        for (int c = 0; c < Q_SLOTS; ++c)
            if ((tid & 63) == 0) wave_max[c][tid >> 6] = m[c];
        __syncthreads();
        const int waves = group >> 6;
        const int first = (tid >> 6) & ~(waves - 1);
#pragma unroll
        for (int c = 0; c < Q_SLOTS; ++c)
            for (int j = 0; j < waves; ++j) m[c] = fmaxf(m[c], wave_max[c][first + j]);
    }
#pragma unroll
    for (int c = 0; c < Q_SLOTS; ++c) {
        const int64_t e0 = (((int64_t)blockIdx.x * Q_SLOTS + c) * THREADS + tid) * 8;
        // every lane computes its codes (the cell lookup reads other lanes' registers, so no lane
        // may drop out before it); lanes past the end hold zeros and store nothing
        const float inv = __fdiv_rn(1.0f, m[c]);
        uint32_t word = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t hi = nf4_code(__fmul_rn(v[c][2 * j], inv), cc);
            const uint32_t lo = nf4_code(__fmul_rn(v[c][2 * j + 1], inv), cc);
            word |= ((hi << 4) | lo) << (8 * j);
        }
        if (e0 >= n) continue;
        if ((tid & (group - 1)) == 0) absmax[e0 >> block_log2] = m[c];
        if (e0 + 8 <= n) {
            reinterpret_cast<uint32_t*>(packed)[e0 / 8] = word;
        } else {
            const int64_t nbytes = (n + 1) / 2;
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (e0 / 2 + j < nbytes) packed[e0 / 2 + j] = (uint8_t)(word >> (8 * j));
        }
    }
}

// Eight elements of output from one 32-bit word of codes.
template <bool STREAM>
__device__ __forceinline__ void dequant8_store(uint32_t word, float s, const float* lut, void* out, int out_dtype,
                                               int64_t e0, int64_t n) {
    const bool full = e0 + 8 <= n;
    float v[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t byte = (word >> (8 * j)) & 0xffu;
        v[2 * j] = __fmul_rn(lut[byte >> 4], s);
        v[2 * j + 1] = __fmul_rn(lut[byte & 15u], s);
    }
    if (out_dtype == F32) {
        float* o = reinterpret_cast<float*>(out);
        if (full) {
            store16<STREAM>(o + e0, __float_as_uint(v[0]), __float_as_uint(v[1]), __float_as_uint(v[2]), __float_as_uint(v[3]));
            store16<STREAM>(o + e0 + 4, __float_as_uint(v[4]), __float_as_uint(v[5]), __float_as_uint(v[6]), __float_as_uint(v[7]));
        } else {
            for (int j = 0; j < 8; ++j)
                if (e0 + j < n) o[e0 + j] = v[j];
        }
    } else {
        uint32_t h[8];
#pragma unroll
        for (int j = 0; j < 8; ++j)
            h[j] = out_dtype == BF16 ? f32_to_bf16_bits(v[j]) : (uint32_t)__half_as_ushort(__float2half_rn(v[j]));
        uint16_t* o = reinterpret_cast<uint16_t*>(out);
        if (full) {
            store16<STREAM>(o + e0, h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16));
        } else {
            for (int j = 0; j < 8; ++j)
                if (e0 + j < n) o[e0 + j] = (uint16_t)h[j];
        }
    }
}

// A workgroup covers DQ_SLOTS consecutive spans of 2048 elements; a thread owns 8 consecutive
// elements of each span, so every load and store of a wave is contiguous, and the loads of all
// spans are in flight before the first store.
constexpr int DQ_SLOTS = 4;

template <bool NESTED, bool STREAM>
__global__ __launch_bounds__(256) void dequantize_kernel(const uint8_t* __restrict__ packed,
                                                         const float* __restrict__ absmax, NestedAbsmax nq,
                                                         const float* __restrict__ lut16, int64_t n, int block_log2,
                                                         void* __restrict__ out, int out_dtype) {
    __shared__ float lut[16];
    const int tid = threadIdx.x;
    if (tid < 16) lut[tid] = lut16[tid];
    uint32_t word[DQ_SLOTS];
    float s[DQ_SLOTS];
#pragma unroll
    for (int c = 0; c < DQ_SLOTS; ++c) {
        const int64_t e0 = (((int64_t)blockIdx.x * DQ_SLOTS + c) * 256 + tid) * 8;
        word[c] = 0;
        s[c] = 0.0f;
        if (e0 >= n) continue;
        const int64_t blk = e0 >> block_log2;
        s[c] = NESTED ? nested_absmax(nq, blk) : absmax[blk];
        if (e0 + 8 <= n) {
            word[c] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(packed) + e0 / 8);
        } else {
            const int64_t nbytes = (n + 1) / 2;
            for (int j = 0; j < 4; ++j)
                if (e0 / 2 + j < nbytes) word[c] |= (uint32_t)packed[e0 / 2 + j] << (8 * j);
        }
    }
    __syncthreads();
#pragma unroll
    for (int c = 0; c < DQ_SLOTS; ++c) {
        const int64_t e0 = (((int64_t)blockIdx.x * DQ_SLOTS + c) * 256 + tid) * 8;
        if (e0 < n) dequant8_store<STREAM>(word[c], s[c], lut, out, out_dtype, e0, n);
    }
}

// One workgroup per nested block: r = absmax - offset, absmax2 = max|r|, then the nearest entry
// of the 256-entry map (lowest index on ties) for every r * (1/absmax2).
__global__ __launch_bounds__(256) void dq_compress_kernel(const float* __restrict__ absmax, int64_t nblocks,
                                                          int nested_log2, const float* __restrict__ map256,
                                                          float offset, uint8_t* __restrict__ q,
                                                          float* __restrict__ absmax2) {
    __shared__ float map[256];
    __shared__ float red[4];
    __shared__ int zero_code;
    const int tid = threadIdx.x;
    const int nested = 1 << nested_log2;
    const int64_t base = (int64_t)blockIdx.x << nested_log2;
    map[tid] = map256[tid];
    if (tid == 0) zero_code = 256;  // sentinel: the map holds no 0.0 (then an all-zero block stores code 0)
    __syncthreads();
    if (map[tid] == 0.0f) atomicMin(&zero_code, tid);

    float m = 0.0f;
    for (int i = tid; i < nested; i += 256) {
        const int64_t idx = base + i;
        if (idx < nblocks) m = fmaxf(m, fabsf(__fsub_rn(absmax[idx], offset)));
    }
    for (int off = 1; off < 64; off <<= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
    if ((tid & 63) == 0) red[tid >> 6] = m;
    __syncthreads();
    m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    if (tid == 0) absmax2[blockIdx.x] = m;

    const float inv = __fdiv_rn(1.0f, m);
    for (int i = tid; i < nested; i += 256) {
        const int64_t idx = base + i;
        if (idx >= nblocks) continue;
        int best = zero_code == 256 ? 0 : zero_code;
        if (m != 0.0f) {
            const float s = __fmul_rn(__fsub_rn(absmax[idx], offset), inv);
            float bestd = INFINITY;
            best = 0;
            for (int j = 0; j < 256; ++j) {
                const float d = fabsf(__fsub_rn(s, map[j]));
                if (d < bestd) {
                    bestd = d;
                    best = j;
                }
            }
        }
        q[idx] = (uint8_t)best;
    }
}

__global__ __launch_bounds__(256) void dq_reconstruct_kernel(NestedAbsmax nq, int64_t nblocks,
                                                             float* __restrict__ absmax) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < nblocks) absmax[i] = nested_absmax(nq, i);
}

}  // namespace

hipError_t launch_quantize(const void* w, int w_dtype, int64_t n, int block_log2, uint8_t* packed, float* absmax,
                           hipStream_t stream) {
    if (n == 0) return hipSuccess;
    if (block_log2 == 12) {
        const int64_t grid = (n + 4096 * Q_SLOTS - 1) / (4096 * Q_SLOTS);
        hipLaunchKernelGGL(quantize_kernel<512>, dim3((unsigned)grid), dim3(512), 0, stream, w, w_dtype, n, block_log2,
                           packed, absmax);
    } else {
        const int64_t grid = (n + 2048 * Q_SLOTS - 1) / (2048 * Q_SLOTS);
        hipLaunchKernelGGL(quantize_kernel<256>, dim3((unsigned)grid), dim3(256), 0, stream, w, w_dtype, n, block_log2,
                           packed, absmax);
    }
    return hipGetLastError();
}

hipError_t launch_dequantize(const uint8_t* packed, const float* absmax, const NestedAbsmax& nested,
                             const float* lut16, int64_t n, int block_log2, void* out, int out_dtype,
                             hipStream_t stream) {
    if (n == 0) return hipSuccess;
    const int64_t grid = (n + 2048 * DQ_SLOTS - 1) / (2048 * DQ_SLOTS);
    // An output that fits in the 256 MB last-level cache is written with ordinary stores, so that the
    // GEMM that usually follows finds it there; a larger one cannot stay anyway and is streamed
    // (non-temporal stores: 20 % faster on their own, 5 % slower for that GEMM).
    const int64_t out_bytes = n * (out_dtype == F32 ? 4 : 2);
    const bool stream_out = out_bytes > ((int64_t)192 << 20);
    const dim3 g((unsigned)grid), b(256);
    if (nested.q) {
        if (stream_out)
            hipLaunchKernelGGL((dequantize_kernel<true, true>), g, b, 0, stream, packed, absmax, nested, lut16, n, block_log2, out, out_dtype);
        else
            hipLaunchKernelGGL((dequantize_kernel<true, false>), g, b, 0, stream, packed, absmax, nested, lut16, n, block_log2, out, out_dtype);
    } else {
        if (stream_out)
            hipLaunchKernelGGL((dequantize_kernel<false, true>), g, b, 0, stream, packed, absmax, nested, lut16, n, block_log2, out, out_dtype);
        else
            hipLaunchKernelGGL((dequantize_kernel<false, false>), g, b, 0, stream, packed, absmax, nested, lut16, n, block_log2, out, out_dtype);
    }
    return hipGetLastError();
}

hipError_t launch_dq_compress(const float* absmax, int64_t nblocks, int nested_log2, const float* map256,
                              float offset, uint8_t* q, float* absmax2, hipStream_t stream) {
    if (nblocks == 0) return hipSuccess;
    const int64_t grid = (nblocks + (1 << nested_log2) - 1) >> nested_log2;
    hipLaunchKernelGGL(dq_compress_kernel, dim3((unsigned)grid), dim3(256), 0, stream, absmax, nblocks, nested_log2,
                       map256, offset, q, absmax2);
    return hipGetLastError();
}

hipError_t launch_dq_reconstruct(const NestedAbsmax& nested, int64_t nblocks, float* absmax, hipStream_t stream) {
    if (nblocks == 0) return hipSuccess;
    const int64_t grid = (nblocks + 255) / 256;
    hipLaunchKernelGGL(dq_reconstruct_kernel, dim3((unsigned)grid), dim3(256), 0, stream, nested, nblocks, absmax);
    return hipGetLastError();
}

}  // namespace nf4
