// Pieces shared by the three decode-shape kernels (row-streaming, four weight rows per lane quad, MFMA tiles).
#pragma once

#include "nf4_common.h"

namespace nf4 {

constexpr int GEMV_THREADS = 512;  // 8 waves; two workgroups per CU
constexpr int GEMV_WAVES = GEMV_THREADS / 64;

// What a wave's first requests depend on -- code book, x, codes, absmax, N, K, M -- travels ahead of the argument
// structs as scalars.  This library is built with -mllvm -amdgpu-kernarg-preload-count: the leading scalar arguments of
// a kernel (up to 14 dwords; structs are passed by reference and never qualify) then arrive in SGPRs with the wave, and
// the kernel requests its code-book entry, x and first weights without first waiting for a load from the argument
// block.  Measured on the row kernel, one row of x: [6144, 4096] 7.1 -> 6.8 us, [14336, 4096] 11.2 -> 10.7,
// [4096, 14336] 11.5 -> 11.1, [28672, 4096] 17.0 -> 16.6; a 161-linear decode step 1.764 -> 1.715 ms.
// 11 dwords here; a kernel adds up to three of its launch plan.
#define NF4_HOT_PARAMS                                                                                          \
    const float *hot_lut, const uint16_t *hot_x, const uint8_t *hot_packed, const float *hot_absmax, int hot_N, \
        int hot_K, int hot_M_log2
// (with nested absmax the slot of the absmax pointer carries the pointer to their 8-bit codes)
#define NF4_HOT_VALUES(a)                                                                                              \
    (a).lut16, (a).x, (a).packed, ((a).nested.q ? reinterpret_cast<const float*>((a).nested.q) : (a).absmax), (a).N, (a).K, \
        ((a).M | ((a).block_log2 << 8))
#define NF4_HOT_NAMES hot_lut, hot_x, hot_packed, hot_absmax, hot_N, hot_K, hot_M_log2

template <bool NESTED>
__device__ __forceinline__ MatmulArgs with_hot_args(const MatmulArgs& in, NF4_HOT_PARAMS) {
    MatmulArgs a = in;
    a.lut16 = hot_lut; a.x = hot_x; a.packed = hot_packed;
    if (NESTED) {
        a.nested.q = reinterpret_cast<const uint8_t*>(hot_absmax);
        a.absmax = nullptr;
    } else {
        a.absmax = hot_absmax;
    }
    a.N = hot_N; a.K = hot_K; a.M = hot_M_log2 & 0xff; a.block_log2 = hot_M_log2 >> 8;
    return a;
}
constexpr int GEMV_TABLE_BYTES = 256 * 256;     // 256 byte values x 64 lanes x 4 B
constexpr int GEMV_COUNTER_BYTES = (int)GEMV_COUNTER_REGION_BYTES;  // split-K arrival counters at the head of the workspace

// Byte -> (16-bit float, 16-bit float) table at the start of LDS.  Entry b holds the code values of the two
// nibbles of b, the high nibble (even element) in the low half, as bf16 (F16 = false) or as fp16 (F16 = true:
// the code book is then exact to 2^-12 instead of 2^-9, see F16Scale).  It is replicated for the
// 64 lanes with a 256-byte stride: lane l reads byte address (b << 8) | (l * 4), so every lane
// owns one bank column and a lookup is conflict-free whatever the data.
// `lut_lane` is lut16[lane & 15], loaded by the caller (early, so that its latency is hidden).
template <bool F16 = false>
__device__ __forceinline__ void build_pair_table(uint8_t* smem, float lut_lane, int lane, int wave) {
    // Every entry is one dword replicated over a 256-byte row.  Sixteen lanes write one row with
    // 16-byte stores, so a wave writes four entries per instruction and its 32 entries in eight.
    const uint32_t lb = F16 ? (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)lut_lane) : f32_to_bf16_bits(lut_lane);
    uint4* table = reinterpret_cast<uint4*>(smem);
    const int sub = lane >> 4;
#pragma unroll
    for (int it = 0; it < 8; ++it) {
        const int e = wave * 32 + it * 4 + sub;
        // high nibble = even element: wave * 2 + (it >> 2), the same for all four entries
        const uint32_t first = __builtin_amdgcn_readlane(lb, wave * 2 + (it >> 2));
        // low nibble = odd element: lane (it * 4 + sub) & 15 holds its code value
        const uint32_t second = (uint32_t)__builtin_amdgcn_ds_bpermute(((it * 4 + sub) & 15) * 4, (int)lb);
        const uint32_t v = first | (second << 16);
        table[e * 16 + (lane & 15)] = make_uint4(v, v, v, v);
    }
}

// The decode kernels for up to eight rows of x multiply on the matrix pipe in fp16: code-book values rounded to
// fp16 (11 significant bits) times x.  A lane converts the bf16 values of x it holds once, when it loads them.  A
// bf16 value is exactly representable in fp16 unless it lies outside fp16's range, so the lane first scales its
// values by the power of two that puts the largest of them into [2^14, 2^15) and multiplies its partial sums by the
// inverse afterwards -- both exact in fp32.  Values 2^28 times smaller than the lane's largest lose bits or vanish;
// their share of the sum is below fp32's resolution of it.
struct F16Scale {
    float to_f16;    // multiply x by this before the conversion
    float from_f16;  // multiply the sums by this
};
// `mx`: the largest of the lane's |x| as fp32 bits (bf16 bits << 16)
__device__ __forceinline__ F16Scale f16_scale_for(uint32_t mx) {
    // biased exponent e of the largest value: scale by 2^(14 - (e - 127)), at most by 2^126 (largest values below
    // 2^-112, an all-zero lane)
    const uint32_t ebits = max(mx >> 23, 141u - 126u);
    F16Scale s;
    s.to_f16 = __uint_as_float((268u - ebits) << 23);
    s.from_f16 = __uint_as_float((ebits - 14u) << 23);
    return s;
}
// running maximum of |x| over bf16 pairs, both halves at once (one v_and, one v_pk_max_u16 per dword) ...
typedef unsigned short u16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ u16x2_t absmax_of_bf16_pair(uint32_t v, u16x2_t mx) {
    return __builtin_elementwise_max(mx, __builtin_bit_cast(u16x2_t, v & 0x7fff7fffu));
}
// ... and the larger half as fp32 bits
__device__ __forceinline__ uint32_t absmax_bits(u16x2_t mx) { return (uint32_t)max(mx.x, mx.y) << 16; }
// two bf16 in a dword -> the same two values times `scale` as fp16 in a dword
__device__ __forceinline__ uint32_t bf16_pair_to_f16(uint32_t v, float scale) {
    typedef __fp16 fp16x2_t __attribute__((ext_vector_type(2)));
    const float lo = __fmul_rn(__uint_as_float(v << 16), scale), hi = __fmul_rn(__uint_as_float(v & 0xffff0000u), scale);
    const fp16x2_t h = __builtin_amdgcn_cvt_pkrtz(lo, hi);
    return __builtin_bit_cast(uint32_t, h);
}

// fp32 variant of the table for the exact kernels: entry b = (lut[b >> 4], lut[b & 15]) as two
// floats, replicated for 32 lane columns with a 256-byte stride; lane l reads byte address
// (b << 8) | ((l & 31) * 8).
__device__ __forceinline__ void build_pair_table_f32(uint8_t* smem, float lut_lane, int lane, int wave) {
    const uint32_t lb = __float_as_uint(lut_lane);
    float2* table = reinterpret_cast<float2*>(smem);
    const int half = lane >> 5;
#pragma unroll 8
    for (int it = 0; it < 16; ++it) {
        const int e0 = wave * 32 + 2 * it;  // lanes 0-31 write entry e0, lanes 32-63 entry e0 + 1
        const uint32_t first = __builtin_amdgcn_readlane(lb, e0 >> 4);
        const uint32_t s0 = __builtin_amdgcn_readlane(lb, e0 & 15);
        const uint32_t s1 = __builtin_amdgcn_readlane(lb, (e0 & 15) + 1);
        table[(e0 + half) * 32 + (lane & 31)] = make_float2(__uint_as_float(first), __uint_as_float(half ? s1 : s0));
    }
}

// K beyond which the decode kernels reproduce the reference's per-weight bf16 rounding exactly.  The cheaper
// arithmetic (rounded code-book value * x on the matrix pipe, block sums scaled by absmax) differs from
// bf16(lut * absmax) * x by the reference's own bf16 rounding of every weight and, where the code book is held in
// bf16 (the tile kernel), by a second, independent one; its distance from the reference grows like sqrt(K).
// Measured sigma for N(0, 1) activations and N(0, 0.02) weights, bf16 code book: 0.0027 / 0.0038 / 0.0047 at K = 4096 /
// 8192 / 14336 -- at K = 14336 the 2e-2 tolerance is 4.2 sigma and about one output in 40 000 crosses it (seen at
// [4096, 14336], M = 16), at K = 8192 it is 5.2 sigma (one in five million).  fp16 code book (row and quad kernels):
// 0.0036 at K = 14336 and no output in a million beyond 0.73 of the tolerance; 0.0038 at K = 16384.
// The kernels therefore come in up to three arithmetic modes, chosen from K: bf16 code book up to K = 8192 (x is
// used as it is loaded), fp16 code book up to 16384 where the kernel has one (x converted once per lane: a few
// hundred VALU instructions per wave, which only longer rows repay), exact beyond.
enum : int { ARITH_BF16 = 0, ARITH_F16 = 1, ARITH_EXACT = 2 };
__host__ __device__ constexpr int gemv_arith_mode(int64_t K, bool has_f16_mode) {
    return K <= 8192 ? ARITH_BF16 : (has_f16_mode && K <= 16384) ? ARITH_F16 : ARITH_EXACT;
}

// Read one table entry.  `addr` is an absolute LDS byte address: the table sits at LDS offset 0
// (the gemv kernels have no static __shared__ data, so their dynamic segment starts there), which
// saves the "+ base" VALU add the compiler emits for every access through an extern __shared__
// array.
__device__ __forceinline__ uint32_t lds_table_read(uint32_t addr) {
    typedef __attribute__((address_space(3))) const uint32_t* lds_u32_ptr;
    return *reinterpret_cast<lds_u32_ptr>((uintptr_t)addr);
}

__device__ __forceinline__ float2 lds_table_read2(uint32_t addr) {
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    typedef __attribute__((address_space(3))) const f32x2_t* lds_f2_ptr;
    const f32x2_t v = *reinterpret_cast<lds_f2_ptr>((uintptr_t)addr);
    return make_float2(v.x, v.y);
}

// One stage of the in-quad transpose: lanes whose `bit` is 0 keep A and receive the partner's A
// into B; lanes whose bit is 1 keep B and receive the partner's B into A.
template <int DPP_CTRL>
__device__ __forceinline__ void quad_exchange(uint32_t& A, uint32_t& B, bool bit) {
    const uint32_t pa = (uint32_t)__builtin_amdgcn_update_dpp((int)A, (int)A, DPP_CTRL, 0xf, 0xf, true);
    const uint32_t pb = (uint32_t)__builtin_amdgcn_update_dpp((int)B, (int)B, DPP_CTRL, 0xf, 0xf, true);
    A = bit ? pb : A;
    B = bit ? B : pa;
}

// 4x4 transpose of r[0..3] across the four lanes of a quad: afterwards r[i] of lane q holds what
// r[q] of lane i (of the same quad) held.
__device__ __forceinline__ void transpose_quad(uint32_t& r0, uint32_t& r1, uint32_t& r2, uint32_t& r3, bool b0,
                                               bool b1) {
    quad_exchange<0xB1>(r0, r1, b0);  // quad_perm [1,0,3,2]
    quad_exchange<0xB1>(r2, r3, b0);
    quad_exchange<0x4E>(r0, r2, b1);  // quad_perm [2,3,0,1]
    quad_exchange<0x4E>(r1, r3, b1);
}

template <typename K>
hipError_t gemv_allow_lds(K kern, int bytes) {
    return hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
}

// row-streaming kernel, M = 1, 2 (nf4_gemv_rows.hip)
size_t gemv_rows_workspace_bytes(int64_t M, int64_t N, int64_t K);
hipError_t gemv_rows_setup();
hipError_t launch_gemv_rows(const MatmulArgs& a, int cus, hipStream_t stream);
bool gemv_rows_epilogue_possible(const MatmulArgs& a);
int gemv_rows_norm_parts(int64_t M, int64_t N, int64_t K, int cus);

// four-weight-rows-per-quad kernel, 3 <= M <= 8 (nf4_gemv_quad.hip)
size_t gemv_quad_workspace_bytes(int64_t M, int64_t N, int64_t K);
hipError_t gemv_quad_setup();
hipError_t launch_gemv_quad(const MatmulArgs& a, int cus, hipStream_t stream);
bool gemv_quad_halves_possible(int64_t N, int64_t K);
hipError_t launch_gemv_quad_halves(const MatmulArgs& a, int cus, hipStream_t stream);
bool gemv_quad_epilogue_possible(const MatmulArgs& a);
int gemv_quad_norm_parts(int64_t M, int64_t N, int64_t K, int cus, bool halves);

// MFMA tile kernel, 5 <= M <= 16 (nf4_gemv_tiles.hip)
size_t gemv_tiles_workspace_bytes(int64_t M, int64_t N, int64_t K);
hipError_t gemv_tiles_setup();
hipError_t launch_gemv_tiles(const MatmulArgs& a, int cus, hipStream_t stream);
bool gemv_tiles_epilogue_possible(const MatmulArgs& a);
int gemv_tiles_norm_parts(int64_t N);

// codes and absmax staged through LDS, 1 <= M <= 16, fp32 absmax, blocksize 64, K % 256 == 0 (nf4_gemv_stage.hip)
bool gemv_stage_possible(const MatmulArgs& a);
size_t gemv_stage_workspace_bytes(int64_t M, int64_t N, int64_t K);
enum : int { GEMV_KERNEL_ROWS = 1, GEMV_KERNEL_QUAD = 2, GEMV_KERNEL_QUAD_HALVES = 3, GEMV_KERNEL_TILES = 4, GEMV_KERNEL_STAGED = 5 };
int gemv_kernel_for(int64_t M, int64_t N, int64_t K, int block_log2, bool nested);
int gemv_plan_cus();  // CU count of the current device, 256 where there is none: what launch plans are judged on
int gemv_stage_norm_parts(int64_t M, int64_t N, int64_t K, int cus);  // EPI_RESID_NORM: partial sums per row of x (0: not served)
int gemv_stage_splits(int64_t K);  // K ranges of the staged kernel: 1 while the sixteen waves of a workgroup cover K (4096)
hipError_t gemv_stage_setup();
hipError_t launch_gemv_stage(const MatmulArgs& a, int cus, hipStream_t stream);

}  // namespace nf4
