// Pieces shared by the three decode-shape kernels (row-streaming, four weight rows per lane quad, MFMA tiles).
#pragma once

#include "nf4_common.h"

namespace nf4 {

constexpr int GEMV_THREADS = 512;  // 8 waves; two workgroups per CU
constexpr int GEMV_WAVES = GEMV_THREADS / 64;
constexpr int GEMV_TABLE_BYTES = 256 * 256;     // 256 byte values x 64 lanes x 4 B
constexpr int GEMV_COUNTER_BYTES = (int)GEMV_COUNTER_REGION_BYTES;  // split-K arrival counters at the head of the workspace

// Byte -> (bf16, bf16) table at the start of LDS.  Entry b holds the code values of the two
// nibbles of b as bf16, the high nibble (even element) in the low half.  It is replicated for the
// 64 lanes with a 256-byte stride: lane l reads byte address (b << 8) | (l * 4), so every lane
// owns one bank column and a lookup is conflict-free whatever the data.
// `lut_lane` is lut16[lane & 15], loaded by the caller (early, so that its latency is hidden).
__device__ __forceinline__ void build_pair_table(uint8_t* smem, float lut_lane, int lane, int wave) {
    // Every entry is one dword replicated over a 256-byte row.  Sixteen lanes write one row with
    // 16-byte stores, so a wave writes four entries per instruction and its 32 entries in eight.
    const uint32_t lb = f32_to_bf16_bits(lut_lane);
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
// arithmetic (bf16(lut) * x on the matrix pipe, block sums scaled by absmax) differs from bf16(lut * absmax) * x by
// two independent bf16 roundings per weight, so its distance from the reference grows like sqrt(K): measured
// sigma 0.0027 / 0.0038 / 0.0047 at K = 4096 / 8192 / 14336 for N(0, 1) activations and N(0, 0.02) weights.  At K = 14336
// the 2e-2 tolerance is 4.2 sigma and about one output in 40 000 crosses it (seen at [4096, 14336], M = 16), at
// K = 8192 it is 5.2 sigma (one in five million).
__host__ __device__ constexpr bool gemv_wants_exact(int64_t K) { return K > 8192; }

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

// four-weight-rows-per-quad kernel, 3 <= M <= 8 (nf4_gemv_quad.hip)
size_t gemv_quad_workspace_bytes(int64_t M, int64_t N, int64_t K);
hipError_t gemv_quad_setup();
hipError_t launch_gemv_quad(const MatmulArgs& a, int cus, hipStream_t stream);

// MFMA tile kernel, 5 <= M <= 16 (nf4_gemv_tiles.hip)
size_t gemv_tiles_workspace_bytes(int64_t M, int64_t N, int64_t K);
hipError_t gemv_tiles_setup();
hipError_t launch_gemv_tiles(const MatmulArgs& a, int cus, hipStream_t stream);

}  // namespace nf4
