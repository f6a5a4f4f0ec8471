// Prefill-shape fused NF4 dequant-matmul for gfx950, M > 16 rows of x.
//
// Replaces the dequantize_4bit + F.linear route of bitsandbytes.matmul_4bit
// (MatMul4Bit.forward), reached from thunder/transforms/quantization.py:39: instead of writing
// the whole bf16 weight to HBM and reading it back, every workgroup expands the NF4 tile it needs
// to bf16 in LDS -- bf16_rne(lut16[code] * absmax), the same value nf4hip_dequantize produces -- and
// contracts it with bf16 MFMA, fp32 accumulation, bf16 output.
//
// Tile: BM (128 or 256 rows of x) x 256 (n) x 64 (k) per workgroup of 512 threads: 8 waves as
// 2 (m) x 4 (n), each BM/2 x 64 outputs, v_mfma_f32_32x32x16_bf16 with A = x and B = W.  LDS holds
// two stages of (BM + 256) rows padded to 144 bytes (128-bit fragment reads without bank
// conflicts) and the code book.  One k step of 64 is one quantisation block per weight row at
// blocksize 64, so a thread's 32 codes share one scale at every supported blocksize.
//
// Pipeline per k step kt: the registers loaded two steps earlier (x rows, codes, absmax of step
// kt + 1) are expanded into the other LDS stage between the MFMAs of step kt, then refilled with
// step kt + 2; one barrier per step.
#include "nf4_common.h"

#include <type_traits>

namespace nf4 {
namespace {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;
typedef float float2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

constexpr int BK = 64;
constexpr int BN = 256;
constexpr int THREADS = 512;
constexpr int ROW_BYTES = BK * 2 + 16;  // padded LDS row
constexpr int LUT_BYTES = 16 * 256;     // 16 fp32 entries, one copy per lane of a wave

template <int BM>
struct Tile {
    static constexpr int XA = BM / 64;  // 16-byte x loads per thread and k step
    static constexpr int A_BYTES = BM * ROW_BYTES;
    static constexpr int STAGE_BYTES = (BM + BN) * ROW_BYTES;
    static constexpr int SMEM_BYTES = LUT_BYTES + 2 * STAGE_BYTES;
    static constexpr int TI = BM / 64;  // 32-row MFMA tiles per wave along m (wave tile BM/2 x 64)
    static constexpr int TJ = 2;        // along n
    static constexpr int HI = TI / 2;   // x tiles per half slice
};

// What one thread holds of a k step on its way from global memory to LDS.
template <int XA>
struct Staged {
    uint4 x[XA];  // XA x 8 bf16 of the x tile
    uint4 w;      // 32 codes of one weight row
    float scale;  // absmax of their block
};

template <bool NESTED, int XA>
__device__ __forceinline__ void load_step(const MatmulArgs& a, Staged<XA>& st, const uint16_t* const (&xrow)[XA],
                                          int64_t e0, int k0) {
#pragma unroll
    for (int u = 0; u < XA; ++u) st.x[u] = load16(xrow[u] + k0);
    const int64_t e = e0 + k0;
    st.w = load16(a.packed + (e >> 1));
    const int64_t blk = e >> a.block_log2;
    st.scale = NESTED ? nested_absmax(a.nested, blk) : a.absmax[blk];
}

__device__ __forceinline__ uint32_t and_or(uint32_t x, uint32_t mask, uint32_t orv) {
    uint32_t r;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(x), "s"(mask), "v"(orv));
    return r;
}

// LDS addresses of the code-book entries of the 8 codes of one dword, in element order (high
// nibble of a byte first).  The book sits at the start of the workgroup's LDS, 256 bytes per
// code, one fp32 per lane: address = book | code << 8 | lane * 4, `book_lane` = book | lane * 4.
__device__ __forceinline__ void lut_addresses(uint32_t d, uint32_t book_lane, uint32_t (&addr)[8]) {
#pragma unroll
    for (int b = 0; b < 4; ++b) {
        addr[2 * b] = and_or(b == 0 ? d << 4 : d >> (8 * b - 4), 0xf00u, book_lane);
        addr[2 * b + 1] = and_or(b == 0 ? d << 8 : b == 1 ? d : d >> (8 * b - 8), 0xf00u, book_lane);
    }
}

__device__ __forceinline__ float lds_f32(uint32_t addr) {
    return *reinterpret_cast<const __attribute__((address_space(3))) float*>(addr);
}

__device__ __forceinline__ uint32_t dword_of(const uint4& w, int p) {
    return p == 0 ? w.x : p == 1 ? w.y : p == 2 ? w.z : w.w;
}

// 8 code-book values of one dword -> 8 bf16 = bf16_rne(value * scale), as 16 bytes
__device__ __forceinline__ uint4 scale_round(const float (&v)[8], float scale) {
    uint32_t o[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const float2_t f = {__fmul_rn(v[2 * c], scale), __fmul_rn(v[2 * c + 1], scale)};
        o[c] = __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2_t));
    }
    return make_uint4(o[0], o[1], o[2], o[3]);
}

template <bool NESTED, int BM>
__global__ __launch_bounds__(THREADS) void gemm_kernel(MatmulArgs a, int m_tiles, int n_tiles) {
    using T = Tile<BM>;
    using St = Staged<T::XA>;
    // 4 KiB alignment: the code-book addresses are formed with OR (lut_addresses)
    extern __shared__ __attribute__((aligned(4096))) uint8_t smem[];
    uint8_t* stages = smem + LUT_BYTES;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave & 1, wn = wave >> 1;

#pragma unroll
    for (int it = 0; it < 2; ++it) {
        const int idx = tid + THREADS * it;  // 1024 dwords: entry idx / 64, lane idx % 64
        reinterpret_cast<float*>(smem)[idx] = a.lut16[idx >> 6];
    }
    typedef __attribute__((address_space(3))) uint8_t* lds_ptr;
    const uint32_t book_lane = (uint32_t)(uintptr_t)(lds_ptr)smem + lane * 4;

    // Workgroups are handed to the 8 XCDs round-robin; give every XCD a contiguous run of tiles,
    // m fastest, so that the m tiles sharing one n tile's weights hit that XCD's L2.
    const int total = m_tiles * n_tiles;
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int chunk = total >> 3, rem = total & 7;
    const int id = xcd * chunk + min(xcd, rem) + slot;
    const int nt = id / m_tiles;
    const int mt = id - nt * m_tiles;
    const int m0 = mt * BM, n0 = nt * BN;

    f32x16 acc[T::TI][T::TJ];
#pragma unroll
    for (int i = 0; i < T::TI; ++i)
#pragma unroll
        for (int j = 0; j < T::TJ; ++j)
#pragma unroll
            for (int q = 0; q < 16; ++q) acc[i][j][q] = 0.0f;

    // Load bases.  x: thread -> row tid / 8 (+ 64 u), 16 bytes tid % 8 of the 128-byte k step; codes:
    // thread -> weight row tid / 2, half tid % 2 of the 64 codes.  Rows beyond M or N are clamped to
    // the last one (their outputs are never stored).
    const uint16_t* xrow[T::XA];
#pragma unroll
    for (int u = 0; u < T::XA; ++u)
        xrow[u] = a.x + (int64_t)min(m0 + (tid >> 3) + 64 * u, a.M - 1) * a.K + (tid & 7) * 8;
    const int64_t e0 = (int64_t)min(n0 + (tid >> 1), a.N - 1) * a.K + (tid & 1) * 32;
    const int a_st = (tid >> 3) * ROW_BYTES + (tid & 7) * 16;               // + 64 u rows
    const int b_st = T::A_BYTES + (tid >> 1) * ROW_BYTES + (tid & 1) * 64;  // + 16 bytes per dword of codes

    const int ksteps = a.K / BK;
    St s0, s1;
    load_step<NESTED>(a, s0, xrow, e0, 0);
    if (ksteps > 1) load_step<NESTED>(a, s1, xrow, e0, BK);
    __syncthreads();  // code book visible
#pragma unroll
    for (int u = 0; u < T::XA; ++u) *reinterpret_cast<uint4*>(stages + a_st + u * 64 * ROW_BYTES) = s0.x[u];
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        uint32_t addr[8];
        float v[8];
        lut_addresses(dword_of(s0.w, p), book_lane, addr);
#pragma unroll
        for (int c = 0; c < 8; ++c) v[c] = lds_f32(addr[c]);
        *reinterpret_cast<uint4*>(stages + b_st + p * 16) = scale_round(v, s0.scale);
    }
    __syncthreads();

    const int frag_row = lane & 31;
    const int frag_k = (lane >> 5) * 16;  // byte offset of this lane's 8 bf16 inside a 16-k slice
    const int a_off = (wm * (BM / 2) + frag_row) * ROW_BYTES + frag_k;
    const int b_off = T::A_BYTES + (wn * (BN / 4) + frag_row) * ROW_BYTES + frag_k;

    // One k step: MFMAs on stage kt & 1 in eight half slices (half of the wave's x tiles, both W
    // tiles, 16 k), the fragments of the next half slice read while the MFMAs of this one run.
    // `stg` (step kt + 1) is expanded into the other stage between them: code-book reads of dword p
    // in half slice 2p; scaling, rounding and the stores in half slice 2p + 1.  `ld` then receives
    // step kt + 2.  The scheduling fences keep each half slice's reads, MFMAs and expansion together.
    auto step = [&](int kt, St& ld, St& stg, auto full) {
        constexpr bool FULL = decltype(full)::value;  // steps kt + 1 and kt + 2 exist
        const uint8_t* cur = stages + (kt & 1) * T::STAGE_BYTES;
        uint8_t* nxt = stages + ((kt + 1) & 1) * T::STAGE_BYTES;
        const bool more = FULL || kt + 1 < ksteps;
        bf16x8 fa[2][T::HI], fb[2][T::TJ];
        auto read_frags = [&](int h) {
            const int kk = h >> 1, ih = h & 1;
#pragma unroll
            for (int i = 0; i < T::HI; ++i)
                fa[h & 1][i] =
                    *reinterpret_cast<const bf16x8*>(cur + a_off + (ih * T::HI + i) * 32 * ROW_BYTES + kk * 32);
#pragma unroll
            for (int j = 0; j < T::TJ; ++j)
                fb[h & 1][j] = *reinterpret_cast<const bf16x8*>(cur + b_off + j * 32 * ROW_BYTES + kk * 32);
        };
        float v[8];
        read_frags(0);
#pragma unroll
        for (int h = 0; h < 8; ++h) {
            if (h < 7) read_frags(h + 1);
#pragma unroll
            for (int i = 0; i < T::HI; ++i)
#pragma unroll
                for (int j = 0; j < T::TJ; ++j)
                    acc[(h & 1) * T::HI + i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                        fa[h & 1][i], fb[h & 1][j], acc[(h & 1) * T::HI + i][j], 0, 0, 0);
            if (more) {
                if ((h & 1) == 0) {
                    uint32_t addr[8];
                    lut_addresses(dword_of(stg.w, h >> 1), book_lane, addr);
#pragma unroll
                    for (int c = 0; c < 8; ++c) v[c] = lds_f32(addr[c]);
                } else {
                    *reinterpret_cast<uint4*>(nxt + b_st + (h >> 1) * 16) = scale_round(v, stg.scale);
                    if ((h >> 1) < T::XA)
                        *reinterpret_cast<uint4*>(nxt + a_st + (h >> 1) * 64 * ROW_BYTES) = stg.x[h >> 1];
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if (FULL || kt + 2 < ksteps) load_step<NESTED>(a, ld, xrow, e0, (kt + 2) * BK);
        __syncthreads();
    };
    // step 0 is in LDS, s1 holds step 1
    int kt = 0;
    for (; kt + 3 < ksteps; kt += 2) {
        step(kt, s0, s1, std::true_type{});      // expands s1 (step kt + 1), loads step kt + 2 into s0
        step(kt + 1, s1, s0, std::true_type{});  // expands s0 (step kt + 2), loads step kt + 3 into s1
    }
    for (; kt + 1 < ksteps; kt += 2) {
        step(kt, s0, s1, std::false_type{});
        step(kt + 1, s1, s0, std::false_type{});
    }
    if (kt < ksteps) step(kt, s0, s1, std::false_type{});

    // acc[i][j][q] = out[m][n], n = lane & 31, m = 8*(q/4) + 4*(lane/32) + q%4 inside the 32x32 tile
#pragma unroll
    for (int j = 0; j < T::TJ; ++j) {
        const int n = n0 + wn * (BN / 4) + j * 32 + (lane & 31);
        if (n >= a.N) continue;
        const float b = a.bias ? bf16_bits_to_f32(a.bias[n]) : 0.0f;
#pragma unroll
        for (int i = 0; i < T::TI; ++i)
#pragma unroll
            for (int q = 0; q < 16; ++q) {
                const int m = m0 + wm * (BM / 2) + i * 32 + 8 * (q >> 2) + 4 * (lane >> 5) + (q & 3);
                if (m < a.M) a.out[(int64_t)m * a.N + n] = (uint16_t)f32_to_bf16_bits(acc[i][j][q] + b);
            }
    }
}

constexpr int MAX_DEVICES = 64;

template <bool NESTED, int BM>
hipError_t launch_tile(const MatmulArgs& a, hipStream_t stream) {
    using T = Tile<BM>;
    static bool ready[MAX_DEVICES] = {};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= MAX_DEVICES) return hipErrorInvalidDevice;
    auto kern = gemm_kernel<NESTED, BM>;
    if (!ready[dev]) {
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                T::SMEM_BYTES);
        if (e != hipSuccess) return e;
        ready[dev] = true;
    }
    const int m_tiles = (a.M + BM - 1) / BM;
    const int n_tiles = (a.N + BN - 1) / BN;
    hipLaunchKernelGGL(kern, dim3((unsigned)(m_tiles * n_tiles)), dim3(THREADS), T::SMEM_BYTES, stream, a, m_tiles,
                       n_tiles);
    return hipGetLastError();
}

}  // namespace

size_t gemm_workspace_bytes(int64_t, int64_t, int64_t) { return 0; }

hipError_t launch_gemm(const MatmulArgs& a, hipStream_t stream) {
    // 128-row tiles while one of them covers x: the weight tile is expanded once per tile of x rows
    if (a.M <= 128) return a.nested.q ? launch_tile<true, 128>(a, stream) : launch_tile<false, 128>(a, stream);
    return a.nested.q ? launch_tile<true, 256>(a, stream) : launch_tile<false, 256>(a, stream);
}

}  // namespace nf4
