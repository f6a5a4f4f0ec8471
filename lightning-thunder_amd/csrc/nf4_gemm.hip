// Prefill-shape fused NF4 dequant-matmul for gfx950, M > 16 rows of x.
//
// Replaces the dequantize_4bit + F.linear route of bitsandbytes.matmul_4bit
// (MatMul4Bit.forward), reached from thunder/transforms/quantization.py:39: instead of writing
// the whole bf16 weight to HBM and reading it back, every workgroup expands the NF4 tile it needs
// to bf16 in LDS -- bf16_rne(lut16[code] * absmax), the same value nf4hip_dequantize produces -- and
// contracts it with bf16 MFMA, fp32 accumulation, bf16 output.
//
// Tile: 128 (m) x 128 (n) x 64 (k) per workgroup of 256 threads (2 x 2 waves, 64 x 64 each),
// v_mfma_f32_32x32x16_bf16 with A = x and B = W, LDS double-buffered, rows padded to 144 bytes so
// that the 128-bit fragment reads are bank-conflict free.  One k step of 64 is exactly one
// quantisation block per weight row (blocksize 64), so the scale is one value per row per step.
#include "nf4_common.h"

namespace nf4 {
namespace {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;
typedef float float2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

constexpr int BM = 128, BN = 128, BK = 64;
constexpr int THREADS = 256;
constexpr int ROW_BYTES = BK * 2 + 16;                 // padded LDS row
constexpr int TILE_BYTES = (BM + BN) * ROW_BYTES;      // one stage: x tile then W tile
constexpr int LUT_BYTES = 16 * 256;                    // 16 fp32 entries replicated for 64 lanes
constexpr int SMEM_BYTES = 2 * TILE_BYTES + LUT_BYTES;

struct Staged {
    uint4 x[4];   // 4 x 8 bf16 of the x tile
    uint4 w;      // 32 codes of one weight row
    float scale;  // absmax of that row's block
};

template <bool NESTED>
__device__ __forceinline__ void load_tiles(const MatmulArgs& a, Staged& st, int m0, int n0, int k0, int tid) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int row = (tid >> 3) + 32 * u;
        const int seg = tid & 7;
        const int m = m0 + row;
        st.x[u] = m < a.M ? *reinterpret_cast<const uint4*>(a.x + (int64_t)m * a.K + k0 + seg * 8) : make_uint4(0, 0, 0, 0);
    }
    const int row = min(n0 + (tid >> 1), a.N - 1);
    const int half = tid & 1;
    const int64_t e = (int64_t)row * a.K + k0 + half * 32;
    st.w = load16_stream(a.packed + (e >> 1));
    const int64_t blk = e >> a.block_log2;
    st.scale = NESTED ? nested_absmax(a.nested, blk) : a.absmax[blk];
}

__device__ __forceinline__ void store_tiles(const Staged& st, uint8_t* stage, const uint8_t* lutrep, int tid) {
    // x tile
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int row = (tid >> 3) + 32 * u;
        const int seg = tid & 7;
        *reinterpret_cast<uint4*>(stage + row * ROW_BYTES + seg * 16) = st.x[u];
    }
    // W tile: 32 codes -> 32 bf16
    const int lane4 = (tid & 63) * 4;
    const int row = tid >> 1, half = tid & 1;
    uint8_t* dst = stage + (BM + row) * ROW_BYTES + half * 64;
    const uint32_t d[4] = {st.w.x, st.w.y, st.w.z, st.w.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        uint32_t o[4];
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const uint32_t byte = (d[j] >> (8 * b)) & 0xffu;
            const float v0 = *reinterpret_cast<const float*>(lutrep + (((byte >> 4) << 8) | lane4));
            const float v1 = *reinterpret_cast<const float*>(lutrep + (((byte & 15u) << 8) | lane4));
            float2_t f = {__fmul_rn(v0, st.scale), __fmul_rn(v1, st.scale)};
            o[b] = __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2_t));
        }
        *reinterpret_cast<uint4*>(dst + j * 16) = make_uint4(o[0], o[1], o[2], o[3]);
    }
}

template <bool NESTED>
__global__ __launch_bounds__(THREADS) void gemm_kernel(MatmulArgs a, int m_tiles, int n_tiles) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint8_t* lutrep = smem + 2 * TILE_BYTES;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;

    // fp32 code book replicated per lane: address = code << 8 | lane * 4
#pragma unroll
    for (int it = 0; it < 4; ++it) {
        const int idx = tid + THREADS * it;  // 1024 dwords
        reinterpret_cast<float*>(lutrep)[idx] = a.lut16[idx >> 6];
    }

    // Workgroups are handed to the 8 XCDs round-robin; remap so that the m tiles of one n tile
    // (which share the same weights) run on the same XCD and hit its L2.
    int id = blockIdx.x;
    const int total = m_tiles * n_tiles;
    if ((total & 7) == 0) id = (id & 7) * (total >> 3) + (id >> 3);
    const int nt = id / m_tiles;
    const int mt = id - nt * m_tiles;
    const int m0 = mt * BM, n0 = nt * BN;

    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int q = 0; q < 16; ++q) acc[i][j][q] = 0.0f;

    const int ksteps = a.K / BK;
    Staged st;
    load_tiles<NESTED>(a, st, m0, n0, 0, tid);
    __syncthreads();  // lutrep visible
    store_tiles(st, smem, lutrep, tid);
    __syncthreads();

    const int frag_row = lane & 31;
    const int frag_k = (lane >> 5) * 16;  // byte offset of this lane's 8 bf16 inside a 16-k slice
    for (int kt = 0; kt < ksteps; ++kt) {
        uint8_t* cur = smem + (kt & 1) * TILE_BYTES;
        uint8_t* nxt = smem + ((kt + 1) & 1) * TILE_BYTES;
        if (kt + 1 < ksteps) load_tiles<NESTED>(a, st, m0, n0, (kt + 1) * BK, tid);
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
            bf16x8 fa[2], fb[2];
#pragma unroll
            for (int i = 0; i < 2; ++i)
                fa[i] = *reinterpret_cast<const bf16x8*>(cur + (wm * 64 + i * 32 + frag_row) * ROW_BYTES + kk * 32 + frag_k);
#pragma unroll
            for (int j = 0; j < 2; ++j)
                fb[j] = *reinterpret_cast<const bf16x8*>(cur + (BM + wn * 64 + j * 32 + frag_row) * ROW_BYTES + kk * 32 + frag_k);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < ksteps) store_tiles(st, nxt, lutrep, tid);
        __syncthreads();
    }

    // epilogue: acc[i][j][q] = out[m][n], n = lane & 31, m = 8*(q/4) + 4*(lane/32) + q%4 inside the 32x32 tile
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int n = n0 + wn * 64 + j * 32 + (lane & 31);
        if (n >= a.N) continue;
        const float b = a.bias ? bf16_bits_to_f32(a.bias[n]) : 0.0f;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int q = 0; q < 16; ++q) {
                const int m = m0 + wm * 64 + i * 32 + 8 * (q >> 2) + 4 * (lane >> 5) + (q & 3);
                if (m < a.M) a.out[(int64_t)m * a.N + n] = (uint16_t)f32_to_bf16_bits(acc[i][j][q] + b);
            }
    }
}

template <typename K>
hipError_t allow_big_lds(K kern) {
    return hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                               SMEM_BYTES);
}

constexpr int MAX_DEVICES = 64;
bool g_ready[MAX_DEVICES] = {};

}  // namespace

size_t gemm_workspace_bytes(int64_t, int64_t, int64_t) { return 0; }

hipError_t launch_gemm(const MatmulArgs& a, hipStream_t stream) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= MAX_DEVICES) return hipErrorInvalidDevice;
    if (!g_ready[dev]) {
        if ((e = allow_big_lds(gemm_kernel<false>)) != hipSuccess) return e;
        if ((e = allow_big_lds(gemm_kernel<true>)) != hipSuccess) return e;
        g_ready[dev] = true;
    }
    const int m_tiles = (a.M + BM - 1) / BM;
    const int n_tiles = (a.N + BN - 1) / BN;
    const dim3 grid((unsigned)(m_tiles * n_tiles));
    if (a.nested.q)
        hipLaunchKernelGGL(gemm_kernel<true>, grid, dim3(THREADS), SMEM_BYTES, stream, a, m_tiles, n_tiles);
    else
        hipLaunchKernelGGL(gemm_kernel<false>, grid, dim3(THREADS), SMEM_BYTES, stream, a, m_tiles, n_tiles);
    return hipGetLastError();
}

}  // namespace nf4
