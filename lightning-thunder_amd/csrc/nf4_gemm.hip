// Prefill-shape fused NF4 dequant-matmul for gfx950, M > 16 rows of x.
//
// Replaces the dequantize_4bit + F.linear route of bitsandbytes.matmul_4bit
// (MatMul4Bit.forward), reached from thunder/transforms/quantization.py:39: instead of writing
// the whole bf16 weight to HBM and reading it back, every wave expands the NF4 codes it needs to
// bf16 in registers -- bf16_rne(lut16[code] * absmax), the same value nf4hip_dequantize produces --
// and contracts them with bf16 MFMA, fp32 accumulation, bf16 output.
//
// Tile: BM (64, 128 or 256 rows of x) x 256 (n) x 64 (k) per workgroup of 512 threads.  Wave w of 8
// owns weight rows 32 w .. + 31 of the tile against all BM rows of x: BM / 32 accumulators of
// v_mfma_f32_32x32x16_bf16 with A = x (from LDS) and B = W (from this wave's registers).  A lane
// loads 16 bytes = 32 codes of one weight row per k step; each of its four dwords becomes the B
// fragment of one 16-k slice, so the weights never pass through LDS.  The k order inside a step
// follows the codes (lane half h, slice s: k = 32 h + 8 s .. + 7) and the x fragments are read from
// LDS in the same order.  LDS holds two stages of BM rows of x padded to 144 bytes (128-bit
// fragment reads without bank conflicts) and the code book as a table of pairs: for every byte
// value the two fp32 entries of its codes, in 32 copies laid out so that the 32 lanes the LDS serves
// together never share a bank -- one ds_read_b64 per byte of codes.
//
// Up to 128 rows of x (one tile of x rows) K is split over up to 8 workgroups per weight tile when the
// weight has too few tiles for the chip; their fp32 partial tiles meet in the workspace and the last
// one to arrive adds them in split order.
//
// Pipeline per k step kt: x rows of step kt + 1 go from registers to the other LDS stage at the
// top of the step and the registers are refilled with step kt + 2; codes and absmax run two steps
// ahead in two register sets; the B fragment of slice s + 1 is expanded between the MFMAs of slice
// s (pair-book reads in its first half, scaling and rounding in its second); one barrier per step.
#include "nf4_gemv.h"

#include <type_traits>

namespace nf4 {
namespace {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;
typedef float float2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4v __attribute__((ext_vector_type(4)));

constexpr int BK = 64;
constexpr int BN = 256;
constexpr int THREADS = 512;
constexpr int ROW_BYTES = BK * 2 + 16;  // padded LDS row
constexpr int LUT_BYTES = 256 * 256;    // byte -> (fp32, fp32) of its two codes, 32 copies: 256 B per byte value

template <int BM>
struct Tile {
    static constexpr int XA = BM / 64;  // 16-byte x loads per thread and k step
    static constexpr int STAGE_BYTES = BM * ROW_BYTES;
    static constexpr int SMEM_BYTES = LUT_BYTES + 2 * STAGE_BYTES;
    static constexpr int TI = BM / 32;  // 32-row MFMA tiles per wave (every wave covers all BM rows)
    static constexpr int HI = TI / 2;   // x tiles per half slice
};

struct Codes {
    uint4 w;      // 32 codes of one weight row
    float scale;  // absmax of their block
    uint32_t q;   // nested absmax only: the 8-bit absmax code of the step this set is loaded with next
};

template <bool NESTED>
__device__ __forceinline__ void load_codes(const MatmulArgs& a, Codes& c, int64_t e) {
    c.w = load16(a.packed + (e >> 1));
    const int64_t blk = e >> a.block_log2;
    c.scale = NESTED ? nested_absmax(a.nested, blk) : a.absmax[blk];
}

// Nested absmax inside the k loop: the 8-bit code is fetched one step before the two look-ups that
// depend on it, so that no load in the loop waits for another (same arithmetic as nested_absmax).
__device__ __forceinline__ void load_absmax_code(const MatmulArgs& a, Codes& c, int64_t e) {
    c.q = a.nested.q[e >> a.block_log2];
}
__device__ __forceinline__ void load_codes_staged(const MatmulArgs& a, Codes& c, int64_t e) {
    c.w = load16(a.packed + (e >> 1));
    const int64_t blk = e >> a.block_log2;
    const float m = a.nested.map256[c.q];
    const float s = a.nested.absmax2[blk >> a.nested.nested_log2];
    c.scale = __fadd_rn(__fmul_rn(m, s), a.nested.offset);
}

__device__ __forceinline__ uint32_t and_or(uint32_t x, uint32_t mask, uint32_t orv) {
    uint32_t r;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(x), "s"(mask), "v"(orv));
    return r;
}

// The pair book: for every byte value (two codes) the two fp32 code-book entries, high nibble first,
// in 32 copies: address = book | byte << 8 | copy << 3.  A lane uses copy lane % 32, so the 32 lanes
// that the LDS serves together hit 32 different bank pairs whatever their bytes are.
__device__ __forceinline__ void lut_addresses(uint32_t d, uint32_t book_lane, uint32_t (&addr)[4]) {
    addr[0] = and_or(d << 8, 0xff00u, book_lane);
    addr[1] = and_or(d, 0xff00u, book_lane);
    addr[2] = and_or(d >> 8, 0xff00u, book_lane);
    addr[3] = and_or(d >> 16, 0xff00u, book_lane);
}

__device__ __forceinline__ float2_t lds_f32x2(uint32_t addr) {
    return *reinterpret_cast<const __attribute__((address_space(3))) float2_t*>(addr);
}

__device__ __forceinline__ uint32_t dword_of(const uint4& w, int p) {
    return p == 0 ? w.x : p == 1 ? w.y : p == 2 ? w.z : w.w;
}

// 8 code-book values of one dword -> 8 bf16 = bf16_rne(value * scale): one MFMA B fragment
__device__ __forceinline__ bf16x8 scale_round(const float (&v)[8], float scale) {
    u32x4v o;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const float2_t f = {__fmul_rn(v[2 * c], scale), __fmul_rn(v[2 * c + 1], scale)};
        o[c] = __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2_t));
    }
    return __builtin_bit_cast(bf16x8, o);
}

// 8 waves, wave w: all BM rows of x by weight rows n0 + 32 w .. + 31.  Lane l holds weight row l % 32,
// codes 32 (l / 32) .. + 31 of the k step; its dword s is the B fragment of slice s, covering
// k = 32 (l / 32) + 8 s .. + 7, and the x fragments are read from LDS in the same k order.
template <bool NESTED, int BM>
__global__ __launch_bounds__(THREADS) void gemm_kernel(MatmulArgs a, int m_tiles, int n_tiles, int splits,
                                                           uint32_t* counters, float* partials) {
    using T = Tile<BM>;
    extern __shared__ __attribute__((aligned(4096))) uint8_t smem[];
    uint8_t* stages = smem + LUT_BYTES;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;

    // pair book: thread tid writes copy tid % 32 of the 16 byte values (it << 4) | (tid / 32)
    {
        const float second = a.lut16[tid >> 5];
#pragma unroll
        for (int it = 0; it < 16; ++it) {
            const float2_t pair = {a.lut16[it], second};
            *reinterpret_cast<float2_t*>(smem + (((it << 4) | (tid >> 5)) << 8) + ((tid & 31) << 3)) = pair;
        }
    }
    typedef __attribute__((address_space(3))) uint8_t* lds_ptr;
    const uint32_t book_lane = (uint32_t)(uintptr_t)(lds_ptr)smem + (lane & 31) * 8;

    const int total = m_tiles * n_tiles;
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int chunk = total >> 3, rem = total & 7;
    const int id = xcd * chunk + min(xcd, rem) + slot;
    const int nt = id / m_tiles;
    const int mt = id - nt * m_tiles;
    const int m0 = mt * BM, n0 = nt * BN;
    // K split over blockIdx.y: this workgroup's steps start at k_base
    const int ksteps = a.K / BK / splits;
    const int k_base = blockIdx.y * ksteps * BK;

    f32x16 acc[T::TI];
#pragma unroll
    for (int i = 0; i < T::TI; ++i)
#pragma unroll
        for (int q = 0; q < 16; ++q) acc[i][q] = 0.0f;

    const uint16_t* xrow[T::XA];
#pragma unroll
    for (int u = 0; u < T::XA; ++u)
        xrow[u] = a.x + (int64_t)min(m0 + (tid >> 3) + 64 * u, a.M - 1) * a.K + k_base + (tid & 7) * 8;
    const int a_st = (tid >> 3) * ROW_BYTES + (tid & 7) * 16;  // + 64 u rows
    const int64_t e0 = (int64_t)min(n0 + wave * 32 + (lane & 31), a.N - 1) * a.K + k_base + (lane >> 5) * 32;
    const int a_off = (lane & 31) * ROW_BYTES + (lane >> 5) * 64;  // + 32 i rows, + 16 bytes per slice

    uint4 xa[T::XA];
    Codes c0, c1;
#pragma unroll
    for (int u = 0; u < T::XA; ++u) xa[u] = load16(xrow[u]);
    load_codes<NESTED>(a, c0, e0);
    if (ksteps > 1) load_codes<NESTED>(a, c1, e0 + BK);
    if (NESTED && ksteps > 2) load_absmax_code(a, c0, e0 + 2 * BK);
    __syncthreads();  // code book visible
#pragma unroll
    for (int u = 0; u < T::XA; ++u) *reinterpret_cast<uint4*>(stages + a_st + u * 64 * ROW_BYTES) = xa[u];
    if (ksteps > 1) {
#pragma unroll
        for (int u = 0; u < T::XA; ++u) xa[u] = load16(xrow[u] + BK);
    }
    bf16x8 fb;
    {
        uint32_t addr[4];
        float v[8];
        lut_addresses(c0.w.x, book_lane, addr);
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const float2_t p = lds_f32x2(addr[c]);
            v[2 * c] = p.x;
            v[2 * c + 1] = p.y;
        }
        fb = scale_round(v, c0.scale);
    }
    __syncthreads();

    // One k step.  `cur` holds the codes of step kt (dword 0 already expanded into fb), `nxt` those
    // of step kt + 1; xa holds the x rows of step kt + 1.
    auto step = [&](int kt, Codes& cur, Codes& nxt, auto full) {
        constexpr bool FULL = decltype(full)::value;  // steps kt + 1 and kt + 2 exist
        const uint8_t* st = stages + (kt & 1) * T::STAGE_BYTES;
        uint8_t* st_next = stages + ((kt + 1) & 1) * T::STAGE_BYTES;
        const bool more = FULL || kt + 1 < ksteps;
        const bool more2 = FULL || kt + 2 < ksteps;
        if (more) {
#pragma unroll
            for (int u = 0; u < T::XA; ++u) *reinterpret_cast<uint4*>(st_next + a_st + u * 64 * ROW_BYTES) = xa[u];
        }
        if (more2) {
#pragma unroll
            for (int u = 0; u < T::XA; ++u) xa[u] = load16(xrow[u] + (kt + 2) * BK);
        }
        bf16x8 fa[2][T::HI];
        auto read_frags = [&](int h) {  // half slice h: slice h / 2, x tiles (h % 2) * HI ..
#pragma unroll
            for (int i = 0; i < T::HI; ++i)
                fa[h & 1][i] = *reinterpret_cast<const bf16x8*>(st + a_off + ((h & 1) * T::HI + i) * 32 * ROW_BYTES +
                                                                (h >> 1) * 16);
        };
        float v[8];
        bf16x8 fbn = fb;
        read_frags(0);
#pragma unroll
        for (int h = 0; h < 8; ++h) {
            const int kk = h >> 1;
            if (h < 7) read_frags(h + 1);
#pragma unroll
            for (int i = 0; i < T::HI; ++i)
                acc[(h & 1) * T::HI + i] =
                    __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[h & 1][i], fb, acc[(h & 1) * T::HI + i], 0, 0, 0);
            // the B fragment of the next slice: dword kk + 1 of this step, or dword 0 of the next step
            if (kk < 3 || more) {
                const Codes& src = kk < 3 ? cur : nxt;
                if ((h & 1) == 0) {
                    uint32_t addr[4];
                    lut_addresses(dword_of(src.w, (kk + 1) & 3), book_lane, addr);
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        const float2_t p = lds_f32x2(addr[c]);
                        v[2 * c] = p.x;
                        v[2 * c + 1] = p.y;
                    }
                } else {
                    fbn = scale_round(v, src.scale);
                }
            }
            if (h == 6 && more2) {  // cur's dwords are used up
                if (NESTED) {
                    load_codes_staged(a, cur, e0 + (int64_t)(kt + 2) * BK);
                    if (kt + 3 < ksteps) load_absmax_code(a, nxt, e0 + (int64_t)(kt + 3) * BK);
                } else {
                    load_codes<false>(a, cur, e0 + (int64_t)(kt + 2) * BK);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            if (h & 1) fb = fbn;
        }
        __syncthreads();
    };
    int kt = 0;
    for (; kt + 3 < ksteps; kt += 2) {
        step(kt, c0, c1, std::true_type{});
        step(kt + 1, c1, c0, std::true_type{});
    }
    for (; kt + 1 < ksteps; kt += 2) {
        step(kt, c0, c1, std::false_type{});
        step(kt + 1, c1, c0, std::false_type{});
    }
    if (kt < ksteps) step(kt, c0, c1, std::false_type{});

    if (splits > 1) {
        // Partial sums of this K split go to the workspace in register order ([i][q][thread]: coalesced);
        // the last split to arrive for the tile adds all of them in split order (deterministic) and
        // writes the result.  Ordering without L2-wide fences: agent-scope stores go through to L2, every
        // store of the workgroup has completed (s_waitcnt, barrier) before its arrival is counted, and the
        // last workgroup reads with agent-scope loads, which bypass its CU's L1.
        float* tile_part = partials + (int64_t)id * splits * (T::TI * 16 * THREADS);
        float* mine = tile_part + (int64_t)blockIdx.y * (T::TI * 16 * THREADS);
#pragma unroll
        for (int i = 0; i < T::TI; ++i)
#pragma unroll
            for (int q = 0; q < 16; ++q)
                __hip_atomic_store(mine + (i * 16 + q) * THREADS + tid, acc[i][q], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        publish_partials();
        __syncthreads();
        uint32_t* flag = reinterpret_cast<uint32_t*>(smem);
        if (tid == 0) *flag = __hip_atomic_fetch_add(&counters[id], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        acquire_partials();
        if (*flag != (uint32_t)(splits - 1)) return;
        // G splits' worth of loads are issued before the first add, so the merge costs a few memory
        // round trips instead of one per split
        constexpr int G = BM <= 64 ? 8 : 4;
#pragma unroll
        for (int i = 0; i < T::TI; ++i) {
            float sum[16];
#pragma unroll
            for (int q = 0; q < 16; ++q) sum[q] = 0.0f;
            for (int sp0 = 0; sp0 < splits; sp0 += G) {
                float v[G][16];
#pragma unroll
                for (int g = 0; g < G; ++g) {
                    const int sp = min(sp0 + g, splits - 1);
                    const float* src = tile_part + (int64_t)sp * (T::TI * 16 * THREADS) + i * 16 * THREADS + tid;
#pragma unroll
                    for (int q = 0; q < 16; ++q)
                        v[g][q] = __hip_atomic_load(src + q * THREADS, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
#pragma unroll
                for (int g = 0; g < G; ++g)
                    if (sp0 + g < splits) {
#pragma unroll
                        for (int q = 0; q < 16; ++q) sum[q] += v[g][q];
                    }
            }
#pragma unroll
            for (int q = 0; q < 16; ++q) acc[i][q] = sum[q];
        }
        if (tid == 0) __hip_atomic_store(&counters[id], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }

    // acc[i][q] = out[m][n], n = lane & 31, m = 8*(q/4) + 4*(lane/32) + q%4 inside the 32x32 tile
    const int n = n0 + wave * 32 + (lane & 31);
    if (n < a.N) {
        const float b = a.bias ? bf16_bits_to_f32(a.bias[n]) : 0.0f;
#pragma unroll
        for (int i = 0; i < T::TI; ++i)
#pragma unroll
            for (int q = 0; q < 16; ++q) {
                const int m = m0 + i * 32 + 8 * (q >> 2) + 4 * (lane >> 5) + (q & 3);
                if (m < a.M) a.out[(int64_t)m * a.N + n] = (uint16_t)f32_to_bf16_bits(acc[i][q] + b);
            }
    }
}

constexpr int MAX_DEVICES = 64;
// arrival counters at the head of the workspace: the same region as the decode kernels', so that one
// zero-initialised workspace serves both (partial sums never land where the other expects zeroed counters)
constexpr size_t GEMM_COUNTER_BYTES = GEMV_COUNTER_BYTES;

// K splits for up to 128 rows of x (one tile of x rows): as many workgroups as fit the chip's 256 CUs in
// one round when the weight has few 256-row tiles; the k steps divide evenly and every split keeps at
// least 4.
int gemm_splits(int64_t M, int64_t N, int64_t K) {
    if (M > 128) return 1;
    const int64_t tiles = (N + BN - 1) / BN;
    const int64_t ksteps = K / BK;
    int best = 1;
    for (int s = 2; s <= 8; ++s)
        if (tiles * s <= 256 && ksteps % s == 0 && ksteps / s >= 4) best = s;
    return best;
}

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
    const int splits = gemm_splits(a.M, a.N, a.K);
    uint32_t* counters = static_cast<uint32_t*>(a.workspace);
    float* partials = splits > 1 ? reinterpret_cast<float*>(static_cast<uint8_t*>(a.workspace) + GEMM_COUNTER_BYTES) : nullptr;
    hipLaunchKernelGGL(kern, dim3((unsigned)(m_tiles * n_tiles), (unsigned)splits), dim3(THREADS), T::SMEM_BYTES, stream, a,
                       m_tiles, n_tiles, splits, counters, partials);
    return hipGetLastError();
}

}  // namespace

size_t gemm_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    if (M > 128) return M * K * 2 < ((int64_t)1 << 32) ? gemm_wide_workspace_bytes(M, N, K) : 0;
    const int splits = gemm_splits(M, N, K);
    if (splits == 1) return 0;
    const int64_t bm = M <= 64 ? 64 : 128;
    return GEMM_COUNTER_BYTES + (size_t)((N + BN - 1) / BN) * splits * bm * BN * sizeof(float);
}

void gemm_plan(int64_t M, int64_t N, int64_t K, int plan[4]) {
    if (M > 128 && M * K * 2 < ((int64_t)1 << 32)) return gemm_wide_plan(M, N, K, plan);
    const int bm = M <= 64 ? 64 : M <= 128 ? 128 : 256;
    const int64_t tiles = ((M + bm - 1) / bm) * ((N + BN - 1) / BN);
    plan[0] = bm;
    plan[1] = (int)tiles;
    plan[2] = gemm_splits(M, N, K);
    plan[3] = (int)tiles * plan[2];
}

hipError_t launch_gemm(const MatmulArgs& a, hipStream_t stream) {
    // the smallest tile height that covers x with one tile: the weight tile is expanded once per tile of x rows
    if (a.M <= 64) return a.nested.q ? launch_tile<true, 64>(a, stream) : launch_tile<false, 64>(a, stream);
    if (a.M <= 128) return a.nested.q ? launch_tile<true, 128>(a, stream) : launch_tile<false, 128>(a, stream);
    // more rows: the kernel of nf4_gemm_wide.hip, whose x loads address x with 32-bit offsets
    if ((int64_t)a.M * a.K * 2 < ((int64_t)1 << 32)) return launch_gemm_wide(a, stream);
    return a.nested.q ? launch_tile<true, 256>(a, stream) : launch_tile<false, 256>(a, stream);
}

}  // namespace nf4
