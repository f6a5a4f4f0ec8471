// Decode-shape fused NF4 dequant-matmul for gfx950, 5 <= M <= 16 rows of x (MFMA tiles), and the
// dispatch between it, the row-streaming kernel (M = 1) and the four-rows-per-quad kernel (M = 2..4).
//
// Replaces bitsandbytes' gemv_4bit (kgemm_4bit_inference_naive), the kernel that
// bitsandbytes.matmul_4bit picks for a single-row x; call site
// thunder/transforms/quantization.py:39.
//
// The kernel is HBM-bound: per weight it moves 4 bits of code plus 1/blocksize of an fp32 absmax.
// Design (one wave64 = one 16-row tile of W, all of the workgroup's K range):
//
//  * Weight stream.  Lane (c = lane & 15, g = lane >> 4) owns row n0 + c and loads 16 bytes
//    (32 codes) at byte offset 16*g of every 64-byte chunk of that row, so the four lanes of a row
//    read 64 contiguous bytes and two loads per step cover a full 128-byte line.  Loads are issued
//    one phase (512 k) ahead of their use and never pass through LDS.
//  * Code -> bf16.  A 256-entry table indexed by a whole packed BYTE returns both bf16 code values
//    of that byte as one dword (first element in the low half, as MFMA wants it).  The table is
//    replicated for all 64 lanes with a 256-byte stride, so its LDS address is
//    (byte << 8) | (lane * 4): one v_perm_b32 per byte, and every lane hits its own bank column.
//  * Contraction.  v_mfma_f32_16x16x32_bf16 with A = x (rows m) and B = W (columns n).  The k order
//    inside an MFMA is free as long as A and B agree, which lets a lane feed the four dwords of its
//    16-byte load to four different MFMAs.  A 4x4 dword transpose across the four lanes of a row
//    (v_permlane32_swap + v_permlane16_swap) makes every MFMA cover 32 CONSECUTIVE k, so that two
//    MFMAs = one 64-element quantisation block, whose partial sum is then scaled by absmax.
//    With B = W the accumulator of a lane belongs to the lane's own row, so that scale is the one
//    the lane loaded itself: 4 FMAs per block, no cross-lane traffic.
//  * x.  The workgroup stages x[0:16, 512 k] per phase into LDS already permuted into MFMA
//    A-operand order (rows >= M stay zero), so the inner loop reads it with linear ds_read_b128.
//  * K split.  When N alone cannot fill the chip, K is split over workgroups; partial sums go to a
//    workspace and the last workgroup to finish a row group (device-scope counter) adds them in a
//    fixed order, so the result does not depend on scheduling.
#include "nf4_gemv.h"

namespace nf4 {
namespace {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

constexpr int THREADS = GEMV_THREADS;
constexpr int WAVES = GEMV_WAVES;
constexpr int TABLE_BYTES = GEMV_TABLE_BYTES;
constexpr int PHASE_K = 512;                // k per phase (two steps of 256)
constexpr int XOPS_BYTES = 16 * PHASE_K * 2;  // x operands of one phase, 16 rows
constexpr int SMEM_BYTES = TABLE_BYTES + XOPS_BYTES;
constexpr int COUNTER_BYTES = GEMV_COUNTER_BYTES;

struct Plan {
    int tiles;        // ceil(N / 16)
    int tile_groups;  // ceil(tiles / 8): one workgroup handles 8 tiles = 128 rows
    int splits;       // K splits across workgroups
    int phases;       // phases per split
    int ntasks;       // tile_groups * splits
};

struct PhaseRegs {
    uint4 w[2][2];    // [step][chunk]: 32 codes each
    float4 s[2];      // [step]: absmax of the 4 blocks of the step (or raw data to build them)
    uint4 x[2];       // this thread's share of the x operands of the phase
};

// 4x4 dword transpose across the lanes {c, c+16, c+32, c+48}: afterwards element a of lane g holds
// what element g of lane a held.
__device__ __forceinline__ void transpose_g(uint32_t d[4]) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {  // lane bit 5 <-> element bit 1
        auto r = __builtin_amdgcn_permlane32_swap(d[j], d[j + 2], false, false);
        d[j] = r[0];
        d[j + 2] = r[1];
    }
#pragma unroll
    for (int j = 0; j < 4; j += 2) {  // lane bit 4 <-> element bit 0
        auto r = __builtin_amdgcn_permlane16_swap(d[j], d[j + 1], false, false);
        d[j] = r[0];
        d[j + 1] = r[1];
    }
}

template <bool B64, bool NESTED>
__device__ __forceinline__ void load_phase(const MatmulArgs& a, PhaseRegs& r, const uint8_t* wrow, int64_t row_elem0,
                                           int kphase, int tid) {
    // wrow = first byte of this lane's share of its row; row_elem0 = flat index of the row's first
    // element; kphase = absolute k at which the phase starts
    // weights: 4 x 16 B, streaming
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int c = 0; c < 2; ++c)
            r.w[s][c] = load16_stream(wrow + (kphase >> 1) + s * 128 + c * 64);
    // absmax of the 8 blocks of 64 k in this phase
#pragma unroll
    for (int s = 0; s < 2; ++s) {
        const int64_t e = row_elem0 + kphase + s * 256;
        if (NESTED) {
            if (B64) {
                const int64_t b = e >> 6;
                const uint32_t q = *reinterpret_cast<const uint32_t*>(a.nested.q + b);
                r.s[s].x = __uint_as_float(q);
                r.s[s].y = a.nested.absmax2[b >> a.nested.nested_log2];
            } else {
                // all four 64-k sub-blocks of a step share one or two blocks: resolve at use
                r.s[s].x = nested_absmax(a.nested, e >> a.block_log2);
                r.s[s].y = nested_absmax(a.nested, (e + 64) >> a.block_log2);
                r.s[s].z = nested_absmax(a.nested, (e + 128) >> a.block_log2);
                r.s[s].w = nested_absmax(a.nested, (e + 192) >> a.block_log2);
            }
        } else if (B64) {
            r.s[s] = *reinterpret_cast<const float4*>(a.absmax + (e >> 6));
        } else {
            r.s[s].x = a.absmax[e >> a.block_log2];
            r.s[s].y = a.absmax[(e + 64) >> a.block_log2];
            r.s[s].z = a.absmax[(e + 128) >> a.block_log2];
            r.s[s].w = a.absmax[(e + 192) >> a.block_log2];
        }
    }
    // x operands: slot = tid + 512*u -> (chunk, a, g, m); rows >= M are never loaded (stay zero in LDS)
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        const int slot = tid + THREADS * u;
        const int m = slot & 15, gg = (slot >> 4) & 3, aa = (slot >> 6) & 3, chunk = slot >> 8;
        if (m < a.M)
            r.x[u] = *reinterpret_cast<const uint4*>(a.x + (int64_t)m * a.K + kphase + chunk * 128 + aa * 32 + gg * 8);
    }
}

template <bool B64, bool NESTED>
__device__ __forceinline__ void compute_phase(const MatmulArgs& a, const PhaseRegs& r, const uint8_t* smem, int lane,
                                              f32x4& acc) {
    const uint32_t lane4 = (uint32_t)lane * 4u;
    const uint4* xops = reinterpret_cast<const uint4*>(smem + TABLE_BYTES);
#pragma unroll
    for (int s = 0; s < 2; ++s) {
        float sc[4];
        if (NESTED && B64) {
            const uint32_t q = __float_as_uint(r.s[s].x);
            const float a2 = r.s[s].y;
#pragma unroll
            for (int j = 0; j < 4; ++j)
                sc[j] = __fadd_rn(__fmul_rn(a.nested.map256[(q >> (8 * j)) & 0xffu], a2), a.nested.offset);
        } else {
            sc[0] = r.s[s].x; sc[1] = r.s[s].y; sc[2] = r.s[s].z; sc[3] = r.s[s].w;
        }
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            uint32_t d[4] = {r.w[s][c].x, r.w[s][c].y, r.w[s][c].z, r.w[s][c].w};
            transpose_g(d);
            f32x4 blk = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int aa = 0; aa < 4; ++aa) {
                uint32_t p[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    // LDS byte address = (byte j of d[aa]) << 8 | lane*4
                    const uint32_t addr = __builtin_amdgcn_perm(d[aa], lane4, 0x0c0c0400u | ((uint32_t)j << 8));
                    p[j] = lds_table_read(addr);
                }
                const uint4 xa = xops[((s * 2 + c) * 4 + aa) * 64 + lane];
                const uint4 wb = make_uint4(p[0], p[1], p[2], p[3]);
                blk = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, xa),
                                                              __builtin_bit_cast(bf16x8, wb), blk, 0, 0, 0);
                if (aa & 1) {
                    const float scale = sc[c * 2 + (aa >> 1)];
#pragma unroll
                    for (int q = 0; q < 4; ++q) acc[q] = fmaf(scale, blk[q], acc[q]);
                    blk = f32x4{0.f, 0.f, 0.f, 0.f};
                }
            }
            // keep the scheduler from hoisting the next chunk's table reads over this one: the
            // kernel has a 128-VGPR budget (4 waves per SIMD)
            __builtin_amdgcn_sched_barrier(0);
        }
    }
}

template <bool B64, bool NESTED>
__global__ __launch_bounds__(THREADS, 4) void gemv_kernel(MatmulArgs a, Plan p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    // The first word of the x-operand buffer doubles as the "last workgroup" flag of the split-K
    // epilogue: it is only written after the barrier that follows the last compute of a task, and
    // slot 0 (row 0 of x) is rewritten by the next phase anyway.
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col = lane & 15, g = lane >> 4;

    build_pair_table(smem, a.lut16[lane & 15], lane, wave);
    {
        uint4* xops = reinterpret_cast<uint4*>(smem + TABLE_BYTES);
        xops[tid] = make_uint4(0, 0, 0, 0);
        xops[tid + THREADS] = make_uint4(0, 0, 0, 0);
    }

    unsigned* counters = reinterpret_cast<unsigned*>(a.workspace);
    float* partial = reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(a.workspace) + COUNTER_BYTES);

    for (int task = blockIdx.x; task < p.ntasks; task += gridDim.x) {
        const int tg = task / p.splits;
        const int ks = task - tg * p.splits;
        const int tile = tg * WAVES + wave;
        const int n0 = tile * 16;
        const int row = min(n0 + col, a.N - 1);
        const int kbase = ks * p.phases * PHASE_K;
        const int64_t row_elem0 = (int64_t)row * a.K;
        const uint8_t* wrow = a.packed + (row_elem0 >> 1) + g * 16;

        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        PhaseRegs ra, rb;
        load_phase<B64, NESTED>(a, ra, wrow, row_elem0, kbase, tid);

        auto phase = [&](int ph, PhaseRegs& cur, PhaseRegs& nxt) {
            __syncthreads();  // every wave is done with the previous x operands (and the table is built)
            {
                uint4* xops = reinterpret_cast<uint4*>(smem + TABLE_BYTES);
#pragma unroll
                for (int u = 0; u < 2; ++u)
                    if (((tid + THREADS * u) & 15) < a.M) xops[tid + THREADS * u] = cur.x[u];
            }
            __syncthreads();
            if (ph + 1 < p.phases) load_phase<B64, NESTED>(a, nxt, wrow, row_elem0, kbase + (ph + 1) * PHASE_K, tid);
            compute_phase<B64, NESTED>(a, cur, smem, lane, acc);
        };
        for (int ph = 0; ph < p.phases; ph += 2) {
            phase(ph, ra, rb);
            if (ph + 1 < p.phases) phase(ph + 1, rb, ra);
        }

        // ---- epilogue: lane holds out[m = 4g + q][n = n0 + col] ----
        const int n = n0 + col;
        if (p.splits == 1) {
            if (n < a.N) {
                const float b = a.bias ? bf16_bits_to_f32(a.bias[n]) : 0.0f;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int m = 4 * g + q;
                    if (m < a.M) a.out[(int64_t)m * a.N + n] = (uint16_t)f32_to_bf16_bits(acc[q] + b);
                }
            }
        } else {
            // Partial sums cross workgroups (and XCDs, whose L2s are not coherent with each other)
            // through agent-scope relaxed atomics only: such stores write through and such loads
            // bypass stale lines, so no L2-wide write-back/invalidate fence is needed.  Ordering:
            // every store has completed (s_waitcnt) before the workgroup bumps the counter.
            if (n < a.N) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int m = 4 * g + q;
                    if (m < a.M)
                        __hip_atomic_store(&partial[((int64_t)ks * a.M + m) * a.N + n], acc[q], __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT);
                }
            }
            __builtin_amdgcn_s_waitcnt(0);
            __syncthreads();
            int* flag = reinterpret_cast<int*>(smem + TABLE_BYTES);
            if (tid == 0) {
                const unsigned prev =
                    __hip_atomic_fetch_add(&counters[tg], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                *flag = (prev == (unsigned)p.splits - 1u);
            }
            __syncthreads();
            const bool is_last = *flag != 0;
            if (is_last) {
                const int rows = min(WAVES * 16, a.N - tg * WAVES * 16);
                for (int idx = tid; idx < rows * a.M; idx += THREADS) {
                    const int m = idx / rows;
                    const int nn = tg * WAVES * 16 + (idx - m * rows);
                    float sum = 0.0f;
                    for (int k2 = 0; k2 < p.splits; ++k2)
                        sum += __hip_atomic_load(&partial[((int64_t)k2 * a.M + m) * a.N + nn], __ATOMIC_RELAXED,
                                                 __HIP_MEMORY_SCOPE_AGENT);
                    if (a.bias) sum += bf16_bits_to_f32(a.bias[nn]);
                    a.out[(int64_t)m * a.N + nn] = (uint16_t)f32_to_bf16_bits(sum);
                }
                if (tid == 0) __hip_atomic_store(&counters[tg], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
}

// Work split.  `slots` = workgroups resident at once (two per CU).
Plan make_plan(int64_t N, int64_t K, int slots) {
    Plan p;
    p.tiles = (int)((N + 15) / 16);
    p.tile_groups = (p.tiles + WAVES - 1) / WAVES;
    const int phases_total = (int)(K / PHASE_K);
    int best = 1;
    for (int s = 1; s <= phases_total; ++s)
        if (phases_total % s == 0 && (int64_t)p.tile_groups * s <= slots) best = s;
    p.splits = best;
    p.phases = phases_total / best;
    p.ntasks = p.tile_groups * p.splits;
    return p;
}

constexpr int MAX_DEVICES = 64;
int g_num_cus[MAX_DEVICES] = {};  // 0 = not set up yet; set once per device (benign if set twice)

// CU count of the current device; on first use on a device also raises the kernels' LDS limit.
hipError_t device_setup(int* cus_out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= MAX_DEVICES) return hipErrorInvalidDevice;
    if (!g_num_cus[dev]) {
        int cus = 0;
        e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
        if (e != hipSuccess) return e;
        if ((e = gemv_tiles_setup()) != hipSuccess) return e;
        if ((e = gemv_rows_setup()) != hipSuccess) return e;
        if ((e = gemv_quad_setup()) != hipSuccess) return e;
        g_num_cus[dev] = cus > 0 ? cus : 256;
    }
    *cus_out = g_num_cus[dev];
    return hipSuccess;
}

}  // namespace

size_t gemv_tiles_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    if (M <= 0 || N <= 0 || K <= 0 || K % PHASE_K) return COUNTER_BYTES;
    // the largest split any device-dependent plan can choose is bounded by the slot count
    const int64_t max_splits = K / PHASE_K;
    const int64_t tile_groups = ((N + 15) / 16 + WAVES - 1) / WAVES;
    int64_t splits = 1;
    for (int64_t s = 1; s <= max_splits; ++s)
        if (max_splits % s == 0 && tile_groups * s <= 2 * 1024) splits = s;  // covers devices up to 1024 CUs
    return (size_t)COUNTER_BYTES + (splits > 1 ? (size_t)splits * (size_t)M * (size_t)N * sizeof(float) : 0);
}

hipError_t gemv_tiles_setup() {
    hipError_t e;
    if ((e = gemv_allow_lds(gemv_kernel<false, false>, SMEM_BYTES)) != hipSuccess) return e;
    if ((e = gemv_allow_lds(gemv_kernel<true, false>, SMEM_BYTES)) != hipSuccess) return e;
    if ((e = gemv_allow_lds(gemv_kernel<false, true>, SMEM_BYTES)) != hipSuccess) return e;
    return gemv_allow_lds(gemv_kernel<true, true>, SMEM_BYTES);
}

hipError_t launch_gemv_tiles(const MatmulArgs& a, int cus, hipStream_t stream) {
    const int slots = 2 * cus;
    Plan p = make_plan(a.N, a.K, slots);
    if (p.tile_groups > COUNTER_BYTES / 4 && p.splits > 1) p.splits = 1, p.phases = a.K / PHASE_K, p.ntasks = p.tile_groups;
    const int grid = p.ntasks < slots ? p.ntasks : slots;
    const bool b64 = a.block_log2 == 6;
    const bool nested = a.nested.q != nullptr;
    auto kern = b64 ? (nested ? gemv_kernel<true, true> : gemv_kernel<true, false>)
                    : (nested ? gemv_kernel<false, true> : gemv_kernel<false, false>);
    hipLaunchKernelGGL(kern, dim3(grid), dim3(THREADS), SMEM_BYTES, stream, a, p);
    return hipGetLastError();
}

// ---- dispatch -------------------------------------------------------------------------------

size_t gemv_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    if (M == 1) return gemv_rows_workspace_bytes(M, N, K);
    return M <= 4 ? gemv_quad_workspace_bytes(M, N, K) : gemv_tiles_workspace_bytes(M, N, K);
}

hipError_t launch_gemv(const MatmulArgs& a, hipStream_t stream) {
    int cus = 0;
    const hipError_t e = device_setup(&cus);
    if (e != hipSuccess) return e;
    if (a.M == 1) return launch_gemv_rows(a, cus, stream);
    return a.M <= 4 ? launch_gemv_quad(a, cus, stream) : launch_gemv_tiles(a, cus, stream);
}

}  // namespace nf4
