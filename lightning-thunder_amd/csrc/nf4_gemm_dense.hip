// Dense bf16 GEMM for gfx950: out[M, N] = x[M, K] . w[N, K]^T (+ bias), fp32 accumulation, bf16 output.
//
// The second half of the dequantize_4bit + F.linear route of bitsandbytes.matmul_4bit (MatMul4Bit.forward, reached
// from thunder/transforms/quantization.py:39): it follows nf4hip_dequantize, whose bf16 weight it reads, and
// replaces the library GEMM behind torch.nn.functional.linear on that route.
//
// Tile 256 rows of x by 256 weight rows by 64 k per workgroup of FOUR waves, one per SIMD; wave (wm, wn) owns the
// 128 x 128 quarter: sixteen accumulators of v_mfma_f32_32x32x16_bf16 (256 registers, which the compiler keeps in
// the accumulation file) and eight fragment reads per sixteen MFMAs.  What the kernel is built around, all measured
// on this part with the MFMAs of one 16-k slice as the clock (16 x 32 cycles per wave):
//  * Both operands go from global memory straight into LDS (buffer_load_dwordx4 ... lds), two stages of 64 KB.
//    A load instruction of a wave fills 1 KB = eight rows of 128 bytes; 16-byte pieces are XOR-swizzled inside a row
//    and the rows of odd chunks swap places pairwise, so that the sixteen lanes a 128-bit fragment read serves
//    together hit sixteen different 16-byte bank groups.  Rows of 128 bytes, not 64: with a 32-k step every cache
//    line is requested twice, a k step apart, and the kernel loses a seventh of its rate.
//  * The CU's one address unit takes about 14.5 cycles per such load.  The sixteen loads a wave issues per k step
//    are therefore spread: eight (x) behind every other MFMA of the step's last slice -- the stage they refill is
//    free from the barrier that precedes that slice -- and eight (w) behind every other MFMA of the next step's
//    first slice.  All sixteen behind the last slice make that slice take 930 cycles instead of 512.
//  * One barrier per k step, before the last slice (its fragments are in registers by then).
//  * Fragments of the next slice are read behind the first eight MFMAs of a slice into a second register set.
//  * The tile leaves through LDS as bf16 and is stored in 16-byte pieces that cover whole 512-byte rows.
// Calls with at most 128 tiles cut every tile in two along k; the halves meet in the workspace without either
// workgroup waiting for the other (same protocol as the fused kernel's two-piece tiles).
#include "nf4_gemv.h"

#include <type_traits>

namespace nf4 {
namespace {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;
typedef float float2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) void* lds_void_ptr;

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int OPER_BYTES = 256 * BK * 2;     // one operand of one stage: 32 KB
constexpr int STAGE_BYTES = 2 * OPER_BYTES;  // 64 KB
constexpr int SMEM_BYTES = 2 * STAGE_BYTES;  // 128 KB
constexpr int THREADS = 256;
[[maybe_unused]] constexpr int GROUP_M = 8;  // x-row tiles that run next to each other (tile numbering in the kernel)
constexpr int SLOT_FLOATS = BM * BN;

struct DenseSchedule {
    int m_tiles, n_tiles, tiles;
    int pieces;          // 1 or 2 pieces per tile along k
    uint32_t* counters;  // two per tile, zero between calls
    float* partials;     // two slots of 256 x 256 floats per tile
};

__device__ __forceinline__ bf16x8 lds_frag(uint32_t addr) {
    return *reinterpret_cast<const __attribute__((address_space(3))) bf16x8*>(addr);
}

// Tile number -> (x-row tile, weight-row tile), inside the kernel: workgroups are handed out to the XCDs in turn and
// every XCD gets a contiguous run of tile numbers; numbers run through GROUP_M x-row tiles first, then through the
// weight-row tiles, so the 32 tiles an XCD works on at a time share eight tiles of x and four of w in its L2.
template <bool TWO_PIECES>
__global__ __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(1, 1)))
void gemm_dense_kernel(DenseArgs a, DenseSchedule sch) {
    // The body exists in the device pass only: the host pass cannot instantiate the buffer-resource type.
#if defined(__HIP_DEVICE_COMPILE__)
    extern __shared__ __attribute__((aligned(4096))) uint8_t smem[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;

    // ---- what this workgroup works on ----
    constexpr int PIECES = TWO_PIECES ? 2 : 1;
    const int total = sch.tiles * PIECES;
    int u = blockIdx.x;
    {
        const int full = total & ~7;
        if (u < full) u = (u & 7) * (full >> 3) + (u >> 3);
    }
    const int piece = u / sch.tiles;
    const int tile = u - piece * sch.tiles;
    int mt, nt;
    {
        const int width = GROUP_M * sch.n_tiles;
        const int group = tile / width;
        const int first = group * GROUP_M;
        const int size = min(sch.m_tiles - first, GROUP_M);
        const int in = tile - group * width;
        mt = first + in % size;
        nt = in / size;
    }
    const int m0 = mt * BM, n0 = nt * BN;
    const int ksteps_all = a.K / BK;
    const int kfirst = piece * ksteps_all / PIECES;
    const int ksteps = (piece + 1) * ksteps_all / PIECES - kfirst;

    // Buffer resources that start at the tile's first row: offsets inside a tile fit 32 bits whatever the tensor's size.
    const uint32_t row_bytes = (uint32_t)a.K * 2u;
    auto bytes_from = [&](int64_t rows_left) { return (int)(uint32_t)min((int64_t)0xfffff000, rows_left * (int64_t)row_bytes); };
    const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(a.x + (int64_t)m0 * a.K), 0,
                                                                        bytes_from(a.M - m0), 0x00020000);
    const __amdgpu_buffer_rsrc_t wr = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(a.w + (int64_t)n0 * a.K), 0,
                                                                        bytes_from(a.N - n0), 0x00020000);
    // Wave v loads chunks 8 v .. 8 v + 7 of either operand (eight rows of 128 bytes each).  Row rr of chunk c sits in
    // 128-byte slot rr ^ (c & 1), its 16-byte piece p at position p ^ rr; lane l of a load writes slot l / 8,
    // position l % 8, so it fetches row (l / 8) ^ (c & 1), piece (l % 8) ^ row.  Rows beyond the tensor repeat its
    // last row (their results are never stored).
    uint32_t xo[8], wo[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int c = 8 * wave + j;
        const int rr = (lane >> 3) ^ (c & 1);
        const uint32_t in_row = (uint32_t)(((lane & 7) ^ rr) << 4) + (uint32_t)kfirst * (BK * 2);
        xo[j] = (uint32_t)min(8 * c + rr, a.M - 1 - m0) * row_bytes + in_row;
        wo[j] = (uint32_t)min(8 * c + rr, a.N - 1 - n0) * row_bytes + in_row;
    }
    auto load_one = [&](int kt, int stage, int j) {  // j = 0..7: chunks of x, 8..15: chunks of w
        const uint32_t st = stage * STAGE_BYTES + 8 * wave * 1024;
        if (j < 8)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(xr, (lds_void_ptr)(uintptr_t)(st + j * 1024), 16, xo[j], kt * (BK * 2), 0, 0);
        else
            __builtin_amdgcn_raw_ptr_buffer_load_lds(wr, (lds_void_ptr)(uintptr_t)(st + OPER_BYTES + (j - 8) * 1024), 16,
                                                     wo[j - 8], kt * (BK * 2), 0, 0);
    };

    // Fragment of 32-row block b, slice s: row 32 b + l % 32 lies in chunk 4 b + (l % 32) / 8 (parity that of (l % 32) / 8)
    // at slot (row % 8) ^ parity; its piece 4 (l / 32) + s sits at position piece ^ (row % 8).  (The k order inside
    // a step is the same for both operands, which is all the contraction needs.)
    const int fr = lane & 31, fh = lane >> 5;
    const uint32_t frow = (uint32_t)((fr >> 3) * 1024 + (((fr & 7) ^ ((fr >> 3) & 1)) << 7));
    uint32_t a_off[4], b_off[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) {
        const uint32_t pos = (uint32_t)((((fh << 2) | s) ^ (fr & 7)) << 4);
        a_off[s] = (uint32_t)(16 * wm * 1024) + frow + pos;
        b_off[s] = (uint32_t)(OPER_BYTES + 16 * wn * 1024) + frow + pos;
    }

    f32x16 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int g = 0; g < 4; ++g)
#pragma unroll
            for (int q = 0; q < 16; ++q) acc[i][g][q] = 0.0f;

#pragma unroll
    for (int j = 0; j < 16; ++j) load_one(0, 0, j);
#pragma unroll
    for (int j = 0; j < 8; ++j) load_one(1, 1, j);  // x of step 1 (every piece has two steps or more); w follows in step 0
    asm volatile("s_waitcnt vmcnt(8)\n\ts_barrier" ::: "memory");

    bf16x8 fa[2][4], fb[2][4];
#pragma unroll
    for (int i = 0; i < 4; ++i) fa[0][i] = lds_frag(a_off[0] + i * 4096);
#pragma unroll
    for (int g = 0; g < 4; ++g) fb[0][g] = lds_frag(b_off[0] + g * 4096);

    // One k step = four slices; slice s uses fragment set s % 2.  Before slice 3 the one barrier of the step: every
    // wave has received its fragment reads of this stage and its loads of the next step have landed (nothing else
    // of this wave is in flight then).  Behind the MFMAs of slice 3 the stage is refilled with x of step kt + 2 and
    // the first fragments of step kt + 1 are read; w of step kt + 2 follows behind slice 0 of step kt + 1.
    auto step = [&](int kt, auto stage, auto full) {
        constexpr int ST = decltype(stage)::value;
        constexpr bool FULL = decltype(full)::value;  // steps up to kt + 2 exist
        constexpr uint32_t st = ST * STAGE_BYTES;
        constexpr uint32_t st_next = (ST ^ 1) * STAGE_BYTES;
        const bool more = FULL || kt + 1 < ksteps;
        const bool more2 = FULL || kt + 2 < ksteps;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const int cur = s & 1, nxt = cur ^ 1;
            if (s == 3) {
                __builtin_amdgcn_sched_barrier(0);
                asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
                __builtin_amdgcn_sched_barrier(0);
            }
            const uint32_t nb = s < 3 ? st + b_off[(s + 1) & 3] : st_next + b_off[0];
            const uint32_t na = s < 3 ? st + a_off[(s + 1) & 3] : st_next + a_off[0];
            const bool pre = s < 3 || more;
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                const int i = j >> 2, g = j & 3;
                acc[i][g] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[cur][i], fb[cur][g], acc[i][g], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
                if (pre) {
                    if (j < 4) fb[nxt][j] = lds_frag(nb + j * 4096);
                    else if (j < 8) fa[nxt][j - 4] = lds_frag(na + (j - 4) * 4096);
                }
                if ((j & 1) == 0) {
                    if (s == 3 && more2) load_one(kt + 2, ST, j >> 1);
                    if (s == 0 && more) load_one(kt + 1, ST ^ 1, 8 + (j >> 1));
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };
    using S0 = std::integral_constant<int, 0>;
    using S1 = std::integral_constant<int, 1>;
    int kt = 0;
    for (; kt + 4 <= ksteps; kt += 2) {
        step(kt, S0{}, std::true_type{});
        step(kt + 1, S1{}, std::true_type{});
    }
    for (; kt < ksteps; kt += 2) {
        step(kt, S0{}, std::false_type{});
        if (kt + 1 < ksteps) step(kt + 1, S1{}, std::false_type{});
    }
    __syncthreads();  // every wave has received its last fragment reads: LDS is free

    // ---- one of two pieces of a tile: meet the other one in the workspace ----
    // Two counters per tile, zero between calls: P counts published partials, T hands out tickets.  The holder of the
    // second ticket looks at P: if the other piece's partial is published already it adds it to its registers and
    // writes the tile.  Otherwise it stores its own partial like the first one did, and whoever raises P to two adds
    // the other partial to its registers and writes the tile.  Either way the tile is a + b with the two halves'
    // fp32 sums as a and b, so the result does not depend on who arrives when; nobody waits for anybody.
    bool write_tile = true;
    if (TWO_PIECES) {
        uint32_t* cP = sch.counters + 2 * tile;
        uint32_t* cT = cP + 1;
        float* mine = sch.partials + (int64_t)(2 * tile + piece) * SLOT_FLOATS;
        const float* other = sch.partials + (int64_t)(2 * tile + (piece ^ 1)) * SLOT_FLOATS;
        volatile uint32_t* flag = reinterpret_cast<volatile uint32_t*>(smem);
        if (tid == 0) {
            const uint32_t ticket = __hip_atomic_fetch_add(cT, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            uint32_t ok = 0;
            if (ticket == 1) ok = __hip_atomic_load(cP, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 1u;
            *flag = ok;
        }
        __syncthreads();
        bool add_other = *flag != 0;
        acquire_partials();
        __syncthreads();
        if (!add_other) {
#pragma unroll
            for (int f = 0; f < 16; ++f)
#pragma unroll
                for (int q = 0; q < 16; ++q)
                    __hip_atomic_store(mine + (f * 16 + q) * THREADS + tid, acc[f >> 2][f & 3][q], __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
            publish_partials();
            __syncthreads();
            if (tid == 0) *flag = __hip_atomic_fetch_add(cP, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1u;
            __syncthreads();
            add_other = *flag == 2u;
            acquire_partials();
            __syncthreads();
        }
        if (add_other) {
#pragma unroll
            for (int f = 0; f < 16; ++f) {
                float v[16];
#pragma unroll
                for (int q = 0; q < 16; ++q)
                    v[q] = __hip_atomic_load(other + (f * 16 + q) * THREADS + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
                for (int q = 0; q < 16; ++q) acc[f >> 2][f & 3][q] += v[q];
            }
            if (tid == 0) {
                __hip_atomic_store(cP, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(cT, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        write_tile = add_other;
    }

    // ---- the tile: bf16 into LDS, then 16-byte stores that cover whole rows ----
    // acc[i][g][q] = out[m][n], n = 128 wn + 32 g + l % 32, m = 128 wm + 32 i + 8 (q / 4) + 4 (l / 32) + q % 4.  Rows q and
    // q + 1 of a lane are rounded into one dword, lanes l and l ^ 1 exchange dwords (DPP) and v_perm_b32 leaves the
    // even lane with columns (n, n + 1) of row q and the odd lane with the same columns of row q + 1: one ds_write_b32
    // per two outputs.  Row r starts at 512 r; its dword c sits at c ^ 16 f(r), f(r) = r % 2 + 2 (r / 4 % 2), which keeps
    // 16-byte pieces whole and sends the four rows one write instruction touches to four different bank groups.
    if (write_tile) {
        const uint32_t sel = (lane & 1) ? 0x03020706u : 0x05040100u;
        const uint32_t wf = (uint32_t)((lane & 1) | (fh << 1));
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int nl = 128 * wn + 32 * g + fr;
            const int n = n0 + nl;
            const float b = (a.bias && n < a.N) ? bf16_bits_to_f32(a.bias[n]) : 0.0f;
            uint8_t* wbase = smem + (128 * wm + 4 * fh + (lane & 1)) * 512 + ((((uint32_t)nl >> 1) ^ (wf << 4)) << 2);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
#pragma unroll
                for (int q = 0; q < 16; q += 2) {
                    const float2_t f = {acc[i][g][q] + b, acc[i][g][q + 1] + b};
                    const uint32_t mine = __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2_t));
                    const uint32_t theirs = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)mine, 0xB1, 0xf, 0xf, true);
                    const uint32_t packed = __builtin_amdgcn_perm(theirs, mine, sel);
                    *reinterpret_cast<uint32_t*>(wbase + (32 * i + 8 * (q >> 2) + (q & 2)) * 512) = packed;
                }
            }
        }
        __syncthreads();
        const bool vec = (a.N & 7) == 0;
#pragma unroll 4
        for (int it = 0; it < BM / (THREADS / 32); ++it) {
            const int r = it * (THREADS / 32) + (tid >> 5);
            const int p = tid & 31;
            const int f2 = (r & 1) | (((r >> 2) & 1) << 1);
            const uint4 v = *reinterpret_cast<const uint4*>(smem + r * 512 + ((p ^ (f2 << 2)) << 4));
            const int m = m0 + r;
            const int n = n0 + p * 8;
            if (m < a.M) {
                uint16_t* dst = a.out + (int64_t)m * a.N + n;
                if (vec) {
                    if (n < a.N) store16<false>(dst, v.x, v.y, v.z, v.w);
                } else {
                    const uint32_t d[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if (n + e < a.N) dst[e] = (uint16_t)(d[e >> 1] >> (16 * (e & 1)));
                }
            }
        }
    }
#endif  // __HIP_DEVICE_COMPILE__
}

constexpr int MAX_DEVICES = 64;

DenseSchedule dense_schedule(int64_t M, int64_t N, int64_t K, size_t workspace_bytes) {
    DenseSchedule s{};
    s.m_tiles = (int)((M + BM - 1) / BM);
    s.n_tiles = (int)((N + BN - 1) / BN);
    s.tiles = s.m_tiles * s.n_tiles;
    // Two pieces per tile where that puts idle CUs to work and leaves every piece sixteen k steps or more.
    s.pieces = (s.tiles <= 128 && K / BK >= 32) ? 2 : 1;
    if (s.pieces == 2 && workspace_bytes < gemm_dense_workspace_bytes(M, N, K)) s.pieces = 1;
    return s;
}

}  // namespace

bool gemm_dense_possible(int64_t M, int64_t N, int64_t K) {
    if (M < 1 || N < 1 || K < 2 * BK || K % BK != 0) return false;
    if (K > (1 << 20)) return false;  // 256 rows of 2 K bytes stay far below the 32-bit offsets of a tile's buffer resource
    const int64_t tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
    return tiles * 2 < (int64_t)1 << 30;
}

size_t gemm_dense_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    const int64_t tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
    if (!(tiles <= 128 && K / BK >= 32)) return 0;
    return (size_t)GEMV_COUNTER_BYTES + (size_t)tiles * 2 * SLOT_FLOATS * sizeof(float);
}

void gemm_dense_plan(int64_t M, int64_t N, int64_t K, int plan[4]) {
    const DenseSchedule s = dense_schedule(M, N, K, ~(size_t)0);
    plan[0] = BM;
    plan[1] = s.tiles;
    plan[2] = s.pieces;
    plan[3] = s.tiles * s.pieces;
}

hipError_t launch_gemm_dense(const DenseArgs& a, hipStream_t stream) {
    static bool ready[MAX_DEVICES] = {};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= MAX_DEVICES) return hipErrorInvalidDevice;
    if (!ready[dev]) {
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_dense_kernel<false>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                SMEM_BYTES);
        if (e != hipSuccess) return e;
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_dense_kernel<true>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                SMEM_BYTES);
        if (e != hipSuccess) return e;
        ready[dev] = true;
    }
    DenseSchedule sch = dense_schedule(a.M, a.N, a.K, a.workspace ? a.workspace_bytes : 0);
    if (sch.tiles * 2 > (int)(GEMV_COUNTER_BYTES / sizeof(uint32_t))) sch.pieces = 1;
    sch.counters = static_cast<uint32_t*>(a.workspace);
    sch.partials = a.workspace ? reinterpret_cast<float*>(static_cast<uint8_t*>(a.workspace) + GEMV_COUNTER_BYTES) : nullptr;
    if (sch.pieces == 2)
        hipLaunchKernelGGL(gemm_dense_kernel<true>, dim3((unsigned)(sch.tiles * 2)), dim3(THREADS), SMEM_BYTES, stream, a, sch);
    else
        hipLaunchKernelGGL(gemm_dense_kernel<false>, dim3((unsigned)sch.tiles), dim3(THREADS), SMEM_BYTES, stream, a, sch);
    return hipGetLastError();
}

}  // namespace nf4
