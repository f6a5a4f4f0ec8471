// Decode-shape fused NF4 dequant-matmul for gfx950, 3 <= M <= 8 rows of x (any M from 1 works).
//
// Replaces bitsandbytes' gemv_4bit (kgemm_4bit_inference_naive), the kernel that
// bitsandbytes.matmul_4bit picks for a single-row x; call site
// thunder/transforms/quantization.py:39.
//
// HBM-bound: 0.5 byte of codes + 4/blocksize bytes of absmax per weight, each read exactly once.
//
//  * Lane mapping.  A wave works on FOUR weight rows at a time.  Lane l = 4*s + r holds row r of the
//    group and k segment s (32 consecutive k): one 16-byte load per lane, and the 16 lanes of a row
//    read 256 contiguous bytes.  CPW such loads (512 k each) cover the wave's k range; the 8 waves
//    of a workgroup are (waves along K) x (row groups), so a workgroup streams whole rows.
//  * v_mfma_f32_4x4x4_16b_bf16 computes one 4x4x4 product per group of 4 lanes: A row i comes from
//    lane i of the quad (4 weights of weight-row i), B column j from lane j (4 values of x row j at
//    the same k).  C[i][j] = weight-row i . x-row j, so ALL 16 results of the quad are wanted and
//    M = 2, 3, 4 cost exactly what M = 1 costs.  Lane j keeps x row j in registers (rows >= M: 0);
//    a workgroup keeps one K split for all its tasks, so x is read once per kernel, in contiguous
//    1 KB requests, and put into that layout by a 4x4 transpose inside every quad.
//    M = 5..8 (XS = 2): lane j also keeps x row j + 4, and every dequantised weight fragment feeds a
//    second MFMA (a wave then takes one or two loads per row group like the others: pick_cpw).
//  * Code -> bf16: 256-entry LDS table indexed by a whole packed byte, both code values as one
//    dword, replicated per lane with a 256-byte stride: address (byte << 8) | lane*4 is one
//    v_perm_b32 and bank-conflict free.
//  * Scale: a lane's 32 weights share one absmax; the 8-MFMA partial of row i is scaled by the
//    absmax lane i of the quad loaded (a DPP quad broadcast folded into the FMA).  EXACT variant
//    (K > 8192): fp32 table, every weight rounded as bf16(lut * absmax) before the MFMA, which is
//    the reference's dequantisation bit for bit.
//  * Reduction over the 16 k segments: a transposing butterfly leaves the 16 (row, m) totals of the
//    group in lanes 0..15; per-(row, wave) sums are parked in LDS and added in a fixed order.
//  * K larger than one workgroup covers is split over workgroups; partial sums cross workgroups
//    through agent-scope relaxed atomics and a counter (no L2-wide fences), added in a fixed order
//    by the last workgroup to arrive.
#include <type_traits>

#include "decode_math.h"
#include "nf4_gemv.h"

namespace nf4 {
namespace {

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

constexpr int PART_BYTES = 16 * 1024;  // per-(row, wave, m) partial sums of one band
constexpr int SMEM_BYTES = GEMV_TABLE_BYTES + PART_BYTES;
constexpr int LOAD_K = 512;            // k covered by one wave-wide 16-byte load (16 segments of 32)
constexpr int FLAG_OFFSET = GEMV_TABLE_BYTES + PART_BYTES - 16;
constexpr int MAP_BYTES = 1024;         // nested absmax only: the 256-entry map, taken from the end of the partial sums
constexpr int MAP_OFFSET = FLAG_OFFSET - MAP_BYTES;
// kernels with an epilogue (fp32 absmax only): sums of squares per (row of x, wave), below the flag
constexpr int SUMSQ_BYTES = 8 * GEMV_WAVES * 4;
constexpr int SUMSQ_OFFSET = FLAG_OFFSET - 16 - SUMSQ_BYTES;

struct QuadPlan {
    int waves_k;          // waves of a workgroup along K
    int row_groups;       // 4-row groups processed concurrently by a workgroup = 8 / waves_k
    int splits;           // K splits across workgroups
    int groups_per_band;  // 4-row groups of one task
    int nbands;
    int ntasks;           // nbands * splits
    int aligned;          // K % blocksize == 0
};

#define NF4_DPP(v, ctrl, bank, keep_old) \
    __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, keep_old), __builtin_bit_cast(int, v), ctrl, 0xf, bank, false))
// every lane of the quad reads a valid lane: no "old" value is needed, which lets the compiler fold
// the DPP into the instruction that uses the result
#define NF4_QUAD_BCAST(v, ctrl) \
    __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v), __builtin_bit_cast(int, v), ctrl, 0xf, 0xf, true))

// value of `v` in lane (lane ^ 4); DPP shifts by 4 inside a row of 16, direction chosen per bank of 4
__device__ __forceinline__ float lane_xor4(float v) {
    float o = NF4_DPP(v, 0x104 /*row_shl:4*/, 0x5, v);  // banks 1, 3 are overwritten below
    return NF4_DPP(v, 0x114 /*row_shr:4*/, 0xa, o);
}

// t[0..3]: this lane's partial sums for weight rows 0..3 of the group (and x row lane & 3).
// Returns in every lane the total over the 16 k segments of weight row 2*bit3 + bit2 (bits of lane).
__device__ __forceinline__ float reduce_rows(const float t[4], int lane) {
    const bool b2 = lane & 4, b3 = lane & 8;
    float w[2];
#pragma unroll
    for (int p = 0; p < 2; ++p) {  // rows (0,1) and (2,3): lane bit 2 picks the row the lane keeps
        const float keep = b2 ? t[2 * p + 1] : t[2 * p];
        const float send = b2 ? t[2 * p] : t[2 * p + 1];
        w[p] = keep + lane_xor4(send);
    }
    const float keep = b3 ? w[1] : w[0];
    const float send = b3 ? w[0] : w[1];
    float y = keep + NF4_DPP(send, 0x128 /*row_ror:8*/, 0xf, send);
    y += __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((lane ^ 16) << 2, __builtin_bit_cast(int, y)));
    y += __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((lane ^ 32) << 2, __builtin_bit_cast(int, y)));
    return y;
}

// EPI (Epilogue flags; fp32 absmax): what the thread that finishes an output does with it; with K split over
// workgroups that thread belongs to the last workgroup to arrive.  For the sums of squares of EPI_RESID_NORM a thread
// keeps to one row of x (m = tid % MP, MP the power of two that holds M), lanes of equal m are added by a butterfly
// and the waves in order.
template <int CPW, int U, int XS, bool NESTED, int MODE, int EPI = EPI_NONE>
__global__ __launch_bounds__(GEMV_THREADS, 4) void gemv_quad_kernel(NF4_HOT_PARAMS, int hot_plan, int hot_groups_per_band, int hot_ntasks,
                                                                     MatmulArgs a_rest, QuadPlan p_rest) {
    // (arguments in SGPRs at wave start; the structs supply what is wanted later)
    MatmulArgs a = with_hot_args<NESTED>(a_rest, NF4_HOT_NAMES);
    QuadPlan p = p_rest;
    p.waves_k = hot_plan & 0xf; p.row_groups = (hot_plan >> 4) & 0xf; p.aligned = (hot_plan >> 8) & 1; p.splits = hot_plan >> 9;
    p.groups_per_band = hot_groups_per_band; p.ntasks = hot_ntasks;
    static_assert(EPI == EPI_NONE || !NESTED, "epilogues come with fp32 absmax only");
    constexpr bool EXACT = MODE == ARITH_EXACT, F16 = MODE == ARITH_F16;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t lane4 = (uint32_t)lane * 4u;
    const uint32_t lane8 = (uint32_t)(lane & 31) * 8u;
    const int ri = lane & 3;        // weight row inside the group of 4, and the x row this lane feeds
    const uint32_t kseg = 32u * (uint32_t)(lane >> 2);

    // the code-book entry this lane contributes to the LDS table: requested first, used last
    const float lut_mine = a.lut16[lane & 15];

    float* part = reinterpret_cast<float*>(smem + GEMV_TABLE_BYTES);
    int* flag = reinterpret_cast<int*>(smem + FLAG_OFFSET);
    unsigned* counters = reinterpret_cast<unsigned*>(a.workspace);
    float* partial = reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(a.workspace) + GEMV_COUNTER_BYTES);

    // Nine to sixteen rows of x on a small weight: two workgroups per task, blockIdx.y picks rows 0..7 or 8..15 of x
    // (the launcher only does this when K is not split across workgroups, so the halves share nothing)
    if (gridDim.y > 1) {
        const int mb = 8 * (int)blockIdx.y;
        a.x += (int64_t)mb * a.K;
        a.out += (int64_t)mb * ((EPI & EPI_SILU_PAIRS) ? a.N / 2 : a.N);
        a.M = min(a.M - mb, 8);
        if (EPI & EPI_ROWSCALE) a.epi.in_sumsq += (int64_t)mb * a.epi.in_parts;
        if (EPI & EPI_RESID_NORM) {
            a.epi.resid_in += (int64_t)mb * a.N;
            a.epi.resid_out += (int64_t)mb * a.N;
            a.epi.xnext_out += (int64_t)mb * a.N;
            a.epi.out_sumsq += (int64_t)mb * p.nbands;
        }
    }
    float* sumsq_s = reinterpret_cast<float*>(smem + SUMSQ_OFFSET);
    // which K chunk a wave takes rotates with the workgroup: every workgroup reads all of x, and workgroups that start
    // together would otherwise ask the same L2 channel for the same piece at the same time ([4096, 4096], 8 rows: 8.2 -> 7.8 us)
    const int cw = (wave + (int)blockIdx.x) % p.waves_k;
    const int rg = wave / p.waves_k;
    const int64_t K = a.K;
    const int M = a.M;
    const int step = p.row_groups;

    // The grid is a multiple of the number of K splits, so every task of this workgroup has the same
    // split and x is read once, with the first task.
    const int ks = (int)blockIdx.x % p.splits;
    const int64_t kw0 = (int64_t)(ks * p.waves_k + cw) * (CPW * LOAD_K);
    uint32_t xr[XS][CPW][16];  // x rows `ri`, `ri + 4`, ...: this lane's 32 k of every load
    float unscale[XS];         // fp16 arithmetic: what undoes the scaling of the lane's x values
#pragma unroll
    for (int h = 0; h < XS; ++h) unscale[h] = 1.0f;

    auto run_task = [&](const int task, auto first_tag) {
        constexpr bool FIRST = decltype(first_tag)::value;
        const int band = task / p.splits;
        const int g_begin = band * p.groups_per_band;
        const int g_end = min((a.N + 3) / 4, g_begin + p.groups_per_band);
        const bool wave_on = rg < p.row_groups && kw0 < K && g_begin + rg < g_end;
        const int cnt = wave_on ? (g_end - g_begin - rg + step - 1) / step : 0;  // groups of this wave
        bool lane_on[CPW];
#pragma unroll
        for (int c = 0; c < CPW; ++c) lane_on[c] = wave_on && kw0 + c * LOAD_K + kseg < K;

        // sq: absmax of the lane's block; nested: its 8-bit code (resolved through the LDS copy of
        // the map when the slot is consumed, so that issuing a load never waits for another) and
        // s2 the second-level absmax
        uint4 wq[U][CPW];
        float sq[U][CPW];
        float s2[NESTED ? U : 1][CPW];
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int c = 0; c < CPW; ++c) {
                wq[u][c] = make_uint4(0, 0, 0, 0);
                sq[u][c] = 0.0f;
                if (NESTED) s2[u][c] = 0.0f;
            }
        // group i of this wave is g_begin + rg + i * step; its rows are 4 * group + ri
        auto issue = [&](int u, int i) {
            const int row = min(4 * (g_begin + rg + i * step) + ri, a.N - 1);
            const int64_t e0 = (int64_t)row * K + kw0 + kseg;
#pragma unroll
            for (int c = 0; c < CPW; ++c)
                if (lane_on[c]) {
                    const int64_t e = e0 + c * LOAD_K;
                    wq[u][c] = load16_stream(a.packed + (e >> 1));
                    const int64_t blk = e >> a.block_log2;
                    if (NESTED) {
                        sq[u][c] = __uint_as_float((uint32_t)a.nested.q[blk]);
                        s2[u][c] = a.nested.absmax2[blk >> a.nested.nested_log2];
                    } else {
                        sq[u][c] = load_f32_stream(a.absmax + blk);
                    }
                }
        };
        // First task: x.  Row by row, lane l takes elements [8 l, 8 l + 8) of the load's 512: one
        // contiguous 1 KB per request.  (Every lane reading its own 64 bytes would touch 64 cache lines
        // per request instead of 16, and with 16 waves per CU the address unit would then pace the
        // whole kernel.)  These requests go out ahead of the weights: they are served by the L2 while
        // the first weights are on their way from HBM.
        uint4 xraw[XS][CPW][4];
        float lut = lut_mine;
        if constexpr (FIRST) {
            // The wait for the code-book entry belongs here, where nothing else is in flight: the
            // loads below sit under branches, so a wait placed after them would be for all of them,
            // and the table is to be built while they are in flight.
            asm volatile("" : "+v"(lut));
#pragma unroll
            for (int c = 0; c < CPW; ++c) {
                // a lane beyond K (or an idle wave) reads the end of the row; the value is dropped below
                const int64_t kc = kw0 + c * LOAD_K + 8 * lane;
                const uint16_t* xb = a.x + min(kc, K - 8);
#pragma unroll
                for (int h = 0; h < XS; ++h)
#pragma unroll
                    for (int r = 0; r < 4; ++r)  // rows >= M: every lane reads x[0] (one cache line)
                        xraw[h][c][r] = load16(4 * h + r < M ? xb + (int64_t)(4 * h + r) * K : a.x);
            }
        }
        // get the weight stream going before anything else happens
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (u < cnt) issue(u, u);

        // EPI_ROWSCALE: the producer's partial sums of squares, requested behind the first weights (they are wanted
        // last: in front of x they would hold x back); wave w adds up row w of x -- in_parts <= 512 values, eight per
        // lane -- once the task's rows are done
        float ssp[8];
        if constexpr (FIRST && (EPI & EPI_ROWSCALE) != 0) {
#pragma unroll
            for (int j = 0; j < 8; ++j)
                ssp[j] = (wave < M && lane + 64 * j < a.epi.in_parts) ? a.epi.in_sumsq[wave * a.epi.in_parts + lane + 64 * j] : 0.0f;
        }
        // first task: the table is built while the loads are in flight
        if constexpr (FIRST) {
            if (EXACT)
                build_pair_table_f32(smem, lut, lane, wave);
            else
                build_pair_table<F16>(smem, lut, lane, wave);
            if (NESTED && tid < 256) reinterpret_cast<float*>(smem + MAP_OFFSET)[tid] = a.nested.map256[tid];
        }
        __syncthreads();  // table built (first task) / previous task's epilogue done with `part`
        if constexpr (FIRST) {
            // The four lanes of a quad hold the quad's 32 k of rows 4h..4h+3 in four pieces each; a 4x4
            // transpose inside the quad hands lane `ri` the four pieces of row 4h + `ri`.
#pragma unroll
            for (int h = 0; h < XS; ++h)
#pragma unroll
                for (int c = 0; c < CPW; ++c) {
                    const bool in = rg < p.row_groups && kw0 + c * LOAD_K + 8 * lane < K;
                    uint32_t v[4][4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const bool keep = in && 4 * h + r < M;
                        v[r][0] = keep ? xraw[h][c][r].x : 0u; v[r][1] = keep ? xraw[h][c][r].y : 0u;
                        v[r][2] = keep ? xraw[h][c][r].z : 0u; v[r][3] = keep ? xraw[h][c][r].w : 0u;
                    }
#pragma unroll
                    for (int d = 0; d < 4; ++d) transpose_quad(v[0][d], v[1][d], v[2][d], v[3][d], lane & 1, lane & 2);
#pragma unroll
                    for (int j = 0; j < 4; ++j)
#pragma unroll
                        for (int d = 0; d < 4; ++d) xr[h][c][4 * j + d] = v[j][d];
                }
            if (F16) {  // the lane's x values become fp16, scaled into range per row of x
#pragma unroll
                for (int h = 0; h < XS; ++h) {
                    u16x2_t mx = {0, 0};
#pragma unroll
                    for (int c = 0; c < CPW; ++c)
#pragma unroll
                        for (int q = 0; q < 16; ++q) mx = absmax_of_bf16_pair(xr[h][c][q], mx);
                    const F16Scale fs = f16_scale_for(absmax_bits(mx));
#pragma unroll
                    for (int c = 0; c < CPW; ++c)
#pragma unroll
                        for (int q = 0; q < 16; ++q) xr[h][c][q] = bf16_pair_to_f16(xr[h][c][q], fs.to_f16);
                    unscale[h] = fs.from_f16;
                }
            }
        }

        for (int i0 = 0; i0 < cnt; i0 += U) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                float tot[XS][4];
#pragma unroll
                for (int h = 0; h < XS; ++h)
#pragma unroll
                    for (int i = 0; i < 4; ++i) tot[h][i] = 0.0f;
                // take the slot's contents, then refill it at once: the load is in flight while the
                // table lookups and MFMAs below run
                uint32_t dd[CPW][4];
                float ss[CPW];
#pragma unroll
                for (int c = 0; c < CPW; ++c) {
                    dd[c][0] = wq[u][c].x; dd[c][1] = wq[u][c].y; dd[c][2] = wq[u][c].z; dd[c][3] = wq[u][c].w;
                    ss[c] = sq[u][c];
                    if (NESTED)
                        ss[c] = __fadd_rn(__fmul_rn(reinterpret_cast<const float*>(smem + MAP_OFFSET)[__float_as_uint(ss[c])], s2[u][c]),
                                          a.nested.offset);
                }
                const int i = i0 + u;
                if (i + U < cnt) issue(u, i + U);  // else the slot keeps its stale contents: its results are dropped
#pragma unroll
                for (int c = 0; c < CPW; ++c) {
                    const uint32_t* d = dd[c];
                    const float s = ss[c];
                    uint32_t pr[16];
#pragma unroll
                    for (int q = 0; q < 4; ++q)
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            const uint32_t sel = 0x0c0c0400u | ((uint32_t)j << 8);
                            if (EXACT) {
                                // bf16(lut[c] * absmax) per weight, the value nf4hip_dequantize produces
                                const float2 v = lds_table_read2(__builtin_amdgcn_perm(d[q], lane8, sel));
                                f32x2 f = {__fmul_rn(v.x, s), __fmul_rn(v.y, s)};
                                pr[4 * q + j] = __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
                            } else {
                                pr[4 * q + j] = lds_table_read(__builtin_amdgcn_perm(d[q], lane4, sel));
                            }
                        }
#pragma unroll
                    for (int h = 0; h < XS; ++h) {  // the dequantised weights serve every set of four x rows
                        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                        for (int t = 0; t < 8; ++t) {
                            const uint2 wa = make_uint2(pr[2 * t], pr[2 * t + 1]);
                            const uint2 xb = make_uint2(xr[h][c][2 * t], xr[h][c][2 * t + 1]);
                            if (!F16)
                                acc = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(s16x4, wa),
                                                                             __builtin_bit_cast(s16x4, xb), acc, 0, 0, 0);
                            else
                                acc = __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(f16x4, wa),
                                                                         __builtin_bit_cast(f16x4, xb), acc, 0, 0, 0);
                        }
                        if (EXACT) {
#pragma unroll
                            for (int i = 0; i < 4; ++i) tot[h][i] += acc[i];
                        } else {
                            // acc[i] belongs to weight row i, whose absmax lane i of this quad holds
                            tot[h][0] = fmaf(NF4_QUAD_BCAST(s, 0x00), acc[0], tot[h][0]);
                            tot[h][1] = fmaf(NF4_QUAD_BCAST(s, 0x55), acc[1], tot[h][1]);
                            tot[h][2] = fmaf(NF4_QUAD_BCAST(s, 0xAA), acc[2], tot[h][2]);
                            tot[h][3] = fmaf(NF4_QUAD_BCAST(s, 0xFF), acc[3], tot[h][3]);
                        }
                    }
                }
                const int grow = 2 * ((lane >> 3) & 1) + ((lane >> 2) & 1);
#pragma unroll
                for (int h = 0; h < XS; ++h) {
                    if (F16) {
#pragma unroll
                        for (int i = 0; i < 4; ++i) tot[h][i] *= unscale[h];
                    }
                    // lanes 0..15: row 2*b3+b2 of the group, x row 4h + ri
                    const float total = reduce_rows(tot[h], lane);
                    if (lane < 16 && 4 * h + ri < M && i < cnt)
                        part[(((rg + i * step) * 4 + grow) * p.waves_k + cw) * M + 4 * h + ri] = total;
                }
            }
        }
        if constexpr (FIRST && (EPI & EPI_ROWSCALE) != 0) {
            float ss = ((ssp[0] + ssp[1]) + (ssp[2] + ssp[3])) + ((ssp[4] + ssp[5]) + (ssp[6] + ssp[7]));
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
            if (lane == 0) sumsq_s[wave] = ss;  // rows of x beyond M: 0
        }
        __syncthreads();

        // ---- band epilogue: add the waves of every row in a fixed order ----
        const int r_begin = 4 * g_begin;
        const int nrows = min(a.N, 4 * g_end) - r_begin;
        // the last split may own fewer waves along K than the others
        const int wave_k = CPW * LOAD_K;
        const int nwk = min(p.waves_k, (int)((K + wave_k - 1) / wave_k) - ks * p.waves_k);
        // What happens to the finished sums; `sum_of(r, m)`: the sum of output (row r of the band, row m of x) over K.
        auto finish = [&](auto sum_of) {
            auto finished = [&](int r, int m) {
                float sum = sum_of(r, m);
                // 1 / rms of row m of x, from the sum of squares the first task left in LDS
                if (EPI & EPI_ROWSCALE) sum *= rsqrtf(sumsq_s[m] / (float)K + a.epi.eps);
                if (a.bias) sum += bf16_bits_to_f32(a.bias[r_begin + r]);
                return sum;
            };
            if (EPI & EPI_SILU_PAIRS) {
                // rows 2j, 2j + 1 of the band: gate j, up j (a band is a whole number of four-row groups)
                for (int idx = tid; idx < (nrows / 2) * M; idx += GEMV_THREADS) {
                    const int j = idx / M, m = idx - j * M;
                    const float g = nf4x::round_bf16(finished(2 * j, m)), u = nf4x::round_bf16(finished(2 * j + 1, m));
                    a.out[(int64_t)m * (a.N / 2) + r_begin / 2 + j] = (uint16_t)nf4x::silu_mul_bf16(g, u);
                }
            } else if (EPI & EPI_RESID_NORM) {
                const int MP = M <= 1 ? 1 : M <= 2 ? 2 : M <= 4 ? 4 : 8;  // thread = (m = tid % MP, rows tid / MP + i * 512 / MP)
                const int m = tid % MP;
                float ss = 0.0f;
                if (m < M)
                    for (int r = tid / MP; r < nrows; r += GEMV_THREADS / MP) {
                        const int64_t at = (int64_t)m * a.N + r_begin + r;
                        const float d = nf4x::round_bf16(finished(r, m));
                        const float res = nf4x::resid_add(bf16_bits_to_f32(a.epi.resid_in[at]), d);
                        a.epi.resid_out[at] = (uint16_t)f32_to_bf16_bits(res);
                        a.epi.xnext_out[at] = (uint16_t)f32_to_bf16_bits(res * bf16_bits_to_f32(a.epi.norm_weight[r_begin + r]));
                        ss = fmaf(res, res, ss);
                    }
                for (int o = 32; o >= MP; o >>= 1) ss += __shfl_xor(ss, o, 64);  // lanes of equal m
                if (lane < MP) sumsq_s[lane * GEMV_WAVES + wave] = ss;
                __syncthreads();
                if (tid < M) {
                    float tot = 0.0f;
#pragma unroll
                    for (int w = 0; w < GEMV_WAVES; ++w) tot += sumsq_s[tid * GEMV_WAVES + w];
                    a.epi.out_sumsq[tid * p.nbands + band] = tot;
                }
            } else {
                for (int idx = tid; idx < nrows * M; idx += GEMV_THREADS) {
                    const int r = idx / M, m = idx - r * M;
                    a.out[(int64_t)m * a.N + r_begin + r] = (uint16_t)f32_to_bf16_bits(finished(r, m));
                }
            }
        };
        if (p.splits == 1) {
            finish([&](int r, int m) {
                float sum = 0.0f;
                for (int c = 0; c < nwk; ++c) sum += part[(r * p.waves_k + c) * M + m];
                return sum;
            });
        } else {
            for (int idx = tid; idx < nrows * M; idx += GEMV_THREADS) {
                const int r = idx / M, m = idx - r * M;
                float sum = 0.0f;
                for (int c = 0; c < nwk; ++c) sum += part[(r * p.waves_k + c) * M + m];
                __hip_atomic_store(&partial[((int64_t)ks * M + m) * a.N + r_begin + r], sum, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
            }
            publish_partials();
            __syncthreads();
            if (tid == 0) {
                const unsigned prev =
                    __hip_atomic_fetch_add(&counters[band], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                *flag = (prev == (unsigned)p.splits - 1u);
            }
            __syncthreads();
            acquire_partials();
            if (*flag != 0) {
                finish([&](int r, int m) {
                    float sum = 0.0f;
                    for (int k2 = 0; k2 < p.splits; ++k2)
                        sum += __hip_atomic_load(&partial[((int64_t)k2 * M + m) * a.N + r_begin + r], __ATOMIC_RELAXED,
                                                 __HIP_MEMORY_SCOPE_AGENT);
                    return sum;
                });
                if (tid == 0) __hip_atomic_store(&counters[band], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    };

    int task = blockIdx.x;
    if (task < p.ntasks) {
        run_task(task, std::true_type{});
        for (task += gridDim.x; task < p.ntasks; task += gridDim.x) run_task(task, std::false_type{});
    }
}

// k per wave = 512 * CPW: the fewest loads per wave with which the workgroup's 8 waves cover K, i.e. without splitting K
// over workgroups -- one up to K = 4096, two up to 8192 (four rows of x, CPW 1 vs 2: [6144, 4096] 7.2 vs 9.2 us,
// [4096, 4096] 6.2 vs 7.1; eight rows at [8192, 8192], 2 vs 1: 14.7 vs 16.4).  Longer K is split either way: two loads
// with up to four rows of x ([8192, 8192]-like shapes measured 13 vs 15 us), one with eight (x then takes 64 of the
// 128 registers at two loads; [4096, 14336]: 17.8 vs 19.0 us).
int pick_cpw(int64_t M, int64_t K) {
    if (K <= GEMV_WAVES * LOAD_K) return 1;
    if (K <= 2 * GEMV_WAVES * LOAD_K) return 2;
    return M > 4 ? 1 : 2;
}

int quad_splits(int64_t M, int64_t K) {
    const int64_t wave_k = (int64_t)pick_cpw(M, K) * LOAD_K;
    const int64_t nwk = (K + wave_k - 1) / wave_k;
    return (int)((nwk + GEMV_WAVES - 1) / GEMV_WAVES);
}

QuadPlan make_quad_plan(int M, int64_t N, int64_t K, int block_log2, int slots, bool nested, bool epi = false) {
    QuadPlan p;
    p.aligned = (K & (((int64_t)1 << block_log2) - 1)) == 0;
    const int64_t wave_k = (int64_t)pick_cpw(M, K) * LOAD_K;
    const int nwk = (int)((K + wave_k - 1) / wave_k);
    p.splits = quad_splits(M, K);
    p.waves_k = (nwk + p.splits - 1) / p.splits;
    p.row_groups = GEMV_WAVES / p.waves_k;
    const int groups = (int)((N + 3) / 4);
    const int part_bytes = PART_BYTES - 64 - (nested ? MAP_BYTES : 0) - (epi ? SUMSQ_BYTES + 16 : 0);
    const int cap = (part_bytes / (4 * p.waves_k * M * 4)) / p.row_groups * p.row_groups;
    int bands_target = slots / p.splits;
    if (bands_target < 1) bands_target = 1;
    // one task per resident workgroup if its partial sums fit in LDS, else 2, 3, ... balanced rounds
    int gpb = cap;
    for (int rounds = 1; rounds <= 64; ++rounds) {
        int g = (groups + rounds * bands_target - 1) / (rounds * bands_target);
        g = (g + p.row_groups - 1) / p.row_groups * p.row_groups;
        if (g <= cap) {
            gpb = g;
            break;
        }
    }
    if (gpb < p.row_groups) gpb = p.row_groups;
    p.groups_per_band = gpb;
    p.nbands = (groups + gpb - 1) / gpb;
    p.ntasks = p.nbands * p.splits;
    return p;
}

template <int CPW, int U, int XS, bool NESTED, int EPI>
hipError_t launch_u(const MatmulArgs& a, const QuadPlan& p, int grid, hipStream_t stream, int halves = 1) {
    const int mode = gemv_arith_mode(a.K, true);
    const dim3 g((unsigned)grid, (unsigned)halves);
    if (mode == ARITH_EXACT)
        hipLaunchKernelGGL((gemv_quad_kernel<CPW, U, XS, NESTED, ARITH_EXACT, EPI>), g, dim3(GEMV_THREADS), SMEM_BYTES, stream, NF4_HOT_VALUES(a),
                           p.waves_k | (p.row_groups << 4) | (p.aligned << 8) | (p.splits << 9), p.groups_per_band, p.ntasks, a, p);
    else if (mode == ARITH_F16)
        hipLaunchKernelGGL((gemv_quad_kernel<CPW, U, XS, NESTED, ARITH_F16, EPI>), g, dim3(GEMV_THREADS), SMEM_BYTES, stream, NF4_HOT_VALUES(a),
                           p.waves_k | (p.row_groups << 4) | (p.aligned << 8) | (p.splits << 9), p.groups_per_band, p.ntasks, a, p);
    else
        hipLaunchKernelGGL((gemv_quad_kernel<CPW, U, XS, NESTED, ARITH_BF16, EPI>), g, dim3(GEMV_THREADS), SMEM_BYTES, stream, NF4_HOT_VALUES(a),
                           p.waves_k | (p.row_groups << 4) | (p.aligned << 8) | (p.splits << 9), p.groups_per_band, p.ntasks, a, p);
    return hipGetLastError();
}

// U = row groups in flight per wave besides the one being worked on (a slot is refilled as soon as its codes are
// copied out).  ONE is the fastest: measured against two, four and eight, four rows of x: [4096, 4096] 7.5-7.8 vs
// 8.3-8.8 us, [14336, 4096] 12.3 vs 13.4-14.3, [28672, 4096] 17.1-17.5 vs 18.5-21.0, [4096, 14336] 13.8 vs 14.3-15.6,
// lm_head the same; eight rows of x: [14336, 4096] 12.9-13.3 vs 14.2-15.1, the others the same.  More requests in
// flight per wave only queue up behind each other (32 KB per CU are under way as it is) and cost registers.
template <int CPW, int XS, bool NESTED, int EPI>
hipError_t launch_c(const MatmulArgs& a, const QuadPlan& p, int grid, hipStream_t stream, int halves = 1) {
    return launch_u<CPW, 1, XS, NESTED, EPI>(a, p, grid, stream, halves);
}

template <bool NESTED, int EPI>
hipError_t launch_e(const MatmulArgs& a, const QuadPlan& p, int grid, hipStream_t stream, int halves = 1) {
    if (a.M > 4 || halves > 1)  // (a half is planned as eight rows of x)
        return pick_cpw(8, a.K) == 1 ? launch_c<1, 2, NESTED, EPI>(a, p, grid, stream, halves)
                                     : launch_c<2, 2, NESTED, EPI>(a, p, grid, stream, halves);
    return pick_cpw(a.M, a.K) == 1 ? launch_c<1, 1, NESTED, EPI>(a, p, grid, stream) : launch_c<2, 1, NESTED, EPI>(a, p, grid, stream);
}

template <bool NESTED>
hipError_t launch_n(const MatmulArgs& a, const QuadPlan& p, int grid, hipStream_t stream, int halves = 1) {
    if constexpr (!NESTED) {
        switch (a.epi.flags) {
            case EPI_ROWSCALE: return launch_e<false, EPI_ROWSCALE>(a, p, grid, stream, halves);
            case EPI_ROWSCALE | EPI_SILU_PAIRS: return launch_e<false, EPI_ROWSCALE | EPI_SILU_PAIRS>(a, p, grid, stream, halves);
            case EPI_SILU_PAIRS: return launch_e<false, EPI_SILU_PAIRS>(a, p, grid, stream, halves);
            case EPI_RESID_NORM: return launch_e<false, EPI_RESID_NORM>(a, p, grid, stream, halves);
        }
    }
    if (a.epi.flags != EPI_NONE) return hipErrorNotSupported;
    return launch_e<NESTED, EPI_NONE>(a, p, grid, stream, halves);
}

template <int CPW, int U, int XS, int MODE>
hipError_t allow_lds_epi() {
    hipError_t e;
    if ((e = gemv_allow_lds(gemv_quad_kernel<CPW, U, XS, false, MODE, EPI_NONE>, SMEM_BYTES)) != hipSuccess) return e;
    if ((e = gemv_allow_lds(gemv_quad_kernel<CPW, U, XS, true, MODE, EPI_NONE>, SMEM_BYTES)) != hipSuccess) return e;
    if ((e = gemv_allow_lds(gemv_quad_kernel<CPW, U, XS, false, MODE, EPI_ROWSCALE>, SMEM_BYTES)) != hipSuccess) return e;
    if ((e = gemv_allow_lds(gemv_quad_kernel<CPW, U, XS, false, MODE, EPI_ROWSCALE | EPI_SILU_PAIRS>, SMEM_BYTES)) != hipSuccess) return e;
    if ((e = gemv_allow_lds(gemv_quad_kernel<CPW, U, XS, false, MODE, EPI_SILU_PAIRS>, SMEM_BYTES)) != hipSuccess) return e;
    return gemv_allow_lds(gemv_quad_kernel<CPW, U, XS, false, MODE, EPI_RESID_NORM>, SMEM_BYTES);
}

template <int CPW, int U, int XS>
hipError_t allow_lds_cu() {
    hipError_t e;
    if ((e = allow_lds_epi<CPW, U, XS, ARITH_BF16>()) != hipSuccess) return e;
    if ((e = allow_lds_epi<CPW, U, XS, ARITH_F16>()) != hipSuccess) return e;
    return allow_lds_epi<CPW, U, XS, ARITH_EXACT>();
}

int quad_slots(int cus) {
    int slots = 2 * cus;
    return slots > GEMV_COUNTER_BYTES / 4 ? GEMV_COUNTER_BYTES / 4 : slots;
}

}  // namespace

size_t gemv_quad_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    const int s = quad_splits(M, K);
    return (size_t)GEMV_COUNTER_BYTES + (s > 1 ? (size_t)s * (size_t)M * (size_t)N * sizeof(float) : 0);
}

hipError_t gemv_quad_setup() {
    hipError_t e;
    if ((e = allow_lds_cu<1, 1, 1>()) != hipSuccess) return e;
    if ((e = allow_lds_cu<2, 1, 1>()) != hipSuccess) return e;
    if ((e = allow_lds_cu<2, 1, 2>()) != hipSuccess) return e;
    return allow_lds_cu<1, 1, 2>();
}

// Nine to sixteen rows of x as two halves of up to eight, one workgroup each per task (the weight is read twice, the
// second time mostly from the caches): for small weights, where the tile kernel's start-up costs more than that.
bool gemv_quad_halves_possible(int64_t N, int64_t K) { return K % LOAD_K == 0 && quad_splits(8, K) == 1; }

hipError_t launch_gemv_quad_halves(const MatmulArgs& a, int cus, hipStream_t stream) {
    if (a.M <= 8 || a.M > 16 || !gemv_quad_halves_possible(a.N, a.K)) return hipErrorInvalidValue;
    if (!gemv_quad_epilogue_possible(a)) return hipErrorNotSupported;
    // each half has the chip to itself in the plan: the two halves of a task then run side by side
    int slots = cus;
    const QuadPlan p = make_quad_plan(8, a.N, a.K, a.block_log2, slots, a.nested.q != nullptr, a.epi.flags != EPI_NONE);
    if (p.splits != 1) return hipErrorInvalidValue;
    int grid = p.ntasks < slots ? p.ntasks : slots;
    return a.nested.q ? launch_n<true>(a, p, grid, stream, 2) : launch_n<false>(a, p, grid, stream, 2);
}

// epilogues of the quad kernel: fp32 absmax; (gate, up) pairs need an even N; the producer's partial sums one per thread
bool gemv_quad_epilogue_possible(const MatmulArgs& a) {
    if (a.epi.flags == EPI_NONE) return true;
    if (a.nested.q) return false;
    if ((a.epi.flags & EPI_ROWSCALE) && a.epi.in_parts > GEMV_THREADS) return false;
    return !(a.epi.flags & EPI_SILU_PAIRS) || a.N % 2 == 0;
}

// bands of the plan an EPI_RESID_NORM call runs with (`halves`: nine to sixteen rows of x as two halves of eight)
int gemv_quad_norm_parts(int64_t M, int64_t N, int64_t K, int cus, bool halves) {
    const QuadPlan p = halves ? make_quad_plan(8, N, K, 6, cus, false, true) : make_quad_plan((int)M, N, K, 6, quad_slots(cus), false, true);
    if (p.splits > 1 && p.nbands > GEMV_COUNTER_BYTES / 4) return 0;
    return p.nbands;
}

hipError_t launch_gemv_quad(const MatmulArgs& a, int cus, hipStream_t stream) {
    if (!gemv_quad_epilogue_possible(a)) return hipErrorNotSupported;
    const int slots = quad_slots(cus);
    const QuadPlan p = make_quad_plan(a.M, a.N, a.K, a.block_log2, slots, a.nested.q != nullptr, a.epi.flags != EPI_NONE);
    // one arrival counter per band when K is split across workgroups
    if (p.splits > 1 && p.nbands > GEMV_COUNTER_BYTES / 4) return hipErrorInvalidValue;
    int grid = p.ntasks < slots ? p.ntasks : slots;
    grid -= grid % p.splits;  // every workgroup keeps one K split (ntasks is a multiple of splits)
    if (grid < p.splits) grid = p.splits;
    return a.nested.q ? launch_n<true>(a, p, grid, stream) : launch_n<false>(a, p, grid, stream);
}

}  // namespace nf4
