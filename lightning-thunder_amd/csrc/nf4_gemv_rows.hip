// Decode-shape fused NF4 dequant-matmul for gfx950, M = 1 and 2 (any M <= 4 works): the GEMV proper.
//
// Replaces bitsandbytes' gemv_4bit (kgemm_4bit_inference_naive), the kernel that
// bitsandbytes.matmul_4bit picks for a single-row x; call site
// thunder/transforms/quantization.py:39.
//
// HBM-bound: 0.5 byte of codes + 4/blocksize bytes of absmax per weight, each read exactly once.
//
//  * Weight stream.  A wave reads one weight row at a time, 1 KB per load instruction: lane l takes
//    the 16 bytes (32 codes) at k = chunk*2048 + 32*l.  Consecutive lanes read consecutive bytes, so
//    every load is a fully coalesced 1 KB burst; U rows are kept in flight per wave.
//  * x stays in registers.  A wave works on one 2048-wide k chunk for all its rows, so each lane
//    keeps its 32 x values (16 dwords of bf16 pairs) per row of x for the whole task.
//  * Code -> bf16.  A 256-entry LDS table indexed by a whole packed BYTE returns both bf16 code
//    values of that byte as one dword (even element in the low half).  The table is replicated for
//    all 64 lanes with a 256-byte stride, so the LDS address is (byte << 8) | (lane * 4): one
//    v_perm_b32 per byte and no bank conflicts.
//  * Multiply-accumulate on the matrix pipe.  v_mfma_f32_4x4x4_16b_bf16 computes 16 independent
//    4x4x4 products, one per group of 4 lanes.  Lane i of a group supplies row i of A (4 of its own
//    weights) and column i of B (the 4 matching x values), so the DIAGONAL element C[i][i] is lane
//    i's own dot product; the off-diagonal 3/4 of the result is discarded.  Eight such MFMAs cover
//    a lane's 32 weights and leave the VALU with the table addressing only.
//  * Scale.  The 32 weights of a lane share one quantisation block, so absmax multiplies the lane's
//    partial sum once.  This differs from the reference's dequantise-then-multiply only in where the
//    bf16 rounding happens; the difference grows like sqrt(K), so for K > 8192 an exact variant
//    rounds every weight as bf16(lut * absmax) before the MFMA (fp32 table, two multiplies and one
//    convert per byte more).
//  * Reduction.  Per-lane partial sums of 8 (row, m) pairs are reduced together by a transposing
//    butterfly (DPP for the four in-row levels, ds_bpermute for the two cross-row levels); the
//    result of (row, chunk, m) is parked in LDS, and after the band is done the chunks are added in
//    a fixed order.
//  * K > 16384 is split over two or more workgroups; partial sums cross workgroups through
//    agent-scope relaxed atomics and a counter (no L2-wide fences), added in a fixed order by the
//    last workgroup to arrive.
#include "decode_math.h"
#include "nf4_gemv.h"

namespace nf4 {
namespace {

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

constexpr int PART_BYTES = 16 * 1024;  // per-(row, chunk, m) partial sums of one band
constexpr int SMEM_BYTES = GEMV_TABLE_BYTES + PART_BYTES;
constexpr int CHUNK_K = 2048;          // k covered by one wave-wide 16-byte load
constexpr int FLAG_OFFSET = GEMV_TABLE_BYTES + PART_BYTES - 16;
constexpr int MAP_BYTES = 1024;         // nested absmax only: the 256-entry map, taken from the end of the partial sums
constexpr int MAP_OFFSET = FLAG_OFFSET - MAP_BYTES;
// kernels with an epilogue (fp32 absmax only): sums of squares per (row of x, wave), below the flag
constexpr int SUMSQ_BYTES = 2 * GEMV_WAVES * 4;
constexpr int SUMSQ_OFFSET = FLAG_OFFSET - 16 - SUMSQ_BYTES;
constexpr int PRE_BYTES = GEMV_THREADS * 4;  // EPI_RESID_NORM: a dword per thread
constexpr int PRE_OFFSET = SUMSQ_OFFSET - PRE_BYTES;

struct RowsPlan {
    int chunks;         // k chunks handled by one workgroup (waves along K)
    int row_lanes;      // rows processed concurrently by one workgroup = 8 / chunks
    int splits;         // K splits across workgroups
    int rows_per_band;  // rows of one task
    int nbands;
    int ntasks;         // nbands * splits
    int aligned;        // K % blocksize == 0: the block index splits into a row part and a k part
};

#define NF4_DPP(v, ctrl) \
    __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, 0xf, 0xf, true))

// v[0..7] hold per-lane partial sums of 8 independent quantities.  Returns, in every lane, the
// 64-lane total of quantity id(lane) = 4 * ((lane >> 2) & 1) ... see `reduce8_id`.
// Stage A/B/C halve the number of registers by letting lane bit 0/1/2 choose which quantity the
// lane keeps (the partner lane sends its share of it); the remaining three levels are plain sums.
__device__ __forceinline__ float reduce8(const float v[8], int lane) {
    const bool b0 = lane & 1, b1 = lane & 2, b2 = lane & 4;
    float w[4], z[2];
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const float keep = b0 ? v[2 * p + 1] : v[2 * p];
        const float send = b0 ? v[2 * p] : v[2 * p + 1];
        w[p] = keep + NF4_DPP(send, 0xB1);  // quad_perm [1,0,3,2]: lane ^ 1
    }
#pragma unroll
    for (int p = 0; p < 2; ++p) {
        const float keep = b1 ? w[2 * p + 1] : w[2 * p];
        const float send = b1 ? w[2 * p] : w[2 * p + 1];
        z[p] = keep + NF4_DPP(send, 0x4E);  // quad_perm [2,3,0,1]: lane ^ 2
    }
    const float keep = b2 ? z[1] : z[0];
    const float send = b2 ? z[0] : z[1];
    // lane ^ 4 inside a row of 16: shift by 4 in the direction that stays inside the group of 8
    float other = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, send), 0x104 /*row_shl:4*/, 0xf, 0x5, false));
    other = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, other), __builtin_bit_cast(int, send), 0x114 /*row_shr:4*/, 0xf, 0xa, false));
    float y = keep + other;
    y += NF4_DPP(y, 0x128);  // row_ror:8: lane ^ 8
    y += __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((lane ^ 16) << 2, __builtin_bit_cast(int, y)));
    y += __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((lane ^ 32) << 2, __builtin_bit_cast(int, y)));
    return y;
}
// quantity whose total `reduce8` leaves in `lane`: bit 0 of the lane picks v[odd], bit 1 the second
// pair, bit 2 the second half
__device__ __forceinline__ int reduce8_id(int lane) { return (lane & 1) | ((lane & 2) ? 2 : 0) | ((lane & 4) ? 4 : 0); }

// MODE (gemv_arith_mode): ARITH_BF16 / ARITH_F16: the table holds the code book rounded to bf16 / fp16 in pairs, x is
//                used as bf16 / converted to fp16 per lane, and absmax scales the 32-weight partial sum.
//                ARITH_EXACT: the table holds fp32 pairs and every weight is rounded like the reference's
//                dequantisation, bf16(lut * absmax), before it is multiplied (more VALU work).
// PAIRED (fp32 absmax, K a multiple of the blocksize): one absmax load serves TWO rows in flight -- the two lanes
//                that share a block fetch that block's absmax of the even and of the odd slot's row, and each slot
//                reads its value from the right lane through a DPP operand.  The 4-byte loads cost more than their
//                share of the bytes (a vector memory instruction per KB of codes: the lm_head ran 5 us faster without
//                them); this halves their number (lm_head 59.7 -> 58.4 us, [28672, 8192] 29.8 -> 28.0 with one row of x).
// EPI (Epilogue flags; fp32 absmax, K not split over workgroups): what the thread that finishes an output does with
//                it.  EPI_ROWSCALE: the producer's partial sums of squares are added up once per workgroup (one per
//                thread, butterfly per wave, waves in order) while the first weights are on their way.
//                EPI_RESID_NORM: a thread's outputs all belong to one row of x (M divides the workgroup size), so its
//                squares add up in a register; lanes of equal m are added by a butterfly, waves in order.
template <int M, int U, bool NESTED, int MODE, bool PAIRED, int EPI = EPI_NONE>
__global__ __launch_bounds__(GEMV_THREADS, 4) void gemv_rows_kernel(NF4_HOT_PARAMS, int hot_plan, int hot_rows_per_band, int hot_ntasks,
                                                                     MatmulArgs a_rest, RowsPlan p_rest) {
    // (arguments in SGPRs at wave start; the structs supply what is wanted later)
    const MatmulArgs a = with_hot_args<NESTED>(a_rest, NF4_HOT_NAMES);
    RowsPlan p = p_rest;
    p.chunks = hot_plan & 0xf; p.row_lanes = (hot_plan >> 4) & 0xf; p.aligned = (hot_plan >> 8) & 1; p.splits = hot_plan >> 9;
    p.rows_per_band = hot_rows_per_band; p.ntasks = hot_ntasks;
    static_assert(EPI == EPI_NONE || (!NESTED && GEMV_THREADS % M == 0 && M <= 2), "epilogues: fp32 absmax, M = 1, 2");
    constexpr bool EXACT = MODE == ARITH_EXACT, F16 = MODE == ARITH_F16;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t lane4 = (uint32_t)lane * 4u;
    const uint32_t lane8 = (uint32_t)(lane & 31) * 8u;

    // the code-book entry this lane contributes to the LDS table: requested first, used last
    const float lut_mine = a.lut16[lane & 15];
    bool table_built = false;

    float* part = reinterpret_cast<float*>(smem + GEMV_TABLE_BYTES);
    int* flag = reinterpret_cast<int*>(smem + FLAG_OFFSET);
    unsigned* counters = reinterpret_cast<unsigned*>(a.workspace);
    float* partial = reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(a.workspace) + GEMV_COUNTER_BYTES);

    const int cw = wave % p.chunks;   // this wave's chunk inside the workgroup's K range
    const int rl = wave / p.chunks;   // this wave's row lane
    const int64_t K = a.K;
    const int step = p.row_lanes;
    float* sumsq_s = reinterpret_cast<float*>(smem + SUMSQ_OFFSET);
    uint32_t* pre_s = reinterpret_cast<uint32_t*>(smem + PRE_OFFSET);

    for (int task = blockIdx.x; task < p.ntasks; task += gridDim.x) {
        const int band = task / p.splits;
        const int ks = task - band * p.splits;
        const int r_begin = band * p.rows_per_band;
        const int r_end = min(a.N, r_begin + p.rows_per_band);
        const int64_t kchunk = (int64_t)(ks * p.chunks + cw) * CHUNK_K;
        const uint32_t klane = 32u * (uint32_t)lane;
        const bool wave_on = rl < p.row_lanes && kchunk < K && r_begin + rl < r_end;
        const bool lane_on = wave_on && kchunk + klane < K;
        const int cnt = wave_on ? (r_end - r_begin - rl + step - 1) / step : 0;  // rows of this wave

        // What the epilogue needs from memory is requested first, ahead of x and the weights.  EPI_ROWSCALE (first
        // task): this thread's share of the producer's partial sums of squares, added up once the task's rows are
        // done.  EPI_RESID_NORM: residual and norm weight of the thread's first output (it rarely has a second), parked
        // in LDS before the first barrier (the wave's oldest requests: waiting for them waits for nothing else).
        const bool first_task = !table_built;
        float ssp[M];
        uint32_t pre_res = 0, pre_w = 0;
#pragma unroll
        for (int m = 0; m < M; ++m) {
            ssp[m] = 0.0f;
            if ((EPI & EPI_ROWSCALE) && first_task && tid < a.epi.in_parts) ssp[m] = a.epi.in_sumsq[m * a.epi.in_parts + tid];
        }
        if ((EPI & EPI_RESID_NORM) && tid < (r_end - r_begin) * M) {
            pre_res = a.epi.resid_in[(int64_t)(tid % M) * a.N + r_begin + tid / M];
            pre_w = a.epi.norm_weight[r_begin + tid / M];
        }
        // x for this lane's 32 k, all M rows
        uint32_t xr[M][16];
#pragma unroll
        for (int m = 0; m < M; ++m)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                uint4 v = make_uint4(0, 0, 0, 0);
                if (lane_on) v = *reinterpret_cast<const uint4*>(a.x + m * K + kchunk + klane + 8 * q);
                xr[m][4 * q + 0] = v.x; xr[m][4 * q + 1] = v.y; xr[m][4 * q + 2] = v.z; xr[m][4 * q + 3] = v.w;
            }
        // sq: absmax of the lane's block; nested: its 8-bit code (resolved through the LDS copy of
        // the map when the slot is consumed, so that issuing a load never waits for another) and
        // s2 the second-level absmax
        uint4 wq[U];
        float sq[U];
        float s2[NESTED ? U : 1];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            wq[u] = make_uint4(0, 0, 0, 0);
            sq[u] = 0.0f;
            if (NESTED) s2[u] = 0.0f;
        }
        // row i of this wave is r_begin + rl + i * step
        auto issue = [&](int u, int i) {
                const int row = r_begin + rl + i * step;
                if (lane_on) {
                    const uint8_t* rowp = a.packed + (((int64_t)row * K + kchunk) >> 1);  // uniform
                    wq[u] = load16_stream(rowp + (klane >> 1));
                    int64_t blk;
                    if (p.aligned)
                        blk = (((int64_t)row * K + kchunk) >> a.block_log2) + (klane >> a.block_log2);
                    else
                        blk = ((int64_t)row * K + kchunk + klane) >> a.block_log2;
                    if (NESTED) {
                        sq[u] = __uint_as_float((uint32_t)a.nested.q[blk]);
                        s2[u] = a.nested.absmax2[blk >> a.nested.nested_log2];
                    } else if (!PAIRED) {
                        sq[u] = load_f32_stream(a.absmax + blk);
                    } else if ((u & 1) == 0) {
                        // even lanes: this row; odd lanes: the row of slot u + 1 (the wave's next row, if it has one)
                        const int row2 = r_begin + rl + min(i + 1, cnt - 1) * step;
                        const int64_t blk2 = (((int64_t)row2 * K + kchunk) >> a.block_log2) + (klane >> a.block_log2);
                        sq[u] = load_f32_stream(a.absmax + ((lane & 1) ? blk2 : blk));
                    }
                }
            };
        // get the weight stream going before anything else happens
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (u < cnt) issue(u, u);

        if (!table_built) {  // first task only: overlaps with the loads above
            if (EXACT)
                build_pair_table_f32(smem, lut_mine, lane, wave);
            else
                build_pair_table<F16>(smem, lut_mine, lane, wave);
            if (NESTED && tid < 256) reinterpret_cast<float*>(smem + MAP_OFFSET)[tid] = a.nested.map256[tid];
            table_built = true;
        }
        if (EPI & EPI_RESID_NORM) {
            // (the two values are first looked at here: without this the compiler moves the shift up to the loads, and the
            // wait for them in front of the requests for x and the weights)
            asm volatile("" : "+v"(pre_res), "+v"(pre_w));
            pre_s[tid] = pre_res | (pre_w << 16);  // a slot per thread, read back by the same thread
        }
        __syncthreads();  // table built (first task) / previous task's epilogue done with `part`

        // fp16 arithmetic: the lane's x values become fp16, scaled into range per row of x (here, behind the requests for
        // the first weights, so that the conversion runs while they are under way)
        float unscale[M];
#pragma unroll
        for (int m = 0; m < M; ++m) {
            unscale[m] = 1.0f;
            if (F16) {
                u16x2_t mx = {0, 0};
#pragma unroll
                for (int q = 0; q < 16; ++q) mx = absmax_of_bf16_pair(xr[m][q], mx);
                const F16Scale fs = f16_scale_for(absmax_bits(mx));
#pragma unroll
                for (int q = 0; q < 16; ++q) xr[m][q] = bf16_pair_to_f16(xr[m][q], fs.to_f16);
                unscale[m] = fs.from_f16;
            }
        }


        if (cnt > 0) {
            for (int i0 = 0; i0 < cnt; i0 += U) {
                float res[U * M];
                float s_odd = 0.0f;
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const uint32_t d[4] = {wq[u].x, wq[u].y, wq[u].z, wq[u].w};
                    float s = sq[u];
                    if (PAIRED) {
                        if ((u & 1) == 0) {
                            const int both = __builtin_bit_cast(int, sq[u]);
                            s = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(both, both, 0xA0, 0xf, 0xf, true));  // quad_perm [0,0,2,2]
                            s_odd = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(both, both, 0xF5, 0xf, 0xf, true));  // quad_perm [1,1,3,3]
                        } else {
                            s = s_odd;
                        }
                    }
                    if (NESTED)
                        s = __fadd_rn(__fmul_rn(reinterpret_cast<const float*>(smem + MAP_OFFSET)[__float_as_uint(s)], s2[u]),
                                      a.nested.offset);
                    if (i0 + u + U < cnt) {
                        issue(u, i0 + u + U);
                    } else {  // slot is dead from here on; say so, or the compiler keeps copies alive
                        wq[u] = make_uint4(0, 0, 0, 0);
                        sq[u] = 0.0f;
                        if (NESTED) s2[u] = 0.0f;
                    }
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
                    for (int m = 0; m < M; ++m) {
                        f32x4 c = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                        for (int t = 0; t < 8; ++t) {
                            const uint2 wa = make_uint2(pr[2 * t], pr[2 * t + 1]);
                            const uint2 xb = make_uint2(xr[m][2 * t], xr[m][2 * t + 1]);
                            if (!F16)
                                c = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(s16x4, wa),
                                                                           __builtin_bit_cast(s16x4, xb), c, 0, 0, 0);
                            else
                                c = __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(f16x4, wa),
                                                                       __builtin_bit_cast(f16x4, xb), c, 0, 0, 0);
                        }
                        // diagonal element of this lane's 4x4 block
                        const float c01 = (lane & 1) ? c[1] : c[0];
                        const float c23 = (lane & 1) ? c[3] : c[2];
                        const float diag = (lane & 2) ? c23 : c01;
                        res[u * M + m] = EXACT ? diag : diag * (s * unscale[m]);
                    }
                }
                // reduce the U*M per-lane results over the wave, 8 at a time
#pragma unroll
                for (int g8 = 0; g8 < (U * M + 7) / 8; ++g8) {
                    float v8[8];
#pragma unroll
                    for (int e = 0; e < 8; ++e) v8[e] = (g8 * 8 + e < U * M) ? res[g8 * 8 + e] : 0.0f;
                    const float total = reduce8(v8, lane);
                    const int id = g8 * 8 + reduce8_id(lane);  // = u * M + m
                    const int u = id / M, m = id - u * M;
                    const int i = i0 + u;
                    if (lane < 8 && id < U * M && i < cnt)
                        part[((rl + i * step) * p.chunks + cw) * M + m] = total;
                }
            }
        }
        // EPI_ROWSCALE: the partial sums requested at the top have long arrived; nothing has looked at them so far
        if ((EPI & EPI_ROWSCALE) && first_task) {
#pragma unroll
            for (int m = 0; m < M; ++m) {
                float ss = ssp[m];
#pragma unroll
                for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
                if (lane == 0) sumsq_s[m * GEMV_WAVES + wave] = ss;
            }
        }
        __syncthreads();

        // ---- band epilogue: add the chunks of every row in a fixed order ----
        const int nrows = r_end - r_begin;
        // the last split may own fewer chunks than the others
        const int nchunks = min(p.chunks, (int)((K + CHUNK_K - 1) / CHUNK_K) - ks * p.chunks);
        float rstd[M];  // EPI_ROWSCALE: 1 / rms of every row of x, from the wave sums left in LDS by the first task
#pragma unroll
        for (int m = 0; m < M; ++m) {
            rstd[m] = 1.0f;
            if (EPI & EPI_ROWSCALE) {
                float tot = 0.0f;
#pragma unroll
                for (int w = 0; w < GEMV_WAVES; ++w) tot += sumsq_s[m * GEMV_WAVES + w];
                rstd[m] = rsqrtf(tot / (float)K + a.epi.eps);
            }
        }
        // finished sum of output (r, m) of this band, bias included
        auto finished = [&](int r, int m) {
            float sum = 0.0f;
            for (int c = 0; c < nchunks; ++c) sum += part[(r * p.chunks + c) * M + m];
            if (EPI & EPI_ROWSCALE) sum *= rstd[m];
            if (a.bias) sum += bf16_bits_to_f32(a.bias[r_begin + r]);
            return sum;
        };
        if (EPI & EPI_SILU_PAIRS) {
            // rows 2j, 2j + 1 of the band: gate j, up j (bands start and end on even rows)
            for (int idx = tid; idx < (nrows / 2) * M; idx += GEMV_THREADS) {
                const int j = idx / M, m = idx - j * M;
                const float g = nf4x::round_bf16(finished(2 * j, m)), u = nf4x::round_bf16(finished(2 * j + 1, m));
                a.out[(int64_t)m * (a.N / 2) + r_begin / 2 + j] = (uint16_t)nf4x::silu_mul_bf16(g, u);
            }
        } else if (EPI & EPI_RESID_NORM) {
            float ss = 0.0f;  // every output of this thread has m = tid % M
            for (int idx = tid; idx < nrows * M; idx += GEMV_THREADS) {
                const int r = idx / M, m = idx - r * M;
                const int64_t at = (int64_t)m * a.N + r_begin + r;
                const float d = nf4x::round_bf16(finished(r, m));
                const bool pre = idx == tid;
                const uint32_t parked = pre_s[tid];
                const float old = bf16_bits_to_f32(pre ? parked & 0xffffu : (uint32_t)a.epi.resid_in[at]);
                const float nw = bf16_bits_to_f32(pre ? parked >> 16 : (uint32_t)a.epi.norm_weight[r_begin + r]);
                const float res = nf4x::resid_add(old, d);
                a.epi.resid_out[at] = (uint16_t)f32_to_bf16_bits(res);
                a.epi.xnext_out[at] = (uint16_t)f32_to_bf16_bits(res * nw);
                ss = fmaf(res, res, ss);
            }
#pragma unroll
            for (int o = 32; o >= M; o >>= 1) ss += __shfl_xor(ss, o, 64);  // lanes of equal m (M = 1, 2)
            if (lane < M) sumsq_s[lane * GEMV_WAVES + wave] = ss;
            __syncthreads();
            if (tid < M) {
                float tot = 0.0f;
#pragma unroll
                for (int w = 0; w < GEMV_WAVES; ++w) tot += sumsq_s[tid * GEMV_WAVES + w];
                a.epi.out_sumsq[tid * p.nbands + band] = tot;
            }
        } else if (p.splits == 1) {
            for (int idx = tid; idx < nrows * M; idx += GEMV_THREADS) {
                const int r = idx / M, m = idx - r * M;
                a.out[(int64_t)m * a.N + r_begin + r] = (uint16_t)f32_to_bf16_bits(finished(r, m));
            }
        } else {
            for (int idx = tid; idx < nrows * M; idx += GEMV_THREADS) {
                const int r = idx / M, m = idx - r * M;
                float sum = 0.0f;
                for (int c = 0; c < nchunks; ++c) sum += part[(r * p.chunks + c) * M + m];
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
                for (int idx = tid; idx < nrows * M; idx += GEMV_THREADS) {
                    const int r = idx / M, m = idx - r * M;
                    const int n = r_begin + r;
                    float sum = 0.0f;
                    for (int k2 = 0; k2 < p.splits; ++k2)
                        sum += __hip_atomic_load(&partial[((int64_t)k2 * M + m) * a.N + n], __ATOMIC_RELAXED,
                                                 __HIP_MEMORY_SCOPE_AGENT);
                    if (a.bias) sum += bf16_bits_to_f32(a.bias[n]);
                    a.out[(int64_t)m * a.N + n] = (uint16_t)f32_to_bf16_bits(sum);
                }
                if (tid == 0) __hip_atomic_store(&counters[band], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
}

int rows_splits(int64_t K) {
    const int64_t nch = (K + CHUNK_K - 1) / CHUNK_K;
    return (int)((nch + GEMV_WAVES - 1) / GEMV_WAVES);
}

RowsPlan make_rows_plan(int M, int64_t N, int64_t K, int block_log2, int slots, bool nested, int epi = EPI_NONE) {
    RowsPlan p;
    p.aligned = (K & (((int64_t)1 << block_log2) - 1)) == 0;
    const int nch = (int)((K + CHUNK_K - 1) / CHUNK_K);
    p.splits = rows_splits(K);
    p.chunks = (nch + p.splits - 1) / p.splits;
    p.row_lanes = GEMV_WAVES / p.chunks;
    // rows of a band come in multiples of `unit`: the row lanes, and whole (gate, up) pairs where those are merged
    const int unit = (epi & EPI_SILU_PAIRS) && p.row_lanes % 2 ? 2 * p.row_lanes : p.row_lanes;
    const int part_bytes = PART_BYTES - 64 - (nested ? MAP_BYTES : 0) - (epi ? SUMSQ_BYTES + 16 + PRE_BYTES : 0);
    const int cap = (part_bytes / (p.chunks * M * 4)) / unit * unit;
    int bands_target = slots / p.splits;
    if (bands_target < 1) bands_target = 1;
    // one task per resident workgroup if its partial sums fit in LDS, else 2, 3, ... balanced rounds
    int64_t rpb = cap;
    for (int rounds = 1; rounds <= 64; ++rounds) {
        int64_t r = (N + (int64_t)rounds * bands_target - 1) / ((int64_t)rounds * bands_target);
        r = (r + unit - 1) / unit * unit;
        if (r <= cap) {
            rpb = r;
            break;
        }
    }
    if (rpb < unit) rpb = unit;
    p.rows_per_band = (int)rpb;
    p.nbands = (int)((N + rpb - 1) / rpb);
    p.ntasks = p.nbands * p.splits;
    return p;
}

template <int M, int U, bool NESTED, bool PAIRED, int EPI>
hipError_t launch_p(const MatmulArgs& a, const RowsPlan& p, int grid, hipStream_t stream) {
    const int mode = gemv_arith_mode(a.K, true);
    if (mode == ARITH_EXACT)
        hipLaunchKernelGGL((gemv_rows_kernel<M, U, NESTED, ARITH_EXACT, PAIRED, EPI>), dim3(grid), dim3(GEMV_THREADS), SMEM_BYTES, stream, NF4_HOT_VALUES(a),
                           p.chunks | (p.row_lanes << 4) | (p.aligned << 8) | (p.splits << 9), p.rows_per_band, p.ntasks, a, p);
    else if (mode == ARITH_F16)
        hipLaunchKernelGGL((gemv_rows_kernel<M, U, NESTED, ARITH_F16, PAIRED, EPI>), dim3(grid), dim3(GEMV_THREADS), SMEM_BYTES, stream, NF4_HOT_VALUES(a),
                           p.chunks | (p.row_lanes << 4) | (p.aligned << 8) | (p.splits << 9), p.rows_per_band, p.ntasks, a, p);
    else
        hipLaunchKernelGGL((gemv_rows_kernel<M, U, NESTED, ARITH_BF16, PAIRED, EPI>), dim3(grid), dim3(GEMV_THREADS), SMEM_BYTES, stream, NF4_HOT_VALUES(a),
                           p.chunks | (p.row_lanes << 4) | (p.aligned << 8) | (p.splits << 9), p.rows_per_band, p.ntasks, a, p);
    return hipGetLastError();
}

template <int M, int U, bool NESTED, int EPI>
hipError_t launch_u(const MatmulArgs& a, const RowsPlan& p, int grid, hipStream_t stream) {
    if constexpr (!NESTED && M == 1)  // measured: 1-2 us on weights of 30 MB and more with one row of x, a loss with two
        if (p.aligned) return launch_p<M, U, false, true, EPI>(a, p, grid, stream);
    return launch_p<M, U, NESTED, false, EPI>(a, p, grid, stream);
}

// U = rows in flight per wave.  Four KB per wave, 64 KB per CU, cover the memory system's latency; eight rows in
// flight (every one of the 128 registers in use, any further live value spilt) measured 0.3-0.5 us slower on the
// 33-117 MB weights and 2.5 us slower on [28672, 8192].  Two rows of x: two rows in flight ([28672, 4096] 16.7-17.2 vs
// 17.9-18.6 us, [4096, 14336] 12.7 vs 13.4; four rows in flight and two rows of x leave no register free).
template <int M, bool NESTED, int EPI>
hipError_t launch_m(const MatmulArgs& a, const RowsPlan& p, int grid, hipStream_t stream) {
    const int cnt = p.rows_per_band / p.row_lanes;  // rows per wave and task
    if constexpr (M == 1) {
        if (cnt >= 4) return launch_u<1, 4, NESTED, EPI>(a, p, grid, stream);
    }
    return launch_u<M, 2, NESTED, EPI>(a, p, grid, stream);
}

template <bool NESTED, int EPI>
hipError_t launch_n(const MatmulArgs& a, const RowsPlan& p, int grid, hipStream_t stream) {
    // M = 3 and 4 are served by the four-rows-per-quad kernel
    return a.M == 2 ? launch_m<2, NESTED, EPI>(a, p, grid, stream) : launch_m<1, NESTED, EPI>(a, p, grid, stream);
}

template <int M, int U, int MODE, int EPI>
hipError_t allow_lds_epi() {
    hipError_t e;
    if ((e = gemv_allow_lds(gemv_rows_kernel<M, U, false, MODE, false, EPI>, SMEM_BYTES)) != hipSuccess) return e;
    if constexpr (M == 1)
        if ((e = gemv_allow_lds(gemv_rows_kernel<M, U, false, MODE, true, EPI>, SMEM_BYTES)) != hipSuccess) return e;
    return hipSuccess;
}

template <int M, int U, int MODE>
hipError_t allow_lds_mode() {
    hipError_t e;
    if ((e = allow_lds_epi<M, U, MODE, EPI_NONE>()) != hipSuccess) return e;
    if ((e = allow_lds_epi<M, U, MODE, EPI_ROWSCALE>()) != hipSuccess) return e;
    if ((e = allow_lds_epi<M, U, MODE, EPI_ROWSCALE | EPI_SILU_PAIRS>()) != hipSuccess) return e;
    if ((e = allow_lds_epi<M, U, MODE, EPI_SILU_PAIRS>()) != hipSuccess) return e;
    if ((e = allow_lds_epi<M, U, MODE, EPI_RESID_NORM>()) != hipSuccess) return e;
    return gemv_allow_lds(gemv_rows_kernel<M, U, true, MODE, false>, SMEM_BYTES);
}

template <int M, int U>
hipError_t allow_lds_mu() {
    hipError_t e;
    if ((e = allow_lds_mode<M, U, ARITH_BF16>()) != hipSuccess) return e;
    if ((e = allow_lds_mode<M, U, ARITH_F16>()) != hipSuccess) return e;
    return allow_lds_mode<M, U, ARITH_EXACT>();
}

template <int M>
hipError_t allow_lds_m() {
    if constexpr (M == 1) {  // four rows in flight: one row of x only (launch_m)
        const hipError_t e = allow_lds_mu<M, 4>();
        if (e != hipSuccess) return e;
    }
    return allow_lds_mu<M, 2>();
}

}  // namespace

size_t gemv_rows_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    const int s = rows_splits(K);
    return (size_t)GEMV_COUNTER_BYTES + (s > 1 ? (size_t)s * (size_t)M * (size_t)N * sizeof(float) : 0);
}

hipError_t gemv_rows_setup() {
    hipError_t e;
    if ((e = allow_lds_m<1>()) != hipSuccess) return e;
    return allow_lds_m<2>();
}

// epilogues of the row kernel: fp32 absmax, whole rows of x in one workgroup; (gate, up) pairs need an even N
bool gemv_rows_epilogue_possible(const MatmulArgs& a) {
    if (a.epi.flags == EPI_NONE) return true;
    if (a.nested.q || rows_splits(a.K) != 1) return false;
    if ((a.epi.flags & EPI_ROWSCALE) && a.epi.in_parts > GEMV_THREADS) return false;
    return !(a.epi.flags & EPI_SILU_PAIRS) || a.N % 2 == 0;
}

int gemv_rows_norm_parts(int64_t M, int64_t N, int64_t K, int cus) {
    if (rows_splits(K) != 1) return 0;
    int slots = 2 * cus;
    if (slots > GEMV_COUNTER_BYTES / 4) slots = GEMV_COUNTER_BYTES / 4;
    return make_rows_plan((int)M, N, K, 6, slots, false, EPI_RESID_NORM).nbands;
}

hipError_t launch_gemv_rows(const MatmulArgs& a, int cus, hipStream_t stream) {
    if (!gemv_rows_epilogue_possible(a)) return hipErrorNotSupported;
    int slots = 2 * cus;
    if (slots > GEMV_COUNTER_BYTES / 4) slots = GEMV_COUNTER_BYTES / 4;
    const RowsPlan p = make_rows_plan(a.M, a.N, a.K, a.block_log2, slots, a.nested.q != nullptr, a.epi.flags);
    // one arrival counter per band when K is split across workgroups
    if (p.splits > 1 && p.nbands > GEMV_COUNTER_BYTES / 4) return hipErrorInvalidValue;
    const int grid = p.ntasks < slots ? p.ntasks : slots;
    switch (a.epi.flags) {
        case EPI_NONE: return a.nested.q ? launch_n<true, EPI_NONE>(a, p, grid, stream) : launch_n<false, EPI_NONE>(a, p, grid, stream);
        case EPI_ROWSCALE: return launch_n<false, EPI_ROWSCALE>(a, p, grid, stream);
        case EPI_ROWSCALE | EPI_SILU_PAIRS: return launch_n<false, EPI_ROWSCALE | EPI_SILU_PAIRS>(a, p, grid, stream);
        case EPI_SILU_PAIRS: return launch_n<false, EPI_SILU_PAIRS>(a, p, grid, stream);
        case EPI_RESID_NORM: return launch_n<false, EPI_RESID_NORM>(a, p, grid, stream);
    }
    return hipErrorNotSupported;
}

}  // namespace nf4
