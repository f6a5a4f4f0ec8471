// Decode-shape fused NF4 dequant-matmul for gfx950, 5 <= M <= 16 rows of x: MFMA tiles.
//
// Replaces bitsandbytes' gemv_4bit / small-batch matmul_4bit, call site
// thunder/transforms/quantization.py:39.
//
// The kernel is HBM-bound: per weight it moves 4 bits of code plus 1/blocksize of an fp32 absmax.
// One workgroup (8 waves) per CU; wave w of a workgroup owns the w-th 16-row tile of each of the
// workgroup's 128-row tile groups.  The x operands of one K slice are resident in LDS in MFMA
// order, so the waves run unsynchronised except when the slice changes.  Tile groups are taken
// in batches of up to four whose accumulators all live in registers: the batch sweeps the slices
// of the workgroup's K range one after the other, so a long K costs a re-staging of x per slice
// and batch, not a round trip of partial sums.  Weight loads run through a four-slot register
// ring (one 512-k phase of one tile per slot) that stays full across tile, slice and batch
// boundaries.
//
//  * Weight stream.  Per phase a lane issues four 16-byte loads; in load i, lane l reads row
//    4*((l>>2)&3) + i of the tile at byte (l>>4)*64 + (l&3)*16 of the row's 256-byte phase slice,
//    so four ADJACENT lanes read 64 contiguous bytes (one L1 request instead of four) and one load
//    instruction covers four rows x 256 contiguous bytes.
//  * Into MFMA order, in registers.  A 4x4 transpose inside each lane quad (DPP quad_perm +
//    select) exchanges "load index" with "lane & 3", after which lane l holds row l & 15; a 4x4
//    transpose across lanes {c, c+16, c+32, c+48} (v_permlane32_swap, v_permlane16_swap) then
//    makes every MFMA cover 32 CONSECUTIVE k, so two MFMAs = one 64-element quantisation block.
//  * Code -> bf16.  256-entry byte -> (bf16, bf16) LDS table replicated per lane: one v_perm_b32
//    builds the address, one ds_read_b32 returns two MFMA-ready values.
//  * Contraction.  v_mfma_f32_16x16x32_bf16, A = x (rows m), B = W (columns n): the accumulator of
//    a lane belongs to the lane's own weight row, so the absmax scale of a block is one the lane
//    loaded itself (4 FMAs per block).
//  * x.  Up to 80 KB resident: 5 phases of 16 rows, or 10 phases of 8 rows when M <= 8 (lanes of
//    rows >= 8 then re-read rows 0..7; an MFMA output row depends on its own A row only, and rows
//    >= M are never stored).  XOR-swizzled so that both the scattered staging writes and the
//    linear operand reads are conflict-free.
//  * K split.  Only when N alone cannot fill the chip is K also split over workgroups; partial
//    sums then go to a workspace and the last WAVE to finish a tile (device-scope counter per
//    tile) adds them in a fixed order, so the result does not depend on scheduling.
#include "decode_math.h"
#include "nf4_gemv.h"

namespace nf4 {
namespace {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

constexpr int THREADS = GEMV_THREADS;
constexpr int WAVES = GEMV_WAVES;
constexpr int TABLE_BYTES = GEMV_TABLE_BYTES;
constexpr int PHASE_K = 512;                 // k per phase
constexpr int XBYTES_MAX = 80 * 1024;        // resident x operands
constexpr int ITEMS_MAX = 512;               // longest work list of a workgroup (one entry per thread)
constexpr int ITEMS_OFFSET = TABLE_BYTES + XBYTES_MAX;
constexpr int UNSCALE_OFFSET = ITEMS_OFFSET + ITEMS_MAX * 16;  // fp16 mode: 16 floats, what undoes the scaling of each row of x
constexpr int SUMSQ_OFFSET = UNSCALE_OFFSET + 64;  // EPI_ROWSCALE: the sum of squares of each row of x, 16 floats
constexpr int SMEM_BYTES = SUMSQ_OFFSET + 64;
constexpr int COUNTER_BYTES = GEMV_COUNTER_BYTES;
constexpr int SLOTS = 4;                     // ring slots = accumulator sets = largest batch

struct Plan {
    int tile_groups;   // ceil(N / 128)
    int splits;        // K ranges across workgroups
    int range_phases;  // phases per K range (the last range may be shorter)
    int total_phases;  // K / 512
    int tg_step;       // gridDim.x / splits: distance between a workgroup's consecutive tile groups
};

struct PhaseRegs {
    uint4 w[4];   // [load]: 32 codes each
    float4 s[2];  // absmax of the 8 blocks of the phase (or raw data to build them)
};

// One entry of a workgroup's work list: one 512-k phase of one tile group, or a gap.
//
// Order of the list: batch, slice, phase, tile group of the batch.  Tile groups are taken in batches of
// 4, then 2, then 1; entry i uses ring slot and accumulator set i & 3, so with batches of 1, 2 or 4
// tile groups a slot always meets the same tile group.  Every slice of a batch starts at a multiple
// of 4 (gaps pad the previous one), so a change of slice is only ever met at slot 0.  Odd batches
// walk the slices backwards, so the slice a batch ends with is the one the next batch starts with.
// The list is a pure function of the entry index: every workgroup writes its own into LDS once, one
// entry per thread, and the waves then read it instead of carrying cursors through the loop.
struct Item {
    int tg;    // tile group
    int kabs;  // first k of the phase
    int info;  // see below
    int k0;    // first k of the phase's slice
};
constexpr int ITEM_PHS_MASK = 0xf;      // bits 0-3: phase within its slice
constexpr int ITEM_NB_SHIFT = 4;        // bits 4-6: tile groups in the batch (1, 2, 4)
constexpr int ITEM_GAP = 1 << 7;        // nothing to do in this slot
constexpr int ITEM_RESTAGE = 1 << 8;    // first entry of a slice that is not resident yet (always at slot 0)
constexpr int ITEM_END = 1 << 9;        // last entry of its batch
constexpr int ITEM_NPH_SHIFT = 12;      // bits 12-15: phases of the slice

struct ListShape {
    int G;         // tile groups of this workgroup
    int rph;       // phases of its K range
    int nsl;       // slices of the range
    int last;      // phases of the last slice
    int r0;        // first phase of the range
    int tg0;       // first tile group
    int tg_step;   // distance between consecutive tile groups
    int nitems;    // entries, gaps included (a multiple of 4)
};

__device__ __host__ constexpr int ceil4(int v) { return (v + 3) & ~3; }

// entries of one batch of nb tile groups
template <int CAP>
__device__ __host__ constexpr int batch_length(int nsl, int last, int nb) {
    return (nsl - 1) * ceil4(CAP * nb) + ceil4(last * nb);
}

template <int CAP>
__device__ __host__ constexpr int list_length(int G, int nsl, int last) {
    const int full = G >> 2, rem = G & 3;
    int n = full * batch_length<CAP>(nsl, last, 4);
    if (rem == 1) n += batch_length<CAP>(nsl, last, 1);
    if (rem >= 2) n += batch_length<CAP>(nsl, last, 2);
    if (rem == 3) n += batch_length<CAP>(nsl, last, 1);
    return n;
}

template <int CAP>
__device__ __forceinline__ Item make_item(const ListShape& ls, int i) {
    const int LB4 = batch_length<CAP>(ls.nsl, ls.last, 4);
    const int full = ls.G >> 2, rem = ls.G & 3;
    int batch, k, nb, bi;
    if (i < full * LB4) {
        batch = i / LB4;
        k = i - batch * LB4;
        nb = 4;
        bi = 4 * batch;
    } else {
        const int j = i - full * LB4;
        const int nb0 = rem == 1 ? 1 : 2;
        const int L0 = batch_length<CAP>(ls.nsl, ls.last, nb0);
        batch = full;
        bi = 4 * full;
        if (j < L0) {
            nb = nb0;
            k = j;
        } else {  // rem == 3: the single tile group after the pair
            nb = 1;
            k = j - L0;
            batch += 1;
            bi += 2;
        }
    }
    const int Lf = ceil4(CAP * nb), Ll = ceil4(ls.last * nb);
    int sl, kk;
    if (!(batch & 1)) {  // forwards: the full slices, then the last one
        const int head = (ls.nsl - 1) * Lf;
        if (k < head) {
            sl = k / Lf;
            kk = k - sl * Lf;
        } else {
            sl = ls.nsl - 1;
            kk = k - head;
        }
    } else {  // backwards: the last slice first
        if (k < Ll) {
            sl = ls.nsl - 1;
            kk = k;
        } else {
            const int q = (k - Ll) / Lf;
            sl = ls.nsl - 2 - q;
            kk = k - Ll - q * Lf;
        }
    }
    const int nph = sl == ls.nsl - 1 ? ls.last : CAP;
    const int t = kk & (nb - 1);
    const int phs = kk >> (nb >> 1);  // nb = 1, 2, 4 -> shift 0, 1, 2
    const bool final_slice = (batch & 1) ? sl == 0 : sl == ls.nsl - 1;
    Item it;
    it.tg = ls.tg0 + (bi + t) * ls.tg_step;
    it.kabs = (ls.r0 + sl * CAP + phs) * PHASE_K;
    it.k0 = (ls.r0 + sl * CAP) * PHASE_K;
    it.info = (phs & ITEM_PHS_MASK) | (nb << ITEM_NB_SHIFT) | ((nph & 0xf) << ITEM_NPH_SHIFT);
    if (kk >= nph * nb) it.info |= ITEM_GAP;
    if (kk == 0 && k != 0) it.info |= ITEM_RESTAGE;
    if (final_slice && kk == nph * nb - 1) it.info |= ITEM_END;
    return it;
}

// Lane-dependent constants of the load side.
struct LaneLoad {
    uint32_t woff[4];  // per load: byte offset from the tile's first byte of the phase
    uint32_t s_off;    // absmax blocks from the tile's first row to the lane's row
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

// `on` (wave-uniform, all ones or zero) switches a request off without a branch: with on = 0 every
// lane reads the first bytes of the phase (one cache line per instruction) and the slot's contents
// are never used.
template <bool B64, bool NESTED>
__device__ __forceinline__ void load_phase(const MatmulArgs& a, PhaseRegs& r, const LaneLoad& ll, int n0c, int kabs,
                                           uint32_t on = 0xffffffffu) {
    // n0c = first row actually read for the tile, kabs = first k of the phase (both wave-uniform)
    const int64_t e0 = (int64_t)n0c * a.K + kabs;
    const uint8_t* wp = a.packed + (e0 >> 1);
    const uint32_t s_off = ll.s_off & on;
#pragma unroll
    for (int i = 0; i < 4; ++i) r.w[i] = load16_stream(wp + (ll.woff[i] & on));
    if (NESTED) {
        if (B64) {
            const int64_t b = (e0 >> 6) + s_off;
            const uint2 q = *reinterpret_cast<const uint2*>(a.nested.q + b);
            r.s[0].x = __uint_as_float(q.x);
            r.s[0].y = __uint_as_float(q.y);
            // 8 consecutive blocks starting at a multiple of 8 share one nested block (>= 64 blocks)
            r.s[0].z = a.nested.absmax2[b >> a.nested.nested_log2];
        } else {
            const int64_t b = ((int64_t)n0c * a.K >> a.block_log2) + s_off;
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                r.s[j].x = nested_absmax(a.nested, b + ((kabs + j * 256) >> a.block_log2));
                r.s[j].y = nested_absmax(a.nested, b + ((kabs + j * 256 + 64) >> a.block_log2));
                r.s[j].z = nested_absmax(a.nested, b + ((kabs + j * 256 + 128) >> a.block_log2));
                r.s[j].w = nested_absmax(a.nested, b + ((kabs + j * 256 + 192) >> a.block_log2));
            }
        }
    } else if (B64) {
        const float* sp = a.absmax + (e0 >> 6) + s_off;
        // (ordinary loads: a phase takes 32 bytes of a row's absmax line, the next phases the rest of it from the caches)
        r.s[0] = *reinterpret_cast<const float4*>(sp);
        r.s[1] = *reinterpret_cast<const float4*>(sp + 4);
    } else {
        const float* sp = a.absmax + ((int64_t)n0c * a.K >> a.block_log2) + s_off;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            r.s[j].x = sp[(kabs + j * 256) >> a.block_log2];
            r.s[j].y = sp[(kabs + j * 256 + 64) >> a.block_log2];
            r.s[j].z = sp[(kabs + j * 256 + 128) >> a.block_log2];
            r.s[j].w = sp[(kabs + j * 256 + 192) >> a.block_log2];
        }
    }
}

// LDS layout of the resident x operands.  One phase = 16 MFMAs (j); MFMA j reads, for lane
// (gg = lane >> 4, m = lane & 15), the 16 bytes x[m][32 j + 8 gg .. + 8].  With R rows held
// (R = 16, or 8 when M <= 8) a phase takes R KB and the slot of (j, gg, m) is
//     j * 4R + gg * R + ((m ^ ((j & 1) << 2 | gg)) & (R - 1)):
// linear in the lane up to an XOR inside each R-slot group, so operand reads are conflict-free,
// and the XOR spreads the eight consecutive 8-k pieces that eight adjacent staging lanes write
// (same m, piece & 7 = 0..7) over all banks.
template <int R>
__device__ __forceinline__ uint32_t xslot_bytes(int m, int piece) {
    const int j = piece >> 2, gg = piece & 3;
    return (uint32_t)(j * 4 * R + gg * R + ((m ^ (((j & 1) << 2) | gg)) & (R - 1))) * 16u;
}

// The codes of one phase in MFMA order plus the scales of its 8 blocks: what is left of a ring slot
// once its registers have been handed back to the next load.
struct PhaseOperands {
    uint32_t d[4][4];  // d[q][p] = bytes [64 p + 16 q + 4 (lane >> 4), +4) of row (lane & 15)
    float sc[8];
};

template <bool B64, bool NESTED, bool STEADY>
__device__ __forceinline__ void prepare_phase(const MatmulArgs& a, PhaseRegs& r, int lane, PhaseOperands& o) {
    const bool b0 = lane & 1, b1 = lane & 2;
    float* sc = o.sc;
    if (NESTED && B64) {
        const uint32_t q0 = __float_as_uint(r.s[0].x), q1 = __float_as_uint(r.s[0].y);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const uint32_t code = ((j < 4 ? q0 : q1) >> (8 * (j & 3))) & 0xffu;
            sc[j] = __fadd_rn(__fmul_rn(a.nested.map256[code], r.s[0].z), a.nested.offset);
        }
    } else {
        const float in[8] = {r.s[0].x, r.s[0].y, r.s[0].z, r.s[0].w, r.s[1].x, r.s[1].y, r.s[1].z, r.s[1].w};
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            // STEADY: real moves.  The compiler would rename registers instead and then rotate the
            // slot's registers at the back edge of the steady loop, which needs the data of the
            // load just issued and so waits for it.
            if (STEADY)
                asm volatile("v_mov_b32 %0, %1" : "=v"(sc[j]) : "v"(in[j]));
            else
                sc[j] = in[j];
        }
    }

    // in-quad transpose, one dword column at a time: load index <-> lane & 3
    transpose_quad(r.w[0].x, r.w[1].x, r.w[2].x, r.w[3].x, b0, b1);
    transpose_quad(r.w[0].y, r.w[1].y, r.w[2].y, r.w[3].y, b0, b1);
    transpose_quad(r.w[0].z, r.w[1].z, r.w[2].z, r.w[3].z, b0, b1);
    transpose_quad(r.w[0].w, r.w[1].w, r.w[2].w, r.w[3].w, b0, b1);
    // now w[q] = bytes [64 * (lane >> 4) + 16 * q, +16) of row (lane & 15)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        o.d[q][0] = r.w[q].x; o.d[q][1] = r.w[q].y; o.d[q][2] = r.w[q].z; o.d[q][3] = r.w[q].w;
        transpose_g(o.d[q]);
    }
}

// MFMA j = 4p + q of the phase covers k [32j, 32j + 32) and uses d[q][p].
// EXACT (K > 8192): fp32 table, every weight rounded as bf16(lut * absmax) before the MFMA -- the
// reference's dequantisation bit for bit -- and the MFMAs accumulate straight into acc.
template <int R, int MODE>
__device__ __forceinline__ void contract_phase(const PhaseOperands& o, const uint8_t* xph, int lane, f32x4& acc) {
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    constexpr bool EXACT = MODE == ARITH_EXACT, F16 = MODE == ARITH_F16;
    const uint32_t lane4 = (uint32_t)lane * 4u;
    const uint32_t lane8 = (uint32_t)(lane & 31) * 8u;
    const int gg = lane >> 4, m = lane & 15;
    const uint32_t xoff_even = (uint32_t)(gg * R + ((m ^ gg) & (R - 1))) * 16u;
    const uint32_t xoff_odd = (uint32_t)(gg * R + ((m ^ (4 | gg)) & (R - 1))) * 16u;

    // The 16 MFMAs of a phase in the order s = 0..15: p = s >> 2, then the two blocks of p interleaved
    // (block h = s & 1, MFMA qq = (s >> 1) & 1 of the block), so that consecutive MFMAs never depend on
    // each other.  Operands are fetched from LDS one MFMA ahead of their use.
    struct Ops {
        uint32_t t[4];
        float2 tf[4];
        uint4 xa;
    };
    auto fetch = [&](int s, Ops& f) __attribute__((always_inline)) {
        const int p = s >> 2, h = s & 1, qq = (s >> 1) & 1;
        const int q = 2 * h + qq;
        const int j = 4 * p + q;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const uint32_t sel = 0x0c0c0400u | ((uint32_t)b << 8);
            if (EXACT)
                f.tf[b] = lds_table_read2(__builtin_amdgcn_perm(o.d[q][p], lane8, sel));
            else
                f.t[b] = lds_table_read(__builtin_amdgcn_perm(o.d[q][p], lane4, sel));
        }
        f.xa = *reinterpret_cast<const uint4*>(xph + j * (64 * R) + (qq ? xoff_odd : xoff_even));
    };
    constexpr int AHEAD = 1;  // MFMAs between the fetch of an operand set and its use
    Ops ops[AHEAD + 1];
#pragma unroll
    for (int s = 0; s < AHEAD; ++s) fetch(s, ops[s]);
    f32x4 blk[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
#pragma unroll
    for (int s = 0; s < 16; ++s) {
        if (s + AHEAD < 16) fetch(s + AHEAD, ops[(s + AHEAD) % (AHEAD + 1)]);
        const int p = s >> 2, h = s & 1, qq = (s >> 1) & 1;
        const float scale = o.sc[2 * p + h];
        Ops& f = ops[s % (AHEAD + 1)];
        if (EXACT) {
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                const f32x2_t v = {__fmul_rn(f.tf[b].x, scale), __fmul_rn(f.tf[b].y, scale)};
                f.t[b] = __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
            }
        }
        const uint4 wb = make_uint4(f.t[0], f.t[1], f.t[2], f.t[3]);
        if (EXACT) {
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, f.xa), __builtin_bit_cast(bf16x8, wb),
                                                          acc, 0, 0, 0);
        } else {
            const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
            if (F16)
                blk[h] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, f.xa),
                                                                __builtin_bit_cast(f16x8, wb), qq ? blk[h] : zero, 0, 0, 0);
            else
                blk[h] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, f.xa),
                                                                 __builtin_bit_cast(bf16x8, wb), qq ? blk[h] : zero, 0, 0, 0);
            // the block of the PREVIOUS pair that just completed is scaled here, one MFMA later
            if (qq == 1 && h == 1) {
#pragma unroll
                for (int hh = 0; hh < 2; ++hh) {
                    const float sc = o.sc[2 * p + hh];
#pragma unroll
                    for (int i = 0; i < 4; ++i) acc[i] = fmaf(sc, blk[hh][i], acc[i]);
                }
            }
        }
    }
}

// Staging of one slice of x.  One (row, phase) of x = 64 pieces of 16 bytes = 1 KB contiguous,
// handled by one wave: wave w takes rows w and w + 8 (the latter only exists in the 16-row layout),
// all phases of the slice, i.e. at most ten units.  All loads are issued before the first LDS
// write.
constexpr int XUNITS = XBYTES_MAX / 1024 / WAVES;  // units per wave: 10 in both layouts

template <int R>
__device__ __forceinline__ void load_x_slice(const MatmulArgs& a, uint4 (&v)[XUNITS], int k0, int n, int lane, int wave) {
    constexpr int CAP = XBYTES_MAX / (R * 1024);
#pragma unroll
    for (int u = 0; u < XUNITS; ++u) {
        // outside the slice or the matrix: re-read a valid unit, the value is dropped
        const int m = min(wave + 8 * (u / CAP), a.M - 1);
        const int pp = min(u % CAP, n - 1);
        v[u] = load16(a.x + (int64_t)m * a.K + k0 + pp * PHASE_K + lane * 8);
    }
}

template <int R>
__device__ __forceinline__ void store_x_slice(const MatmulArgs& a, const uint4 (&v)[XUNITS], uint8_t* xlds, int n,
                                              int lane, int wave) {
    constexpr int CAP = XBYTES_MAX / (R * 1024);
#pragma unroll
    for (int u = 0; u < XUNITS; ++u) {
        const int m = wave + 8 * (u / CAP), ph = u % CAP;
        if (m < a.M && ph < n) *reinterpret_cast<uint4*>(xlds + ph * (R * 1024) + xslot_bytes<R>(m, lane)) = v[u];
    }
}

// fp16 mode (the launcher picks it only when the workgroup's K range is ONE slice, so that a row of x keeps one scale
// for everything its accumulators see): a wave holds whole rows of the slice -- row `wave` in units [0, CAP), row
// wave + 8 in units [CAP, 2 CAP) -- finds each row's largest |x|, scales the row into fp16's range by a power of two
// (f16_scale_for), converts it, and leaves what undoes the scaling in `unscale[row]` for the end of the batch.
template <int R>
__device__ __forceinline__ void scale_x_slice_to_f16(uint4 (&v)[XUNITS], int n, uint8_t* unscale, int lane, int wave) {
    constexpr int CAP = XBYTES_MAX / (R * 1024);
#pragma unroll
    for (int rg = 0; rg < XUNITS / CAP; ++rg) {
        u16x2_t mx = {0, 0};
#pragma unroll
        for (int pp = 0; pp < CAP; ++pp) {
            const uint4& w = v[rg * CAP + pp];
            if (pp < n) {  // units beyond the slice hold a re-read valid unit: harmless, but keep the maximum the slice's own
                mx = absmax_of_bf16_pair(w.x, mx); mx = absmax_of_bf16_pair(w.y, mx);
                mx = absmax_of_bf16_pair(w.z, mx); mx = absmax_of_bf16_pair(w.w, mx);
            }
        }
        uint32_t m = absmax_bits(mx);
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) m = max(m, (uint32_t)__shfl_xor((int)m, off));
        const F16Scale fs = f16_scale_for(m);
#pragma unroll
        for (int pp = 0; pp < CAP; ++pp) {
            uint4& w = v[rg * CAP + pp];
            w.x = bf16_pair_to_f16(w.x, fs.to_f16); w.y = bf16_pair_to_f16(w.y, fs.to_f16);
            w.z = bf16_pair_to_f16(w.z, fs.to_f16); w.w = bf16_pair_to_f16(w.w, fs.to_f16);
        }
        if (lane == 0) reinterpret_cast<float*>(unscale)[wave + 8 * rg] = fs.from_f16;
    }
}

// STEADY (long work lists): the slots are refilled without branches and groups of four entries that
// follow each other without a restage or a batch end run in an inner loop that holds nothing else.
// The compiler can then count the loads in flight and waits for ONE slot where it otherwise waits for
// everything in flight at the top of every group (loads under branches, and the stores of a batch
// end, which complete out of order with loads).  The price is a drain when that loop is entered and
// switched-off requests at the end of the list, which short lists cannot afford.
// EPI (Epilogue flags; fp32 absmax, blocksize 64): what the lane that finishes an output does with it -- at the end of
// a batch, or in the wave that reduces a tile when K is split over workgroups.  A tile is 16 weight rows: the two
// rows of a (gate, up) pair sit in neighbouring lanes, and EPI_RESID_NORM leaves one partial sum of squares per tile
// (added over the tile's 16 lanes by a butterfly), so what a partial sum holds does not depend on which workgroup
// finished the tile.
template <bool B64, bool NESTED, int R, int MODE, bool STEADY, int EPI = EPI_NONE>
__global__ __launch_bounds__(THREADS, 2) void gemv_tiles_kernel(NF4_HOT_PARAMS, int hot_splits, int hot_range_phases, int hot_tg_step,
                                                                MatmulArgs a_rest) {
    // (arguments in SGPRs at wave start; the struct supplies what is wanted later)
    const MatmulArgs a = with_hot_args<NESTED>(a_rest, NF4_HOT_NAMES);
    Plan p;
    p.tile_groups = (a.N + 16 * WAVES - 1) / (16 * WAVES);
    p.total_phases = a.K / PHASE_K;
    p.splits = hot_splits; p.range_phases = hot_range_phases; p.tg_step = hot_tg_step;
    static_assert(EPI == EPI_NONE || (B64 && !NESTED), "epilogues: fp32 absmax, blocksize 64");
    constexpr bool EXACT = MODE == ARITH_EXACT, F16 = MODE == ARITH_F16;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    constexpr int CAP = XBYTES_MAX / (R * 1024);  // phases of x that fit
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col = lane & 15, g = lane >> 4;

    const float lut_lane = a.lut16[lane & 15];

    // this workgroup's K range and tile groups
    const int ks = (int)blockIdx.x % p.splits;
    ListShape ls;
    ls.tg0 = (int)blockIdx.x / p.splits;
    ls.tg_step = p.tg_step;
    ls.r0 = ks * p.range_phases;                             // first phase of the range

    LaneLoad ll;
    {
        // rows of a tile are read from n0c = max(min(n0, N - 16), 0) on, so only N < 16 needs a clamp
        const uint32_t lane_bytes = (uint32_t)(lane >> 4) * 64u + (uint32_t)(lane & 3) * 16u;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            ll.woff[i] = (uint32_t)min(((lane >> 2) & 3) * 4 + i, a.N - 1) * (uint32_t)(a.K >> 1) + lane_bytes;
        ll.s_off = (uint32_t)min(col, a.N - 1) * (uint32_t)(a.K >> a.block_log2);
    }
    auto first_row = [&](int tg) {  // first row read for the wave's tile of a tile group
        const int n0 = (tg * WAVES + wave) * 16;
        return max(min(n0, a.N - 16), 0);
    };
    const Item* items = reinterpret_cast<const Item*>(smem + ITEMS_OFFSET);
    auto read_item = [&](int i) {  // wave-uniform LDS read, moved to scalar registers
        const int4 v = *reinterpret_cast<const int4*>(items + i);
        Item it;
        it.tg = __builtin_amdgcn_readfirstlane(v.x);
        it.kabs = __builtin_amdgcn_readfirstlane(v.y);
        it.info = __builtin_amdgcn_readfirstlane(v.z);
        it.k0 = __builtin_amdgcn_readfirstlane(v.w);
        return it;
    };

    PhaseRegs ring[SLOTS];

    // Prologue.  Loads return in issue order, so x (slice 0 of the range) is requested BEFORE the
    // ring is filled: its latency is then that of an idle memory system.  The work list is written
    // next (one entry per thread), and the ring is filled from it while the table is built.
    ls.rph = min(p.range_phases, p.total_phases - ls.r0);    // phases in the range
    ls.nsl = (ls.rph + CAP - 1) / CAP;                       // x slices in the range
    ls.last = ls.rph - (ls.nsl - 1) * CAP;                   // phases of the last slice
    ls.G = ls.tg0 < p.tile_groups ? (p.tile_groups - 1 - ls.tg0) / p.tg_step + 1 : 0;
    ls.nitems = list_length<CAP>(ls.G, ls.nsl, ls.last);
    const int cn = ls.nitems;  // <= ITEMS_MAX, guaranteed by the launcher
    float* sumsq_s = reinterpret_cast<float*>(smem + SUMSQ_OFFSET);
    {
        // EPI_ROWSCALE: this thread's share of the producer's partial sums of squares, the first requests of all
        // (wave w adds up rows w and w + 8 of x: in_parts <= 512 values each, eight per lane)
        float ssp[R / 8][8];
        if (EPI & EPI_ROWSCALE) {
#pragma unroll
            for (int h = 0; h < R / 8; ++h)
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const int m = wave + 8 * h;
                    ssp[h][j] = (m < a.M && lane + 64 * j < a.epi.in_parts) ? a.epi.in_sumsq[m * a.epi.in_parts + lane + 64 * j] : 0.0f;
                }
        }
        uint4 xv[XUNITS];
        const int nph0 = ls.nsl == 1 ? ls.last : CAP;
        load_x_slice<R>(a, xv, ls.r0 * PHASE_K, nph0, lane, wave);
        if (tid < cn) {
            const Item it = make_item<CAP>(ls, tid);
            reinterpret_cast<int4*>(smem + ITEMS_OFFSET)[tid] = make_int4(it.tg, it.kabs, it.info, it.k0);
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < SLOTS; ++j) {
            if constexpr (STEADY) {
                const Item it = read_item(j);
                const bool on = j < cn && !(it.info & ITEM_GAP);
                load_phase<B64, NESTED>(a, ring[j], ll, first_row(on ? it.tg : ls.tg0),
                                        on ? it.kabs : ls.r0 * PHASE_K, on ? 0xffffffffu : 0u);
            } else if (j < cn) {
                const Item it = read_item(j);
                if (!(it.info & ITEM_GAP)) load_phase<B64, NESTED>(a, ring[j], ll, first_row(it.tg), it.kabs);
            }
        }
        if (EXACT)
            build_pair_table_f32(smem, lut_lane, lane, wave);
        else
            build_pair_table<F16>(smem, lut_lane, lane, wave);
        if (F16) scale_x_slice_to_f16<R>(xv, nph0, smem + UNSCALE_OFFSET, lane, wave);
        store_x_slice<R>(a, xv, smem + TABLE_BYTES, nph0, lane, wave);
        if (EPI & EPI_ROWSCALE) {
#pragma unroll
            for (int h = 0; h < R / 8; ++h) {
                const float* v = ssp[h];
                float ss = ((v[0] + v[1]) + (v[2] + v[3])) + ((v[4] + v[5]) + (v[6] + v[7]));
#pragma unroll
                for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
                if (lane == 0) sumsq_s[wave + 8 * h] = ss;  // rows of x beyond M: 0
            }
        }
        __syncthreads();
    }
    // 1 / rms of row m of x (EPI_ROWSCALE)
    auto rstd_of = [&](int m) { return rsqrtf(sumsq_s[m] / (float)a.K + a.epi.eps); };
    const int ntiles = (a.N + 15) / 16;  // EPI_RESID_NORM: partial sums per row of x
    // The lane's finished sums of one tile: v[j] belongs to row m_of(j) of x and weight row n (valid: the lane owns a
    // row of the matrix here).  Every lane of the wave takes part (the pair exchange and the butterfly need them all).
    auto emit = [&](const float* v, int cnt, auto m_of, int n, bool valid, int tile) {
        const float b = (a.bias && valid) ? bf16_bits_to_f32(a.bias[n]) : 0.0f;
        for (int j = 0; j < cnt; ++j) {
            const int m = m_of(j);
            const bool on = valid && m < a.M;
            float val = v[j];
            if (EPI & EPI_ROWSCALE) val *= rstd_of(min(m, R - 1));
            val += b;
            if (EPI & EPI_SILU_PAIRS) {
                // the lane of the odd row hands its value to the lane of the even row (N is even, tiles start on even rows)
                const float mine = nf4x::round_bf16(val);
                const float other = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, mine), 0xB1, 0xf, 0xf, true));
                if (on && !(n & 1)) a.out[(int64_t)m * (a.N / 2) + n / 2] = (uint16_t)nf4x::silu_mul_bf16(mine, other);
            } else if (EPI & EPI_RESID_NORM) {
                float sq = 0.0f;
                if (on) {
                    const int64_t at = (int64_t)m * a.N + n;
                    const float res = nf4x::resid_add(bf16_bits_to_f32(a.epi.resid_in[at]), nf4x::round_bf16(val));
                    a.epi.resid_out[at] = (uint16_t)f32_to_bf16_bits(res);
                    a.epi.xnext_out[at] = (uint16_t)f32_to_bf16_bits(res * bf16_bits_to_f32(a.epi.norm_weight[n]));
                    sq = res * res;
                }
#pragma unroll
                for (int o = 8; o > 0; o >>= 1) sq += __shfl_xor(sq, o, 64);  // the 16 rows of the tile
                if (col == 0 && m < a.M && tile < ntiles) a.epi.out_sumsq[m * ntiles + tile] = sq;
            } else if (on) {
                a.out[(int64_t)m * a.N + n] = (uint16_t)f32_to_bf16_bits(val);
            }
        }
    };

    unsigned* counters = reinterpret_cast<unsigned*>(a.workspace);
    float* partial = reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(a.workspace) + COUNTER_BYTES);

    f32x4 acc[SLOTS];
#pragma unroll
    for (int j = 0; j < SLOTS; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};

    {
        for (int base = 0; base < cn; base += SLOTS) {
            int end_info = 0, end_tg = 0;
            {
                // a new slice always starts at slot 0
                const Item it0 = read_item(base);
                if (it0.info & ITEM_RESTAGE) {
                    uint4 xv[XUNITS];
                    const int n = (it0.info >> ITEM_NPH_SHIFT) & 0xf;
                    load_x_slice<R>(a, xv, it0.k0, n, lane, wave);
                    __syncthreads();  // every wave is done with the slice that was resident
                    store_x_slice<R>(a, xv, smem + TABLE_BYTES, n, lane, wave);
                    __syncthreads();
                }
            }
            if constexpr (STEADY) {
                __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the steady loop is entered with nothing in flight
                for (;;) {
#pragma unroll
                    for (int j = 0; j < SLOTS; ++j) {
                        const Item it = read_item(base + j);
                        const Item nx = read_item(min(base + j + SLOTS, cn - 1));
                        const bool refill = base + j + SLOTS < cn && !(nx.info & ITEM_GAP);
                        // codes out of the slot, the slot refilled at once, both without a branch (a
                        // gap's operands are not used)
                        PhaseOperands o;
                        prepare_phase<B64, NESTED, true>(a, ring[j], lane, o);
                        load_phase<B64, NESTED>(a, ring[j], ll, first_row(refill ? nx.tg : ls.tg0),
                                                refill ? nx.kabs : ls.r0 * PHASE_K, refill ? 0xffffffffu : 0u);
                        if (!(it.info & ITEM_GAP)) {
                            contract_phase<R, MODE>(o, smem + TABLE_BYTES + (it.info & ITEM_PHS_MASK) * (R * 1024), lane,
                                                     acc[j]);
                            if (it.info & ITEM_END) {
                                end_info = it.info;
                                end_tg = it.tg;
                            }
                        }
                    }
                    if ((end_info & ITEM_END) || base + SLOTS >= cn) break;
                    if (read_item(base + SLOTS).info & ITEM_RESTAGE) break;
                    base += SLOTS;
                }
            } else {
#pragma unroll
            for (int j = 0; j < SLOTS; ++j) {
                const Item it = read_item(base + j);
                Item nx;
                nx.info = ITEM_GAP;
                if (base + j + SLOTS < cn) nx = read_item(base + j + SLOTS);
                if (!(it.info & ITEM_GAP)) {
                    PhaseOperands o;
                    prepare_phase<B64, NESTED, false>(a, ring[j], lane, o);
                    // the slot's registers are free again: refill before the long part of the work
                    if (!(nx.info & ITEM_GAP)) load_phase<B64, NESTED>(a, ring[j], ll, first_row(nx.tg), nx.kabs);
                    contract_phase<R, MODE>(o, smem + TABLE_BYTES + (it.info & ITEM_PHS_MASK) * (R * 1024), lane, acc[j]);
                    if (it.info & ITEM_END) {
                        end_info = it.info;
                        end_tg = it.tg;
                    }
                } else if (!(nx.info & ITEM_GAP)) {
                    load_phase<B64, NESTED>(a, ring[j], ll, first_row(nx.tg), nx.kabs);
                }
            }
            }
            if (!(end_info & ITEM_END)) continue;
            const int fin_nb = (end_info >> ITEM_NB_SHIFT) & 7;
            const int fin_tg0 = end_tg - (fin_nb - 1) * ls.tg_step;  // the batch's first tile group

        // ---- end of a batch: slot j holds tile group j % nb; lane holds out[m = 4g + i][row] ----
        if (fin_nb == 1) {
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[0][i] = (acc[0][i] + acc[1][i]) + (acc[2][i] + acc[3][i]);
        } else if (fin_nb == 2) {
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[0][i] += acc[2][i], acc[1][i] += acc[3][i];
        }
        if (F16) {  // back from the per-row scaling of x (rows 4 g .. 4 g + 3 are this lane's)
            const float4 us = *reinterpret_cast<const float4*>(smem + UNSCALE_OFFSET + 16 * g);
#pragma unroll
            for (int t = 0; t < SLOTS; ++t) {
                acc[t][0] *= us.x; acc[t][1] *= us.y; acc[t][2] *= us.z; acc[t][3] *= us.w;
            }
        }
#pragma unroll
        for (int t = 0; t < SLOTS; ++t) {
            if (t < fin_nb) {
                const int tile = (fin_tg0 + t * ls.tg_step) * WAVES + wave;
                const int n0 = tile * 16;
                const int n = max(min(n0, a.N - 16), 0) + col;  // the lane's row
                const bool mine = n >= n0 && n < a.N;
                if (p.splits == 1) {
                    const float v4[4] = {acc[t][0], acc[t][1], acc[t][2], acc[t][3]};
                    emit(v4, 4, [&](int i) { return 4 * g + i; }, n, mine, tile);
                } else if (n0 < a.N) {
                    // Partial sums cross workgroups (and XCDs, whose L2s are not coherent with each
                    // other) through agent-scope relaxed atomics only: such stores write through
                    // and such loads bypass stale lines, so no L2-wide write-back/invalidate is
                    // needed.  Ordering: a tile belongs to ONE wave per K range, so the hand-off is per
                    // wave: every store of the wave has completed (publish_partials) before the wave bumps
                    // the tile's counter; the wave that finds splits - 1 there reduces.
                    if (mine) {
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const int m = 4 * g + i;
                            if (m < a.M)
                                __hip_atomic_store(&partial[((int64_t)ks * a.M + m) * a.N + n], acc[t][i],
                                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        }
                    }
                    publish_partials();
                    unsigned prev = 0;
                    if (lane == 0)
                        prev = __hip_atomic_fetch_add(&counters[tile], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    prev = __builtin_amdgcn_readfirstlane(prev);
                    acquire_partials();
                    if (prev == (unsigned)p.splits - 1u) {
                        // the lane's R / 4 outputs of the 16 x M tile; the loads of eight slices of all
                        // of them are in flight together, the adds run in slice order
                        constexpr int OUTS = R / 4;
                        const int nn = n0 + col;
                        const float* p0[OUTS];
                        float sum[OUTS];
#pragma unroll
                        for (int o = 0; o < OUTS; ++o) {
                            const int m = min(g + 4 * o, a.M - 1);
                            p0[o] = &partial[(int64_t)m * a.N + min(nn, a.N - 1)];
                            sum[o] = 0.0f;
                        }
                        const int64_t stride = (int64_t)a.M * a.N;
                        for (int k2 = 0; k2 < p.splits; k2 += 8) {
                            float v[OUTS][8];
#pragma unroll
                            for (int j = 0; j < 8; ++j) {
                                const int64_t off = (int64_t)min(k2 + j, p.splits - 1) * stride;
#pragma unroll
                                for (int o = 0; o < OUTS; ++o)
                                    v[o][j] = __hip_atomic_load(p0[o] + off, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            }
#pragma unroll
                            for (int j = 0; j < 8; ++j)
#pragma unroll
                                for (int o = 0; o < OUTS; ++o) sum[o] += k2 + j < p.splits ? v[o][j] : 0.0f;
                        }
                        emit(sum, OUTS, [&](int o) { return g + 4 * o; }, min(nn, a.N - 1), nn < a.N, tile);
                        if (lane == 0)
                            __hip_atomic_store(&counters[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
                }
            }
                acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
        }
    }
}

constexpr int rows_held(int64_t M) {
    return M <= 8 ? 8 : 16;
}

// Work split.  K is split into ranges over workgroups only to fill the chip: the number of ranges
// minimises rounds x (phases per range + fixed cost) on a device of NOMINAL_SLOTS CUs, one
// workgroup per CU, where a split adds the partial sums' round trip to the fixed cost.  The choice
// does not depend on the device at hand, so that the workspace size is a function of the shape
// alone; the grid does (correctness never depends on how many workgroups are resident).
constexpr int NOMINAL_SLOTS = 256;

// Work lists at least this long run the STEADY variant of the kernel (measured: it gains 3-8 % from 16
// entries on and costs up to 2 us on lists of four).
constexpr int STEADY_MIN_ITEMS = 16;

int grid_for(int64_t ntasks, int splits, int slots) {
    int grid = (int)(ntasks < slots ? ntasks : slots);
    grid -= grid % splits;
    return grid < splits ? splits : grid;
}

Plan make_plan(int64_t M, int64_t N, int64_t K) {
    Plan p;
    p.tile_groups = (int)((N + 16 * WAVES - 1) / (16 * WAVES));
    p.total_phases = (int)(K / PHASE_K);
    const int cap = XBYTES_MAX / (rows_held(M) * 1024);
    double best_cost = 1e30;
    int best_rp = p.total_phases;
    for (int rp = p.total_phases; rp >= 1; --rp) {
        const int splits = (p.total_phases + rp - 1) / rp;
        if ((p.total_phases + splits - 1) / splits != rp) continue;  // same split, shorter last range
        if (splits > 1 && (int64_t)p.tile_groups * WAVES > COUNTER_BYTES / 4) break;
        const int64_t ntasks = (int64_t)p.tile_groups * splits;
        const int grid = grid_for(ntasks, splits, NOMINAL_SLOTS);
        const int64_t rounds = (ntasks + grid - 1) / grid;
        const int restages = (rp + cap - 1) / cap;
        const double fixed = 1.0 + 0.5 * restages + (splits > 1 ? (double)M / 18.0 + 1.0 : 0.0);
        const double cost = (double)rounds * (rp + fixed);
        if (cost < best_cost - 1e-9) best_cost = cost, best_rp = rp;
    }
    p.range_phases = best_rp;
    p.splits = (p.total_phases + best_rp - 1) / best_rp;
    p.tg_step = 0;  // set with the grid
    return p;
}

}  // namespace

size_t gemv_tiles_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    if (M <= 0 || N <= 0 || K <= 0 || K % PHASE_K) return COUNTER_BYTES;
    const Plan p = make_plan(M, N, K);
    return (size_t)COUNTER_BYTES + (p.splits > 1 ? (size_t)p.splits * (size_t)M * (size_t)N * sizeof(float) : 0);
}

template <bool B64, bool NESTED, bool STEADY>
hipError_t allow_rx() {
    hipError_t e;
    if ((e = gemv_allow_lds(gemv_tiles_kernel<B64, NESTED, 8, ARITH_BF16, STEADY>, SMEM_BYTES)) != hipSuccess) return e;
    if ((e = gemv_allow_lds(gemv_tiles_kernel<B64, NESTED, 16, ARITH_BF16, STEADY>, SMEM_BYTES)) != hipSuccess) return e;
    if ((e = gemv_allow_lds(gemv_tiles_kernel<B64, NESTED, 8, ARITH_F16, STEADY>, SMEM_BYTES)) != hipSuccess) return e;
    if ((e = gemv_allow_lds(gemv_tiles_kernel<B64, NESTED, 16, ARITH_F16, STEADY>, SMEM_BYTES)) != hipSuccess) return e;
    if ((e = gemv_allow_lds(gemv_tiles_kernel<B64, NESTED, 8, ARITH_EXACT, STEADY>, SMEM_BYTES)) != hipSuccess) return e;
    return gemv_allow_lds(gemv_tiles_kernel<B64, NESTED, 16, ARITH_EXACT, STEADY>, SMEM_BYTES);
}

template <bool B64, bool NESTED>
hipError_t allow_both() {
    const hipError_t e = allow_rx<B64, NESTED, false>();
    return e != hipSuccess ? e : allow_rx<B64, NESTED, true>();
}

template <int EPI, bool STEADY>
hipError_t allow_epi() {
    hipError_t e;
    if ((e = gemv_allow_lds(gemv_tiles_kernel<true, false, 8, ARITH_BF16, STEADY, EPI>, SMEM_BYTES)) != hipSuccess) return e;
    if ((e = gemv_allow_lds(gemv_tiles_kernel<true, false, 16, ARITH_BF16, STEADY, EPI>, SMEM_BYTES)) != hipSuccess) return e;
    if ((e = gemv_allow_lds(gemv_tiles_kernel<true, false, 8, ARITH_F16, STEADY, EPI>, SMEM_BYTES)) != hipSuccess) return e;
    if ((e = gemv_allow_lds(gemv_tiles_kernel<true, false, 16, ARITH_F16, STEADY, EPI>, SMEM_BYTES)) != hipSuccess) return e;
    if ((e = gemv_allow_lds(gemv_tiles_kernel<true, false, 8, ARITH_EXACT, STEADY, EPI>, SMEM_BYTES)) != hipSuccess) return e;
    return gemv_allow_lds(gemv_tiles_kernel<true, false, 16, ARITH_EXACT, STEADY, EPI>, SMEM_BYTES);
}

hipError_t gemv_tiles_setup() {
    hipError_t e;
    if ((e = allow_both<false, false>()) != hipSuccess) return e;
    if ((e = allow_both<true, false>()) != hipSuccess) return e;
    if ((e = allow_both<false, true>()) != hipSuccess) return e;
    if ((e = allow_both<true, true>()) != hipSuccess) return e;
    if ((e = allow_epi<EPI_ROWSCALE, false>()) != hipSuccess || (e = allow_epi<EPI_ROWSCALE, true>()) != hipSuccess) return e;
    if ((e = allow_epi<EPI_ROWSCALE | EPI_SILU_PAIRS, false>()) != hipSuccess) return e;
    if ((e = allow_epi<EPI_ROWSCALE | EPI_SILU_PAIRS, true>()) != hipSuccess) return e;
    if ((e = allow_epi<EPI_SILU_PAIRS, false>()) != hipSuccess || (e = allow_epi<EPI_SILU_PAIRS, true>()) != hipSuccess) return e;
    if ((e = allow_epi<EPI_RESID_NORM, false>()) != hipSuccess) return e;
    return allow_epi<EPI_RESID_NORM, true>();
}

template <int R, int MODE, bool STEADY>
hipError_t launch_rs(const MatmulArgs& a, const Plan& p, int grid, hipStream_t stream) {
    const bool b64 = a.block_log2 == 6;
    const bool nested = a.nested.q != nullptr;
    auto kern = b64 ? (nested ? gemv_tiles_kernel<true, true, R, MODE, STEADY> : gemv_tiles_kernel<true, false, R, MODE, STEADY>)
                    : (nested ? gemv_tiles_kernel<false, true, R, MODE, STEADY>
                              : gemv_tiles_kernel<false, false, R, MODE, STEADY>);
    switch (a.epi.flags) {  // epilogues: fp32 absmax and blocksize 64 (gemv_tiles_epilogue_possible)
        case EPI_NONE: break;
        case EPI_ROWSCALE: kern = gemv_tiles_kernel<true, false, R, MODE, STEADY, EPI_ROWSCALE>; break;
        case EPI_ROWSCALE | EPI_SILU_PAIRS: kern = gemv_tiles_kernel<true, false, R, MODE, STEADY, EPI_ROWSCALE | EPI_SILU_PAIRS>; break;
        case EPI_SILU_PAIRS: kern = gemv_tiles_kernel<true, false, R, MODE, STEADY, EPI_SILU_PAIRS>; break;
        case EPI_RESID_NORM: kern = gemv_tiles_kernel<true, false, R, MODE, STEADY, EPI_RESID_NORM>; break;
        default: return hipErrorNotSupported;
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(THREADS), SMEM_BYTES, stream, NF4_HOT_VALUES(a), p.splits, p.range_phases, p.tg_step, a);
    return hipGetLastError();
}

template <int R, int MODE>
hipError_t launch_r(const MatmulArgs& a, const Plan& p, int grid, bool steady, hipStream_t stream) {
    return steady ? launch_rs<R, MODE, true>(a, p, grid, stream) : launch_rs<R, MODE, false>(a, p, grid, stream);
}

template <int MODE>
hipError_t launch_m(const MatmulArgs& a, const Plan& p, int grid, bool steady, hipStream_t stream) {
    return rows_held(a.M) == 8 ? launch_r<8, MODE>(a, p, grid, steady, stream) : launch_r<16, MODE>(a, p, grid, steady, stream);
}

// epilogues of the tile kernel: fp32 absmax, blocksize 64; (gate, up) pairs need an even N; the producer's partial
// sums one per thread; a partial sum of squares per tile of 16 weight rows, at most one per thread of the consumer
bool gemv_tiles_epilogue_possible(const MatmulArgs& a) {
    if (a.epi.flags == EPI_NONE) return true;
    if (a.nested.q || a.block_log2 != 6) return false;
    if ((a.epi.flags & EPI_ROWSCALE) && a.epi.in_parts > THREADS) return false;
    if ((a.epi.flags & EPI_RESID_NORM) && gemv_tiles_norm_parts(a.N) == 0) return false;
    return !(a.epi.flags & EPI_SILU_PAIRS) || a.N % 2 == 0;
}

int gemv_tiles_norm_parts(int64_t N) {
    const int64_t tiles = (N + 15) / 16;
    return tiles <= THREADS ? (int)tiles : 0;
}

hipError_t launch_gemv_tiles(const MatmulArgs& a, int cus, hipStream_t stream) {
    if (!gemv_tiles_epilogue_possible(a)) return hipErrorNotSupported;
    Plan p = make_plan(a.M, a.N, a.K);
    const int grid = grid_for((int64_t)p.tile_groups * p.splits, p.splits, cus < 1024 ? cus : 1024);
    p.tg_step = grid / p.splits;
    // the longest work list of a workgroup (the one that owns the most tile groups and a full K range)
    // must fit in LDS
    const int cap = XBYTES_MAX / (rows_held(a.M) * 1024);
    const int G = (p.tile_groups + p.tg_step - 1) / p.tg_step;
    const int nsl = (p.range_phases + cap - 1) / cap;
    const int last = p.range_phases - (nsl - 1) * cap;
    const int n = rows_held(a.M) == 8 ? list_length<10>(G, nsl, last) : list_length<5>(G, nsl, last);
    if (n > ITEMS_MAX) return hipErrorInvalidValue;
    const bool steady = n >= STEADY_MIN_ITEMS;
    // fp16 arithmetic needs one scale per row of x for everything an accumulator sees: only when the workgroup's K
    // range is a single slice of x (otherwise the exact variant serves 8192 < K <= 16384 too)
    const int mode = gemv_arith_mode(a.K, nsl == 1);
    if (mode == ARITH_EXACT) return launch_m<ARITH_EXACT>(a, p, grid, steady, stream);
    if (mode == ARITH_F16) return launch_m<ARITH_F16>(a, p, grid, steady, stream);
    return launch_m<ARITH_BF16>(a, p, grid, steady, stream);
}

}  // namespace nf4
