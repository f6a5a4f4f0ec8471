// Decode-shape fused NF4 dequant-matmul for gfx950, 1 <= M <= 16 rows of x, blocksize 64, fp32 absmax, K a multiple
// of 256: codes AND absmax are staged through LDS by LDS-direct loads, so that every byte of the weight stream is
// requested in whole 128-byte lines, no register holds data in flight, and the layout the MFMA wants costs nothing.
//
// Replaces bitsandbytes' gemv_4bit (kgemm_4bit_inference_naive) / small-batch matmul_4bit, call site
// thunder/transforms/quantization.py:39.
//
// HBM-bound: 0.5 byte of codes + 1/16 byte of absmax per weight, each read exactly once.
//
//  * One workgroup of 16 waves per CU.  Wave w owns k slice w of the workgroup's K range: 256 consecutive k =
//    128 bytes of codes (one cache line) and 16 bytes of absmax (four blocks) of every weight row.  Its slice of x
//    (16 rows x 256 k) sits in 32 registers as the A operands of eight v_mfma_f32_16x16x32_bf16 for the whole kernel.
//    A workgroup streams a contiguous range of weight rows, 16 at a time (a tile).
//  * Codes.  buffer_load_dwordx4 ... lds: one instruction moves 8 rows x 128 bytes (eight whole lines) from HBM into
//    a wave-private ring of five 1 KB slots (two of them feed the tile being multiplied, three are in flight).  The
//    16-byte pieces of a line are stored XOR-swizzled by row, so that the MFMA-order reads below are conflict-free.
//  * absmax.  The 16 rows x 16 waves x 16 bytes a tile needs are contiguous per row (256 bytes); wave r fetches row r
//    with one 16-lane LDS-direct load two tiles ahead, into one of three 4 KB buffers, pieces XOR-swizzled by row;
//    every wave then reads its four block scales of a row with one conflict-free ds_read_b128.
//  * Into MFMA order for free.  Lane (n = lane & 15, g = lane >> 4) supplies the B operand of weight row n.  For
//    block b of the slice it reads 8 bytes -- half (g & 1) of 16-byte piece 2b + (g >> 1) -- whose two dwords feed the
//    two MFMAs of the block; the A operands were loaded from x in the same k order, so no transposes are needed, and
//    the two MFMAs of a block cover exactly its 64 k: the block sum is scaled by absmax afterwards (4 FMAs).
//  * Code -> bf16.  256-entry byte -> (bf16, bf16) LDS table replicated for 32 lane columns with a 256-byte stride
//    (address = (byte << 8) | column * 4: one v_perm_b32); the unused second half of every 256-byte row holds the
//    buffers of the cross-wave reduction.
//  * Reduction.  The sixteen waves hold sixteen partial 16 x 16 tiles (one per k slice).  They go to LDS (double
//    buffered, one barrier per tile); wave m adds the sixteen partials of row m of x in a fixed order, adds the bias,
//    rounds and stores 16 consecutive outputs -- one tile late: it asks for the partials of tile t - 1 at the top of
//    tile t and adds them up at its end, so that the reads' latency hides behind the tile's own work.
//  * K > 4096 is split over workgroups (each keeps its slice of x): the sums of a K range go to the workspace as they
//    are finished (agent-scope stores, nothing waits for them); after its last tile a workgroup counts its arrival
//    (one counter per row range), and the last of a row range's workgroups adds the ranges in order and stores.
//
//  * Epilogues (K not split): wave m may scale its finished sums of row m by 1 / rms (EPI_ROWSCALE: the producer's
//    partial sums of squares are added up once per workgroup, by wave m for its row, while the first weights are on their
//    way) and merge (gate, up) pairs of outputs into SiLU(gate) * up (EPI_SILU_PAIRS: the odd row's lane hands its value
//    to the even row's lane), with the roundings of the two-step route.
//
// What keeps the waits exact: every wave issues the same sequence of vector memory operations per tile (one absmax
// load, then two code loads at the end), also where a load is not needed (rows are clamped into the workgroup's
// range), so the hand-counted s_waitcnt vmcnt(n) below always name the same operations.
#include "decode_math.h"
#include "nf4_gemv.h"

namespace nf4 {
namespace {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;
typedef __attribute__((address_space(3))) void* lds_void_ptr;

constexpr int ST_WAVES = 16;
constexpr int ST_THREADS = ST_WAVES * 64;
constexpr int SLICE_K = 256;                 // k per wave
constexpr int SLOT_BYTES = 1024;             // one LDS-direct load: 8 rows x 128 B
constexpr int RING_SLOTS = 5;
constexpr int TABLE_SPAN = 256 * 256;        // table rows of 256 B: first half table, second half reduction buffers
constexpr int RING_OFF = TABLE_SPAN;
constexpr int ABS_OFF = RING_OFF + ST_WAVES * RING_SLOTS * SLOT_BYTES;
constexpr int ABS_BYTES = 16 * ST_WAVES * 16;  // 16 rows x 16 waves x 16 B
constexpr int ABS_BUFS = 3;
// bias of the workgroup's rows (bf16), fetched once: a load into a register inside the tile loop would have the compiler
// wait for every load of the ring behind it
constexpr int BIAS_OFF = ABS_OFF + ABS_BUFS * ABS_BYTES;
constexpr int BIAS_ROWS = 1024;
// EPI_RESID_NORM while one workgroup covers K: the residual of the workgroup's outputs (M rows of x times its weight rows)
// and the norm weight of its rows, bf16, fetched once like the bias: at most RESID_SLOTS values, (M + 1) * rows
constexpr int RESID_OFF = BIAS_OFF + BIAS_ROWS * 2;
constexpr int RESID_SLOTS = 1024;
constexpr int RESID_MAX_ROWS = 128;  // (one 4-byte-per-lane request of a wave covers a row of x: 64 lanes x 2 values)
constexpr int ST_SMEM_BYTES = RESID_OFF + RESID_SLOTS * 2;  // 64 + 80 + 12 + 2 + 2 = 160 KB
// nested absmax: the same 12 KB hold three buffers of 8-bit absmax codes (16 rows x 64 bytes, rows 80 bytes apart so that
// the sixteen rows a wave reads spread over the banks), the 256-entry map and the second-level absmax of the workgroup's
// blocks
constexpr int ABSQ_ROW = 80;
constexpr int ABSQ_BYTES = 16 * ABSQ_ROW;
constexpr int MAP_OFF = ABS_OFF + ABS_BUFS * ABSQ_BYTES;
constexpr int AM2_OFF = MAP_OFF + 256 * 4;
constexpr int AM2_MAX = 1024;  // second-level absmax values one workgroup may need
static_assert(AM2_OFF + AM2_MAX * 4 <= BIAS_OFF, "the nested tables live where the fp32 absmax buffers are");
constexpr int RED_BUF_BYTES = ST_WAVES * 1024;                 // per buffer: 16 rows of x, a plane of 16 waves x 16 weight rows x 4 B each
static_assert(2 * RED_BUF_BYTES <= TABLE_SPAN / 2, "reduction buffers live in the table's unused half rows");
static_assert(ST_SMEM_BYTES <= 160 * 1024, "LDS of one CU");

struct StagePlan {
    int rows_per_wg;    // weight rows of one workgroup (a multiple of 8)
    int wgs_per_split;  // workgroups that share one K range
    int splits;         // K ranges
    int slices_per_split;  // 256-k slices of one K range (<= 16); the last range may hold fewer
};

// byte offset in LDS of byte `o` of the reduction buffers: the second half of the table's 256-byte rows
__device__ __forceinline__ uint32_t red_addr(uint32_t o) { return ((o >> 7) << 8) | 0x80u | (o & 127u); }

__device__ __forceinline__ uint32_t lds_read_u32(uint32_t addr) {
    typedef __attribute__((address_space(3))) const uint32_t* p_t;
    return *reinterpret_cast<p_t>((uintptr_t)addr);
}
__device__ __forceinline__ uint32_t lds_read_u16(uint32_t addr) {
    typedef __attribute__((address_space(3))) const uint16_t* p_t;
    return *reinterpret_cast<p_t>((uintptr_t)addr);
}
__device__ __forceinline__ float lds_read_f32(uint32_t addr) {
    typedef __attribute__((address_space(3))) const float* p_t;
    return *reinterpret_cast<p_t>((uintptr_t)addr);
}
__device__ __forceinline__ uint2 lds_read_u32x2(uint32_t addr) {
    typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
    typedef __attribute__((address_space(3))) const u32x2_t* p_t;
    const u32x2_t v = *reinterpret_cast<p_t>((uintptr_t)addr);
    return make_uint2(v.x, v.y);
}
__device__ __forceinline__ float4 lds_read_f32x4(uint32_t addr) {
    typedef float f32x4_t __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) const f32x4_t* p_t;
    const f32x4_t v = *reinterpret_cast<p_t>((uintptr_t)addr);
    return make_float4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void lds_write_f32(uint32_t addr, float v) {
    typedef __attribute__((address_space(3))) float* p_t;
    *reinterpret_cast<p_t>((uintptr_t)addr) = v;
}
__device__ __forceinline__ void lds_write_f32x4(uint32_t addr, f32x4 v) {
    typedef float f32x4_t __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) f32x4_t* p_t;
    const f32x4_t w = {v[0], v[1], v[2], v[3]};
    *reinterpret_cast<p_t>((uintptr_t)addr) = w;
}

// wait until at most N of this wave's vector memory operations are outstanding (they complete in order)
template <int N>
__device__ __forceinline__ void wait_vm() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
__device__ __forceinline__ void wait_lds() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

// 4 bytes per active lane from a buffer straight into LDS at lds_base + lane * 4
__device__ __forceinline__ void dma4(__amdgpu_buffer_rsrc_t rsrc, uint32_t lds_base, uint32_t lane_offset, uint32_t wave_offset) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_void_ptr)(uintptr_t)lds_base, 4, lane_offset, wave_offset, 0, 2 /* nt */);
}

// 16 bytes per active lane from a buffer straight into LDS at lds_base + lane * 16 (nontemporal); the byte offset is a
// per-lane part that never changes (a register) plus a wave-uniform part (a scalar register: no vector arithmetic
// per load)
__device__ __forceinline__ void dma16(__amdgpu_buffer_rsrc_t rsrc, uint32_t lds_base, uint32_t lane_offset, uint32_t wave_offset) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_void_ptr)(uintptr_t)lds_base, 16, lane_offset, wave_offset, 0, 2 /* nt */);
}

// float -> bf16 bits, round to nearest even (v_cvt_pk_bf16_f32)
__device__ __forceinline__ uint32_t bf16_bits_hw(float f) {
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    const f32x2_t v = {f, f};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t)) & 0xffffu;
}

// MGROUPS: lane groups of four rows of x that carry rows < M: ceil(M / 4).  EPI: the epilogue flags of the call.
// F16 (8192 < K <= 16384, where sums of bf16 code-book values drift past the matmul's tolerance): the table holds the
// code book rounded to fp16, and the wave's slice of x is converted to fp16 once, every row scaled by a power of two
// that puts its largest value of the slice just below 2^15 (exact for bf16 inputs); a wave's sums are scaled back before
// they leave for the reduction.
// NESTED: absmax arrives as 8-bit codes (one byte per block, a quarter of the bytes) and is reconstructed per lane and
// tile as map[code] * absmax2[block / nested blocksize] + offset, each rounded once, like everywhere else.
template <int MGROUPS, int EPI, bool F16 = false, bool NESTED = false>
__global__ __launch_bounds__(ST_THREADS, 1) void gemv_stage_kernel(NF4_HOT_PARAMS, int hot_rows_per_wg, int hot_wgs_per_split,
                                                                     int hot_splits_slices, MatmulArgs a_rest) {
#if defined(__HIP_DEVICE_COMPILE__)
    const MatmulArgs a = with_hot_args<NESTED>(a_rest, NF4_HOT_NAMES);
    const int splits = hot_splits_slices & 0xffff, slices_per_split = hot_splits_slices >> 16;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15, g = lane >> 4;
    const int M = a.M, N = a.N, K = a.K;
    const int row_bytes = K >> 1;

    // this workgroup's K range and rows
    const int split = (int)blockIdx.x % splits;
    const int part = (int)blockIdx.x / splits;
    const int r0 = part * hot_rows_per_wg;
    const int r1 = min(N, r0 + hot_rows_per_wg);
    const int rmax = r1 - 1;                       // rows beyond the range are clamped to its last row
    const int halves = (r1 - r0 + 7) >> 3;         // 8-row loads
    const int tiles = (halves + 1) >> 1;
    const int total_slices = K / SLICE_K;
    const int slice0 = split * slices_per_split;
    const int nslices = min(slices_per_split, total_slices - slice0);  // k slices of this range
    const bool wave_on = wave < nslices;
    const int slice = slice0 + (wave_on ? wave : 0);  // (a wave without a slice runs on slice 0 and contributes zeros)

    const __amdgpu_buffer_rsrc_t codes_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(a.packed), 0, (int)(uint32_t)((int64_t)N * row_bytes), 0x00020000);
    const __amdgpu_buffer_rsrc_t abs_rsrc =
        NESTED ? __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(a.nested.q), 0, (int)(uint32_t)((int64_t)N * (K >> 6)), 0x00020000)
               : __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(a.absmax), 0, (int)(uint32_t)((int64_t)N * (K >> 6) * 4), 0x00020000);

    // bias of this workgroup's rows into LDS, 128 rows per wave: the oldest request of the wave, so no count below
    // changes with it (reads past the end of the bias return zeros; those rows are never stored).  Where K is split
    // the workgroup that adds the ranges reads the bias from memory after its last tile.
    const bool bias_staged = a.bias && splits == 1;
    if (bias_staged && wave * 128 < r1 - r0) {
        const __amdgpu_buffer_rsrc_t bias_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(a.bias), 0, (int)(2 * N), 0x00020000);
        dma4(bias_rsrc, BIAS_OFF + wave * 256, (uint32_t)(r0 + wave * 128) * 2u + (uint32_t)lane * 4u, 0);
    }
    // EPI_ROWSCALE: wave m's share of the partial sums of squares of row m of x (at most 512: eight per lane), all
    // requested here and added up after the first barrier (a loop that adds as it loads waits for a round trip per
    // 64 partial sums before the wave's first weight request: 1.8 us of a launch whose producer had 512 workgroups)
    float ssp[8];
    if (EPI & EPI_ROWSCALE) {
#pragma unroll
        for (int j = 0; j < 8; ++j)
            ssp[j] = (wave < M && lane + 64 * j < a.epi.in_parts) ? a.epi.in_sumsq[wave * a.epi.in_parts + lane + 64 * j] : 0.0f;
    }
    // EPI_RESID_NORM with one K range: wave m fetches the residual of row m of x for the workgroup's rows, wave 0 the
    // norm weight of those rows as well (row M of the staging area); rows past the tensors read as zeros or as the
    // next row's values and are never stored
    const int rpw = hot_rows_per_wg;
    const bool resid_staged = (EPI & EPI_RESID_NORM) && splits == 1;
    if (resid_staged) {
        const uint32_t lane2 = (uint32_t)lane * 4u;
        if (wave < M && 2 * lane < rpw) {
            const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(a.epi.resid_in), 0, (int)(2 * M * N), 0x00020000);
            dma4(rs, RESID_OFF + wave * rpw * 2, (uint32_t)(wave * N + r0) * 2u + lane2, 0);
        }
        if (wave == 0 && 2 * lane < rpw) {
            const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(a.epi.norm_weight), 0, (int)(2 * N), 0x00020000);
            dma4(rs, RESID_OFF + M * rpw * 2, (uint32_t)r0 * 2u + lane2, 0);
        }
    }
    // the two code-book values of this thread's table entry (entry tid >> 2): requested next, so that waiting for them
    // later waits for nothing that is requested after them
    const float lut_hi = a.lut16[tid >> 6], lut_lo = a.lut16[(tid >> 2) & 15];
    // nested absmax: this thread's entry of the map and of the workgroup's second-level absmax (blocks of the rows r0 ..
    // r1 - 1 in this K range are consecutive per row; their second-level indices run from am2_first on)
    const int kblocks = K >> 6;
    const int am2_first = NESTED ? (int)(((int64_t)r0 * kblocks + slice0 * 4) >> a.nested.nested_log2) : 0;
    float map_mine = 0.0f, am2_mine = 0.0f;
    if (NESTED) {
        const int am2_last = (int)(((int64_t)rmax * kblocks + (slice0 + nslices) * 4 - 1) >> a.nested.nested_log2);
        if (tid < 256) map_mine = a.nested.map256[tid];
        if (tid <= am2_last - am2_first) am2_mine = a.nested.absmax2[am2_first + tid];
    }
    asm volatile("" ::: "memory");

    // ---- x: the A operands of the wave's eight MFMAs, loaded once -------------------------------------------------
    // MFMA (b, h) of block b covers k = slice * 256 + 64 b + 16 g' + 8 h + [0, 8) over the four lane groups g'
    bf16x8 xa[4][2];
    {
        const uint16_t* xrow = a.x + (int64_t)min(n, M - 1) * K + slice * SLICE_K + 16 * g;
#pragma unroll
        for (int b = 0; b < 4; ++b)
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const uint4 v = load16(xrow + 64 * b + 8 * h);
                xa[b][h] = __builtin_bit_cast(bf16x8, v);
            }
    }

    // ---- load side: lane constants ----------------------------------------------------------------------------------
    // code loads: lane i takes row (i >> 3) of the 8-row half tile and the 16-byte piece (i & 7) ^ f(row in tile),
    // f(n) = n >> 1 (rows 0..7: the even half tile; rows 8..15: the odd one)
    // The lane's share of the offset is fixed for the whole launch; which half tile is a wave-uniform offset.  A half
    // tile beyond the workgroup's range is replaced by its last one (rows of a workgroup come in whole half tiles, so
    // nothing outside the weight is ever addressed).
    const int lrow = lane >> 3;
    const uint32_t ccol = (uint32_t)lrow * (uint32_t)row_bytes + (uint32_t)slice * 128u;
    const uint32_t clane_even = ccol + ((uint32_t)((lane & 7) ^ (lrow >> 1)) << 4);
    const uint32_t clane_odd = ccol + ((uint32_t)((lane & 7) ^ (4 + (lrow >> 1))) << 4);
    const uint32_t ring = RING_OFF + wave * (RING_SLOTS * SLOT_BYTES);
    auto load_codes = [&](int h, bool odd, int slot) {  // half tile h of this workgroup into ring slot `slot` (odd = h & 1)
        const uint32_t base = (uint32_t)(r0 + 8 * min(h, halves - 1)) * (uint32_t)row_bytes;
        dma16(codes_rsrc, ring + slot * SLOT_BYTES, odd ? clane_odd : clane_even, base);
    };
    // absmax loads: wave r fetches row r of a tile, lanes 0..15 the pieces of the range's k slices; lane q stores
    // piece q ^ r at position q (readers of slice w look at position w ^ row)
    const uint32_t abs_row_bytes = (uint32_t)(K >> 6) * 4u;
    const int apiece = (lane & 15) ^ wave;
    const bool abs_lane = lane < 16 && apiece < nslices;
    const uint32_t alane = (uint32_t)(slice0 + apiece) * 16u;
    // (nested: lane i fetches the four code bytes of slice i of the row, 64 consecutive bytes in all)
    const bool absq_lane = lane < nslices;
    const uint32_t aqlane = (uint32_t)(slice0 + lane) * 4u;
    auto load_absmax = [&](int t) {
        const int row = min(r0 + 16 * t + wave, rmax);
        if (NESTED) {
            if (absq_lane) dma4(abs_rsrc, ABS_OFF + (t % ABS_BUFS) * ABSQ_BYTES + wave * ABSQ_ROW, aqlane, (uint32_t)row * (uint32_t)kblocks);
        } else {
            if (abs_lane) dma16(abs_rsrc, ABS_OFF + (t % ABS_BUFS) * ABS_BYTES + wave * 256, alane, (uint32_t)row * abs_row_bytes);
        }
    };

    // ---- get the stream going: absmax of tiles 0 and 1, the first five half tiles -----------------------------------
    load_absmax(0);
    load_absmax(1);
#pragma unroll
    for (int h = 0; h < RING_SLOTS; ++h) load_codes(h, h & 1, h);

    // ---- byte -> (bf16, bf16) table: entry e = tid >> 2, 32 bytes per thread -----------------------------------------
    {
        const uint32_t vb = F16 ? (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)lut_hi) | ((uint32_t)__builtin_bit_cast(uint16_t, (_Float16)lut_lo) << 16)
                                : f32_to_bf16_bits(lut_hi) | (f32_to_bf16_bits(lut_lo) << 16);
        const float v = __uint_as_float(vb);
        const uint32_t dst = (uint32_t)(tid >> 2) * 256u + (uint32_t)(tid & 3) * 32u;  // (the table starts at LDS address 0)
        lds_write_f32x4(dst, f32x4{v, v, v, v});
        lds_write_f32x4(dst + 16, f32x4{v, v, v, v});
    }
    // a wave without a slice contributes zeros to every sum: written once, into both reduction buffers
    // Reduction buffers: the sum of wave w for (row m of x, weight row n) is dword (16 w + n) ^ (16 * ((m >> 2) & 1)) of
    // plane m (1 KB).  Only the 32 banks of the table rows' second halves are there to be used; with this order both
    // the writers (lane (n, g): m = 4g .. 4g + 3, a plane each) and the readers (lane (n, G): waves G, G + 4, G + 8,
    // G + 12 of one plane) put two lanes on a bank, the least possible.  Planes are 2 KB of LDS addresses apart, the
    // four waves a reader adds 512 bytes.
    constexpr uint32_t RED_PLANE = (1024u >> 7) << 8;
    const uint32_t red_w0 = red_addr((uint32_t)(4 * g) * 1024u + (uint32_t)((16 * wave + n) ^ ((g & 1) << 4)) * 4u);
    auto write_partials = [&](uint32_t at, const f32x4& v) {
#pragma unroll
        for (int i = 0; i < 4; ++i) lds_write_f32(at + (uint32_t)i * RED_PLANE, v[i]);
    };
    if (!wave_on && g < MGROUPS) {
        write_partials(red_w0, f32x4{0.f, 0.f, 0.f, 0.f});
        write_partials(red_w0 + ((RED_BUF_BYTES >> 7) << 8), f32x4{0.f, 0.f, 0.f, 0.f});
    }
    wait_vm<RING_SLOTS>();  // everything older than the five code loads: x, code book, absmax of tiles 0 and 1
    if (NESTED) {
        if (tid < 256) lds_write_f32(MAP_OFF + tid * 4, map_mine);
        lds_write_f32(AM2_OFF + tid * 4, am2_mine);
    }
    // (x is in its registers from here on: said once, so that the loop does not carry waits for it)
#pragma unroll
    for (int b = 0; b < 4; ++b) asm volatile("" ::"v"(xa[b][0]), "v"(xa[b][1]));
    // fp16 arithmetic: the lane's 64 values of row n of x -> fp16, scaled by what the row's largest value in this slice
    // (over the four lane groups) allows; unscale[i] undoes it for output row 4g + i of this lane's sums
    float unscale[4] = {1.0f, 1.0f, 1.0f, 1.0f};
    if constexpr (F16) {
        u16x2_t mx = {0, 0};
#pragma unroll
        for (int b = 0; b < 4; ++b)
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const uint4 v = __builtin_bit_cast(uint4, xa[b][h]);
                mx = absmax_of_bf16_pair(v.x, mx);
                mx = absmax_of_bf16_pair(v.y, mx);
                mx = absmax_of_bf16_pair(v.z, mx);
                mx = absmax_of_bf16_pair(v.w, mx);
            }
        uint32_t mb = absmax_bits(mx);
        mb = max(mb, (uint32_t)__shfl_xor((int)mb, 16, 64));
        mb = max(mb, (uint32_t)__shfl_xor((int)mb, 32, 64));
        const F16Scale fs = f16_scale_for(mb);
#pragma unroll
        for (int b = 0; b < 4; ++b)
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                uint4 v = __builtin_bit_cast(uint4, xa[b][h]);
                v.x = bf16_pair_to_f16(v.x, fs.to_f16);
                v.y = bf16_pair_to_f16(v.y, fs.to_f16);
                v.z = bf16_pair_to_f16(v.z, fs.to_f16);
                v.w = bf16_pair_to_f16(v.w, fs.to_f16);
                xa[b][h] = __builtin_bit_cast(bf16x8, v);
            }
#pragma unroll
        for (int i = 0; i < 4; ++i) unscale[i] = __shfl(fs.from_f16, 4 * g + i, 64);
    }
    wait_lds();
    __builtin_amdgcn_s_barrier();

    float rstd = 1.0f;  // EPI_ROWSCALE: 1 / rms of row `wave` of the producer's residual stream
    if (EPI & EPI_ROWSCALE) {
        float ssq = ssp[0];  // (sums of squares: 0 + ssp[0] has the same bits, and no addition is left where the load is)
#pragma unroll
        for (int j = 1; j < 8; ++j) ssq += ssp[j];
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) ssq += __shfl_xor(ssq, o, 64);
        rstd = rsqrtf(ssq / (float)K + a.epi.eps);
    }

    // ---- read side: lane constants ------------------------------------------------------------------------------------
    const uint32_t col4 = (uint32_t)(lane & 31) * 4u;
    const int f = n >> 1;
    // codes of block b: 8 bytes at piece (2b + (g >> 1)) ^ f, half (g & 1), of row n & 7 of the even (n < 8) / odd half
    // tile.  The odd half tile's slot follows the even one's, except where the ring wraps (slots 4 and 0): one address
    // per block for either case, the slot itself is a constant offset of the read.
    uint32_t cread[4], cread_wrap[4];
    {
        const uint32_t c0 = ring + (uint32_t)(n & 7) * 128u + ((uint32_t)((g >> 1) ^ f) << 4) + (uint32_t)(g & 1) * 8u;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            cread[b] = (c0 ^ (uint32_t)(b << 5)) + (n < 8 ? 0u : (uint32_t)SLOT_BYTES);
            cread_wrap[b] = (c0 ^ (uint32_t)(b << 5)) + (n < 8 ? (uint32_t)((RING_SLOTS - 1) * SLOT_BYTES) : 0u);
        }
    }
    const uint32_t aread = NESTED ? ABS_OFF + (uint32_t)n * ABSQ_ROW + (uint32_t)(wave_on ? wave : 0) * 4u
                                  : ABS_OFF + (uint32_t)(n * 16 + ((wave_on ? wave : 0) ^ n)) * 16u;
    // nested: the lane's first block of tile 0 (its four blocks never straddle a nested block: both start at multiples of 4)
    const uint32_t blk0 = (uint32_t)(r0 + n) * (uint32_t)kblocks + (uint32_t)slice * 4u;
    const bool reducer = wave < M;  // wave m finishes row m of x
    unsigned* counters = reinterpret_cast<unsigned*>(a.workspace);
    float* partial = reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(a.workspace) + GEMV_COUNTER_BYTES);

    // The two reduction buffers are 32 KB of LDS addresses apart: a wave's write address and a finishing wave's read
    // address change buffers by flipping that bit.  Tile t is written into buffer t & 1.
    constexpr uint32_t RED_FLIP = (RED_BUF_BYTES >> 7) << 8;
    uint32_t red_w = red_w0;
    // Finishing a tile (wave m, row m of x): lane (n, G = g) reads the partial sums of waves G, G + 4, G + 8, G + 12 ...
    uint32_t red_r = red_addr((uint32_t)wave * 1024u + (uint32_t)((16 * g + n) ^ (((wave >> 2) & 1) << 4)) * 4u);
    struct Pending {
        float p[4];
        uint32_t bias;         // of row r0 + 16 t + n, bf16 bits
        uint32_t resid, normw;  // EPI_RESID_NORM, one K range: residual of (row m of x, that row) and the row's norm weight
    };
    uint32_t bias_r = BIAS_OFF + (uint32_t)n * 2u;
    uint32_t resid_r = RESID_OFF + (uint32_t)(min(wave, M - 1) * rpw + n) * 2u;
    uint32_t normw_r = RESID_OFF + (uint32_t)(M * rpw + n) * 2u;
    auto read_partials = [&]() {  // of the oldest tile not yet finished
        Pending pd;
#pragma unroll
        for (int q = 0; q < 4; ++q) pd.p[q] = lds_read_f32(red_r + (uint32_t)q * 512u);
        red_r ^= RED_FLIP;
        pd.bias = 0;
        if (bias_staged) {
            pd.bias = lds_read_u16(bias_r);
            bias_r += 32;
        }
        pd.resid = pd.normw = 0;
        if (resid_staged) {
            pd.resid = lds_read_u16(resid_r);
            pd.normw = lds_read_u16(normw_r);
            resid_r += 32;
            normw_r += 32;
        }
        return pd;
    };
    // where row r0 + n of this workgroup sits in row m of the output, in bytes; stores go through a buffer that ends
    // with the workgroup's last row, so that the rows of a last, half-filled tile are dropped by the range check
    const uint32_t out_lane = (uint32_t)(r0 + n) * 2u;
    const bool pairs = (EPI & EPI_SILU_PAIRS) != 0;
    const __amdgpu_buffer_rsrc_t out_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        a.out + (int64_t)(reducer ? wave : 0) * (pairs ? (N >> 1) : N), 0, pairs ? r1 : 2 * r1, 0x00020000);
    // (EPI_RESID_NORM, one K range: the two tensors the epilogue stores instead of `out`, same rows, same range check)
    const __amdgpu_buffer_rsrc_t resid_out_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        ((EPI & EPI_RESID_NORM) ? a.epi.resid_out : a.out) + (int64_t)(reducer ? wave : 0) * N, 0, 2 * r1, 0x00020000);
    const __amdgpu_buffer_rsrc_t xnext_out_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        ((EPI & EPI_RESID_NORM) ? a.epi.xnext_out : a.out) + (int64_t)(reducer ? wave : 0) * N, 0, 2 * r1, 0x00020000);
    float resid_ss = 0.0f;  // sum of squares of the new residual over this lane's rows (lanes 0..15 of wave m: row m of x)
    // ... adds them in that order, then the four lane groups (two register swaps across the wave: no LDS round trip),
    // and stores the 16 outputs
    auto finish_tile = [&](int t, const Pending& pd) {
        const int m = wave;
        float sum = ((pd.p[0] + pd.p[1]) + pd.p[2]) + pd.p[3];
        {
            const uint32_t v = __float_as_uint(sum);
            const auto r = __builtin_amdgcn_permlane16_swap(v, v, false, false);  // rows 1, 3 of the first <-> rows 0, 2 of the second
            sum = __uint_as_float(r[0]) + __uint_as_float(r[1]);               // lanes l and l ^ 16
            const uint32_t w = __float_as_uint(sum);
            const auto r2 = __builtin_amdgcn_permlane32_swap(w, w, false, false);
            sum = __uint_as_float(r2[0]) + __uint_as_float(r2[1]);             // lanes l and l ^ 32
        }
        if (splits == 1) {
            const uint32_t at = out_lane + 32u * (uint32_t)t;  // byte offset of row r0 + 16 t + n
            if (EPI & EPI_ROWSCALE) sum *= rstd;
            if (a.bias) sum += bf16_bits_to_f32((uint16_t)pd.bias);
            if (EPI & EPI_RESID_NORM) {
                // d = bf16(sum + bias); r = bf16(resid + d) -> resid_out; bf16(r * w_next) -> xnext_out; r^2 into the
                // workgroup's share of row m's sum of squares
                const float d = nf4x::round_bf16(sum);
                const float res = nf4x::resid_add(bf16_bits_to_f32(pd.resid), d);
                if (g == 0) {
                    __builtin_amdgcn_raw_buffer_store_b16((short)f32_to_bf16_bits(res), resid_out_rsrc, at, 0, 0);
                    __builtin_amdgcn_raw_buffer_store_b16((short)f32_to_bf16_bits(res * bf16_bits_to_f32(pd.normw)), xnext_out_rsrc, at, 0, 0);
                    if (r0 + 16 * t + n < r1) resid_ss = fmaf(res, res, resid_ss);
                }
            } else
            if (EPI & EPI_SILU_PAIRS) {
                // rows 2j, 2j + 1 = gate j, up j: the even row's lane takes the odd row's value (lane ^ 1)
                const float mine = nf4x::round_bf16(sum);
                const float other = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, mine), 0xB1, 0xf, 0xf, true));
                if (g == 0 && !(n & 1))
                    __builtin_amdgcn_raw_buffer_store_b16((short)nf4x::silu_mul_bf16(mine, other), out_rsrc, at >> 1, 0, 0);
            } else if (g == 0) {
                __builtin_amdgcn_raw_buffer_store_b16((short)bf16_bits_hw(sum), out_rsrc, at, 0, 0);
            }
        } else {
            // K split over workgroups: this wave's 16 sums of (tile, m) go to the workspace (a store that is visible to
            // every workgroup once acknowledged); the ranges meet after the last tile
            const int row = r0 + 16 * t + n;
            if (g == 0 && row < r1)
                __hip_atomic_store(&partial[((int64_t)split * M + m) * N + row], sum, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    };

    // two blocks of the slice, their MFMAs interleaved (independent accumulators), scaled into acc
    auto two_blocks = [&](const uint2& ca, const uint2& cb, const bf16x8 (&xa0)[2], const bf16x8 (&xa1)[2], float sa, float sb,
                          f32x4& acc) {
        f32x4 c0 = {0.f, 0.f, 0.f, 0.f}, c1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const uint32_t d0 = h ? ca.y : ca.x, d1 = h ? cb.y : cb.x;
            uint32_t w0[4], w1[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t sel = 0x0c0c0400u | ((uint32_t)j << 8);
                w0[j] = lds_read_u32(__builtin_amdgcn_perm(d0, col4, sel));
                w1[j] = lds_read_u32(__builtin_amdgcn_perm(d1, col4, sel));
            }
            const uint4 p0 = make_uint4(w0[0], w0[1], w0[2], w0[3]), p1 = make_uint4(w1[0], w1[1], w1[2], w1[3]);
            if constexpr (F16) {
                c0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, xa0[h]), __builtin_bit_cast(f16x8, p0), c0, 0, 0, 0);
                c1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, xa1[h]), __builtin_bit_cast(f16x8, p1), c1, 0, 0, 0);
            } else {
                c0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa0[h], __builtin_bit_cast(bf16x8, p0), c0, 0, 0, 0);
                c1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa1[h], __builtin_bit_cast(bf16x8, p1), c1, 0, 0, 0);
            }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] = fmaf(c0[i], sa, acc[i]);
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] = fmaf(c1[i], sb, acc[i]);
    };

    auto tile_body = [&](int t, auto s0_tag, auto s1_tag, auto first_tag) {
        constexpr int S0 = decltype(s0_tag)::value, S1 = decltype(s1_tag)::value;
        constexpr bool FIRST = decltype(first_tag)::value;  // tile 0: nothing to finish yet
        static_assert(S1 == (S0 + 1) % RING_SLOTS, "the odd half tile's slot follows the even one's");
        // Codes of this tile have landed.  A wave's LOADS in issue order: absmax 0, 1, half tiles 0..4, then per tile t'
        // absmax t' + 2, half tiles 2t' + 5, 2t' + 6.  The youngest load this tile needs is half tile 2t + 1 (first code
        // load of tile t - 2); younger are the second code load of tile t - 2 and the three loads of tile t - 1: four
        // (three in tile 0).  A finishing wave's stores are counted by the same counter but may complete in any order
        // with respect to loads: the count assumes none is outstanding, which is exact when they have completed and waits
        // for a load or two more than needed when they have not.
        if (FIRST)
            wait_vm<3>();
        else
            wait_vm<4>();

        // this tile's codes and scales into registers, so that their LDS slots can be refilled while the tile is multiplied
        uint2 cd[4];
#pragma unroll
        for (int b = 0; b < 4; ++b) cd[b] = S1 > S0 ? lds_read_u32x2(cread[b] + S0 * SLOT_BYTES) : lds_read_u32x2(cread_wrap[b]);
        float4 am4;
        uint32_t aq4 = 0;
        float am2 = 0.0f;
        if (NESTED) {
            aq4 = lds_read_u32(aread + (t % ABS_BUFS) * ABSQ_BYTES);
            am2 = lds_read_f32(AM2_OFF + ((((blk0 + (uint32_t)t * 16u * (uint32_t)kblocks) >> a.nested.nested_log2) - (uint32_t)am2_first) << 2));
        } else {
            am4 = lds_read_f32x4(aread + (t % ABS_BUFS) * ABS_BYTES);
        }
        // the previous tile's partial sums (all written before the barrier that ended it): requested now, added up
        // between the halves of this tile
        Pending pd;
        if (!FIRST && reducer) pd = read_partials();

        if (NESTED) {
            const float off = a.nested.offset;
            am4.x = __fadd_rn(__fmul_rn(lds_read_f32(MAP_OFF + ((aq4 & 0xffu) << 2)), am2), off);
            am4.y = __fadd_rn(__fmul_rn(lds_read_f32(MAP_OFF + (((aq4 >> 8) & 0xffu) << 2)), am2), off);
            am4.z = __fadd_rn(__fmul_rn(lds_read_f32(MAP_OFF + (((aq4 >> 16) & 0xffu) << 2)), am2), off);
            am4.w = __fadd_rn(__fmul_rn(lds_read_f32(MAP_OFF + ((aq4 >> 24) << 2)), am2), off);
        }
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        two_blocks(cd[0], cd[1], xa[0], xa[1], am4.x, am4.y, acc);

        // Everything this tile reads from its ring slots and its absmax buffer is in registers (LDS reads return in
        // order, the scales were requested last): the slots are refilled while the second half is multiplied.  The
        // absmax request goes into the buffer tile t - 1 used; every wave is past the barrier that ended it.
        asm volatile("" ::"v"(cd[2].x), "v"(cd[3].y), "v"(am4.w));
        load_absmax(t + 2);
        load_codes(2 * t + RING_SLOTS, true, S0);
        load_codes(2 * t + RING_SLOTS + 1, false, S1);

        // the previous tile is finished here, between the two halves, so that its chain of additions, swaps and the
        // store runs in the shadow of the second half's table reads
        if (!FIRST && reducer) finish_tile(t - 1, pd);

        two_blocks(cd[2], cd[3], xa[2], xa[3], am4.z, am4.w, acc);
        if constexpr (F16) {
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[i] *= unscale[i];
        }
        if (g < MGROUPS && wave_on) write_partials(red_w, acc);
        red_w ^= RED_FLIP;

        // absmax of tile t + 1 (requested one tile ago) has landed in every wave before anyone reads it: younger loads are
        // the two code loads of the previous tile and this tile's three
        wait_vm<5>();
        wait_lds();
        __builtin_amdgcn_s_barrier();
    };

    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    using I3 = std::integral_constant<int, 3>;
    using I4 = std::integral_constant<int, 4>;
    tile_body(0, I0{}, I1{}, std::true_type{});
    for (int t = 1; t < tiles; t += RING_SLOTS) {
        tile_body(t, I2{}, I3{}, std::false_type{});
        if (t + 1 < tiles) tile_body(t + 1, I4{}, I0{}, std::false_type{});
        if (t + 2 < tiles) tile_body(t + 2, I1{}, I2{}, std::false_type{});
        if (t + 3 < tiles) tile_body(t + 3, I3{}, I4{}, std::false_type{});
        if (t + 4 < tiles) tile_body(t + 4, I0{}, I1{}, std::false_type{});
    }
    if (reducer) finish_tile(tiles - 1, read_partials());
    if (resid_staged && reducer) {
        // lanes 0..15 hold the rows n, n + 16, ... of the workgroup: added in a fixed order, one slot per workgroup
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) resid_ss += __shfl_xor(resid_ss, o, 64);
        if (lane == 0) a.epi.out_sumsq[wave * hot_wgs_per_split + part] = resid_ss;
    }
    wait_vm<0>();  // loads issued past the end of the range still target this workgroup's LDS
    if (splits > 1) {
        // The workgroups that share these rows (one per K range) count their arrival once all their partial sums have
        // been acknowledged; whichever comes last adds the ranges in order, for every row of x, and stores the outputs.
        // (the flag sits where the absmax buffers were: nothing is in flight towards LDS any more)
        publish_partials();
        __syncthreads();
        if (tid == 0) {
            const unsigned prev = __hip_atomic_fetch_add(&counters[part], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            lds_write_f32(ABS_OFF, prev == (unsigned)splits - 1u ? 1.0f : 0.0f);
        }
        __syncthreads();
        acquire_partials();
        if (lds_read_f32(ABS_OFF) != 0.0f && (EPI & EPI_RESID_NORM)) {
            // wave m takes row m of x: residual add, norm weight, and the sum of squares of the new residual over this
            // workgroup's rows (lanes in a fixed order) as partial sum `part` of the row
            if (reducer) {
                const int m = wave;
                float ss = 0.0f;
                for (int row = r0 + lane; row < r1; row += 64) {
                    float tot = 0.0f;
                    for (int s = 0; s < splits; ++s)
                        tot += __hip_atomic_load(&partial[((int64_t)s * M + m) * N + row], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    if (a.bias) tot += bf16_bits_to_f32(a.bias[row]);
                    const int64_t at = (int64_t)m * N + row;
                    const float d = nf4x::round_bf16(tot);
                    const float res = nf4x::resid_add(bf16_bits_to_f32(a.epi.resid_in[at]), d);
                    a.epi.resid_out[at] = (uint16_t)f32_to_bf16_bits(res);
                    a.epi.xnext_out[at] = (uint16_t)f32_to_bf16_bits(res * bf16_bits_to_f32(a.epi.norm_weight[row]));
                    ss = fmaf(res, res, ss);
                }
#pragma unroll
                for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
                if (lane == 0) a.epi.out_sumsq[m * hot_wgs_per_split + part] = ss;
            }
            if (tid == 0) __hip_atomic_store(&counters[part], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else if (lds_read_f32(ABS_OFF) != 0.0f) {
            const int nrows = r1 - r0;
            for (int idx = tid; idx < nrows * M; idx += ST_THREADS) {
                const int m = idx / nrows, row = r0 + idx - m * nrows;
                float tot = 0.0f;
                for (int s = 0; s < splits; ++s)
                    tot += __hip_atomic_load(&partial[((int64_t)s * M + m) * N + row], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (a.bias) tot += bf16_bits_to_f32(a.bias[row]);
                a.out[(int64_t)m * N + row] = (uint16_t)f32_to_bf16_bits(tot);
            }
            if (tid == 0) __hip_atomic_store(&counters[part], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
#endif
}

int stage_splits(int64_t K) { return (int)((K / SLICE_K + ST_WAVES - 1) / ST_WAVES); }

StagePlan make_stage_plan(int64_t N, int64_t K, int cus) {
    StagePlan p;
    p.splits = stage_splits(K);
    const int total = (int)(K / SLICE_K);
    p.slices_per_split = (total + p.splits - 1) / p.splits;
    int wgs = cus / p.splits;
    if (wgs < 1) wgs = 1;
    // contiguous row ranges in units of 8 rows (one load)
    const int unit = 8;
    int64_t rows = (N + wgs - 1) / wgs;
    rows = (rows + unit - 1) / unit * unit;
    p.rows_per_wg = (int)rows;
    p.wgs_per_split = (int)((N + rows - 1) / rows);
    return p;
}

template <int MG, int EPI, bool F16 = false, bool NESTED = false>
hipError_t launch_mg_epi(const MatmulArgs& a, const StagePlan& p, hipStream_t stream) {
    hipLaunchKernelGGL((gemv_stage_kernel<MG, EPI, F16, NESTED>), dim3((unsigned)(p.wgs_per_split * p.splits)), dim3(ST_THREADS), ST_SMEM_BYTES, stream,
                       NF4_HOT_VALUES(a), p.rows_per_wg, p.wgs_per_split, p.splits | (p.slices_per_split << 16), a);
    return hipGetLastError();
}

template <int MG>
hipError_t launch_mg(const MatmulArgs& a, const StagePlan& p, hipStream_t stream) {
    if (a.nested.q) {
        if (a.epi.flags != EPI_NONE) return hipErrorNotSupported;
        return gemv_arith_mode(a.K, true) == ARITH_F16 ? launch_mg_epi<MG, EPI_NONE, true, true>(a, p, stream)
                                                       : launch_mg_epi<MG, EPI_NONE, false, true>(a, p, stream);
    }
    if (gemv_arith_mode(a.K, true) == ARITH_F16)
        return a.epi.flags == EPI_NONE         ? launch_mg_epi<MG, EPI_NONE, true>(a, p, stream)
               : a.epi.flags == EPI_RESID_NORM ? launch_mg_epi<MG, EPI_RESID_NORM, true>(a, p, stream)
                                               : hipErrorNotSupported;
    switch (a.epi.flags) {
        case EPI_RESID_NORM: return launch_mg_epi<MG, EPI_RESID_NORM>(a, p, stream);
        case EPI_NONE: return launch_mg_epi<MG, EPI_NONE>(a, p, stream);
        case EPI_ROWSCALE: return launch_mg_epi<MG, EPI_ROWSCALE>(a, p, stream);
        case EPI_SILU_PAIRS: return launch_mg_epi<MG, EPI_SILU_PAIRS>(a, p, stream);
        case EPI_ROWSCALE | EPI_SILU_PAIRS: return launch_mg_epi<MG, EPI_ROWSCALE | EPI_SILU_PAIRS>(a, p, stream);
    }
    return hipErrorNotSupported;
}

template <int MG>
hipError_t allow_lds_mg() {
    hipError_t e;
    if ((e = gemv_allow_lds(gemv_stage_kernel<MG, EPI_NONE>, ST_SMEM_BYTES)) != hipSuccess) return e;
    if ((e = gemv_allow_lds(gemv_stage_kernel<MG, EPI_NONE, true>, ST_SMEM_BYTES)) != hipSuccess) return e;
    if ((e = gemv_allow_lds(gemv_stage_kernel<MG, EPI_NONE, false, true>, ST_SMEM_BYTES)) != hipSuccess) return e;
    if ((e = gemv_allow_lds(gemv_stage_kernel<MG, EPI_NONE, true, true>, ST_SMEM_BYTES)) != hipSuccess) return e;
    if ((e = gemv_allow_lds(gemv_stage_kernel<MG, EPI_RESID_NORM, true>, ST_SMEM_BYTES)) != hipSuccess) return e;
    if ((e = gemv_allow_lds(gemv_stage_kernel<MG, EPI_RESID_NORM>, ST_SMEM_BYTES)) != hipSuccess) return e;
    if ((e = gemv_allow_lds(gemv_stage_kernel<MG, EPI_ROWSCALE>, ST_SMEM_BYTES)) != hipSuccess) return e;
    if ((e = gemv_allow_lds(gemv_stage_kernel<MG, EPI_SILU_PAIRS>, ST_SMEM_BYTES)) != hipSuccess) return e;
    return gemv_allow_lds(gemv_stage_kernel<MG, EPI_ROWSCALE | EPI_SILU_PAIRS>, ST_SMEM_BYTES);
}

}  // namespace

// What the kernel takes: fp32 absmax, blocksize 64, K a multiple of 256 up to 16384 (fp16 arithmetic beyond 8192; beyond
// 16384 every weight would have to be rounded like the dequantised one), N a multiple of 8 (loads fetch eight whole rows),
// offsets that fit 32 bits; of the epilogues the row scale (at most 512 partial sums) and the (gate, up) pairs (even N)
// while K is not split over workgroups, the residual step where it is and, with one K range, where a workgroup has
// at most 128 weight rows and (M + 1) times as many values fit the 2 KB they are staged in.
// second-level absmax values a workgroup of the plan may need (nested absmax)
static int64_t stage_am2_count(const MatmulArgs& a, const StagePlan& p) {
    const int64_t blocks = (int64_t)p.rows_per_wg * (a.K >> 6);  // from the first block of its first row to the last of its last
    return (blocks >> a.nested.nested_log2) + 2;
}

bool gemv_stage_possible(const MatmulArgs& a) {
    if (a.block_log2 != 6) return false;
    // nested absmax: plain calls; a lane's four blocks must share one second-level value; the workgroup's values fit
    // their table (judged on the plan for the current device's CUs, 256 where there is none)
    if (a.nested.q && (a.epi.flags != EPI_NONE || a.nested.nested_log2 < 2 || stage_am2_count(a, make_stage_plan(a.N, a.K, gemv_plan_cus())) > AM2_MAX))
        return false;
    if (a.M < 1 || a.M > 16 || a.K % SLICE_K || a.K > 16384 || a.N % 8) return false;
    if ((int64_t)a.N * (a.K >> 1) >= ((int64_t)1 << 31)) return false;
    const int splits = stage_splits(a.K);
    // a bias is staged in LDS by 4-byte loads, BIAS_ROWS rows per workgroup (judged on the same plan)
    if (a.bias && splits == 1 && ((reinterpret_cast<uintptr_t>(a.bias) & 3u) || make_stage_plan(a.N, a.K, gemv_plan_cus()).rows_per_wg > BIAS_ROWS))
        return false;
    if (a.epi.flags == EPI_RESID_NORM) {
        // K split: the workgroup that adds the K ranges does the residual step.  One K range: the finishing waves do,
        // on a residual staged in LDS -- a row of x per request, (M + 1) rows of values in all
        if (splits == 1) {
            const int rows = make_stage_plan(a.N, a.K, gemv_plan_cus()).rows_per_wg;
            if (rows > RESID_MAX_ROWS || (a.M + 1) * rows > RESID_SLOTS) return false;
            if ((reinterpret_cast<uintptr_t>(a.epi.resid_in) | reinterpret_cast<uintptr_t>(a.epi.norm_weight)) & 3u) return false;
        }
    } else if (a.epi.flags != EPI_NONE) {
        if ((a.epi.flags & ~(EPI_ROWSCALE | EPI_SILU_PAIRS)) || splits != 1) return false;
        if ((a.epi.flags & EPI_ROWSCALE) && a.epi.in_parts > 512) return false;
        if ((a.epi.flags & EPI_SILU_PAIRS) && a.N % 2) return false;
    }
    return true;  // (one arrival counter per workgroup row range: at most as many as there are CUs)
}

int gemv_stage_splits(int64_t K) { return stage_splits(K); }

// EPI_RESID_NORM: partial sums of squares per row of x = the row ranges of the plan (0: no residual epilogue for this shape)
int gemv_stage_norm_parts(int64_t M, int64_t N, int64_t K, int cus) {
    if (stage_splits(K) == 1) {
        const int rows = make_stage_plan(N, K, cus).rows_per_wg;
        if (rows > RESID_MAX_ROWS || (M + 1) * rows > RESID_SLOTS) return 0;
    }
    return make_stage_plan(N, K, cus).wgs_per_split;
}

size_t gemv_stage_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    const int s = stage_splits(K);
    return (size_t)GEMV_COUNTER_BYTES + (s > 1 ? (size_t)s * (size_t)M * (size_t)N * sizeof(float) : 0);
}

hipError_t gemv_stage_setup() {
    hipError_t e;
    if ((e = allow_lds_mg<1>()) != hipSuccess) return e;
    if ((e = allow_lds_mg<2>()) != hipSuccess) return e;
    if ((e = allow_lds_mg<3>()) != hipSuccess) return e;
    return allow_lds_mg<4>();
}

hipError_t launch_gemv_stage(const MatmulArgs& a, int cus, hipStream_t stream) {
    if (!gemv_stage_possible(a)) return hipErrorNotSupported;
    const StagePlan p = make_stage_plan(a.N, a.K, cus);
    if (a.nested.q && stage_am2_count(a, p) > AM2_MAX) return hipErrorNotSupported;
    if (a.bias && p.splits == 1 && p.rows_per_wg > BIAS_ROWS) return hipErrorNotSupported;
    if (a.epi.flags == EPI_RESID_NORM && p.splits == 1 && (p.rows_per_wg > RESID_MAX_ROWS || (a.M + 1) * p.rows_per_wg > RESID_SLOTS))
        return hipErrorNotSupported;
    switch ((a.M + 3) / 4) {
        case 1: return launch_mg<1>(a, p, stream);
        case 2: return launch_mg<2>(a, p, stream);
        case 3: return launch_mg<3>(a, p, stream);
        default: return launch_mg<4>(a, p, stream);
    }
}

}  // namespace nf4
