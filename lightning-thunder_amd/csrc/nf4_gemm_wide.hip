// Prefill-shape fused NF4 dequant-matmul for gfx950, more than 128 rows of x.
//
// Replaces the dequantize_4bit + F.linear route of bitsandbytes.matmul_4bit (MatMul4Bit.forward),
// reached from thunder/transforms/quantization.py:39, like gemm_kernel in nf4_gemm.hip: every wave
// expands the NF4 codes it needs to bf16 in registers -- bf16_rne(lut16[code] * absmax), the value
// nf4hip_dequantize produces -- and contracts them with v_mfma_f32_32x32x16_bf16, fp32 accumulation,
// bf16 output.  Tile BM (256 or 128 rows of x) x 256 weight rows x 64 k per workgroup of 8 waves; wave w
// owns weight rows 32 w .. + 31 of the tile against all BM rows of x (BM / 32 accumulators), so every
// weight is expanded exactly once per workgroup and never passes through LDS.
//
// What the kernel is built around, all measured on this part:
//  * A SIMD starts one v_mfma_f32_32x32x16_bf16 every 32 cycles, whichever of its waves issues it; an
//    LDS read issued directly behind an MFMA and a few VALU instructions behind that hide in its
//    shadow, the same instructions in the other order do not.  Inside a 16-k slice every MFMA is
//    therefore followed by the x fragment read of the NEXT slice (into the registers the MFMA just
//    read) and by one eighth of the expansion of the next B fragment (4 v_perm_b32 addresses, 4
//    code-book reads, 4 x (2 multiplies + 1 pack)).
//  * x goes from global memory straight into LDS with buffer loads (buffer_load_dwordx4 ... lds: no
//    registers, no ds_write).  Flat-encoded LDS-direct loads would make the compiler turn every wait
//    of the wave into a wait for everything while one is in flight; buffer loads are counted in
//    order with the regular loads.  A load instruction of a wave fills 1 KB = eight rows of 128
//    bytes; 16-byte pieces are XOR-swizzled inside a row and the rows of odd chunks swap places
//    pairwise, so the sixteen lanes that a 128-bit fragment read serves together hit sixteen
//    different 16-byte bank groups without padding.
//  * Three stages of x (96 KB at BM = 256) next to the 64 KB code book -- all of a CU's LDS -- and
//    three register sets of codes: every global load has two full k steps to arrive.  One barrier per
//    k step, placed before the step's last slice: by then a wave has issued all its fragment reads
//    of the current stage (the last slice's were prefetched) and waits, with a counted s_waitcnt, only
//    for its own x loads of the next stage; after the barrier the current stage is refilled for step
//    kt + 3 and the first fragments of step kt + 1 are prefetched behind the last slice's MFMAs.
//  * The clock under this load sits near 1.65 GHz (2.1 GHz with the matrix pipe alone busy): the part is
//    power-limited here, so instructions saved count even where they would hide behind the MFMAs.
#include "nf4_gemv.h"

#include <type_traits>

namespace nf4 {
namespace {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;
typedef float float2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4v __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void* lds_void_ptr;
typedef const __attribute__((address_space(1))) void* global_void_ptr;

[[maybe_unused]] constexpr int BK = 64;
constexpr int BN = 256;
constexpr int BOOK_BYTES = 256 * 256;  // byte -> (fp32, fp32) of its two codes, 32 copies: 256 B per byte value
constexpr int CHUNK_BYTES = 1024;      // eight 128-byte rows of x

// NG = 32-row groups of weight rows per wave; 1 is what is built (8 waves, two per SIMD, 256 registers each)
template <int BM, int NG>
struct Tile {
    static constexpr int WAVES = BN / (32 * NG);
    static constexpr int THREADS = 64 * WAVES;
    static constexpr int TI = BM / 32;                      // 32-row x tiles (every wave covers all of them)
    static constexpr int NM = TI * NG;                      // MFMAs per wave and 16-k slice
    static constexpr int CHUNKS = BM / 8;                   // 1 KB chunks per stage
    static constexpr int XL = CHUNKS / WAVES;               // LDS-direct loads per wave and k step
    static constexpr int STAGE_BYTES = CHUNKS * CHUNK_BYTES;
    static constexpr int SMEM_BYTES = BOOK_BYTES + 3 * STAGE_BYTES;  // 160 KB at BM = 256: all of a CU's LDS
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

// The pair book sits at LDS offset 0 (the kernel has no static __shared__ data, so its dynamic
// segment starts there): for every byte value (two codes) the two fp32 code-book entries, high nibble
// first, in 32 copies: address = byte << 8 | copy << 3.  A lane uses copy lane % 32, so the 32 lanes
// that the LDS serves together hit 32 different bank pairs whatever their bytes are.  One v_perm_b32
// builds an address: byte 0 from book_lane (= copy << 3 < 256), byte 1 = byte j of the code dword.
__device__ __forceinline__ uint32_t book_address(uint32_t d, uint32_t book_lane, int j) {
    return __builtin_amdgcn_perm(d, book_lane, 0x0c0c0400u | ((uint32_t)j << 8));
}

__device__ __forceinline__ float2_t lds_f32x2(uint32_t addr) {
    return *reinterpret_cast<const __attribute__((address_space(3))) float2_t*>(addr);
}
__device__ __forceinline__ bf16x8 lds_frag(uint32_t addr) {
    return *reinterpret_cast<const __attribute__((address_space(3))) bf16x8*>(addr);
}

__device__ __forceinline__ uint32_t dword_of(const uint4& w, int p) {
    return p == 0 ? w.x : p == 1 ? w.y : p == 2 ? w.z : w.w;
}

// two code-book values -> two bf16 = bf16_rne(value * scale) in one dword
__device__ __forceinline__ uint32_t scale_round_pair(float2_t v, float scale) {
    const float2_t f = {__fmul_rn(v.x, scale), __fmul_rn(v.y, scale)};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2_t));
}

// The expansion of one code dword (8 weights of one row) into an MFMA B fragment, cut into eight
// micro-steps so that it can be spread over the MFMAs of the slice before: step 0 builds the four
// book addresses, steps 1 and 2 issue two book reads each, step 3 is empty (the reads' latency),
// steps 4..7 scale and round one pair each.
struct Expansion {
    uint32_t addr[4];
    float2_t v[4];
    u32x4v o;
};
__device__ __forceinline__ void expansion_step(Expansion& x, int t, uint32_t d, float scale, uint32_t book_lane) {
    if (t == 0) {
#pragma unroll
        for (int c = 0; c < 4; ++c) x.addr[c] = book_address(d, book_lane, c);
    } else if (t == 1 || t == 2) {
        x.v[2 * t - 2] = lds_f32x2(x.addr[2 * t - 2]);
        x.v[2 * t - 1] = lds_f32x2(x.addr[2 * t - 1]);
        // keep the address registers alive past the reads: a read whose destination reuses its own address
        // register is later waited for with lgkmcnt(0) instead of its place in the queue
        asm volatile("" ::"v"(x.addr[2 * t - 2]), "v"(x.addr[2 * t - 1]));
    } else if (t >= 4) {
        x.o[t - 4] = scale_round_pair(x.v[t - 4], scale);
    }
}

// WAVES waves, wave w: all BM rows of x by weight rows n0 + 32 NG w .. + 32 NG - 1.  Lane l holds, for
// g < NG, weight row 32 (NG w + g) + l % 32, codes 32 (l / 32) .. + 31 of the k step; dword s of them is the B
// fragment of slice s, covering k = 32 (l / 32) + 8 s .. + 7, and the x fragments are read from LDS in the same
// k order.
//
// Order of issue inside a slice: after every MFMA first the LDS reads (the fragment of the next slice once its
// last user has been issued, book reads), then at most a handful of VALU instructions.
// How the tiles of one call are spread over workgroups (one workgroup per CU at a time, handed out in the order of
// their numbers; GRID CUs).
//   * The first `full` = rounds * GRID tiles are taken whole, one workgroup each.  Tile numbers (m fastest) are
//     dealt so that every XCD -- workgroup b runs on XCD b % 8 -- owns a contiguous run of them: the x-row tiles
//     that share a weight tile meet in one L2.
//   * The remaining `tail_tiles` (fewer than GRID) would leave CUs idle in a last, partial round, so each of them
//     can be cut into `pieces` equal pieces along k (in quanta of `gran` k steps, qpt per tile), one workgroup per
//     piece, numbered piece-major (all first pieces, then all second pieces, ...).  The pieces of a tile meet in
//     the workspace (see the kernel).  pieces == 1: whole tiles.
struct WideSchedule {
    int m_tiles, n_tiles;
    int full, tail_tiles, pieces;
    int qpt, gran;
    uint32_t* counters;  // two per tail tile, zero between calls
    float* partials;     // one slot of BM x 256 floats per piece
};
constexpr int GRID = 256;

template <bool NESTED, int BM, int NG>
__global__ __launch_bounds__(512 / NG) __attribute__((amdgpu_waves_per_eu(3 - NG, 3 - NG)))
void gemm_wide_kernel(MatmulArgs a, WideSchedule sch) {
    // The body exists in the device pass only: the host pass cannot instantiate the buffer-resource type
    // it uses and would then leave the kernel's launch stub undefined.
#if defined(__HIP_DEVICE_COMPILE__)
    using T = Tile<BM, NG>;
    extern __shared__ __attribute__((aligned(4096))) uint8_t smem[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    // pair book: thread tid writes copy tid % 32 of the byte values it * (THREADS / 32) + tid / 32
    {
        constexpr int PER = T::THREADS / 32;
#pragma unroll 4
        for (int it = 0; it < 256 / PER; ++it) {
            const int b = it * PER + (tid >> 5);
            const float2_t pair = {a.lut16[b >> 4], a.lut16[b & 15]};
            *reinterpret_cast<float2_t*>(smem + (b << 8) + ((tid & 31) << 3)) = pair;
        }
    }
    const uint32_t book_lane = (lane & 31) * 8;
    const uint32_t stage0 = BOOK_BYTES;

    // ---- what this workgroup works on: a whole tile, or one piece of a tail tile ----
    const int m_tiles = sch.m_tiles;
    const int ksteps_all = a.K / BK;
    int id, kfirst = 0, ksteps = ksteps_all, tail_tile = -1, piece = 0;
    if ((int)blockIdx.x < sch.full) {
        const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
        id = xcd * (sch.full >> 3) + slot;
    } else {
        const int p = blockIdx.x - sch.full;
        piece = p / sch.tail_tiles;
        tail_tile = p - piece * sch.tail_tiles;
        id = sch.full + tail_tile;
        if (sch.pieces > 1) {
            const int q0 = piece * sch.qpt / sch.pieces, q1 = (piece + 1) * sch.qpt / sch.pieces;
            kfirst = q0 * sch.gran;
            ksteps = (q1 - q0) * sch.gran;
        }
    }
    const bool partial = sch.pieces > 1 && tail_tile >= 0;
    const int nt = id / m_tiles;
    const int mt = id - nt * m_tiles;
    const int m0 = mt * BM, n0 = nt * BN;

    f32x16 acc[T::TI][NG];
#pragma unroll
    for (int i = 0; i < T::TI; ++i)
#pragma unroll
        for (int g = 0; g < NG; ++g)
#pragma unroll
            for (int q = 0; q < 16; ++q) acc[i][g][q] = 0.0f;

    // x: load j of this wave fills chunk c = XL * wave + j = rows 8 c .. + 7 of the stage, 1 KB.  Inside a chunk row
    // rr sits in 128-byte slot rr ^ (c & 1) and its 16-byte piece p at position p ^ rr: the sixteen lanes that a
    // 128-bit fragment read serves together (sixteen consecutive rows, one piece) then hit sixteen different
    // 16-byte bank groups.  Lane l of the load instruction writes slot l / 8, position l % 8 (LDS-direct loads
    // store lane l at 16 l), so it fetches row (l / 8) ^ (c & 1), piece (l % 8) ^ row.
    // The loads are buffer loads (base + per-lane 32-bit offset + scalar offset of the k step): next to regular
    // loads the compiler counts them in order, whereas a flat-encoded LDS-direct load in flight makes it turn
    // every wait of the wave into a wait for everything.  x must be smaller than 4 GB (the launcher checks).
    const __amdgpu_buffer_rsrc_t xrsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(a.x), 0, (int)(uint32_t)((int64_t)a.M * a.K * 2), 0x00020000);
    uint32_t xoff[T::XL];
#pragma unroll
    for (int j = 0; j < T::XL; ++j) {
        const int c = T::XL * wave + j;
        const int rr = (lane >> 3) ^ (c & 1);
        const int row = min(m0 + 8 * c + rr, a.M - 1);
        xoff[j] = (uint32_t)row * (uint32_t)(a.K * 2) + (uint32_t)(((lane & 7) ^ rr) << 4) + (uint32_t)(kfirst * (BK * 2));
    }
    auto load_x_one = [&](int kt, int stage, int j) {  // load j of k step kt into a stage
        const uint32_t st = stage0 + stage * T::STAGE_BYTES + T::XL * wave * CHUNK_BYTES;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(xrsrc, (lds_void_ptr)(uintptr_t)(st + j * CHUNK_BYTES), 16, xoff[j],
                                                 kt * (BK * 2), 0, 0);
    };
    auto load_x = [&](int kt, int stage) {  // k step kt into a stage
#pragma unroll
        for (int j = 0; j < T::XL; ++j) load_x_one(kt, stage, j);
    };
    // fragment of x tile i, slice s: row r = 32 i + l % 32 lies in chunk 4 i + (l % 32) / 8 (whose parity is that of
    // (l % 32) / 8) at slot (r % 8) ^ parity; its piece 4 (l / 32) + s sits at position piece ^ (r % 8).
    const int fr = lane & 31;
    const uint32_t frag_row = (uint32_t)((fr >> 3) * CHUNK_BYTES + (((fr & 7) ^ ((fr >> 3) & 1)) << 7));
    uint32_t frag_off[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) frag_off[s] = stage0 + frag_row + (uint32_t)(((((lane >> 5) << 2) | s) ^ (fr & 7)) << 4);

    int64_t e0[NG];
#pragma unroll
    for (int g = 0; g < NG; ++g)
        e0[g] = (int64_t)min(n0 + (wave * NG + g) * 32 + (lane & 31), a.N - 1) * a.K + (lane >> 5) * 32 + kfirst * BK;

    // Three k steps of x and of codes are under way at any time: stages and code sets rotate with period 3.
    Codes c0[NG], c1[NG], c2[NG];
    load_x(0, 0);
    if (ksteps > 1) load_x(1, 1);
    if (ksteps > 2) load_x(2, 2);
#pragma unroll
    for (int g = 0; g < NG; ++g) {
        load_codes<NESTED>(a, c0[g], e0[g]);
        if (ksteps > 1) load_codes<NESTED>(a, c1[g], e0[g] + BK);
        if (ksteps > 2) load_codes<NESTED>(a, c2[g], e0[g] + 2 * BK);
        if (NESTED && ksteps > 3) load_absmax_code(a, c0[g], e0[g] + 3 * BK);
    }
    __builtin_amdgcn_s_waitcnt(0);  // x of the first steps has landed in LDS (LDS-direct loads count as vector memory)
    __syncthreads();                // ... everyone's, and the code book is visible

    bf16x8 fb[NG], fa[T::TI];
#pragma unroll
    for (int g = 0; g < NG; ++g) {
        Expansion x;
#pragma unroll
        for (int t = 0; t < 8; ++t) expansion_step(x, t, c0[g].w.x, c0[g].scale, book_lane);
        fb[g] = __builtin_bit_cast(bf16x8, x.o);
    }
#pragma unroll
    for (int i = 0; i < T::TI; ++i) fa[i] = lds_frag(frag_off[0] + i * 4 * CHUNK_BYTES);

    // Vector-memory operations a wave issues per k step after its x loads: the code loads of every group.
    constexpr int CODE_LOADS = (NESTED ? 4 : 2) * NG;

    // One k step.  `cur` holds the codes of step kt (dword 0 already expanded into fb), `nxt` those of step
    // kt + 1 (the third set, of step kt + 2, is in flight); fa holds the x fragments of slice 0; stage ST holds x of
    // step kt, the loads of steps kt + 1 and kt + 2 into the other two stages are in flight or done.
    auto step = [&](int kt, auto stage, Codes(&cur)[NG], Codes(&nxt)[NG], auto full) {
        constexpr int ST = decltype(stage)::value;
        constexpr bool FULL = decltype(full)::value;  // steps up to kt + 3 exist
        const uint32_t st = ST * T::STAGE_BYTES;
        const uint32_t st_next = ((ST + 1) % 3) * T::STAGE_BYTES;
        const bool more = FULL || kt + 1 < ksteps;
        const bool more3 = FULL || kt + 3 < ksteps;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            if (s == 3) {
                // The one synchronisation of the step.  Every fragment read of this stage has been issued (slice 3's
                // were prefetched during slice 2) and is complete (lgkmcnt); this wave's x loads of step kt + 1 are
                // complete: loads return in order, and behind them this wave has issued the codes of step kt + 1, x
                // of step kt + 2 and the codes of step kt + 2, of which the last XL + CODE_LOADS may stay in flight.
                // After the barrier all that holds for every wave: stage ST may be refilled, the next stage read.
                __builtin_amdgcn_sched_barrier(0);
                if (FULL)
                    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(T::XL + CODE_LOADS) : "memory");
                else
                    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
                // The codes of step kt + 1 are consumed from here on.  Naming them before the x loads are issued puts
                // the compiler's own wait for them here, where it costs nothing (they are older than what the wait
                // above lets through); behind the x loads it would be a wait for those loads as well.
                if (more) {
#pragma unroll
                    for (int g = 0; g < NG; ++g) asm volatile("" ::"v"(nxt[g].w.x), "v"(nxt[g].scale));
                }
                __builtin_amdgcn_sched_barrier(0);
                __builtin_amdgcn_sched_barrier(0);
            }
            Expansion ex[NG];
            const bool expand = s < 3 || more;  // the B fragments of the next slice: dword s + 1 of cur, or dword 0 of nxt
            const uint32_t next_frag = s < 3 ? st + frag_off[(s + 1) & 3] : st_next + frag_off[0];
#pragma unroll
            for (int j = 0; j < T::NM; ++j) {
                const int i = j / NG, g = j % NG;
                acc[i][g] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[g], acc[i][g], 0, 0, 0);
                // Behind the MFMA: LDS reads first, then VALU work -- except where the VALU work consumes book
                // reads: it then comes first, so that its wait does not include the fragment read just issued.
                // The fragment of the next slice goes into the registers of fa[i] once this slice has no more use
                // for them (the MFMA has read its operands long before the data arrives).  Micro-step t of the
                // next B fragment of group gg belongs to MFMA (8 gg + t) NM / (8 NG).
                auto micro_steps = [&](bool scaling) {
                    if (expand) {
#pragma unroll
                        for (int gg = 0; gg < NG; ++gg)
#pragma unroll
                            for (int t = 0; t < 8; ++t)
                                if (((8 * gg + t) * T::NM) / (8 * NG) == j && (t >= 4) == scaling) {
                                    const Codes& src = s < 3 ? cur[gg] : nxt[gg];
                                    expansion_step(ex[gg], t, dword_of(src.w, (s + 1) & 3), src.scale, book_lane);
                                }
                    }
                };
                micro_steps(true);
                __builtin_amdgcn_sched_barrier(0);
                if (g == NG - 1 && expand) fa[i] = lds_frag(next_frag + i * 4 * CHUNK_BYTES);
                // the refill of this stage, one load behind every SPREAD-th MFMA of the last slice: issued together they
                // would queue up in the CU's one address unit and hold the waves (and their MFMAs) at the issue
                if (s == 3 && more3) {
                    constexpr int SPREAD = T::NM / T::XL;
                    if (j % SPREAD == 0 && j / SPREAD < T::XL) load_x_one(kt + 3, ST, j / SPREAD);
                }
                micro_steps(false);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (s == 3 && more3) {  // cur's dwords are used up: refill it with step kt + 3
#pragma unroll
                for (int g = 0; g < NG; ++g) {
                    if (NESTED) {
                        load_codes_staged(a, cur[g], e0[g] + (int64_t)(kt + 3) * BK);
                        // the set that is refilled next (with step kt + 4) gets its absmax code now
                        if (FULL || kt + 4 < ksteps) load_absmax_code(a, nxt[g], e0[g] + (int64_t)(kt + 4) * BK);
                    } else {
                        load_codes<false>(a, cur[g], e0[g] + (int64_t)(kt + 3) * BK);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            if (expand) {
#pragma unroll
                for (int g = 0; g < NG; ++g) fb[g] = __builtin_bit_cast(bf16x8, ex[g].o);
            }
        }
    };
    using S0 = std::integral_constant<int, 0>;
    using S1 = std::integral_constant<int, 1>;
    using S2 = std::integral_constant<int, 2>;
    int kt = 0;
    for (; kt + 6 < ksteps; kt += 3) {  // FULL: every step of the triple still issues loads (up to step kt + 5) and one more exists
        step(kt, S0{}, c0, c1, std::true_type{});
        step(kt + 1, S1{}, c1, c2, std::true_type{});
        step(kt + 2, S2{}, c2, c0, std::true_type{});
    }
    for (; kt < ksteps; kt += 3) {
        step(kt, S0{}, c0, c1, std::false_type{});
        if (kt + 1 < ksteps) step(kt + 1, S1{}, c1, c2, std::false_type{});
        if (kt + 2 < ksteps) step(kt + 2, S2{}, c2, c0, std::false_type{});
    }

    // acc[i][g][q] = out[m][n], n = 32 (NG wave + g) + lane % 32, m = 32 i + 8 (q / 4) + 4 (lane / 32) + q % 4.
    // The tile leaves through LDS (the x stages are free now), half of its rows at a time, so that global memory
    // sees 16-byte stores that cover whole rows of the tile (512 contiguous bytes per 32 lanes) instead of
    // 2-byte stores in runs of 64 bytes.  Into LDS: rows q and q + 1 of a lane are rounded to one dword, lanes
    // l and l ^ 1 exchange dwords (DPP) and v_perm_b32 leaves the even lane with columns (n, n + 1) of row q and
    // the odd lane with the same columns of row q + 1: one ds_write_b32 per two outputs.  Row r of a half starts at
    // 512 r; its dword c sits at c ^ 16 f(r), f(r) = r % 2 + 2 (r / 4 % 2), which keeps 16-byte pieces whole and
    // sends the four rows one write instruction touches (r, r + 1, r + 4, r + 5) to four different bank groups.
    __syncthreads();  // every wave has issued and received its last fragment reads

    // ---- a piece of a tail tile: meet the tile's other pieces in the workspace ----
    // Pieces are numbered in k order; piece c of tail tile t has a slot of its own (t * pieces + c) for its fp32
    // partial tile in register order ([i][g][q][thread]: coalesced).  Two counters per tile, zero between calls: P
    // counts published partials, T hands out tickets.
    //   * Every piece but the last to finish stores its partial, waits until L2 has it (publish_partials), and only
    //     then counts itself in P.  Whoever raises P to the number of pieces adds all partials from memory, in k
    //     order, and writes the tile.
    //   * Two pieces (the common case): the holder of the second ticket looks at P first; if the other partial is
    //     published already, it adds it to its registers and writes the tile without storing a partial (a + b = b + a
    //     exactly, so the result does not depend on who finishes last).  Otherwise it proceeds like everyone else.
    // No workgroup ever waits for another one.
    bool write_tile = true;
    if (partial) {
        constexpr int SLOT = BM * BN;  // floats
        constexpr int FR = 16 * T::THREADS;  // floats per accumulator fragment
        const int pieces = sch.pieces;
        uint32_t* cP = sch.counters + 2 * tail_tile;
        uint32_t* cT = cP + 1;
        auto slot_of = [&](int c) { return sch.partials + (int64_t)(tail_tile * pieces + c) * SLOT; };
        volatile uint32_t* flag = reinterpret_cast<volatile uint32_t*>(smem + BOOK_BYTES);
        bool in_registers = false;
        if (pieces == 2) {
            if (tid == 0) {
                const uint32_t ticket = __hip_atomic_fetch_add(cT, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                uint32_t ok = 0;
                if (ticket == 1) ok = __hip_atomic_load(cP, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 1u;
                *flag = ok;
            }
            __syncthreads();
            in_registers = *flag != 0;
            acquire_partials();
            __syncthreads();
        }
        bool from_memory = false;
        if (!in_registers) {
            float* mine = slot_of(piece);
#pragma unroll
            for (int i = 0; i < T::TI; ++i)
#pragma unroll
                for (int g = 0; g < NG; ++g)
#pragma unroll
                    for (int q = 0; q < 16; ++q)
                        __hip_atomic_store(mine + ((i * NG + g) * 16 + q) * T::THREADS + tid, acc[i][g][q], __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT);
            publish_partials();
            __syncthreads();
            if (tid == 0) *flag = __hip_atomic_fetch_add(cP, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1u;
            __syncthreads();
            from_memory = *flag == (uint32_t)pieces;
            acquire_partials();
            __syncthreads();
        }
        if (in_registers) {
            const float* other = slot_of(piece ^ 1);
            constexpr int B = 4;  // fragments whose loads are in flight together
#pragma unroll
            for (int f0 = 0; f0 < T::TI * NG; f0 += B) {
                float v[B][16];
#pragma unroll
                for (int f = 0; f < B; ++f)
#pragma unroll
                    for (int q = 0; q < 16; ++q)
                        v[f][q] = __hip_atomic_load(other + ((f0 + f) * 16 + q) * T::THREADS + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
                for (int f = 0; f < B; ++f)
#pragma unroll
                    for (int q = 0; q < 16; ++q) acc[(f0 + f) / NG][(f0 + f) % NG][q] += v[f][q];
            }
        } else if (from_memory) {
            constexpr int G = 4;  // pieces whose loads are in flight together
#pragma unroll
            for (int f = 0; f < T::TI * NG; ++f) {
                float sum[16];
#pragma unroll
                for (int q = 0; q < 16; ++q) sum[q] = 0.0f;
#pragma unroll 1
                for (int c0 = 0; c0 < pieces; c0 += G) {
                    float v[G][16];
#pragma unroll
                    for (int c = 0; c < G; ++c) {
                        const float* src = slot_of(min(c0 + c, pieces - 1)) + f * FR + tid;
#pragma unroll
                        for (int q = 0; q < 16; ++q)
                            v[c][q] = __hip_atomic_load(src + q * T::THREADS, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
#pragma unroll
                    for (int c = 0; c < G; ++c)
                        if (c0 + c < pieces) {
#pragma unroll
                            for (int q = 0; q < 16; ++q) sum[q] += v[c][q];
                        }
                }
#pragma unroll
                for (int q = 0; q < 16; ++q) acc[f / NG][f % NG][q] = sum[q];
            }
        }
        write_tile = in_registers || from_memory;
        if (write_tile && tid == 0) {
            __hip_atomic_store(cP, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(cT, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    if (write_tile) {
        constexpr int HALF_ROWS = BM / 2;
        uint8_t* stage = smem + BOOK_BYTES;
        const uint32_t sel = (lane & 1) ? 0x03020706u : 0x05040100u;
        const int wf = (lane & 1) | ((lane >> 5) << 1);
        const bool vec = (a.N & 7) == 0;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
#pragma unroll
            for (int g = 0; g < NG; ++g) {
                const int nl = (wave * NG + g) * 32 + (lane & 31);
                const int n = n0 + nl;
                const float b = (a.bias && n < a.N) ? bf16_bits_to_f32(a.bias[n]) : 0.0f;
                uint8_t* wbase = stage + (4 * (lane >> 5) + (lane & 1)) * 512 + ((((uint32_t)nl >> 1) ^ ((uint32_t)wf << 4)) << 2);
#pragma unroll
                for (int il = 0; il < T::TI / 2; ++il) {
                    const int i = h * (T::TI / 2) + il;
#pragma unroll
                    for (int q = 0; q < 16; q += 2) {
                        const float2_t f = {acc[i][g][q] + b, acc[i][g][q + 1] + b};
                        const uint32_t mine = __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2_t));
                        const uint32_t theirs = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)mine, 0xB1, 0xf, 0xf, true);
                        const uint32_t packed = __builtin_amdgcn_perm(theirs, mine, sel);
                        *reinterpret_cast<uint32_t*>(wbase + (32 * il + 8 * (q >> 2) + (q & 2)) * 512) = packed;
                    }
                }
            }
            __syncthreads();
#pragma unroll
            for (int it = 0; it < HALF_ROWS / (T::THREADS / 32); ++it) {
                const int r = it * (T::THREADS / 32) + (tid >> 5);
                const int piece = tid & 31;
                const int fr2 = (r & 1) | (((r >> 2) & 1) << 1);
                const uint4 v = *reinterpret_cast<const uint4*>(stage + r * 512 + ((piece ^ (fr2 << 2)) << 4));
                const int m = m0 + h * HALF_ROWS + r;
                const int n = n0 + piece * 8;
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
            if (h == 0) __syncthreads();
        }
    }
#endif  // __HIP_DEVICE_COMPILE__
}

// Bytes of workspace a cut-up tail needs: the counter region and one partial-tile slot per piece.
size_t wide_tail_bytes(int tail_tiles, int pieces, int bm) {
    return (size_t)GEMV_COUNTER_BYTES + (size_t)tail_tiles * pieces * bm * BN * sizeof(float);
}

// The schedule of a call: a pure function of the shape and of the size of the workspace it is given.  With a
// workspace that is too small (or none) the tail tiles are taken whole.
WideSchedule wide_schedule(int64_t M, int64_t N, int64_t K, int bm, size_t workspace_bytes) {
    WideSchedule s{};
    s.m_tiles = (int)((M + bm - 1) / bm);
    s.n_tiles = (int)((N + BN - 1) / BN);
    const int64_t tiles = (int64_t)s.m_tiles * s.n_tiles;
    s.full = (int)(tiles / GRID) * GRID;
    s.tail_tiles = (int)(tiles - s.full);
    const int ksteps = (int)(K / BK);
    s.gran = ksteps % 4 == 0 ? 4 : ksteps % 2 == 0 ? 2 : 1;
    s.qpt = ksteps / s.gran;
    s.pieces = 1;
    if (s.tail_tiles == 0 || s.full > 0 || ksteps < 32) return s;
    const int R = s.tail_tiles;
    // Cutting pays only where it puts idle CUs to work on pieces that stay long: a call with fewer tiles than CUs,
    // at most GRID pieces in all, of 16 k steps or more.  Measured without gain: a partial round behind full
    // rounds cut in two ([28672, 4096], 2048 rows of x: 461 vs 464 us -- the chip is power-limited and a partial
    // round runs at a higher clock), and more than GRID / 2 tiles cut into a long and a short piece each (the
    // short pieces cost more in start-up and hand-off than they save).
    int n = GRID / R;
    if (n > 8) n = 8;
    if (n > ksteps / 16) n = ksteps / 16;
    if (n > s.qpt) n = s.qpt;
    if (n < 2) return s;
    s.pieces = n;
    if (workspace_bytes < wide_tail_bytes(R, s.pieces, bm)) s.pieces = 1;
    return s;
}

constexpr int WIDE_NG = 1;

constexpr int MAX_DEVICES = 64;

template <bool NESTED, int BM>
hipError_t launch_tile(const MatmulArgs& a, hipStream_t stream) {
    using T = Tile<BM, WIDE_NG>;
    static bool ready[MAX_DEVICES] = {};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= MAX_DEVICES) return hipErrorInvalidDevice;
    auto kern = gemm_wide_kernel<NESTED, BM, WIDE_NG>;
    if (!ready[dev]) {
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                T::SMEM_BYTES);
        if (e != hipSuccess) return e;
        ready[dev] = true;
    }
    WideSchedule sch = wide_schedule(a.M, a.N, a.K, BM, a.workspace ? a.workspace_bytes : 0);
    sch.counters = static_cast<uint32_t*>(a.workspace);
    sch.partials = a.workspace ? reinterpret_cast<float*>(static_cast<uint8_t*>(a.workspace) + GEMV_COUNTER_BYTES) : nullptr;
    hipLaunchKernelGGL(kern, dim3((unsigned)(sch.full + sch.tail_tiles * sch.pieces)), dim3(T::THREADS), T::SMEM_BYTES, stream, a, sch);
    return hipGetLastError();
}

}  // namespace

// Rows of x per tile (a pure function of the shape).  The 256-row tile expands every weight half as often, the
// 128-row tile gives twice the workgroups: 256 rows once that makes 160 tiles or more, or when the k loop is long
// enough for the pieces of a cut-up tile to stay long (tiles x k steps >= 28672, e.g. 128 tiles of K = 14336);
// measured on both sides of either bound.
int gemm_wide_tile_rows(int64_t M, int64_t N, int64_t K) {
    const int64_t tiles = ((M + 255) / 256) * ((N + BN - 1) / BN);
    return tiles >= 160 || tiles * (K / BK) >= 28672 ? 256 : 128;
}

// Workspace of a call: none when no tile is cut up.
size_t gemm_wide_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    const int bm = gemm_wide_tile_rows(M, N, K);
    const WideSchedule s = wide_schedule(M, N, K, bm, ~(size_t)0);
    return s.pieces > 1 ? wide_tail_bytes(s.tail_tiles, s.pieces, bm) : 0;
}

void gemm_wide_plan(int64_t M, int64_t N, int64_t K, int plan[4]) {
    const int bm = gemm_wide_tile_rows(M, N, K);
    const WideSchedule s = wide_schedule(M, N, K, bm, ~(size_t)0);
    plan[0] = bm;
    plan[1] = s.m_tiles * s.n_tiles;
    plan[2] = s.pieces;
    plan[3] = s.full + s.tail_tiles * s.pieces;
}

hipError_t launch_gemm_wide(const MatmulArgs& a, hipStream_t stream) {
    const bool nested = a.nested.q != nullptr;
    if (gemm_wide_tile_rows(a.M, a.N, a.K) == 128)
        return nested ? launch_tile<true, 128>(a, stream) : launch_tile<false, 128>(a, stream);
    return nested ? launch_tile<true, 256>(a, stream) : launch_tile<false, 256>(a, stream);
}

}  // namespace nf4
