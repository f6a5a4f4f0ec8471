// Dispatch of the decode-shape fused NF4 dequant-matmul (M <= 16) between its three kernels:
// row-streaming (M = 1, and M = 2 where rows_serve says so, nf4_gemv_rows.hip), four weight rows per lane quad (M = 2..4, and
// M = 5..8 on weights of at most 2^26 elements -- 2^28 with 4096 < K <= 8192 -- and M = 9..16 as two halves of x on
// weights of at most 2^24, nf4_gemv_quad.hip) and MFMA tiles (the rest up to M = 16, nf4_gemv_tiles.hip).
//
// Replaces bitsandbytes' gemv_4bit (kgemm_4bit_inference_naive), the kernel that
// bitsandbytes.matmul_4bit picks for a single-row x; call site
// thunder/transforms/quantization.py:39.
#include <stdlib.h>

#include <atomic>

#include "nf4_gemv.h"

namespace nf4 {
size_t gemv_workspace_bytes_unstaged(int64_t M, int64_t N, int64_t K);
namespace {

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
        if ((e = gemv_stage_setup()) != hipSuccess) return e;
        g_num_cus[dev] = cus > 0 ? cus : 256;
    }
    *cus_out = g_num_cus[dev];
    return hipSuccess;
}

// One row of x: the row kernel.  Two rows: the row kernel where it holds whole rows of x in one workgroup and the
// quad kernel would split K (8192 < K <= 16384: [4096, 14336] 13.5 vs 14.9 us), and on small weights with K <= 4096
// ([4096, 4096] 6.0 vs 6.2); elsewhere the quad kernel, which does two rows of x for the price of four:
// [14336, 4096] 11.3 vs 13.1 us, [28672, 4096] 18.0 vs 19.5, [8192, 8192] 12.1 vs 14.3, [28672, 8192] 27 vs 32.5,
// [8192, 28672] 37 vs 42, lm_head 60-68 vs 67-71.
bool rows_serve(int64_t M, int64_t N, int64_t K) {
    if (M == 1) return true;
    if (M > 2) return false;
    return (K > 8192 && K <= 16384) || (K <= 4096 && N * K <= ((int64_t)1 << 24));
}

// Five to eight rows of x: the quad kernel starts faster (no x staging), the tile kernel streams faster once the weights
// are large; with K = 4096 they cross near 2^26-2^27 weights ([28672, 4096]: 21.9 vs 22.2 us, lm_head 80 vs 64-71).
// With 4096 < K <= 8192 the quad kernel's waves take two loads each and cover K without a split, and it stays ahead
// much longer ([8192, 8192] 14.6 vs 18.8 us, [28672, 8192] 32.3 vs 36.4-38.4).
bool quad_serves(int64_t M, int64_t N, int64_t K) {
    if (M <= 4) return true;  // (what is left of one and two rows of x included)
    if (M > 8) return false;
    return N * K <= ((int64_t)1 << 26) || (K > 4096 && K <= 8192 && N * K <= ((int64_t)1 << 28));
}

// Nine to sixteen rows of x on a small weight (up to 2^24 elements): the quad kernel on two halves of x, whose
// start-up is shorter than the tile kernel's (measured, 16 rows: [1024, 4096] 7.6 vs 10.5 us, [4096, 4096] 10.6 vs 11.5;
// [6144, 4096] 14.6 vs 11.9 the other way round).
bool quad_halves_serve(int64_t M, int64_t N, int64_t K) {
    return M > 8 && N * K <= ((int64_t)1 << 24) && gemv_quad_halves_possible(N, K);
}

// Which launches go to the kernel that stages codes and absmax through LDS (nf4_gemv_stage.hip): -1 the dispatcher's
// own rule, 0 none, 1 every launch that kernel takes.  Preset by the environment variable NF4HIP_STAGE, changed by
// gemv_set_staged (measurements and tests).
std::atomic<int> g_stage_mode{-2};  // -2: not read from the environment yet

int stage_mode() {
    int m = g_stage_mode.load(std::memory_order_relaxed);
    if (m == -2) {
        const char* v = getenv("NF4HIP_STAGE");
        m = (v && *v) ? atoi(v) : -1;  // (set but empty counts as not set)
        if (m < -1 || m > 1) m = -1;
        g_stage_mode.store(m, std::memory_order_relaxed);
    }
    return m;
}

// The dispatcher's own rule, from interleaved timings of both sides (us, staged vs the other kernels, 1 / 4 / 8 / 16 rows
// of x): lm_head [128256, 4096] 47.6 / 48.5 / 49.2 / 54.6 vs 52.4 / 57.7 / 60.9 / 60.8; [28672, 4096] 14.8 / 15.0 / 15.8 / 17.2 vs
// 15.8 / 16.0 / 21.0 / 24.0; [14336, 4096] 11.1 / 11.3 / 11.5 / 12.8 vs 10.3 / 10.2 / 12.8 / 16.9; [6144, 4096] 7.8 / 8.0 / 8.7 / 9.7 vs
// 6.7 / 7.0 / 8.5 / 11.8; [4096, 4096] 6.2 / 6.5 / 7.1 / 8.1 vs 5.1 / 6.3 / 7.7 / 9.4; [1024, 4096] 5.7 / 6.1 / 6.7 / 7.6 vs 4.1 / 4.6 / 5.1 /
// 6.6.  The staged kernel streams faster and starts more slowly (its first tile needs the first requests of all sixteen
// waves): every weight of a hundred million elements or more, from five rows of x on beyond forty million, from nine
// rows on beyond 2^24 (from five where a workgroup's rows are whole tiles).
bool stage_serves(const MatmulArgs& a) {
    const int mode = stage_mode();
    if (mode == 0 || !gemv_stage_possible(a)) return false;
    if (mode == 1) return true;
    const int64_t weights = (int64_t)a.N * a.K;
    // K beyond what the sixteen waves of a workgroup cover (4096) is split over workgroups that meet in the workspace
    // after their last tile, 1-2 us that the other kernels do not pay: [28672, 8192] 26.6 / 27.8 / 29.8 / 29.8 / 33.2 us with
    // 1 / 4 / 8 / 9 / 16 rows of x against 25.5 / 25.7 / 28.9 / 44.0 / 44.2; [8192, 8192] 13.3 / 13.3 / 13.6 / 13.5 / 14.9 against
    // 11.0 / 11.7 / 13.9 / 18.0 / 18.1; [4096, 8192] 10.4 / 10.4 / 10.7 / 10.8 / 12.0 against 7.3 / 9.2 / 10.9 / 13.3 / 13.6; beyond
    // 8192 (fp16 arithmetic on both sides) [4096, 14336] 14.1 / 14.5 / 14.5 / 14.8 / 15.1 / 16.2 with 1 / 4 / 5 / 8 / 9 / 16 rows
    // against 10.6 / 13.9 / 17.0 / 17.2 / 17.4 / 17.8, [8192, 14336] 18.6 / 19.3 / 19.4 / 19.6 / 21.0 / 22.4 against 16.0 / 18.6 /
    // 22.0 / 22.3 / 27.4 / 27.6.
    // Nested absmax (the other kernels resolve the 8-bit codes per lane and load): [28672, 8192] 25.8 / 27.0 / 27.9 / 29.8 / 29.4 /
    // 31.9 with 1 / 4 / 5 / 8 / 9 / 16 rows against 29.8 / 24.5 / 29.6 / 30.6 / 50.7 / 50.0; [8192, 8192] 13.5 / 13.6 / 13.6 / 13.7 / 13.9 / 15.4
    // against 11.6 / 11.8 / 13.9 / 14.2 / 18.5 / 18.6; without a split the lm_head 45.6 / 45.7 / 49.2 / 51.7 with 1 / 4 / 8 / 16 rows
    // against 62.0 / 55.6 / 67.0 / 70.1, [28672, 4096] 14.6 / 14.6 / 15.1 / 17.0 against 17.5 / 15.5 / 22.1 / 24.5, [14336, 4096] 11.0 /
    // 11.0 / 11.4 / 13.0 against 10.6 / 10.1 / 12.5 / 16.6: the same rule, from five rows on with K split.
    // Other shapes, fp32 absmax, staged vs the other kernels with 5 / 8 / 9 / 16 rows: [10240, 8192] 14.2 / 14.7 / 14.9 / 16.7 vs
    // 15.1 / 15.9 / 22.7 / 23.2; [57344, 8192] 52.8 / 53.6 / 54.4 / 60.2 vs 58.7 / 58.4 / 63.7 / 63.6 (1..4 rows: 49-52 vs 45-46);
    // [13824, 5120] 16.1 / 16.7 / 16.8 / 18.5 vs 15.7 / 16.5 / 18.8 / 19.1; [5120, 5120] (26 M weights) loses at every M.
    if (gemv_stage_splits(a.K) > 1) return weights >= ((int64_t)1 << 25) && a.M >= 5;
    if (weights >= 100000000) return true;
    if (weights >= 40000000) return a.M >= 5;
    if (weights < ((int64_t)1 << 24)) return false;
    if (a.M >= 9) return true;
    // 5..8 rows of x: where every workgroup has whole 16-row tiles and all sixteen waves a slice of K -- [4096, 4096]
    // 6.7 / 6.9 / 7.4 us with 5 / 6 / 8 rows against 7.4 / 7.6 / 7.8, [8192, 4096] 8.9 / 8.8 / 9.0 against 9.3 / 9.3 / 9.6; with a
    // half-filled last tile per workgroup [6144, 4096] 8.4 / 8.5 / 8.9 against 8.2 / 8.4 / 8.5, [5120, 4096] 8.2 / 8.2 / 8.6 against
    // 7.9 / 8.2 / 8.4
    return a.M >= 5 && a.K == 4096 && a.N % (256 * 16) == 0;
}

}  // namespace

// ---- dispatch -------------------------------------------------------------------------------

// The CU count the launch plans are made for: the current device's, or 256 (the part this library is written for)
// where no device answers -- what the "is this served" answers are judged on, so that they agree with the launch.
int gemv_plan_cus() {
    int cus = 256;
    if (device_setup(&cus) != hipSuccess) cus = 256;
    return cus;
}


void gemv_set_staged(int mode) { g_stage_mode.store(mode < -1 || mode > 1 ? -1 : mode, std::memory_order_relaxed); }

size_t gemv_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    const size_t staged = K % 256 == 0 && K <= 16384 ? gemv_stage_workspace_bytes(M, N, K) : 0;
    const size_t other = gemv_workspace_bytes_unstaged(M, N, K);
    return staged > other ? staged : other;
}

size_t gemv_workspace_bytes_unstaged(int64_t M, int64_t N, int64_t K) {
    if (rows_serve(M, N, K)) return gemv_rows_workspace_bytes(M, N, K);
    if (quad_halves_serve(M, N, K)) return gemv_quad_workspace_bytes(8, N, K);
    return quad_serves(M, N, K) ? gemv_quad_workspace_bytes(M, N, K) : gemv_tiles_workspace_bytes(M, N, K);
}

bool gemv_epilogue_possible(const MatmulArgs& a) {
    if (a.epi.flags == EPI_NONE) return true;
    if (stage_serves(a)) return true;
    // The same product without an epilogue would go to the staged kernel, which does not have this one: refused, so that
    // a caller who runs the product and the operation one after the other adds to the same sums either way (an
    // epilogue promises the stored roundings of that two-step route)
    {
        MatmulArgs plain = a;
        plain.epi = Epilogue{};
        if (stage_serves(plain)) return false;
    }
    if (rows_serve(a.M, a.N, a.K)) return gemv_rows_epilogue_possible(a);
    if (quad_halves_serve(a.M, a.N, a.K) || quad_serves(a.M, a.N, a.K)) return gemv_quad_epilogue_possible(a);
    return gemv_tiles_epilogue_possible(a);
}

// The number of partial sums is the number of bands of the launch plan, which depends on the device's CU count: the
// current device's (256, the part this library is written for, where no device answers).
int gemv_norm_parts(int64_t M, int64_t N, int64_t K) {
    int cus = 256;
    if (device_setup(&cus) != hipSuccess) cus = 256;
    {
        // where the product by itself goes to the staged kernel, so does the residual epilogue (gemv_epilogue_possible),
        // which that kernel has with K split over workgroups and, for few rows per workgroup, with one K range
        MatmulArgs plain{};
        plain.M = (int)M;
        plain.N = (int)N;
        plain.K = (int)K;
        plain.block_log2 = 6;
        if (stage_serves(plain)) return gemv_stage_norm_parts(M, N, K, cus);
    }
    if (rows_serve(M, N, K)) return gemv_rows_norm_parts(M, N, K, cus);
    if (quad_halves_serve(M, N, K)) return gemv_quad_norm_parts(M, N, K, cus, true);
    if (quad_serves(M, N, K)) return gemv_quad_norm_parts(M, N, K, cus, false);
    return gemv_tiles_norm_parts(N);
}

// Which kernel launch_gemv picks for a call without an epilogue: GEMV_KERNEL_* of nf4_gemv.h.
int gemv_kernel_for(int64_t M, int64_t N, int64_t K, int block_log2, bool nested) {
    MatmulArgs a{};
    a.M = (int)M;
    a.N = (int)N;
    a.K = (int)K;
    a.block_log2 = block_log2;
    static const uint8_t some_codes = 0;
    a.nested.q = nested ? &some_codes : nullptr;  // (only looked at for being non-null)
    a.nested.nested_log2 = 8;                     // (the nested blocksize of the format: 256)
    if (stage_serves(a)) return GEMV_KERNEL_STAGED;
    if (rows_serve(M, N, K)) return GEMV_KERNEL_ROWS;
    if (quad_halves_serve(M, N, K)) return GEMV_KERNEL_QUAD_HALVES;
    return quad_serves(M, N, K) ? GEMV_KERNEL_QUAD : GEMV_KERNEL_TILES;
}

void gemv_plan(int64_t M, int64_t N, int64_t K, int block_log2, bool nested, int plan[4]) {
    plan[0] = gemv_kernel_for(M, N, K, block_log2, nested);
    // (the tile kernel has its fp16 mode only where a workgroup's K range is one slice of x: reported as exact beyond 8192)
    plan[1] = gemv_arith_mode(K, plan[0] != GEMV_KERNEL_TILES);
    plan[2] = 0;
    plan[3] = 0;
}

hipError_t launch_gemv(const MatmulArgs& a, hipStream_t stream) {
    if (!gemv_epilogue_possible(a)) return hipErrorNotSupported;
    int cus = 0;
    const hipError_t e = device_setup(&cus);
    if (e != hipSuccess) return e;
    if (stage_serves(a)) return launch_gemv_stage(a, cus, stream);
    if (rows_serve(a.M, a.N, a.K)) return launch_gemv_rows(a, cus, stream);
    if (quad_halves_serve(a.M, a.N, a.K)) return launch_gemv_quad_halves(a, cus, stream);
    return quad_serves(a.M, a.N, a.K) ? launch_gemv_quad(a, cus, stream) : launch_gemv_tiles(a, cus, stream);
}

}  // namespace nf4
