// Internal declarations shared by the kernel files and the C-ABI front end of libnf4hip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace nf4 {

enum : int { BF16 = 0, F16 = 1, F32 = 2 };

// Nested ("double") quantisation of absmax; all NULL/0 when absmax is given directly as fp32.
struct NestedAbsmax {
    const uint8_t* q;      // [nblocks] 8-bit codes
    const float* absmax2;  // [ceil(nblocks / nested_blocksize)]
    const float* map256;   // [256] dynamic map
    float offset;
    int nested_log2;       // log2(nested_blocksize)
};

// What a decode-shape matmul does with its finished sums besides rounding them (fp32 absmax, K not split over
// workgroups).  Each output is finished by exactly one thread, so nothing here is computed twice.
//   EPI_ROWSCALE    sum[m][n] *= 1 / sqrt(mean_sq[m] + eps) before bias: x is bf16(r * norm_weight) written by an
//                   EPI_RESID_NORM call, in_sumsq [M, in_parts] that call's partial sums of r^2 (mean over this K).
//   EPI_SILU_PAIRS  weight rows 2j / 2j+1 are gate row j / up row j: out [M, N/2], out[m][j] = silu(gate) * up
//                   with the roundings of bf16 linear outputs, a bf16 SiLU and a bf16 product.
//   EPI_RESID_NORM  d = bf16(sum + bias); r = bf16(resid_in + d) -> resid_out; bf16(r * norm_weight) -> xnext_out;
//                   the workgroup's sum of r^2 per row of x -> out_sumsq[m * parts + band]; `out` is not written.
enum : int { EPI_NONE = 0, EPI_ROWSCALE = 1, EPI_SILU_PAIRS = 2, EPI_RESID_NORM = 4 };
struct Epilogue {
    int flags;
    float eps;
    const float* in_sumsq;
    int in_parts;
    const uint16_t* resid_in;     // [M, N]
    const uint16_t* norm_weight;  // [N]
    uint16_t* resid_out;          // [M, N]
    uint16_t* xnext_out;          // [M, N]
    float* out_sumsq;             // [M, gemv_norm_parts(M, N, K)]
};

struct MatmulArgs {
    const uint16_t* x;    // [M, K] bf16
    const uint8_t* packed;  // [N*K/2]
    const float* absmax;  // [N*K/blocksize] or NULL when nested is used
    NestedAbsmax nested;
    const float* lut16;
    const uint16_t* bias;  // [N] bf16 or NULL
    uint16_t* out;         // [M, N] bf16
    int M, N, K;
    int block_log2;  // log2(blocksize)
    void* workspace;
    size_t workspace_bytes;
    Epilogue epi;
};

// Dense bf16 GEMM out[M, N] = x[M, K] . w[N, K]^T (+ bias): the GEMM of the dequantize + linear route.
struct DenseArgs {
    const uint16_t* x;     // [M, K] bf16
    const uint16_t* w;     // [N, K] bf16 (what nf4hip_dequantize wrote)
    const uint16_t* bias;  // [N] bf16 or NULL
    uint16_t* out;         // [M, N] bf16
    int M, N, K;
    void* workspace;
    size_t workspace_bytes;
};

// Launchers (defined next to their kernels).  They assume validated arguments and return the
// hipError_t of the launch.
hipError_t launch_quantize(const void* w, int w_dtype, int64_t n, int block_log2, uint8_t* packed, float* absmax,
                           hipStream_t stream);
hipError_t launch_dequantize(const uint8_t* packed, const float* absmax, const NestedAbsmax& nested,
                             const float* lut16, int64_t n, int block_log2, void* out, int out_dtype,
                             hipStream_t stream);
hipError_t launch_dq_compress(const float* absmax, int64_t nblocks, int nested_log2, const float* map256,
                              float offset, uint8_t* q, float* absmax2, hipStream_t stream);
hipError_t launch_dq_reconstruct(const NestedAbsmax& nested, int64_t nblocks, float* absmax, hipStream_t stream);

// Head of every matmul workspace: the split-K arrival counters (zero between calls).
constexpr size_t GEMV_COUNTER_REGION_BYTES = 65536 * 4;

size_t gemv_workspace_bytes(int64_t M, int64_t N, int64_t K);
hipError_t launch_gemv(const MatmulArgs& a, hipStream_t stream);
void gemv_set_staged(int mode);  // -1 the dispatcher's rule, 0 never, 1 wherever the LDS-staged decode kernel applies
bool gemv_epilogue_possible(const MatmulArgs& a);  // does the kernel that serves (M, N, K) take a.epi?
int gemv_norm_parts(int64_t M, int64_t N, int64_t K);  // partial sums per row of x an EPI_RESID_NORM call writes (0: not served)
size_t gemm_workspace_bytes(int64_t M, int64_t N, int64_t K);
hipError_t launch_gemm(const MatmulArgs& a, hipStream_t stream);
// more than 128 rows of x: one wave per SIMD, 256 x 256 or 128 x 256 tiles (nf4_gemm_wide.hip)
int gemm_wide_tile_rows(int64_t M, int64_t N, int64_t K);
hipError_t launch_gemm_wide(const MatmulArgs& a, hipStream_t stream);
size_t gemm_wide_workspace_bytes(int64_t M, int64_t N, int64_t K);
// The launch plan of the fused GEMM for a shape, as the launchers compute it: plan[0] rows of x per tile (64, 128,
// 256), plan[1] tiles (tiles of x rows times tiles of 256 weight rows), plan[2] pieces a tile is cut into along K,
// plan[3] workgroups launched.
void gemm_wide_plan(int64_t M, int64_t N, int64_t K, int plan[4]);
void gemm_plan(int64_t M, int64_t N, int64_t K, int plan[4]);
// which decode kernel serves a call without an epilogue (GEMV_KERNEL_* of nf4_gemv.h) and its arithmetic mode (ARITH_*)
void gemv_plan(int64_t M, int64_t N, int64_t K, int block_log2, bool nested, int plan[4]);
// dense bf16 GEMM (nf4_gemm_dense.hip): K a multiple of 64, at least 128
bool gemm_dense_possible(int64_t M, int64_t N, int64_t K);
size_t gemm_dense_workspace_bytes(int64_t M, int64_t N, int64_t K);
void gemm_dense_plan(int64_t M, int64_t N, int64_t K, int plan[4]);
hipError_t launch_gemm_dense(const DenseArgs& a, hipStream_t stream);

// ---------------------------------------------------------------------------------------------
// device helpers
// ---------------------------------------------------------------------------------------------

// 16-byte streaming (non-temporal) load: data that is read exactly once should not displace what
// the caches hold for re-use.
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 load16_stream(const void* p) {
    const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}

// 16-byte load as a value (a struct-typed `uint4` copy from global memory becomes a memcpy that keeps
// its destination array in scratch memory).
__device__ __forceinline__ uint4 load16(const void* p) {
    const u32x4_t v = *reinterpret_cast<const u32x4_t*>(p);
    return make_uint4(v.x, v.y, v.z, v.w);
}

// 4-byte and 16-byte streaming loads of fp32 absmax values: like the codes they are read exactly once.
__device__ __forceinline__ float load_f32_stream(const float* p) { return __builtin_nontemporal_load(p); }
__device__ __forceinline__ float4 load_f32x4_stream(const float* p) {
    typedef float f32x4_t __attribute__((ext_vector_type(4)));
    const f32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const f32x4_t*>(p));
    return make_float4(v.x, v.y, v.z, v.w);
}

// 16-byte store, ordinary or streaming (non-temporal: the data is not meant to stay in the caches).
template <bool STREAM>
__device__ __forceinline__ void store16(void* p, uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
    const u32x4_t v = {a, b, c, d};
    if (STREAM)
        __builtin_nontemporal_store(v, reinterpret_cast<u32x4_t*>(p));
    else
        *reinterpret_cast<u32x4_t*>(p) = v;
}

// fp32 -> bf16 bits, round to nearest even (finite inputs; NaN is quieted).
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
    u += 0x7fffu + ((u >> 16) & 1u);
    return u >> 16;
}

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

// Hand-off of split-K partial sums between workgroups, which may run on different XCDs (eight on this part, each with
// an L2 of its own; what they share is the memory-side Infinity Cache and HBM).  The producer stores its partials with
// agent-scope relaxed atomic stores, calls publish_partials(), then counts its arrival with an agent-scope relaxed
// RMW on the band's counter; the last arriver calls acquire_partials() and reads every producer's partials with
// agent-scope relaxed atomic loads.  What is relied on:
//   * EVERY access to the shared words -- partials and counters, writes and reads -- is itself an agent-scope atomic.
//     On this target such an access carries the cache-policy bits that make it coherent across the agent: the store
//     is written through the issuing XCD's L2 to memory, the load and the RMW are served from there and not from a
//     stale line of the reader's L1 or L2.  No plain load or store ever touches these words, so no cache holds a copy
//     that a fence would have to write back or invalidate.
//   * The producer's s_waitcnt(0) makes the wave wait until every one of its stores has been acknowledged, i.e. has
//     reached the level at which agent-scope accesses of other XCDs see it, BEFORE the arrival is counted (where one thread
//     counts for a whole workgroup, a workgroup barrier stands between the waves' waits and that RMW; where a wave
//     counts for itself, the RMW follows its own wait).  The last arriver's loads are issued after its RMW has returned -- a data dependence through the flag --
//     so they are served after every producer's acknowledged stores.
//   * The two fences are there for the COMPILER: no store may sink below the release fence, no load may be hoisted
//     above the acquire fence, and neither may move across the counter RMW between them.  At workgroup scope they
//     order nothing at agent scope in the language's memory model and emit no cache maintenance; the ordering across
//     XCDs comes from the two points above.
//   * An agent-scope fence pair would be the model-blessed spelling, but on this target it writes back and
//     invalidates the whole L2 (measured at 45 us per launch), which nothing here needs.
__device__ __forceinline__ void publish_partials() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0);
}
__device__ __forceinline__ void acquire_partials() { __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup"); }

// Reconstruct one absmax value from its nested form: (map * absmax2) + offset, two roundings.
__device__ __forceinline__ float nested_absmax(const NestedAbsmax& nq, int64_t block) {
    float m = nq.map256[nq.q[block]];
    float s = nq.absmax2[block >> nq.nested_log2];
    return __fadd_rn(__fmul_rn(m, s), nq.offset);
}

}  // namespace nf4
