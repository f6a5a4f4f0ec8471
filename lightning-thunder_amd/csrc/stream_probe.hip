// A kernel that only reads: what one launch can stream from HBM on this part, for bench.py to print next to the decode
// kernels' times (a measuring aid in a library of its own, libnf4hip_probe.so; nothing on the path uses it).
// 512 workgroups of 512 threads (two per CU, as the row kernel runs); a wave reads consecutive 1 KB pieces -- whole
// 128-byte lines, 16 bytes per lane, non-temporal -- four in flight per lane, first from `a`, then from `b` (the codes and
// the absmax of a weight).  What is read is folded into one word per lane that is stored only if it equals a value it
// never takes, so the loads cannot be dropped.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
constexpr int THREADS = 512, WAVES = THREADS / 64, GRID = 512, U = 4;

__global__ __launch_bounds__(THREADS) void stream_read_kernel(const u32x4* __restrict__ a, int64_t a16, const u32x4* __restrict__ b,
                                                              int64_t b16, int per_wave, uint32_t* sink) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t first = ((int64_t)blockIdx.x * WAVES + wave) * per_wave;  // in 1 KB pieces of a followed by b
    const int64_t a_pieces = (a16 + 63) >> 6;
    uint32_t acc = 0;
    for (int i0 = 0; i0 < per_wave; i0 += U) {
        u32x4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int64_t piece = first + i0 + u;
            const bool in_a = piece < a_pieces;
            const int64_t idx = (in_a ? piece : piece - a_pieces) * 64 + lane;
            v[u] = u32x4{0, 0, 0, 0};
            if (i0 + u < per_wave && idx < (in_a ? a16 : b16)) v[u] = __builtin_nontemporal_load((in_a ? a : b) + idx);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) acc += (v[u].x ^ v[u].y) + (v[u].z ^ v[u].w);
    }
    if (acc == 0x9e3779b9u && sink) sink[0] = acc;
}

}  // namespace

// Reads a_bytes from a and b_bytes from b (multiples of 16, 16-byte aligned device pointers; b may be NULL with 0 bytes).
// Returns 0 or the hipError_t of the launch.
extern "C" __attribute__((visibility("default"))) int nf4hip_probe_stream_read(const void* a, int64_t a_bytes, const void* b,
                                                                                int64_t b_bytes, void* sink, void* stream) {
    if (!a || a_bytes < 0 || b_bytes < 0 || (a_bytes | b_bytes) % 16 || (b_bytes && !b)) return (int)hipErrorInvalidValue;
    const int64_t a16 = a_bytes / 16, b16 = b_bytes / 16;
    const int64_t pieces = ((a16 + 63) >> 6) + ((b16 + 63) >> 6);
    const int per_wave = (int)((pieces + (int64_t)GRID * WAVES - 1) / ((int64_t)GRID * WAVES));
    hipLaunchKernelGGL(stream_read_kernel, dim3(GRID), dim3(THREADS), 0, static_cast<hipStream_t>(stream),
                       static_cast<const u32x4*>(a), a16, static_cast<const u32x4*>(b), b16, per_wave, static_cast<uint32_t*>(sink));
    return (int)hipGetLastError();
}
