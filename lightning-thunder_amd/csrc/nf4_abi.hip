// C ABI of libnf4hip.so (declared in include/nf4hip.h): argument validation, then launch.
// Every check runs before the first HIP call so that the error paths are testable without a GPU.
#include <stdarg.h>
#include <stdio.h>

#include <atomic>

#include "../../include/nf4hip.h"
#include "nf4_common.h"

// Scratch of nf4hip_gemv_static: split-K arrival counters and partial sums, in the image of the code
// object instead of a caller's buffer.  Every device that loads the library holds its own copy at its
// own address (zero-filled when the code object is loaded); in host code the name below is only a
// handle for hipGetSymbolAddress, never a device address.
static __device__ __align__(256) unsigned char scratch[NF4HIP_STATIC_SCRATCH_BYTES];

namespace {

constexpr int MAX_DEVICES = 64;
std::atomic<void*> g_scratch_ptr[MAX_DEVICES];  // device address of `scratch` on each device, once resolved

// zero fill as a kernel (a memset node recorded into a captured graph is not reliable on this target)
__global__ void fill_zero_kernel(uint4* p, size_t n16) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n16) p[i] = make_uint4(0u, 0u, 0u, 0u);
}

// Device address of the current device's copy of `scratch`.  The first call on a device resolves it
// and clears the arrival counters at its head (the kernels leave them at zero after every call, so
// this only matters if the process wrote there by other means); later calls cost one hipGetDevice.
hipError_t static_scratch(void** out, hipStream_t stream) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= MAX_DEVICES) return hipErrorInvalidDevice;
    void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        // the set-up below must run, not be recorded: refuse a first call made under stream capture
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        if (stream && hipStreamIsCapturing(stream, &cap) == hipSuccess && cap != hipStreamCaptureStatusNone)
            return hipErrorStreamCaptureUnsupported;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        if (!p) return hipErrorInvalidSymbol;
        const size_t n16 = nf4::GEMV_COUNTER_REGION_BYTES / 16;
        hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)((n16 + 255) / 256)), dim3(256), 0, stream,
                           static_cast<uint4*>(p), n16);
        if ((e = hipGetLastError()) != hipSuccess) return e;
        g_scratch_ptr[dev].store(p, std::memory_order_release);
    }
    *out = p;
    return hipSuccess;
}

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int hip_fail(const char* what, hipError_t e) {
    return fail(NF4HIP_E_HIP, "%s: %s (%d)", what, hipGetErrorString(e), (int)e);
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
bool aligned4(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 3u) == 0; }

// log2 of a supported blocksize, or -1
int block_log2(int blocksize) {
    switch (blocksize) {
        case 64: return 6;
        case 128: return 7;
        case 256: return 8;
        case 512: return 9;
        case 1024: return 10;
        case 2048: return 11;
        case 4096: return 12;
        default: return -1;
    }
}

bool valid_dtype(int d) { return d == NF4HIP_BF16 || d == NF4HIP_F16 || d == NF4HIP_F32; }

int check_nested(const uint8_t* absmax_q, const float* absmax2, const float* map256, int nested_blocksize,
                 int* nested_log2) {
    if (!absmax_q || !absmax2 || !map256) return fail(NF4HIP_E_NULL, "nested absmax: null pointer");
    *nested_log2 = block_log2(nested_blocksize);
    if (*nested_log2 < 0) return fail(NF4HIP_E_BLOCKSIZE, "nested_blocksize %d unsupported", nested_blocksize);
    if (!aligned16(absmax_q) || !aligned16(absmax2) || !aligned4(map256))
        return fail(NF4HIP_E_ALIGN, "nested absmax: absmax_q / absmax2 not 16-byte aligned or map256 not 4-byte aligned");
    return NF4HIP_OK;
}

enum MatmulKind { GEMV, GEMM };

// use_static: the workspace is the library's own `scratch` array (nf4hip_gemv_static)
int matmul_common(MatmulKind kind, const void* x, int x_dtype, int64_t M, const uint8_t* packed, const float* absmax,
                  const nf4::NestedAbsmax* nested, const float* lut16, const void* bias, int64_t N, int64_t K,
                  int blocksize, void* out, void* workspace, size_t workspace_bytes, void* stream,
                  bool use_static = false, const nf4hip_epilogue* epi = nullptr) {
    const char* name = epi ? "nf4hip_gemv_epilogue" : use_static ? "nf4hip_gemv_static" : kind == GEMV ? "nf4hip_gemv" : "nf4hip_gemm";
    if (!x || !packed || !lut16 || !out) return fail(NF4HIP_E_NULL, "%s: null pointer", name);
    if (!nested && !absmax) return fail(NF4HIP_E_NULL, "%s: absmax is null", name);
    if (x_dtype != NF4HIP_BF16)
        return fail(valid_dtype(x_dtype) ? NF4HIP_E_DTYPE : NF4HIP_E_DTYPE, "%s: only bf16 x is fused (got dtype %d)",
                    name, x_dtype);
    const int bl = block_log2(blocksize);
    if (bl < 0) return fail(NF4HIP_E_BLOCKSIZE, "%s: blocksize %d unsupported", name, blocksize);
    if (M <= 0 || N <= 0 || K <= 0) return fail(NF4HIP_E_SHAPE, "%s: M, N, K must be positive", name);
    if (N > INT32_MAX || K > INT32_MAX || M > INT32_MAX) return fail(NF4HIP_E_SHAPE, "%s: dimension too large", name);
    if (kind == GEMV) {
        if (M > 16) return fail(NF4HIP_E_SHAPE, "nf4hip_gemv: M = %lld > 16", (long long)M);
        if (M <= 4 ? K % 32 : K % 512)
            return fail(NF4HIP_E_SHAPE, "nf4hip_gemv: K = %lld is not a multiple of %d (M = %lld)", (long long)K,
                        M <= 4 ? 32 : 512, (long long)M);
        if (M > 4 && K > (1 << 24))
            return fail(NF4HIP_E_SHAPE, "nf4hip_gemv: K = %lld > 2^24 with M > 4 (use nf4hip_gemm)", (long long)K);
    } else {
        if (K % 64) return fail(NF4HIP_E_SHAPE, "nf4hip_gemm: K = %lld is not a multiple of 64", (long long)K);
    }
    if (!(kind == GEMV && M <= 4) && K % blocksize)
        return fail(NF4HIP_E_SHAPE, "%s: blocksize %d does not divide K = %lld", name, blocksize, (long long)K);
    if (!aligned16(x) || !aligned16(packed) || !aligned16(out) || (absmax && !aligned16(absmax)) ||
        (bias && (reinterpret_cast<uintptr_t>(bias) & 1u)) || !aligned4(lut16))
        return fail(NF4HIP_E_ALIGN, "%s: x / packed / absmax / out not 16-byte aligned, lut16 not 4-byte or bias not 2-byte aligned",
                    name);
    const size_t need = kind == GEMV ? nf4::gemv_workspace_bytes(M, N, K) : nf4::gemm_workspace_bytes(M, N, K);
    if (use_static) {
        if (need > (size_t)NF4HIP_STATIC_SCRATCH_BYTES)
            return fail(NF4HIP_E_WORKSPACE,
                        "%s: this shape needs %zu bytes of scratch, the built-in array holds %zu (use nf4hip_gemv with a "
                        "workspace)",
                        name, need, (size_t)NF4HIP_STATIC_SCRATCH_BYTES);
    } else if (need) {
        if (!workspace || workspace_bytes < need)
            return fail(NF4HIP_E_WORKSPACE, "%s: workspace of %zu bytes required, got %zu", name, need,
                        workspace ? workspace_bytes : (size_t)0);
        if (!aligned16(workspace)) return fail(NF4HIP_E_ALIGN, "%s: workspace not 16-byte aligned", name);
    }

    nf4::MatmulArgs a;
    a.x = static_cast<const uint16_t*>(x);
    a.packed = packed;
    a.absmax = absmax;
    a.nested = nested ? *nested : nf4::NestedAbsmax{nullptr, nullptr, nullptr, 0.0f, 0};
    a.lut16 = lut16;
    a.bias = static_cast<const uint16_t*>(bias);
    a.out = static_cast<uint16_t*>(out);
    a.M = (int)M;
    a.N = (int)N;
    a.K = (int)K;
    a.block_log2 = bl;
    a.workspace = workspace;
    a.workspace_bytes = workspace_bytes;
    a.epi = nf4::Epilogue{nf4::EPI_NONE, 0.0f, nullptr, 0, nullptr, nullptr, nullptr, nullptr, nullptr};
    if (epi && epi->flags) {
        const int f = epi->flags;
        const bool scale = f & NF4HIP_EPI_ROWSCALE, pairs = f & NF4HIP_EPI_SILU_PAIRS, resid = f & NF4HIP_EPI_RESID_NORM;
        if ((f & ~(NF4HIP_EPI_ROWSCALE | NF4HIP_EPI_SILU_PAIRS | NF4HIP_EPI_RESID_NORM)) || (resid && (scale || pairs)))
            return fail(NF4HIP_E_SHAPE, "%s: flags %d: RESID_NORM stands alone, ROWSCALE and SILU_PAIRS may be combined", name, f);
        if (scale && (!epi->in_sumsq || epi->in_parts <= 0))
            return fail(NF4HIP_E_NULL, "%s: ROWSCALE needs in_sumsq and in_parts > 0", name);
        if (resid && (!epi->resid_in || !epi->norm_weight || !epi->resid_out || !epi->xnext_out || !epi->out_sumsq))
            return fail(NF4HIP_E_NULL, "%s: RESID_NORM needs resid_in, norm_weight, resid_out, xnext_out and out_sumsq", name);
        if ((scale && !aligned4(epi->in_sumsq)) || (resid && !aligned4(epi->out_sumsq)) ||
            (resid && ((reinterpret_cast<uintptr_t>(epi->resid_in) | reinterpret_cast<uintptr_t>(epi->norm_weight) |
                        reinterpret_cast<uintptr_t>(epi->resid_out) | reinterpret_cast<uintptr_t>(epi->xnext_out)) & 1u)))
            return fail(NF4HIP_E_ALIGN, "%s: an epilogue tensor is not aligned to its element size", name);
        a.epi = nf4::Epilogue{f, epi->eps, epi->in_sumsq, epi->in_parts, static_cast<const uint16_t*>(epi->resid_in),
                              static_cast<const uint16_t*>(epi->norm_weight), static_cast<uint16_t*>(epi->resid_out),
                              static_cast<uint16_t*>(epi->xnext_out), epi->out_sumsq};
        if (!nf4::gemv_epilogue_possible(a))
            return fail(NF4HIP_E_SHAPE, "%s: M = %lld, N = %lld, K = %lld with flags %d is not served (run nf4hip_gemv and the operation by itself)",
                        name, (long long)M, (long long)N, (long long)K, f);
    }
    if (use_static) {
        const hipError_t es = static_scratch(&a.workspace, static_cast<hipStream_t>(stream));
        if (es != hipSuccess) return hip_fail(name, es);
        a.workspace_bytes = NF4HIP_STATIC_SCRATCH_BYTES;
    }
    const hipError_t e = kind == GEMV ? nf4::launch_gemv(a, static_cast<hipStream_t>(stream))
                                      : nf4::launch_gemm(a, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail(name, e);
    return NF4HIP_OK;
}

}  // namespace

extern "C" {

int nf4hip_abi_version(void) { return NF4HIP_ABI_VERSION; }

const char* nf4hip_last_error(void) { return g_err; }

int nf4hip_quantize(const void* w, int w_dtype, int64_t n, int blocksize, uint8_t* packed, float* absmax,
                    void* stream) {
    if (n < 0) return fail(NF4HIP_E_SHAPE, "nf4hip_quantize: n = %lld is negative", (long long)n);
    if (!valid_dtype(w_dtype)) return fail(NF4HIP_E_DTYPE, "nf4hip_quantize: unknown dtype code %d", w_dtype);
    const int bl = block_log2(blocksize);
    if (bl < 0) return fail(NF4HIP_E_BLOCKSIZE, "nf4hip_quantize: blocksize %d unsupported", blocksize);
    if (n == 0) return NF4HIP_OK;
    if (!w || !packed || !absmax) return fail(NF4HIP_E_NULL, "nf4hip_quantize: null pointer");
    if (!aligned16(w) || !aligned16(packed) || !aligned16(absmax))
        return fail(NF4HIP_E_ALIGN, "nf4hip_quantize: pointer not 16-byte aligned");
    const hipError_t e = nf4::launch_quantize(w, w_dtype, n, bl, packed, absmax, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail("nf4hip_quantize", e);
    return NF4HIP_OK;
}

int nf4hip_dequantize(const uint8_t* packed, const float* absmax, const float* lut16, int64_t n, int blocksize,
                      void* out, int out_dtype, void* stream) {
    if (n < 0) return fail(NF4HIP_E_SHAPE, "nf4hip_dequantize: n = %lld is negative", (long long)n);
    if (!valid_dtype(out_dtype)) return fail(NF4HIP_E_DTYPE, "nf4hip_dequantize: unknown dtype code %d", out_dtype);
    const int bl = block_log2(blocksize);
    if (bl < 0) return fail(NF4HIP_E_BLOCKSIZE, "nf4hip_dequantize: blocksize %d unsupported", blocksize);
    if (n == 0) return NF4HIP_OK;
    if (!packed || !absmax || !lut16 || !out) return fail(NF4HIP_E_NULL, "nf4hip_dequantize: null pointer");
    if (!aligned16(packed) || !aligned16(absmax) || !aligned16(out) || !aligned4(lut16))
        return fail(NF4HIP_E_ALIGN, "nf4hip_dequantize: packed / absmax / out not 16-byte aligned or lut16 not 4-byte aligned");
    const nf4::NestedAbsmax none{nullptr, nullptr, nullptr, 0.0f, 0};
    const hipError_t e =
        nf4::launch_dequantize(packed, absmax, none, lut16, n, bl, out, out_dtype, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail("nf4hip_dequantize", e);
    return NF4HIP_OK;
}

int nf4hip_dq_compress(const float* absmax, int64_t nblocks, int nested_blocksize, const float* map256, float offset,
                       uint8_t* absmax_q, float* absmax2, void* stream) {
    if (nblocks < 0) return fail(NF4HIP_E_SHAPE, "nf4hip_dq_compress: nblocks is negative");
    const int nl = block_log2(nested_blocksize);
    if (nl < 0) return fail(NF4HIP_E_BLOCKSIZE, "nf4hip_dq_compress: nested_blocksize %d unsupported", nested_blocksize);
    if (nblocks == 0) return NF4HIP_OK;
    if (!absmax || !map256 || !absmax_q || !absmax2) return fail(NF4HIP_E_NULL, "nf4hip_dq_compress: null pointer");
    if (!aligned16(absmax) || !aligned16(absmax_q) || !aligned16(absmax2) || !aligned4(map256))
        return fail(NF4HIP_E_ALIGN, "nf4hip_dq_compress: absmax / absmax_q / absmax2 not 16-byte aligned or map256 not 4-byte aligned");
    const hipError_t e =
        nf4::launch_dq_compress(absmax, nblocks, nl, map256, offset, absmax_q, absmax2, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail("nf4hip_dq_compress", e);
    return NF4HIP_OK;
}

int nf4hip_dq_reconstruct(const uint8_t* absmax_q, const float* absmax2, const float* map256, float offset,
                          int64_t nblocks, int nested_blocksize, float* absmax, void* stream) {
    if (nblocks < 0) return fail(NF4HIP_E_SHAPE, "nf4hip_dq_reconstruct: nblocks is negative");
    const int nl = block_log2(nested_blocksize);
    if (nl < 0)
        return fail(NF4HIP_E_BLOCKSIZE, "nf4hip_dq_reconstruct: nested_blocksize %d unsupported", nested_blocksize);
    if (nblocks == 0) return NF4HIP_OK;
    if (!absmax_q || !absmax2 || !map256 || !absmax) return fail(NF4HIP_E_NULL, "nf4hip_dq_reconstruct: null pointer");
    if (!aligned16(absmax) || !aligned16(absmax_q) || !aligned16(absmax2) || !aligned4(map256))
        return fail(NF4HIP_E_ALIGN, "nf4hip_dq_reconstruct: absmax / absmax_q / absmax2 not 16-byte aligned or map256 not 4-byte aligned");
    const nf4::NestedAbsmax nq{absmax_q, absmax2, map256, offset, nl};
    const hipError_t e = nf4::launch_dq_reconstruct(nq, nblocks, absmax, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail("nf4hip_dq_reconstruct", e);
    return NF4HIP_OK;
}

int nf4hip_dequantize_dq(const uint8_t* packed, const uint8_t* absmax_q, const float* absmax2, const float* map256,
                         float offset, int nested_blocksize, const float* lut16, int64_t n, int blocksize, void* out,
                         int out_dtype, void* stream) {
    if (n < 0) return fail(NF4HIP_E_SHAPE, "nf4hip_dequantize_dq: n = %lld is negative", (long long)n);
    if (!valid_dtype(out_dtype)) return fail(NF4HIP_E_DTYPE, "nf4hip_dequantize_dq: unknown dtype code %d", out_dtype);
    const int bl = block_log2(blocksize);
    if (bl < 0) return fail(NF4HIP_E_BLOCKSIZE, "nf4hip_dequantize_dq: blocksize %d unsupported", blocksize);
    if (n == 0) return NF4HIP_OK;
    if (!packed || !lut16 || !out) return fail(NF4HIP_E_NULL, "nf4hip_dequantize_dq: null pointer");
    int nl = 0;
    const int rc = check_nested(absmax_q, absmax2, map256, nested_blocksize, &nl);
    if (rc) return rc;
    if (!aligned16(packed) || !aligned16(out) || !aligned4(lut16))
        return fail(NF4HIP_E_ALIGN, "nf4hip_dequantize_dq: packed / out not 16-byte aligned or lut16 not 4-byte aligned");
    const nf4::NestedAbsmax nq{absmax_q, absmax2, map256, offset, nl};
    const hipError_t e =
        nf4::launch_dequantize(packed, nullptr, nq, lut16, n, bl, out, out_dtype, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail("nf4hip_dequantize_dq", e);
    return NF4HIP_OK;
}

size_t nf4hip_gemv_workspace_bytes(int64_t M, int64_t N, int64_t K) { return nf4::gemv_workspace_bytes(M, N, K); }

int nf4hip_gemv_prefer_staged(int mode) {
    if (mode < -1 || mode > 1) return fail(NF4HIP_E_SHAPE, "nf4hip_gemv_prefer_staged: mode %d is not -1, 0 or 1", mode);
    nf4::gemv_set_staged(mode);
    return NF4HIP_OK;
}
size_t nf4hip_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K) { return nf4::gemm_workspace_bytes(M, N, K); }

int nf4hip_gemm_plan(int64_t M, int64_t N, int64_t K, int32_t plan[4]) {
    if (!plan) return fail(NF4HIP_E_NULL, "nf4hip_gemm_plan: plan is null");
    if (M <= 0 || N <= 0 || K <= 0 || N > INT32_MAX || K > INT32_MAX || M > INT32_MAX || K % 64)
        return fail(NF4HIP_E_SHAPE, "nf4hip_gemm_plan: M, N, K must be positive and K a multiple of 64");
    int p[4];
    nf4::gemm_plan(M, N, K, p);
    for (int i = 0; i < 4; ++i) plan[i] = p[i];
    return NF4HIP_OK;
}

int nf4hip_gemv_plan(int64_t M, int64_t N, int64_t K, int blocksize, int nested, int32_t plan[4]) {
    if (!plan) return fail(NF4HIP_E_NULL, "nf4hip_gemv_plan: plan is null");
    const int bl = block_log2(blocksize);
    if (bl < 0) return fail(NF4HIP_E_BLOCKSIZE, "nf4hip_gemv_plan: blocksize %d unsupported", blocksize);
    if (M <= 0 || M > 16 || N <= 0 || K <= 0 || N > INT32_MAX || K > INT32_MAX || (M <= 4 ? K % 32 : K % 512) ||
        (M > 4 && K > (1 << 24)))
        return fail(NF4HIP_E_SHAPE, "nf4hip_gemv_plan: not a shape nf4hip_gemv takes (M = %lld, N = %lld, K = %lld)", (long long)M,
                    (long long)N, (long long)K);
    int p[4];
    nf4::gemv_plan(M, N, K, bl, nested != 0, p);
    for (int i = 0; i < 4; ++i) plan[i] = p[i];
    return NF4HIP_OK;
}

int nf4hip_gemv(const void* x, int x_dtype, int64_t M, const uint8_t* packed, const float* absmax, const float* lut16,
                const void* bias_or_null, int64_t N, int64_t K, int blocksize, void* out, void* workspace,
                size_t workspace_bytes, void* stream) {
    return matmul_common(GEMV, x, x_dtype, M, packed, absmax, nullptr, lut16, bias_or_null, N, K, blocksize, out,
                         workspace, workspace_bytes, stream);
}

int nf4hip_gemv_static(const void* x, int x_dtype, int64_t M, const uint8_t* packed, const float* absmax,
                       const float* lut16, const void* bias_or_null, int64_t N, int64_t K, int blocksize, void* out,
                       void* stream) {
    return matmul_common(GEMV, x, x_dtype, M, packed, absmax, nullptr, lut16, bias_or_null, N, K, blocksize, out,
                         nullptr, 0, stream, true);
}

int nf4hip_gemv_epilogue(const void* x, int x_dtype, int64_t M, const uint8_t* packed, const float* absmax,
                         const float* lut16, const void* bias_or_null, int64_t N, int64_t K, int blocksize, void* out,
                         void* workspace, size_t workspace_bytes, const nf4hip_epilogue* epilogue, void* stream) {
    if (!epilogue) return fail(NF4HIP_E_NULL, "nf4hip_gemv_epilogue: epilogue is null");
    // RESID_NORM writes resid_out / xnext_out instead of out
    if (!out && (epilogue->flags & NF4HIP_EPI_RESID_NORM)) out = epilogue->xnext_out;
    return matmul_common(GEMV, x, x_dtype, M, packed, absmax, nullptr, lut16, bias_or_null, N, K, blocksize, out,
                         workspace, workspace_bytes, stream, false, epilogue);
}

int nf4hip_gemv_epilogue_served(int64_t M, int64_t N, int64_t K, int blocksize, int flags, int in_parts) {
    const int bl = block_log2(blocksize);
    if (bl < 0 || M <= 0 || M > 16 || N <= 0 || K <= 0 || N > INT32_MAX || K > INT32_MAX) return 0;
    if ((M <= 4 ? K % 32 : K % 512) || (M > 4 && (K > (1 << 24) || K % blocksize))) return 0;
    if (flags <= 0 || (flags & ~(NF4HIP_EPI_ROWSCALE | NF4HIP_EPI_SILU_PAIRS | NF4HIP_EPI_RESID_NORM)) ||
        ((flags & NF4HIP_EPI_RESID_NORM) && flags != NF4HIP_EPI_RESID_NORM))
        return 0;
    nf4::MatmulArgs a{};
    a.M = (int)M;
    a.N = (int)N;
    a.K = (int)K;
    a.block_log2 = bl;
    a.epi.flags = flags;
    a.epi.in_parts = in_parts;
    return nf4::gemv_epilogue_possible(a) ? 1 : 0;
}

int nf4hip_gemv_norm_parts(int64_t M, int64_t N, int64_t K) {
    if (M <= 0 || N <= 0 || K <= 0 || M > 16) return 0;
    return nf4::gemv_norm_parts(M, N, K);
}

int nf4hip_gemv_dq(const void* x, int x_dtype, int64_t M, const uint8_t* packed, const uint8_t* absmax_q,
                   const float* absmax2, const float* map256, float offset, int nested_blocksize, const float* lut16,
                   const void* bias_or_null, int64_t N, int64_t K, int blocksize, void* out, void* workspace,
                   size_t workspace_bytes, void* stream) {
    int nl = 0;
    const int rc = check_nested(absmax_q, absmax2, map256, nested_blocksize, &nl);
    if (rc) return rc;
    const nf4::NestedAbsmax nq{absmax_q, absmax2, map256, offset, nl};
    return matmul_common(GEMV, x, x_dtype, M, packed, nullptr, &nq, lut16, bias_or_null, N, K, blocksize, out,
                         workspace, workspace_bytes, stream);
}

int nf4hip_gemm(const void* x, int x_dtype, int64_t M, const uint8_t* packed, const float* absmax, const float* lut16,
                const void* bias_or_null, int64_t N, int64_t K, int blocksize, void* out, void* workspace,
                size_t workspace_bytes, void* stream) {
    return matmul_common(GEMM, x, x_dtype, M, packed, absmax, nullptr, lut16, bias_or_null, N, K, blocksize, out,
                         workspace, workspace_bytes, stream);
}

size_t nf4hip_linear_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    if (M <= 0 || N <= 0 || K <= 0 || !nf4::gemm_dense_possible(M, N, K)) return 0;
    return nf4::gemm_dense_workspace_bytes(M, N, K);
}

int nf4hip_linear_plan(int64_t M, int64_t N, int64_t K, int32_t plan[4]) {
    if (!plan) return fail(NF4HIP_E_NULL, "nf4hip_linear_plan: plan is null");
    if (M <= 0 || N <= 0 || K <= 0 || N > INT32_MAX || K > INT32_MAX || M > INT32_MAX || !nf4::gemm_dense_possible(M, N, K))
        return fail(NF4HIP_E_SHAPE, "nf4hip_linear_plan: M, N, K must be positive and K a multiple of 64, at least 128");
    int p[4];
    nf4::gemm_dense_plan(M, N, K, p);
    for (int i = 0; i < 4; ++i) plan[i] = p[i];
    return NF4HIP_OK;
}

int nf4hip_linear(const void* x, int x_dtype, int64_t M, const void* w, const void* bias_or_null, int64_t N, int64_t K,
                  void* out, void* workspace, size_t workspace_bytes, void* stream) {
    const char* name = "nf4hip_linear";
    if (!x || !w || !out) return fail(NF4HIP_E_NULL, "%s: null pointer", name);
    if (x_dtype != NF4HIP_BF16) return fail(NF4HIP_E_DTYPE, "%s: only bf16 operands (got dtype %d)", name, x_dtype);
    if (M <= 0 || N <= 0 || K <= 0) return fail(NF4HIP_E_SHAPE, "%s: M, N, K must be positive", name);
    if (N > INT32_MAX || K > INT32_MAX || M > INT32_MAX) return fail(NF4HIP_E_SHAPE, "%s: dimension too large", name);
    if (!nf4::gemm_dense_possible(M, N, K))
        return fail(NF4HIP_E_SHAPE, "%s: K = %lld must be a multiple of 64, at least 128", name, (long long)K);
    if (!aligned16(x) || !aligned16(w) || !aligned16(out) || (bias_or_null && (reinterpret_cast<uintptr_t>(bias_or_null) & 1u)))
        return fail(NF4HIP_E_ALIGN, "%s: x / w / out not 16-byte aligned or bias not 2-byte aligned", name);
    const size_t need = nf4::gemm_dense_workspace_bytes(M, N, K);
    if (need) {
        if (!workspace || workspace_bytes < need)
            return fail(NF4HIP_E_WORKSPACE, "%s: workspace of %zu bytes required, got %zu", name, need,
                        workspace ? workspace_bytes : (size_t)0);
        if (!aligned16(workspace)) return fail(NF4HIP_E_ALIGN, "%s: workspace not 16-byte aligned", name);
    }
    nf4::DenseArgs a;
    a.x = static_cast<const uint16_t*>(x);
    a.w = static_cast<const uint16_t*>(w);
    a.bias = static_cast<const uint16_t*>(bias_or_null);
    a.out = static_cast<uint16_t*>(out);
    a.M = (int)M;
    a.N = (int)N;
    a.K = (int)K;
    a.workspace = need ? workspace : nullptr;
    a.workspace_bytes = need ? workspace_bytes : 0;
    const hipError_t e = nf4::launch_gemm_dense(a, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail(name, e);
    return NF4HIP_OK;
}

int nf4hip_gemm_dq(const void* x, int x_dtype, int64_t M, const uint8_t* packed, const uint8_t* absmax_q,
                   const float* absmax2, const float* map256, float offset, int nested_blocksize, const float* lut16,
                   const void* bias_or_null, int64_t N, int64_t K, int blocksize, void* out, void* workspace,
                   size_t workspace_bytes, void* stream) {
    int nl = 0;
    const int rc = check_nested(absmax_q, absmax2, map256, nested_blocksize, &nl);
    if (rc) return rc;
    const nf4::NestedAbsmax nq{absmax_q, absmax2, map256, offset, nl};
    return matmul_common(GEMM, x, x_dtype, M, packed, nullptr, &nq, lut16, bias_or_null, N, K, blocksize, out,
                         workspace, workspace_bytes, stream);
}

}  // extern "C"
