/*
 * nf4hip.h -- C ABI of libnf4hip.so: NF4 blockwise weight-only quantisation kernels for
 * AMD MI355X (gfx950).  Plain pointers and sizes only; no torch types.
 *
 * This is the boundary that replaces the third-party calls made by Thunder's 4-bit path:
 *   thunder/transforms/quantization.py:63     bitsandbytes.functional.quantize_4bit(w, quant_type="nf4")
 *   thunder/transforms/quantization.py:34-39  bitsandbytes.matmul_4bit(x, qweight.t(), bias, quant_state)
 *       -> gemv_4bit                 (single-row x)              -> nf4hip_gemv
 *       -> dequantize_4bit + linear  (everything else)           -> nf4hip_dequantize / nf4hip_gemm
 *
 * Conventions
 *   - Every function returns 0 on success or a negative NF4HIP_E_* code; the text of the last
 *     failure on the calling thread is available from nf4hip_last_error().
 *   - All argument validation happens before the first HIP call, so every error code except
 *     NF4HIP_E_HIP can be reached on a machine without a GPU.
 *   - All data pointers are BORROWED DEVICE pointers; the caller keeps them alive until the work
 *     queued on `stream` has finished.  Outputs are caller-allocated.
 *   - `stream` is a hipStream_t (NULL = the default stream).  Nothing here synchronises the
 *     device, allocates or frees memory, or blocks the host.
 *   - Alignment (else NF4HIP_E_ALIGN): tensors that the kernels read or write in 128-bit pieces -- x, w, packed,
 *     absmax, absmax_q, absmax2, out, workspace -- must be 16-byte aligned; the small tables read element by
 *     element need their natural alignment only: lut16 and map256 4 bytes, bias 2 bytes.
 *   - dtype codes: NF4HIP_BF16 = 0, NF4HIP_F16 = 1, NF4HIP_F32 = 2.
 *   - Weight layout: the [N, K] weight is flattened row-major into n = N*K elements; quantisation
 *     blocks are `blocksize` consecutive elements of that flat view.  `packed` holds two 4-bit
 *     codes per byte, the element with the even index in the HIGH nibble; `absmax` holds one
 *     fp32 per block; `lut16` is the 16-entry fp32 code book (the op's `quant_map` argument).
 */
#ifndef NF4HIP_H
#define NF4HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NF4HIP_ABI_VERSION 6

#define NF4HIP_BF16 0
#define NF4HIP_F16 1
#define NF4HIP_F32 2

#define NF4HIP_OK 0
#define NF4HIP_E_NULL (-1)      /* a required pointer is NULL */
#define NF4HIP_E_DTYPE (-2)     /* dtype code unknown or unsupported by this entry point */
#define NF4HIP_E_BLOCKSIZE (-3) /* blocksize not one of 64,128,256,512,1024,2048,4096 */
#define NF4HIP_E_SHAPE (-4)     /* a size is negative/zero where it may not be, or violates a fast-path rule */
#define NF4HIP_E_ALIGN (-5)     /* a pointer is not aligned as the rules above ask */
#define NF4HIP_E_WORKSPACE (-6) /* workspace missing or smaller than nf4hip_*_workspace_bytes() */
#define NF4HIP_E_HIP (-7)       /* a HIP runtime call failed; text in nf4hip_last_error() */

/* ABI version of the loaded library; the host side refuses a mismatch. */
int nf4hip_abi_version(void);

/* Thread-local description of the last failure on this thread ("" if none). */
const char* nf4hip_last_error(void);

/*
 * Blockwise NF4 quantisation.  Replaces bitsandbytes.functional.quantize_4bit(A, blocksize,
 * quant_type="nf4") as called at thunder/transforms/quantization.py:63.
 *   w        n elements of dtype w_dtype (bf16/f16/f32)
 *   packed   (n+1)/2 bytes out
 *   absmax   ceil(n/blocksize) fp32 out
 * absmax = max|w| per block; code = #{thresholds < w * (1.0f/absmax)}.  n == 0 is a no-op.
 */
int nf4hip_quantize(const void* w, int w_dtype, int64_t n, int blocksize, uint8_t* packed, float* absmax,
                    void* stream);

/*
 * Blockwise NF4 dequantisation.  Replaces bitsandbytes.functional.dequantize_4bit (reached from
 * matmul_4bit, thunder/transforms/quantization.py:39).
 *   out[i] = round_to_nearest_even(out_dtype, lut16[code_i] * absmax[i / blocksize])
 */
int nf4hip_dequantize(const uint8_t* packed, const float* absmax, const float* lut16, int64_t n, int blocksize,
                      void* out, int out_dtype, void* stream);

/*
 * Nested ("double") quantisation of absmax, bitsandbytes' compress_statistics=True.  The
 * reference transform does not call it (thunder/transforms/quantization.py:84 "TODO: double
 * quant support"); provided for 70B-class shapes.
 *   compress:    r = absmax - offset; absmax2[c] = max|r| over nested block c;
 *                absmax_q[b] = argmin_j |r_b * (1.0f/absmax2[c]) - map256[j]|   (lowest j on ties)
 *   reconstruct: absmax[b] = map256[absmax_q[b]] * absmax2[b / nested_blocksize] + offset
 * nested_blocksize must be a power of two in [64, 4096].
 */
int nf4hip_dq_compress(const float* absmax, int64_t nblocks, int nested_blocksize, const float* map256, float offset,
                       uint8_t* absmax_q, float* absmax2, void* stream);
int nf4hip_dq_reconstruct(const uint8_t* absmax_q, const float* absmax2, const float* map256, float offset,
                          int64_t nblocks, int nested_blocksize, float* absmax, void* stream);

/* Same as nf4hip_dequantize with absmax given in nested form. */
int nf4hip_dequantize_dq(const uint8_t* packed, const uint8_t* absmax_q, const float* absmax2, const float* map256,
                         float offset, int nested_blocksize, const float* lut16, int64_t n, int blocksize, void* out,
                         int out_dtype, void* stream);

/*
 * Decode-shape fused dequant-matmul, 1 <= M <= 16.  Replaces bitsandbytes' gemv_4bit
 * (kgemm_4bit_inference_naive), reached from thunder/transforms/quantization.py:39.
 *   out[m][n] = bf16( sum_k x[m][k] * lut16[code(n,k)] * absmax[(n*K+k)/blocksize] + bias[n] )
 *   x    [M, K] bf16 row-major      out  [M, N] bf16 row-major      bias [N] bf16 or NULL
 * Fast-path rules (else NF4HIP_E_SHAPE; the host side then takes dequantize + matmul):
 *   x_dtype == NF4HIP_BF16; M <= 4: K % 32 == 0; M >= 5: K % 512 == 0, blocksize divides K, K <= 2^24.
 * `workspace` must hold nf4hip_gemv_workspace_bytes(M,N,K) bytes, be 16-byte aligned, and have
 * been ZEROED once before its first use; every call leaves it zeroed where that matters, so it
 * can be reused by later calls on the same stream.  Two calls that may overlap in time (different
 * streams) need different workspaces.
 */
size_t nf4hip_gemv_workspace_bytes(int64_t M, int64_t N, int64_t K);
/*
 * Process-wide choice among the decode kernels behind nf4hip_gemv (all give results within the same tolerance of the
 * reference; they differ in how the weight stream reaches the matrix pipe): 1 = the kernel that stages codes and absmax
 * through LDS wherever it applies (fp32 absmax, blocksize 64, K a multiple of 256 up to 8192), 0 = never that kernel,
 * -1 = the library's own rule (the default; the environment variable NF4HIP_STAGE presets it).  For measurements and
 * tests; nf4hip_gemv_workspace_bytes covers every choice.
 */
int nf4hip_gemv_prefer_staged(int mode);
/*
 * Which of the decode kernels nf4hip_gemv launches for a call without an epilogue (no GPU needed; follows
 * nf4hip_gemv_prefer_staged): plan[0] = 1 row-streaming, 2 four weight rows per lane quad, 3 the same on two halves of
 * x, 4 MFMA tiles with x in LDS, 5 codes and absmax staged through LDS; plan[1] = the arithmetic of the call: 0 bf16 code
 * book, 1 fp16 code book, 2 every weight rounded to bf16(code value * absmax) as the reference rounds it; plan[2],
 * plan[3] reserved (0).  `nested` non-zero: the call would go through nf4hip_gemv_dq.  For benchmarks and profiles that
 * attribute time to kernels; results never depend on the choice beyond the tolerance of the call.
 */
int nf4hip_gemv_plan(int64_t M, int64_t N, int64_t K, int blocksize, int nested, int32_t plan[4]);
int nf4hip_gemv(const void* x, int x_dtype, int64_t M, const uint8_t* packed, const float* absmax, const float* lut16,
                const void* bias_or_null, int64_t N, int64_t K, int blocksize, void* out, void* workspace,
                size_t workspace_bytes, void* stream);
int nf4hip_gemv_dq(const void* x, int x_dtype, int64_t M, const uint8_t* packed, const uint8_t* absmax_q,
                   const float* absmax2, const float* map256, float offset, int nested_blocksize, const float* lut16,
                   const void* bias_or_null, int64_t N, int64_t K, int blocksize, void* out, void* workspace,
                   size_t workspace_bytes, void* stream);

/*
 * nf4hip_gemv with an epilogue: the thread that finishes an output also does the element-wise / normalising step
 * that follows (or precedes) the linear in a decoder layer, so that a decode step needs one launch per linear instead
 * of two.  In the reference these steps are fusions of its other executors around bnb_matmul_nf4
 * (thunder/transforms/quantization.py:34-39 has no epilogue); at one to sixteen rows of x each of them costs a launch
 * that takes as long as a small linear.  Every output is finished by exactly one thread, so nothing is computed twice.
 * fp32 absmax only; same rules as nf4hip_gemv otherwise.  What the serving kernel does not take returns
 * NF4HIP_E_SHAPE (run nf4hip_gemv and the step by itself; nf4hip_gemv_epilogue_served answers beforehand):
 * one row of x with K > 16384 (the row kernel wants whole rows of x in one workgroup); a blocksize other than
 * 64 where the MFMA tile kernel serves (nine and more rows of x beyond 2^24 weights, five and more beyond 2^26);
 * RESID_NORM there with N > 8192; SILU_PAIRS with an odd N; ROWSCALE with in_parts > 512.
 *
 *   NF4HIP_EPI_SILU_PAIRS   weight rows 2j and 2j+1 are row j of the gate and of the up projection; out is [M, N/2]:
 *                           out[m][j] = bf16( bf16(silu(g)) * u ), g = bf16(sum[m][2j]), u = bf16(sum[m][2j+1])
 *                           -- what SiLU(gate) * up on the bf16 output of nf4hip_gemv gives, bit for bit.
 *   NF4HIP_EPI_RESID_NORM   d = bf16(sum[m][n] + bias[n]); r = bf16(resid_in[m][n] + d) -> resid_out[m][n];
 *                           bf16(r * norm_weight[n]) -> xnext_out[m][n]; the sum of r^2 over the outputs of one
 *                           workgroup (of one 16-row tile in the tile kernel, of one row range of a launch of the
 *                           LDS-staged kernel) -> out_sumsq[m * parts + i], i < parts =
 *                           nf4hip_gemv_norm_parts(M, N, K); what slot i holds does not depend on timing.
 *                           `out` is not written (NULL accepted).  resid_out may be resid_in.
 *   NF4HIP_EPI_ROWSCALE     x is the xnext_out of a RESID_NORM call and in_sumsq / in_parts its out_sumsq / parts:
 *                           sum[m][n] is multiplied by 1 / sqrt(sum_p in_sumsq[m][p] / K + eps) before the bias, i.e.
 *                           out = linear(rms_norm(r) * norm_weight) with the per-row factor applied to the finished
 *                           sums instead of to every element.  May be combined with SILU_PAIRS.
 */
#define NF4HIP_EPI_ROWSCALE 1
#define NF4HIP_EPI_SILU_PAIRS 2
#define NF4HIP_EPI_RESID_NORM 4
typedef struct nf4hip_epilogue {
    int flags; /* NF4HIP_EPI_* */
    float eps;
    const float* in_sumsq; /* ROWSCALE: [M, in_parts] */
    int in_parts;
    const void* resid_in;    /* RESID_NORM: [M, N] bf16 */
    const void* norm_weight; /* RESID_NORM: [N] bf16 */
    void* resid_out;         /* RESID_NORM: [M, N] bf16 */
    void* xnext_out;         /* RESID_NORM: [M, N] bf16 */
    float* out_sumsq;        /* RESID_NORM: [M, nf4hip_gemv_norm_parts(M, N, K)] */
} nf4hip_epilogue;
/* partial sums per row of x that a RESID_NORM call on the current device writes (0: the shape is not served) */
int nf4hip_gemv_norm_parts(int64_t M, int64_t N, int64_t K);
/* 1 if nf4hip_gemv_epilogue takes this shape with these flags (in_parts: what a ROWSCALE call would pass, else 0),
 * 0 if it would answer NF4HIP_E_SHAPE: for callers that must know before they launch the first kernel of a chain.
 * An epilogue is served by the kernel that serves the shape's plain product or not at all, so that the stored results
 * are those of nf4hip_gemv followed by the step, bit for bit (ROWSCALE excepted, see above). */
int nf4hip_gemv_epilogue_served(int64_t M, int64_t N, int64_t K, int blocksize, int flags, int in_parts);
int nf4hip_gemv_epilogue(const void* x, int x_dtype, int64_t M, const uint8_t* packed, const float* absmax,
                         const float* lut16, const void* bias_or_null, int64_t N, int64_t K, int blocksize, void* out,
                         void* workspace, size_t workspace_bytes, const nf4hip_epilogue* epilogue, void* stream);

/*
 * nf4hip_gemv for callers that cannot allocate or own a workspace (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference:
 * bitsandbytes' gemv_4bit needs no scratch, and the workspace of nf4hip_gemv is this library's own
 * invention.  Same arguments, rules and results as nf4hip_gemv (fp32 absmax), but the split-K
 * counters and partial sums live in an array inside the library's device image,
 * NF4HIP_STATIC_SCRATCH_BYTES per GPU, held from the library's first use on that GPU until the
 * process ends.  The call allocates and frees nothing, on the device or through any library.
 *   - A shape whose nf4hip_gemv_workspace_bytes(M,N,K) exceeds NF4HIP_STATIC_SCRATCH_BYTES is refused
 *     with NF4HIP_E_WORKSPACE (every Llama-3-8B / 70B projection shape fits).
 *   - All calls on one GPU share that GPU's array: two calls that may overlap in time on the same GPU
 *     (different streams, or a graph replayed beside eager calls) race.  The array keeps the last
 *     call's partial sums; the counters at its head are back at zero whenever a call has completed.
 *   - The first call on a GPU resolves the array's address and clears its counters with a small
 *     kernel on `stream`; make that call outside a capture (under capture it fails with NF4HIP_E_HIP
 *     and records nothing).
 */
#define NF4HIP_STATIC_SCRATCH_BYTES (4u << 20)
int nf4hip_gemv_static(const void* x, int x_dtype, int64_t M, const uint8_t* packed, const float* absmax,
                       const float* lut16, const void* bias_or_null, int64_t N, int64_t K, int blocksize, void* out,
                       void* stream);

/*
 * Prefill-shape fused dequant-matmul, M > 16.  Replaces the dequantize_4bit + F.linear route of
 * bitsandbytes.matmul_4bit (MatMul4Bit.forward), reached from thunder/transforms/quantization.py:39.
 * NF4 codes are expanded to bf16 ( bf16(lut16[c] * absmax) ) on chip and contracted with bf16 MFMA,
 * fp32 accumulation, bf16 output.  Same operand layout and fast-path rules as nf4hip_gemv, except
 * K % 64 == 0 and blocksize == 64 ... 4096 dividing K.  Up to 128 rows of x, K may be split over
 * workgroups that meet in `workspace`: nf4hip_gemm_workspace_bytes(M,N,K) bytes (0 = none needed,
 * NULL accepted), under the rules of nf4hip_gemv's workspace -- zeroed once, left zeroed where that
 * matters, one stream at a time; the two kernels may share one workspace.
 */
size_t nf4hip_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K);
/*
 * The launch plan nf4hip_gemm would use for a shape (no GPU needed): plan[0] rows of x per tile (64, 128 or 256),
 * plan[1] tiles (tiles of x rows x tiles of 256 weight rows), plan[2] pieces a tile is cut into along K (they meet in
 * the workspace), plan[3] workgroups launched.  For host code that chooses between this kernel and dequantize +
 * dense GEMM (the choice bitsandbytes.matmul_4bit makes at thunder/transforms/quantization.py:39) without keeping
 * a copy of the launcher's rules.  K must be a multiple of 64.
 */
int nf4hip_gemm_plan(int64_t M, int64_t N, int64_t K, int32_t plan[4]);
int nf4hip_gemm(const void* x, int x_dtype, int64_t M, const uint8_t* packed, const float* absmax, const float* lut16,
                const void* bias_or_null, int64_t N, int64_t K, int blocksize, void* out, void* workspace,
                size_t workspace_bytes, void* stream);
/*
 * Dense linear on a dequantized weight: out[M, N] = x[M, K] . w[N, K]^T (+ bias), bf16 operands, fp32 accumulation,
 * bf16 output.  The GEMM of the dequantize_4bit + torch.nn.functional.linear route of bitsandbytes.matmul_4bit
 * (MatMul4Bit.forward, the route thunder/transforms/quantization.py:39 reaches for more than one row of x): w is
 * what nf4hip_dequantize / nf4hip_dequantize_dq wrote.  K must be a multiple of 64 and at least 128 (NF4HIP_E_SHAPE
 * otherwise: the caller then keeps its own dense GEMM); M and N are free.  Calls with at most 128 tiles of 256 x 256
 * outputs and K >= 2048 cut every tile in two along K and need nf4hip_linear_workspace_bytes(M, N, K) bytes of
 * workspace whose first 256 KiB are zero before the first call (every call leaves them zero); the result is
 * deterministic.  nf4hip_linear_plan: plan[0] rows of x per tile (256), plan[1] tiles, plan[2] pieces per tile,
 * plan[3] workgroups launched (no GPU needed).
 */
size_t nf4hip_linear_workspace_bytes(int64_t M, int64_t N, int64_t K);
int nf4hip_linear_plan(int64_t M, int64_t N, int64_t K, int32_t plan[4]);
int nf4hip_linear(const void* x, int x_dtype, int64_t M, const void* w, const void* bias_or_null, int64_t N, int64_t K,
                  void* out, void* workspace, size_t workspace_bytes, void* stream);
int nf4hip_gemm_dq(const void* x, int x_dtype, int64_t M, const uint8_t* packed, const uint8_t* absmax_q,
                   const float* absmax2, const float* map256, float offset, int nested_blocksize, const float* lut16,
                   const void* bias_or_null, int64_t N, int64_t K, int blocksize, void* out, void* workspace,
                   size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* NF4HIP_H */
