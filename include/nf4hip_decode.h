/* C ABI of libnf4hip_decode.so: the operations between the 4-bit linears of a Llama decode step.
 *
 * These entry points have no counterpart in the reference's bitsandbytes path.  In the reference the
 * same work is done by its other executors around the quantized linear -- attention by
 * thunder/executors/sdpaex.py, norms and element-wise chains as nvFuser / torch.compile fusions
 * (thunder/executors/nvfuserex_impl.py, torch_compile.py) -- and a decode step replayed by
 * thunder/transforms/cudagraph.py:47-226 is then a few launches per layer.  They exist for the
 * decode-step harness (lightning-thunder_amd/decode.py, LlamaConfig.hip_glue): with them the step is
 * bound by the NF4 kernels of include/nf4hip.h instead of ~18 small launches per layer.
 *
 * Conventions as in include/nf4hip.h: 0 on success, -1 on failure with the text available from
 * nf4hip_decode_last_error() on the calling thread; arguments are validated before the first HIP
 * call; device pointers are borrowed; nothing allocates, synchronises or blocks; `stream` is a
 * hipStream_t.  All tensors are bf16, row-major, 16-byte aligned; arithmetic is fp32.
 */
#ifndef NF4HIP_DECODE_H
#define NF4HIP_DECODE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char* nf4hip_decode_last_error(void);

/* x[rows, d] <- bf16(x + delta) (delta may be NULL: x is left as it is), then
 * y[rows, d] <- bf16(x * rsqrt(mean(x^2) + eps) * weight[d]): the residual add and the RMSNorm that
 * follows it.  d % 8 == 0, d <= 16384. */
int nf4hip_decode_add_rmsnorm(void* x, const void* delta_or_null, const void* weight, float eps, int64_t rows,
                              int64_t d, void* y, void* stream);

/* One new token per sequence.  qkv[batch, (n_head + 2 n_kv_head) * head_dim] holds the query heads,
 * then the key heads, then the value heads of the token at position p = *pos (a device scalar, so a
 * captured graph follows the position).  Queries and keys get the rotary embedding
 * out[j] = x[j] cos[p, j] + rotate_half(x)[j] sin[p, j] from the fp32 tables cos/sin[max_seq, head_dim];
 * the new key and value rows are written to kcache / vcache[batch, n_kv_head, max_seq, head_dim] at p;
 * out[batch, n_head * head_dim] <- softmax(q k^T / sqrt(head_dim)) v over cache rows 0..p, query head h
 * reading kv head h / (n_head / n_kv_head).  head_dim 64 or 128; 0 <= p < max_seq <= 32768.
 * When batch * n_head is small the cached keys of a head are split over several workgroups, which
 * meet in `workspace`: nf4hip_decode_attention_workspace_bytes() bytes (0 = none needed, NULL
 * accepted), zero-initialised once by the caller and then owned by one stream at a time -- every call
 * leaves its arrival counters (the first 4096 bytes, whatever the shape) at zero again, so calls of
 * different shapes may share one workspace. */
size_t nf4hip_decode_attention_workspace_bytes(int64_t batch, int n_head, int head_dim);
int nf4hip_decode_attention(const void* qkv, const int64_t* pos, const float* cos, const float* sin, void* kcache,
                            void* vcache, int64_t batch, int n_head, int n_kv_head, int head_dim, int64_t max_seq,
                            void* out, void* workspace, size_t workspace_bytes, void* stream);

/* out[rows, dff] <- bf16(bf16(silu(gate)) * up) with gate = gate_up[:, :dff], up = gate_up[:, dff:];
 * gate_up[rows, 2 dff], dff % 8 == 0. */
int nf4hip_decode_silu_mul(const void* gate_up, int64_t rows, int64_t dff, void* out, void* stream);
/* The same for gate and up interleaved: gate_up[:, 2j] = gate[:, j], gate_up[:, 2j+1] = up[:, j] -- the output of a linear
 * whose weight rows alternate between the gate and the up projection (the layout nf4hip_gemv_epilogue's
 * NF4HIP_EPI_SILU_PAIRS expects). */
int nf4hip_decode_silu_mul_pairs(const void* gate_up, int64_t rows, int64_t dff, void* out, void* stream);

/* Greedy sampling: out[r] <- index of the largest element of logits[r, 0 .. vocab-1] (bf16), the lowest index among
 * equals, a NaN counting as the largest value (torch.argmax's answer).  One workgroup per row, no scratch.
 * pos_or_null: a device counter that the call advances by one after the rows are done (the position of the decode
 * step, so that sampling and bookkeeping are one launch); NULL to leave it out.
 * Several rows need vocab % 8 == 0 (every row 16-byte aligned). */
int nf4hip_decode_argmax(const void* logits, int64_t rows, int64_t vocab, int64_t* out, int64_t* pos_or_null, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* NF4HIP_DECODE_H */
