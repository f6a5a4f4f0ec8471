// The three operations between the 4-bit linears of a Llama decode step (one new token per
// sequence), each as one kernel for gfx950: residual add + RMSNorm, rotary embedding + KV-cache
// update + grouped-query attention over the cache, SiLU(gate) * up; and greedy sampling (row argmax).  In the reference these run as
// fusions of its other executors around the quantized linear (thunder/executors/sdpaex.py for the
// attention, the nvFuser / torch.compile executors for the element-wise and norm work); here they
// exist so that the decode-step harness is bound by the NF4 kernels rather than by ~18 small
// launches per layer.  bf16 in and out, fp32 arithmetic.  C ABI: include/nf4hip_decode.h.
#include <hip/hip_runtime.h>
#include <type_traits>
#include <stdint.h>
#include <stdio.h>

#include <string>

#include "../../include/nf4hip_decode.h"
#include "decode_math.h"

namespace {

__device__ __forceinline__ float bf16_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

__device__ __forceinline__ uint32_t f32_to_bf16(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
    u += 0x7fffu + ((u >> 16) & 1u);
    return u >> 16;
}

__device__ __forceinline__ void unpack8(const uint4& v, float (&f)[8]) {
    const uint32_t d[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        f[2 * i] = __uint_as_float(d[i] << 16);
        f[2 * i + 1] = __uint_as_float(d[i] & 0xffff0000u);
    }
}

__device__ __forceinline__ uint4 pack8(const float (&f)[8]) {
    uint32_t d[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) d[i] = f32_to_bf16(f[2 * i]) | (f32_to_bf16(f[2 * i + 1]) << 16);
    return make_uint4(d[0], d[1], d[2], d[3]);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

constexpr int NORM_THREADS = 512;
constexpr int NORM_MAX_CHUNKS = 4;  // 8 elements per chunk: d <= 512 * 4 * 8 = 16384

// x <- bf16(x + delta) (delta may be null), y <- bf16(x * rsqrt(mean(x^2) + eps) * weight); one
// workgroup per row.
__global__ __launch_bounds__(NORM_THREADS) void add_rmsnorm_kernel(uint16_t* x, const uint16_t* delta,
                                                                   const uint16_t* weight, float eps, int d,
                                                                   uint16_t* y) {
    __shared__ float part[NORM_THREADS / 64];
    const int tid = threadIdx.x;
    const int64_t row = blockIdx.x;
    uint16_t* xr = x + row * d;
    const int chunks = d / 8;
    // every load of the kernel goes out first, the norm weight included: nothing waits on memory twice
    uint4 xv[NORM_MAX_CHUNKS], dv[NORM_MAX_CHUNKS], wv[NORM_MAX_CHUNKS];
#pragma unroll
    for (int c = 0; c < NORM_MAX_CHUNKS; ++c) {
        const int ch = tid + c * NORM_THREADS;
        xv[c] = dv[c] = wv[c] = make_uint4(0, 0, 0, 0);
        if (ch < chunks) {
            xv[c] = *reinterpret_cast<const uint4*>(xr + ch * 8);
            if (delta) dv[c] = *reinterpret_cast<const uint4*>(delta + row * d + ch * 8);
            wv[c] = *reinterpret_cast<const uint4*>(weight + ch * 8);
        }
    }
    float v[NORM_MAX_CHUNKS][8];
    float ss = 0.0f;
#pragma unroll
    for (int c = 0; c < NORM_MAX_CHUNKS; ++c) {
        const int ch = tid + c * NORM_THREADS;
        if (ch < chunks) {
            unpack8(xv[c], v[c]);
            if (delta) {
                float dl[8];
                unpack8(dv[c], dl);
#pragma unroll
                for (int i = 0; i < 8; ++i) v[c][i] = nf4x::resid_add(v[c][i], dl[i]);
                *reinterpret_cast<uint4*>(xr + ch * 8) = pack8(v[c]);
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) ss = fmaf(v[c][i], v[c][i], ss);
        }
    }
    ss = wave_sum(ss);
    if ((tid & 63) == 0) part[tid >> 6] = ss;
    __syncthreads();
    float tot = 0.0f;
#pragma unroll
    for (int w = 0; w < NORM_THREADS / 64; ++w) tot += part[w];
    const float rstd = rsqrtf(tot / (float)d + eps);
#pragma unroll
    for (int c = 0; c < NORM_MAX_CHUNKS; ++c) {
        const int ch = tid + c * NORM_THREADS;
        if (ch < chunks) {
            float w[8], o[8];
            unpack8(wv[c], w);
#pragma unroll
            for (int i = 0; i < 8; ++i) o[i] = v[c][i] * rstd * w[i];
            *reinterpret_cast<uint4*>(y + row * d + ch * 8) = pack8(o);
        }
    }
}

constexpr int ATTN_THREADS = 256;
constexpr int ATTN_XCDS = 8;  // workgroup id % 8 is the XCD a workgroup runs on

// One workgroup per (query head, sequence, split of the cached keys).  The query heads of one kv group read the same
// cached rows: the 1-D grid is laid out so that they are neighbours in dispatch order AND land on one XCD (workgroups go
// to the 8 XCDs round robin, id % 8), i.e. behind one L2 -- the cached rows then come from HBM once instead of once per
// query head.  qkv holds this step's q, k, v
// rows of the sequence; position p = *pos.  The new k (rotated) and v are written to the caches by
// one workgroup of each kv group and used from LDS by all of them, so no workgroup depends on
// another's write.  With more than one split every workgroup leaves (max, sum, unnormalised output)
// in the workspace and the last one to arrive for its (sequence, head) -- an arrival counter in the
// workspace, left at zero again -- merges them.
template <int HD>
__global__ __launch_bounds__(ATTN_THREADS) void attention_decode_kernel(const uint16_t* qkv, const int64_t* pos,
                                                                        const float* cos_t, const float* sin_t,
                                                                        uint16_t* kcache, uint16_t* vcache, int batch,
                                                                        int H, int Hkv, int max_seq, uint16_t* out,
                                                                        int splits, uint32_t* counters, float* partials) {
    constexpr int LPK = HD / 16;            // lanes per key: 16 elements each
    constexpr int KPI = ATTN_THREADS / LPK;  // keys per iteration of the score loop
    constexpr int DG = HD / 8;              // column groups of 8 in the value pass
    constexpr int SG = ATTN_THREADS / DG;   // key groups in the value pass
    extern __shared__ __attribute__((aligned(16))) float lds[];
    float* q_s = lds;                 // [HD] rotated query, pre-scaled
    float* k_s = q_s + HD;            // [HD] new key (rotated, rounded to bf16)
    float* v_s = k_s + HD;            // [HD] new value
    float* red = v_s + HD;            // [8] reductions
    float* acc_s = red + 8;           // [SG][HD] partial outputs
    float* p_s = acc_s + SG * HD;     // [max_seq] scores, then probabilities

    const int tid = threadIdx.x;
    // a stream = (sequence, split, kv head): XCD slot stream_id % 8; its `rep` query heads are 8 workgroup ids apart
    const int rep = H / Hkv;
    const int slot = (int)blockIdx.x & (ATTN_XCDS - 1), outer = (int)blockIdx.x / ATTN_XCDS;
    const int stream_id = (outer / rep) * ATTN_XCDS + slot;
    if (stream_id >= batch * splits * Hkv) return;  // uniform: padding of the last group of eight streams
    const int hk = stream_id % Hkv, split = (stream_id / Hkv) % splits, b = stream_id / (Hkv * splits);
    const int h = hk * rep + outer % rep;
    const int p = (int)*pos;
    if (p < 0 || p >= max_seq) return;  // uniform: a position outside the cache touches nothing
    // this workgroup's cached keys [lo, hi) of 0 .. p-1; the last split also takes the new key p
    const int chunk = (p + splits - 1) / splits;
    const int lo = min(split * chunk, p), hi = min(lo + chunk, p);
    const bool has_new = split == splits - 1;
    const uint16_t* row = qkv + (int64_t)b * (H + 2 * Hkv) * HD;
    uint16_t* kc = kcache + ((int64_t)b * Hkv + hk) * max_seq * HD;
    uint16_t* vc = vcache + ((int64_t)b * Hkv + hk) * max_seq * HD;

    if (tid < HD) {
        const int j = tid, jp = j < HD / 2 ? j + HD / 2 : j - HD / 2;
        const float c = cos_t[(int64_t)p * HD + j], s = sin_t[(int64_t)p * HD + j];
        const float sgn = j < HD / 2 ? -1.0f : 1.0f;
        const uint16_t* qh = row + h * HD;
        const uint16_t* kh = row + (H + hk) * HD;
        const float qr = bf16_to_f32(qh[j]) * c + sgn * bf16_to_f32(qh[jp]) * s;
        const float kr = bf16_to_f32(kh[j]) * c + sgn * bf16_to_f32(kh[jp]) * s;
        const uint32_t kb = f32_to_bf16(kr);
        const uint32_t vb = row[(H + Hkv + hk) * HD + j];
        q_s[j] = bf16_to_f32(f32_to_bf16(qr)) * rsqrtf((float)HD);
        k_s[j] = bf16_to_f32(kb);
        v_s[j] = bf16_to_f32(vb);
        if (h % rep == 0 && split == 0) {
            kc[(int64_t)p * HD + j] = (uint16_t)kb;
            vc[(int64_t)p * HD + j] = (uint16_t)vb;
        }
    }
    __syncthreads();

    // scores of the cached keys 0 .. p-1: LPK lanes per key, four keys per lane in flight (addresses
    // clamped instead of branching, so that the eight loads of a round are issued back to back)
    const int sub = tid % LPK, kslot = tid / LPK;
    float qv[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) qv[i] = q_s[sub * 16 + i];
    float mx = -INFINITY;
    // U keys per lane under way at a time.  A round of requests is a round trip to memory, so with few workgroups per
    // CU (one sequence: 256 workgroups) a workgroup takes as few rounds as its keys need -- eight keys per lane, 256 a
    // round.  With four workgroups per CU the CU's address unit is what the passes wait for, and a round wider than
    // the keys left costs requests for clamped addresses: four per lane there.  The order of the additions does not
    // depend on the width.
    const bool wide = gridDim.x <= 512;
    auto score_pass = [&](auto u_tag) {
        constexpr int U = decltype(u_tag)::value;
        for (int s0 = lo; s0 < hi; s0 += U * KPI) {
            uint4 ka[U], kb[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int s = min(s0 + u * KPI + kslot, hi - 1);
                const uint4* kp = reinterpret_cast<const uint4*>(kc + (int64_t)s * HD + sub * 16);
                ka[u] = kp[0];
                kb[u] = kp[1];
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int s = s0 + u * KPI + kslot;
                float a8[8], b8[8];
                unpack8(ka[u], a8);
                unpack8(kb[u], b8);
                float dot = 0.0f;
#pragma unroll
                for (int i = 0; i < 8; ++i) dot = fmaf(qv[i], a8[i], dot);
#pragma unroll
                for (int i = 0; i < 8; ++i) dot = fmaf(qv[8 + i], b8[i], dot);
#pragma unroll
                for (int o = 1; o < LPK; o <<= 1) dot += __shfl_xor(dot, o, 64);
                if (s < hi) {
                    if (sub == 0) p_s[s] = dot;
                    mx = fmaxf(mx, dot);
                }
            }
        }
    };
    if (hi - lo <= 2 * KPI)
        score_pass(std::integral_constant<int, 2>{});
    else if (hi - lo <= 4 * KPI || !wide)
        score_pass(std::integral_constant<int, 4>{});
    else
        score_pass(std::integral_constant<int, 8>{});
    if (has_new) {  // the new key, from LDS
        float dot = 0.0f;
#pragma unroll
        for (int i = 0; i < 16; ++i) dot = fmaf(qv[i], k_s[sub * 16 + i], dot);
#pragma unroll
        for (int o = 1; o < LPK; o <<= 1) dot += __shfl_xor(dot, o, 64);
        if (tid == 0) p_s[p] = dot;
        mx = fmaxf(mx, dot);
    }
    mx = wave_max(mx);
    if ((tid & 63) == 0) red[tid >> 6] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    float sum = 0.0f;
    for (int s = lo + tid; s < hi + (has_new ? 1 : 0); s += ATTN_THREADS) {
        const int idx = s < hi ? s : p;
        const float e = __expf(p_s[idx] - mx);
        p_s[idx] = e;
        sum += e;
    }
    sum = wave_sum(sum);
    __syncthreads();  // red[0..3] read by everyone, p_s complete
    if ((tid & 63) == 0) red[4 + (tid >> 6)] = sum;

    // values: thread = (key group sg, 8 columns dg); four cached rows per thread in flight
    const int dg = tid % DG, sg = tid / DG;
    float o[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    // (rows per thread under way: as for the keys; a thread adds its rows in the same order whatever the width)
    auto value_pass = [&](auto u_tag) {
        constexpr int U = decltype(u_tag)::value;
        for (int s0 = lo + sg; s0 < hi; s0 += U * SG) {
            uint4 vv[U];
            float w[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int s = s0 + u * SG;
                vv[u] = *reinterpret_cast<const uint4*>(vc + (int64_t)min(s, hi - 1) * HD + dg * 8);
                w[u] = s < hi ? p_s[s] : 0.0f;
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                float vf[8];
                unpack8(vv[u], vf);
#pragma unroll
                for (int i = 0; i < 8; ++i) o[i] = fmaf(w[u], vf[i], o[i]);
            }
        }
    };
    if (hi - lo <= 4 * SG || !wide)
        value_pass(std::integral_constant<int, 4>{});
    else if (hi - lo <= 8 * SG)
        value_pass(std::integral_constant<int, 8>{});
    else
        value_pass(std::integral_constant<int, 12>{});
    if (sg == 0 && has_new) {  // the new value, from LDS
        const float w = p_s[p];
#pragma unroll
        for (int i = 0; i < 8; ++i) o[i] = fmaf(w, v_s[dg * 8 + i], o[i]);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) acc_s[sg * HD + dg * 8 + i] = o[i];
    __syncthreads();
    float t = 0.0f;
    if (tid < HD) {
#pragma unroll 4
        for (int g = 0; g < SG; ++g) t += acc_s[g * HD + tid];
    }
    const float total = red[4] + red[5] + red[6] + red[7];
    uint16_t* dst = out + ((int64_t)b * H + h) * HD;
    if (splits == 1) {
        if (tid < HD) dst[tid] = (uint16_t)f32_to_bf16(t / total);
        return;
    }
    // leave this split's (max, sum, output) and count the arrival.  Ordering without L2-wide fences:
    // agent-scope stores go through to L2; every store of the workgroup has completed (s_waitcnt, then
    // the barrier) before its arrival is counted; the last workgroup reads with agent-scope loads, which
    // bypass its CU's L1.
    const int64_t bh = (int64_t)b * H + h;
    float* mine = partials + (bh * splits + split) * (HD + 2);
    if (tid < HD) __hip_atomic_store(mine + 2 + tid, t, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (tid == 0) {
        __hip_atomic_store(mine, mx, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(mine + 1, total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    // compiler: no store sinks below the release fence, no load rises above the acquire fence;
    // hardware: the s_waitcnt holds the wave until L2 has acknowledged its stores
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (tid == 0)
        red[0] = __uint_as_float(__hip_atomic_fetch_add(&counters[bh], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
    __syncthreads();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    if (__float_as_uint(red[0]) != (uint32_t)(splits - 1)) return;
    if (tid < HD) {
        const float* all = partials + bh * splits * (HD + 2);
        constexpr int MAX_SPLITS = 8;
        float mi[MAX_SPLITS], li[MAX_SPLITS], oi[MAX_SPLITS];
#pragma unroll
        for (int i = 0; i < MAX_SPLITS; ++i) {
            const float* pi = all + min(i, splits - 1) * (HD + 2);
            mi[i] = __hip_atomic_load(pi, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            li[i] = __hip_atomic_load(pi + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            oi[i] = __hip_atomic_load(pi + 2 + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (i >= splits) mi[i] = -INFINITY;
        }
        float m = -INFINITY;
#pragma unroll
        for (int i = 0; i < MAX_SPLITS; ++i) m = fmaxf(m, mi[i]);
        float num = 0.0f, den = 0.0f;
#pragma unroll
        for (int i = 0; i < MAX_SPLITS; ++i) {
            const float w = mi[i] == -INFINITY ? 0.0f : __expf(mi[i] - m);
            den = fmaf(w, li[i], den);
            num = fmaf(w, oi[i], num);
        }
        dst[tid] = (uint16_t)f32_to_bf16(num / den);
    }
    if (tid == 0) __hip_atomic_store(&counters[bh], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// out <- bf16(bf16(silu(gate)) * up).  PAIRS false: gate = gate_up[:, :dff], up = gate_up[:, dff:]; true: gate and up
// interleaved, gate_up[:, 2j] = gate[:, j], gate_up[:, 2j + 1] = up[:, j] (a thread's 8 outputs come from 32 contiguous bytes)
template <bool PAIRS>
__global__ __launch_bounds__(256) void silu_mul_kernel(const uint16_t* gate_up, int64_t rows, int64_t dff, uint16_t* out) {
    const int64_t per_row = dff / 8;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= rows * per_row) return;
    const int64_t r = i / per_row, c = i - r * per_row;
    float g[8], u[8], o[8];
    if (PAIRS) {
        float a[8], b[8];
        unpack8(*reinterpret_cast<const uint4*>(gate_up + r * 2 * dff + c * 16), a);
        unpack8(*reinterpret_cast<const uint4*>(gate_up + r * 2 * dff + c * 16 + 8), b);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            g[k] = a[2 * k]; u[k] = a[2 * k + 1];
            g[4 + k] = b[2 * k]; u[4 + k] = b[2 * k + 1];
        }
    } else {
        unpack8(*reinterpret_cast<const uint4*>(gate_up + r * 2 * dff + c * 8), g);
        unpack8(*reinterpret_cast<const uint4*>(gate_up + r * 2 * dff + dff + c * 8), u);
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) o[k] = bf16_to_f32(nf4x::silu_mul_bf16(g[k], u[k]));
    *reinterpret_cast<uint4*>(out + r * dff + c * 8) = pack8(o);
}

constexpr int ARGMAX_THREADS = 1024;

// Largest element of each row, lowest index on ties, NaN counted as the largest value (what torch.argmax returns);
// one workgroup per row.  Every element becomes a 64-bit key -- the value's bits in an order-preserving form above
// the complemented index -- and the row's answer is the largest key, so the order of the reduction does not matter.
// `pos` (may be null): a position counter that workgroup 0 advances by one, the decode step's bookkeeping.
__global__ __launch_bounds__(ARGMAX_THREADS) void argmax_kernel(const uint16_t* logits, int64_t vocab, int64_t* out,
                                                                 int64_t* pos) {
    __shared__ unsigned long long red[ARGMAX_THREADS / 64];
    const int tid = threadIdx.x;
    const uint16_t* row = logits + (int64_t)blockIdx.x * vocab;
    auto key_of = [](uint32_t bf, int64_t idx) -> unsigned long long {
        uint32_t bits = bf << 16;
        if ((bits << 1) == 0) bits = 0;  // -0.0 and +0.0 compare equal: one key for both, the lower index wins
        uint32_t ord = (bits & 0x80000000u) ? ~bits : bits | 0x80000000u;
        if ((bits & 0x7fffffffu) > 0x7f800000u) ord = 0xffffffffu;  // NaN
        return ((unsigned long long)ord << 32) | (uint32_t)(0xffffffffu - (uint32_t)idx);
    };
    unsigned long long best = 0;
    const int64_t chunks = vocab / 8;
    for (int64_t c0 = tid; c0 < chunks; c0 += 4 * ARGMAX_THREADS) {
        uint4 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {  // four requests in flight; a request past the end re-reads the thread's first
            const int64_t c = c0 + (int64_t)u * ARGMAX_THREADS;
            v[u] = *reinterpret_cast<const uint4*>(row + (c < chunks ? c : c0) * 8);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int64_t c = c0 + (int64_t)u * ARGMAX_THREADS;
            if (c >= chunks) break;
            const uint32_t d[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const unsigned long long k0 = key_of(d[i] & 0xffffu, c * 8 + 2 * i), k1 = key_of(d[i] >> 16, c * 8 + 2 * i + 1);
                best = best > k0 ? best : k0;
                best = best > k1 ? best : k1;
            }
        }
    }
    for (int64_t i = chunks * 8 + tid; i < vocab; i += ARGMAX_THREADS) {  // vocab % 8 elements at the end
        const unsigned long long k = key_of(row[i], i);
        best = best > k ? best : k;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const unsigned long long other = __shfl_xor(best, o, 64);
        best = best > other ? best : other;
    }
    if ((tid & 63) == 0) red[tid >> 6] = best;
    __syncthreads();
    if (tid == 0) {
        for (int w = 1; w < ARGMAX_THREADS / 64; ++w) best = best > red[w] ? best : red[w];
        out[blockIdx.x] = (int64_t)(0xffffffffu - (uint32_t)best);
        if (pos && blockIdx.x == 0) *pos += 1;
    }
}

thread_local char g_err[256] = "";

int fail(const char* msg) {
    snprintf(g_err, sizeof g_err, "%s", msg);
    return -1;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

template <typename K>
hipError_t allow_lds(K kern, size_t bytes) {
    return hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                               (int)bytes);
}

}  // namespace

extern "C" {

__attribute__((visibility("default"))) const char* nf4hip_decode_last_error(void) { return g_err; }

__attribute__((visibility("default"))) int nf4hip_decode_add_rmsnorm(void* x, const void* delta, const void* weight,
                                                                     float eps, int64_t rows, int64_t d, void* y,
                                                                     void* stream) {
    if (!x || !weight || !y) return fail("nf4hip_decode_add_rmsnorm: null pointer");
    if (rows <= 0 || d <= 0 || d % 8 || d > NORM_THREADS * 8 * NORM_MAX_CHUNKS || rows > INT32_MAX)
        return fail("nf4hip_decode_add_rmsnorm: need rows > 0 and d a multiple of 8, at most 16384");
    if (!aligned16(x) || !aligned16(y) || !aligned16(weight) || (delta && !aligned16(delta)))
        return fail("nf4hip_decode_add_rmsnorm: pointer not 16-byte aligned");
    hipLaunchKernelGGL(add_rmsnorm_kernel, dim3((unsigned)rows), dim3(NORM_THREADS), 0, static_cast<hipStream_t>(stream),
                       static_cast<uint16_t*>(x), static_cast<const uint16_t*>(delta),
                       static_cast<const uint16_t*>(weight), eps, (int)d, static_cast<uint16_t*>(y));
    return hipGetLastError() == hipSuccess ? 0 : fail("nf4hip_decode_add_rmsnorm: launch failed");
}

// The arrival counters take a fixed region at the start of the workspace (splits > 1 only for up to
// 512 (sequence, head) pairs), so that calls of different shapes can share one workspace: partial
// results never land where another call expects zeroed counters.
constexpr size_t ATTN_COUNTER_BYTES = 4096;

// splits of the cached keys per (sequence, head): about four workgroups per CU of the chip's 256, so
// that each has a short chain of dependent loads
static int attention_splits(int64_t batch, int n_head) {
    const int64_t wgs = batch * n_head;
    int s = (int)(1024 / (wgs > 0 ? wgs : 1));
    return s < 1 ? 1 : s > 8 ? 8 : s;
}

__attribute__((visibility("default"))) size_t nf4hip_decode_attention_workspace_bytes(int64_t batch, int n_head,
                                                                                      int head_dim) {
    if (batch <= 0 || n_head <= 0 || head_dim <= 0) return 0;
    const int splits = attention_splits(batch, n_head);
    if (splits == 1) return 0;
    return ATTN_COUNTER_BYTES + (size_t)batch * n_head * splits * (head_dim + 2) * sizeof(float);
}

__attribute__((visibility("default"))) int nf4hip_decode_attention(const void* qkv, const int64_t* pos, const float* cos_t,
                                                                   const float* sin_t, void* kcache, void* vcache,
                                                                   int64_t batch, int n_head, int n_kv_head, int head_dim,
                                                                   int64_t max_seq, void* out, void* workspace,
                                                                   size_t workspace_bytes, void* stream) {
    if (!qkv || !pos || !cos_t || !sin_t || !kcache || !vcache || !out) return fail("nf4hip_decode_attention: null pointer");
    if (batch <= 0 || batch > 65535 || n_head <= 0 || n_kv_head <= 0 || n_head % n_kv_head || max_seq <= 0 ||
        max_seq > 32768)
        return fail("nf4hip_decode_attention: need 0 < batch <= 65535, n_head a multiple of n_kv_head, max_seq <= 32768");
    if (head_dim != 64 && head_dim != 128) return fail("nf4hip_decode_attention: head_dim must be 64 or 128");
    if (!aligned16(qkv) || !aligned16(kcache) || !aligned16(vcache) || !aligned16(out))
        return fail("nf4hip_decode_attention: pointer not 16-byte aligned");
    const int splits = attention_splits(batch, n_head);
    const size_t need = nf4hip_decode_attention_workspace_bytes(batch, n_head, head_dim);
    if (need && (!workspace || workspace_bytes < need || !aligned16(workspace)))
        return fail("nf4hip_decode_attention: a zero-initialised, 16-byte aligned workspace of "
                    "nf4hip_decode_attention_workspace_bytes() bytes is required");
    uint32_t* counters = static_cast<uint32_t*>(workspace);
    float* partials = need ? reinterpret_cast<float*>(static_cast<uint8_t*>(workspace) + ATTN_COUNTER_BYTES) : nullptr;
    const int sg = ATTN_THREADS / (head_dim / 8);
    const size_t lds = sizeof(float) * (size_t)(3 * head_dim + 8 + sg * head_dim + max_seq);
    const int64_t streams = batch * splits * n_kv_head;
    const dim3 grid((unsigned)((streams + ATTN_XCDS - 1) / ATTN_XCDS * ATTN_XCDS * (n_head / n_kv_head)));
    // allow the whole 160 KB of LDS once per device (what a launch takes is its own `lds`)
    static bool ready[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return fail("nf4hip_decode_attention: no current device");
    if (!ready[dev]) {
        if (allow_lds(attention_decode_kernel<128>, 160 * 1024) != hipSuccess ||
            allow_lds(attention_decode_kernel<64>, 160 * 1024) != hipSuccess)
            return fail("nf4hip_decode_attention: LDS size");
        ready[dev] = true;
    }
    auto launch = [&](auto kern) {
        hipLaunchKernelGGL(kern, grid, dim3(ATTN_THREADS), lds, static_cast<hipStream_t>(stream),
                           static_cast<const uint16_t*>(qkv), pos, cos_t, sin_t, static_cast<uint16_t*>(kcache),
                           static_cast<uint16_t*>(vcache), (int)batch, n_head, n_kv_head, (int)max_seq, static_cast<uint16_t*>(out),
                           splits, counters, partials);
    };
    if (head_dim == 128)
        launch(attention_decode_kernel<128>);
    else
        launch(attention_decode_kernel<64>);
    return hipGetLastError() == hipSuccess ? 0 : fail("nf4hip_decode_attention: launch failed");
}

static int silu_mul_launch(const char* name, bool pairs, const void* gate_up, int64_t rows, int64_t dff, void* out, void* stream) {
    if (!gate_up || !out) return fail((std::string(name) + ": null pointer").c_str());
    if (rows <= 0 || dff <= 0 || dff % 8) return fail((std::string(name) + ": need rows > 0 and dff a multiple of 8").c_str());
    if (!aligned16(gate_up) || !aligned16(out)) return fail((std::string(name) + ": pointer not 16-byte aligned").c_str());
    const int64_t n = rows * (dff / 8);
    const dim3 grid((unsigned)((n + 255) / 256));
    if (pairs)
        hipLaunchKernelGGL(silu_mul_kernel<true>, grid, dim3(256), 0, static_cast<hipStream_t>(stream),
                           static_cast<const uint16_t*>(gate_up), rows, dff, static_cast<uint16_t*>(out));
    else
        hipLaunchKernelGGL(silu_mul_kernel<false>, grid, dim3(256), 0, static_cast<hipStream_t>(stream),
                           static_cast<const uint16_t*>(gate_up), rows, dff, static_cast<uint16_t*>(out));
    return hipGetLastError() == hipSuccess ? 0 : fail((std::string(name) + ": launch failed").c_str());
}

__attribute__((visibility("default"))) int nf4hip_decode_silu_mul(const void* gate_up, int64_t rows, int64_t dff, void* out,
                                                                  void* stream) {
    return silu_mul_launch("nf4hip_decode_silu_mul", false, gate_up, rows, dff, out, stream);
}

__attribute__((visibility("default"))) int nf4hip_decode_silu_mul_pairs(const void* gate_up, int64_t rows, int64_t dff, void* out,
                                                                        void* stream) {
    return silu_mul_launch("nf4hip_decode_silu_mul_pairs", true, gate_up, rows, dff, out, stream);
}

__attribute__((visibility("default"))) int nf4hip_decode_argmax(const void* logits, int64_t rows, int64_t vocab, int64_t* out,
                                                                int64_t* pos_or_null, void* stream) {
    if (!logits || !out) return fail("nf4hip_decode_argmax: null pointer");
    if (rows <= 0 || vocab <= 0 || rows > INT32_MAX || vocab > 0xffffffffLL)
        return fail("nf4hip_decode_argmax: need 0 < rows < 2^31 and 0 < vocab < 2^32");
    if (!aligned16(logits) || (rows > 1 && vocab % 8))
        return fail("nf4hip_decode_argmax: logits not 16-byte aligned, or several rows whose length is no multiple of 8");
    if ((reinterpret_cast<uintptr_t>(out) & 7u) || (reinterpret_cast<uintptr_t>(pos_or_null) & 7u))
        return fail("nf4hip_decode_argmax: out / pos not 8-byte aligned");
    hipLaunchKernelGGL(argmax_kernel, dim3((unsigned)rows), dim3(ARGMAX_THREADS), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint16_t*>(logits), vocab, out, pos_or_null);
    return hipGetLastError() == hipSuccess ? 0 : fail("nf4hip_decode_argmax: launch failed");
}

}  // extern "C"
