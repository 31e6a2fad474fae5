// Row kernels a decoder needs around the matmuls: RMSNorm, softmax, SiLU*up, residual add, arg-max,
// the packed-weight block permutation and the packed embedding lookup. All fp32, all HBM-bound:
// one pass in, one pass out, reductions inside a workgroup.
//
// Semantics (paths under /root/reference/skainet-backends/skainet-backend-native-cpu/native/src/):
//   rms_norm      out = x / sqrt(mean(x^2) + eps) * gamma      f32_fused.c:255-286
//   layer_norm    (x - mean) / sqrt(var + eps) * gamma + beta  f32_fused.c:255-279
//   softmax_rows  exp(x - max) / sum, or x - (log sum + max)   f32_fused.c:199-222
//   silu_mul      x * (1 / (1 + exp(-x))) * up                 f32_ops.c:222-244 (silu), binary mul
//   argmax        first index of the row maximum               TensorOps.kt:263-277 (ties -> lowest index)
#include "common.h"
#include "../../include/skainet_hip.h"

#include <mutex>

namespace skh {

void* sync_scratch(size_t bytes);   // shim.hip: persistent zero-initialised device memory for cross-workgroup counters

constexpr int ROW_THREADS = 256;

__device__ __forceinline__ float block_sum(float v, float* red) {
    v = wave_sum(v);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < (int)(blockDim.x >> 6); ++i) t += red[i];
    return t;
}
__device__ __forceinline__ float block_max(float v, float* red) {
    v = wave_max(v);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float t = red[0];
    for (int i = 1; i < (int)(blockDim.x >> 6); ++i) t = fmaxf(t, red[i]);
    return t;
}

// One workgroup per row.
__global__ __launch_bounds__(ROW_THREADS) void rms_norm_kernel(const float* __restrict__ in, const float* __restrict__ gamma,
                                                               float* __restrict__ out, int cols, float eps) {
    __shared__ float red[ROW_THREADS / 64];
    const float* x = in + (int64_t)blockIdx.x * cols;
    float* o = out + (int64_t)blockIdx.x * cols;
    float s = 0.f;
    for (int i = threadIdx.x; i < cols; i += blockDim.x) { const float v = x[i]; s = fmaf(v, v, s); }
    s = block_sum(s, red);
    const float scale = 1.0f / sqrtf(s * (1.0f / (float)cols) + eps);
    for (int i = threadIdx.x; i < cols; i += blockDim.x) {
        float y = x[i] * scale;
        if (gamma) y *= gamma[i];
        o[i] = y;
    }
}

// Rows of at most 4 * ROW_THREADS * V floats (cols a multiple of 4, 16-byte aligned): every load of the row is in
// flight at once and the row stays in registers between the two passes, so a single row costs one memory
// round trip instead of one per 256 elements.
template <int V>
__global__ __launch_bounds__(ROW_THREADS) void rms_norm_cached_kernel(const float* __restrict__ in, const float* __restrict__ gamma,
                                                                      float* __restrict__ out, int cols, float eps) {
    __shared__ float red[ROW_THREADS / 64];
    const float4* x = reinterpret_cast<const float4*>(in + (int64_t)blockIdx.x * cols);
    float4* o = reinterpret_cast<float4*>(out + (int64_t)blockIdx.x * cols);
    const float4* g4 = reinterpret_cast<const float4*>(gamma);
    const int c4 = cols >> 2;
    float4 xr[V], gr[V];
#pragma unroll
    for (int j = 0; j < V; ++j) {
        const int i = threadIdx.x + ROW_THREADS * j;
        xr[j] = i < c4 ? x[i] : make_float4(0.f, 0.f, 0.f, 0.f);
        gr[j] = (gamma && i < c4) ? g4[i] : make_float4(1.f, 1.f, 1.f, 1.f);
    }
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < V; ++j) { s = fmaf(xr[j].x, xr[j].x, s); s = fmaf(xr[j].y, xr[j].y, s); s = fmaf(xr[j].z, xr[j].z, s); s = fmaf(xr[j].w, xr[j].w, s); }
    s = block_sum(s, red);
    const float scale = 1.0f / sqrtf(s * (1.0f / (float)cols) + eps);
#pragma unroll
    for (int j = 0; j < V; ++j) {
        const int i = threadIdx.x + ROW_THREADS * j;
        if (i < c4) o[i] = make_float4(xr[j].x * scale * gr[j].x, xr[j].y * scale * gr[j].y, xr[j].z * scale * gr[j].z, xr[j].w * scale * gr[j].w);
    }
}

// out = (x - mean) / sqrt(var + eps) * gamma + beta with the biased variance; gamma / beta may be null.
// Reference: f32_fused.c:255-279 (two passes: mean, then centred sum of squares).
__global__ __launch_bounds__(ROW_THREADS) void layer_norm_kernel(const float* __restrict__ in, const float* __restrict__ gamma,
                                                                 const float* __restrict__ beta, float* __restrict__ out,
                                                                 int cols, float eps) {
    __shared__ float red[ROW_THREADS / 64];
    const float* x = in + (int64_t)blockIdx.x * cols;
    float* o = out + (int64_t)blockIdx.x * cols;
    const float inv_n = 1.0f / (float)cols;
    float s = 0.f;
    for (int i = threadIdx.x; i < cols; i += blockDim.x) s += x[i];
    const float mean = block_sum(s, red) * inv_n;
    float v = 0.f;
    for (int i = threadIdx.x; i < cols; i += blockDim.x) { const float d = x[i] - mean; v = fmaf(d, d, v); }
    const float scale = 1.0f / sqrtf(block_sum(v, red) * inv_n + eps);
    for (int i = threadIdx.x; i < cols; i += blockDim.x) {
        float y = (x[i] - mean) * scale;
        if (gamma) y *= gamma[i];
        if (beta) y += beta[i];
        o[i] = y;
    }
}

__global__ __launch_bounds__(ROW_THREADS) void softmax_rows_kernel(const float* __restrict__ in, float* __restrict__ out,
                                                                   int cols, int log_form) {
    __shared__ float red[ROW_THREADS / 64];
    const float* x = in + (int64_t)blockIdx.x * cols;
    float* o = out + (int64_t)blockIdx.x * cols;
    float m = -INFINITY;
    for (int i = threadIdx.x; i < cols; i += blockDim.x) m = fmaxf(m, x[i]);
    m = block_max(m, red);
    float s = 0.f;
    for (int i = threadIdx.x; i < cols; i += blockDim.x) s += expf(x[i] - m);
    s = block_sum(s, red);
    if (log_form) {
        const float lse = logf(s) + m;
        for (int i = threadIdx.x; i < cols; i += blockDim.x) o[i] = x[i] - lse;
    } else {
        const float inv = s > 0.f ? 1.0f / s : 1.0f;
        for (int i = threadIdx.x; i < cols; i += blockDim.x) o[i] = expf(x[i] - m) * inv;
    }
}

__global__ __launch_bounds__(256) void silu_mul_kernel(const float* __restrict__ gate, const float* __restrict__ up,
                                                       float* __restrict__ out, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) { const float g = gate[i]; out[i] = g * (1.0f / (1.0f + expf(-g))) * up[i]; }
}

// SwiGLU over rows of interleaved (gate, up) pairs: out[i] = silu(gu[2i]) * gu[2i + 1].
__global__ __launch_bounds__(256) void swiglu_pairs_kernel(const float2* __restrict__ gu, float* __restrict__ out, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float2 p = gu[i];
    out[i] = p.x * (1.0f / (1.0f + expf(-p.x))) * p.y;
}

__global__ __launch_bounds__(256) void add_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                  float* __restrict__ out, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = a[i] + b[i];
}

// One workgroup per row; (value, index) pairs reduced with "larger value, then lower index" so ties keep the first.
__global__ __launch_bounds__(ROW_THREADS) void argmax_rows_kernel(const float* __restrict__ in, int cols, int32_t* __restrict__ out) {
    __shared__ float rv[ROW_THREADS / 64];
    __shared__ int ri[ROW_THREADS / 64];
    const float* x = in + (int64_t)blockIdx.x * cols;
    float bv = -INFINITY;
    int bi = 0x7FFFFFFF;
    for (int i = threadIdx.x; i < cols; i += blockDim.x) {
        const float v = x[i];
        if (v > bv || (v == bv && i < bi) || bi == 0x7FFFFFFF) { bv = v; bi = i; }
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
        const float ov = __shfl_xor(bv, m, 64);
        const int oi = __shfl_xor(bi, m, 64);
        if (oi != 0x7FFFFFFF && (bi == 0x7FFFFFFF || ov > bv || (ov == bv && oi < bi))) { bv = ov; bi = oi; }
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) { rv[wave] = bv; ri[wave] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < (int)(blockDim.x >> 6); ++w) {
            if (ri[w] != 0x7FFFFFFF && (bi == 0x7FFFFFFF || rv[w] > bv || (rv[w] == bv && ri[w] < bi))) { bv = rv[w]; bi = ri[w]; }
        }
        out[blockIdx.x] = bi == 0x7FFFFFFF ? 0 : bi;
    }
}

// Few long rows (the logits of a decode step): ARGMAX_SPLIT workgroups per row each reduce a slice to one
// (value, index) pair; the workgroup that finishes last for a row (an agent-scope counter tells it) merges the
// pairs and resets the counter for the next launch. Same ordering rule as above, so ties still keep the first.
constexpr int ARGMAX_SPLIT = 64;
constexpr int ARGMAX_MAX_ROWS = 64;
struct ArgmaxScratch { float val[ARGMAX_MAX_ROWS][ARGMAX_SPLIT]; int idx[ARGMAX_MAX_ROWS][ARGMAX_SPLIT]; unsigned done[ARGMAX_MAX_ROWS]; };

__device__ __forceinline__ void argmax_merge(float& bv, int& bi, float ov, int oi) {
    if (oi != 0x7FFFFFFF && (bi == 0x7FFFFFFF || ov > bv || (ov == bv && oi < bi))) { bv = ov; bi = oi; }
}

__global__ __launch_bounds__(ROW_THREADS) void argmax_split_kernel(const float* __restrict__ in, int cols, int32_t* __restrict__ out,
                                                                   ArgmaxScratch* __restrict__ sc) {
    __shared__ float rv[ROW_THREADS / 64];
    __shared__ int ri[ROW_THREADS / 64];
    __shared__ unsigned ticket;
    const int row = blockIdx.y, part = blockIdx.x;
    const float* x = in + (int64_t)row * cols;
    const int per = ((cols + ARGMAX_SPLIT - 1) / ARGMAX_SPLIT + 3) & ~3;
    const int lo = part * per, hi = min(cols, lo + per);
    float bv = -INFINITY;
    int bi = 0x7FFFFFFF;
    for (int i = lo + threadIdx.x; i < hi; i += blockDim.x) {
        const float v = x[i];
        if (v > bv || bi == 0x7FFFFFFF) { bv = v; bi = i; }     // a thread walks upwards: an equal value later is never lower
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) argmax_merge(bv, bi, __shfl_xor(bv, m, 64), __shfl_xor(bi, m, 64));
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) { rv[wave] = bv; ri[wave] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < ROW_THREADS / 64; ++w) argmax_merge(bv, bi, rv[w], ri[w]);
        __hip_atomic_store(&sc->val[row][part], bv, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(&sc->idx[row][part], bi, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        ticket = __hip_atomic_fetch_add(&sc->done[row], 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (ticket != ARGMAX_SPLIT - 1) return;      // uniform over the workgroup
    if (threadIdx.x < 64) {
        bv = __hip_atomic_load(&sc->val[row][threadIdx.x], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        bi = __hip_atomic_load(&sc->idx[row][threadIdx.x], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1) argmax_merge(bv, bi, __shfl_xor(bv, m, 64), __shfl_xor(bi, m, 64));
        if (threadIdx.x == 0) {
            out[row] = bi == 0x7FFFFFFF ? 0 : bi;
            __hip_atomic_store(&sc->done[row], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}
static_assert(ARGMAX_SPLIT == 64, "the merge step reads one pair per lane of a wave");

// dst (row-major) block (o, b) <- src (input-block-major) block (b, o); 2 bytes per thread-step because
// Q8_0 / Q6_K blocks are only 2-byte aligned.
__global__ __launch_bounds__(256) void relayout_to_row_major_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst,
                                                                    int rows, int bpr, int block_bytes) {
    const int64_t blk = blockIdx.x;   // destination block index o * bpr + b
    const int o = (int)(blk / bpr), b = (int)(blk % bpr);
    const uint16_t* s = reinterpret_cast<const uint16_t*>(src + ((int64_t)b * rows + o) * block_bytes);
    uint16_t* d = reinterpret_cast<uint16_t*>(dst + blk * block_bytes);
    for (int i = threadIdx.x; i < block_bytes / 2; i += blockDim.x) d[i] = s[i];
}

// Rotary position embedding fused with the head-major scatter a KV cache / attention operand needs.
//   in  token t, head h at in + t * in_row_pitch + h * head_dim (a column slice of a projection's token-major output;
//       in_row_pitch == heads * head_dim when the slice is the whole row)
//   out [heads, *, head_dim]: element (h, row0 + t, d) at h * out_head_stride + (row0 + t) * head_dim + d,
//       row0 = *pos_dev (when given) or pos_start: the absolute position of token 0, which is also its cache row
//       when out_row_is_pos != 0 (else rows start at 0).
//   rotate != 0: pairs (x[2i], x[2i+1]) of every head are rotated by (row0 + t) * theta^(-2i / head_dim)
//       (the adjacent-pair convention GGUF Llama weights use); rotate == 0 copies (values of the cache).
// The reference has no RoPE (it lives in the external transformer repo), so this op has no reference parity; the
// tests check it against the closed form in float64.
__global__ __launch_bounds__(256) void rope_scatter_kernel(const float* __restrict__ in, int64_t in_row_pitch,
                                                           float* __restrict__ out, int tokens,
                                                           int heads, int head_dim, int pos_start,
                                                           const int32_t* __restrict__ pos_dev, float theta, int rotate,
                                                           int64_t out_head_stride, int out_row_is_pos) {
    const int half = head_dim >> 1;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;   // one thread per (token, head, pair)
    if (idx >= (int64_t)tokens * heads * half) return;
    const int i = (int)(idx % half);
    const int h = (int)((idx / half) % heads);
    const int t = (int)(idx / ((int64_t)half * heads));
    const int p0 = pos_dev ? pos_dev[0] : pos_start;
    const float2 x = *reinterpret_cast<const float2*>(in + (int64_t)t * in_row_pitch + h * head_dim + 2 * i);
    float2 y = x;
    if (rotate) {
        const float freq = powf(theta, -2.0f * (float)i / (float)head_dim);
        float sn, cs;
        sincosf((float)(p0 + t) * freq, &sn, &cs);
        y = rope_rotate(x.x, x.y, cs, sn);
    }
    const int row = (out_row_is_pos ? p0 : 0) + t;
    *reinterpret_cast<float2*>(out + h * out_head_stride + (int64_t)row * head_dim + 2 * i) = y;
}

// The three scatters of a decoder block in one launch: token rows of [q | k | v] (heads, kv_heads, kv_heads heads of
// head_dim) -> rotated queries [heads, tokens, head_dim], rotated keys and raw values into cache rows p0 + t of
// [kv_heads, kv_capacity, head_dim] caches. p0 = *pos_dev when given, else pos_start.
// A thread owns one (token, pair) and walks ROPE_SLOTS_PER_BLOCK head slots with it: the angle's sine and cosine are
// worked out once per thread instead of once per element (same expressions as before, so the same bits).
constexpr int ROPE_SLOTS_PER_BLOCK = 8;
__global__ __launch_bounds__(256) void rope_qkv_kernel(const float* __restrict__ qkv, float* __restrict__ q_out,
                                                       float* __restrict__ k_cache, float* __restrict__ v_cache, int tokens,
                                                       int heads, int kv_heads, int head_dim, int kv_capacity, int pos_start,
                                                       const int32_t* __restrict__ pos_dev, float theta) {
    const int half = head_dim >> 1;
    const int slots = heads + 2 * kv_heads;
    const uint32_t idx = blockIdx.x * blockDim.x + threadIdx.x;   // one thread per (token, pair); the host checks the count fits 31 bits
    if (idx >= (uint32_t)tokens * (uint32_t)half) return;
    const int i = (int)(idx % (uint32_t)half);
    const int t = (int)(idx / (uint32_t)half);
    const int p0 = pos_dev ? pos_dev[0] : pos_start;
    const float freq = powf(theta, -2.0f * (float)i / (float)head_dim);
    float sn, cs;
    sincosf((float)(p0 + t) * freq, &sn, &cs);
    const int hs0 = blockIdx.y * ROPE_SLOTS_PER_BLOCK;
    float2 x[ROPE_SLOTS_PER_BLOCK];
#pragma unroll
    for (int u = 0; u < ROPE_SLOTS_PER_BLOCK; ++u)
        x[u] = *reinterpret_cast<const float2*>(qkv + ((int64_t)t * slots + min(hs0 + u, slots - 1)) * head_dim + 2 * i);
#pragma unroll
    for (int u = 0; u < ROPE_SLOTS_PER_BLOCK; ++u) {
        const int hs = hs0 + u;
        if (hs >= slots) break;
        float2 y = x[u];
        if (hs < heads + kv_heads) {
            y = rope_rotate(x[u].x, x[u].y, cs, sn);
        }
        float* dst;
        if (hs < heads) dst = q_out + ((int64_t)hs * tokens + t) * head_dim;
        else {
            if (p0 < 0 || p0 + t >= kv_capacity) continue;      // a device-side position past the cache: nothing is written
            if (hs < heads + kv_heads) dst = k_cache + ((int64_t)(hs - heads) * kv_capacity + p0 + t) * head_dim;
            else dst = v_cache + ((int64_t)(hs - heads - kv_heads) * kv_capacity + p0 + t) * head_dim;
        }
        *reinterpret_cast<float2*>(dst + 2 * i) = y;
    }
}

// [heads, tokens, head_dim] -> [tokens, heads * head_dim]: attention output back to the token-major rows a projection takes.
__global__ __launch_bounds__(256) void heads_to_rows_kernel(const float* __restrict__ in, float* __restrict__ out, int heads,
                                                            int tokens, int head_dim) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;   // one thread per float4 of the output
    const int d4 = head_dim >> 2;
    if (idx >= (int64_t)heads * tokens * d4) return;
    const int d = (int)(idx % d4);
    const int h = (int)((idx / d4) % heads);
    const int t = (int)(idx / ((int64_t)d4 * heads));
    reinterpret_cast<float4*>(out)[idx] = reinterpret_cast<const float4*>(in)[((int64_t)h * tokens + t) * d4 + d];
}

__global__ void i32_increment_kernel(int32_t* v, int32_t delta) {
    if (threadIdx.x == 0 && blockIdx.x == 0) v[0] += delta;
}

__global__ void i32_store_at_kernel(int32_t* dst, const int32_t* __restrict__ index, int32_t offset, const int32_t* __restrict__ src) {
    if (threadIdx.x == 0 && blockIdx.x == 0) dst[index[0] + offset] = src[0];
}

// (cos, sin) of (*pos) * theta^(-2i / head_dim) for i < head_dim / 2: the rotation table of one decode position, computed
// once per token and read by every layer's q/k/v epilogue (same expressions as rope_qkv_kernel, so the same bits).
__global__ void rope_table_kernel(const int32_t* __restrict__ pos, float theta, int head_dim, float2* __restrict__ table) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= head_dim / 2) return;
    float sn, cs;
    sincosf((float)pos[0] * powf(theta, -2.0f * (float)i / (float)head_dim), &sn, &cs);
    table[i] = make_float2(cs, sn);
}
int launch_rope_table(const int32_t* pos, float theta, int head_dim, float* table) {
    if (head_dim <= 0 || (head_dim & 1)) return set_error("rope_table: head_dim must be positive and even; got %d", head_dim);
    rope_table_kernel<<<dim3((head_dim / 2 + 63) / 64), dim3(64), 0, current_stream()>>>(pos, theta, head_dim, reinterpret_cast<float2*>(table));
    SKH_CHECK(hipGetLastError());
    return 0;
}

// End of a greedy decode step in one launch: the position and the key count advance by one and the token just
// sampled is appended to the log at the new position. The position saturates at `capacity` (the cache's row count, the
// log holds capacity + 1 entries): a step replayed past the end writes nothing anywhere and the host sees pos == capacity.
__global__ void decode_advance_kernel(int32_t* pos, int32_t* kv_len, const int32_t* __restrict__ token, int32_t* log, int32_t capacity) {
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        const int32_t p = pos[0] + 1;
        if (p > capacity) return;
        pos[0] = p;
        kv_len[0] = min(kv_len[0] + 1, capacity);
        log[p] = token[0];
    }
}
int launch_decode_advance(int32_t* pos, int32_t* kv_len, const int32_t* token, int32_t* log, int32_t capacity) {
    if (capacity <= 0) return set_error("decode_advance: capacity must be positive; got %d", capacity);
    decode_advance_kernel<<<dim3(1), dim3(64), 0, current_stream()>>>(pos, kv_len, token, log, capacity);
    SKH_CHECK(hipGetLastError());
    return 0;
}

int launch_rope_scatter(const float* in, int64_t in_row_pitch, float* out, int tokens, int heads, int head_dim, int pos_start,
                        const int32_t* pos_dev, float theta, int rotate, int64_t out_head_stride, int out_row_is_pos) {
    if (tokens <= 0 || heads <= 0 || head_dim <= 0) return 0;
    if ((head_dim & 1) || (in_row_pitch & 1)) return set_error("rope: head_dim and the row pitch must be even; got %d, %lld", head_dim, (long long)in_row_pitch);
    const int64_t n = (int64_t)tokens * heads * (head_dim / 2);
    rope_scatter_kernel<<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, current_stream()>>>(
        in, in_row_pitch, out, tokens, heads, head_dim, pos_start, pos_dev, theta, rotate, out_head_stride, out_row_is_pos);
    SKH_CHECK(hipGetLastError());
    return 0;
}
int launch_rope_qkv(const float* qkv, float* q_out, float* k_cache, float* v_cache, int tokens, int heads, int kv_heads,
                    int head_dim, int kv_capacity, int pos_start, const int32_t* pos_dev, float theta) {
    if (tokens <= 0 || heads <= 0 || kv_heads <= 0 || head_dim <= 0) return 0;
    if (head_dim & 1) return set_error("rope: head_dim must be even; got %d", head_dim);
    if (!pos_dev && (pos_start < 0 || pos_start + tokens > kv_capacity))
        return set_error("rope_qkv: positions [%d, %d) do not fit a cache of %d rows", pos_start, pos_start + tokens, kv_capacity);
    const int64_t n = (int64_t)tokens * (head_dim / 2);
    if (n >= (int64_t)1 << 31) return set_error("rope_qkv: %d tokens x %d pairs exceed the 31-bit thread index", tokens, head_dim / 2);
    const int slot_blocks = (heads + 2 * kv_heads + ROPE_SLOTS_PER_BLOCK - 1) / ROPE_SLOTS_PER_BLOCK;
    rope_qkv_kernel<<<dim3((unsigned)((n + 255) / 256), slot_blocks), dim3(256), 0, current_stream()>>>(
        qkv, q_out, k_cache, v_cache, tokens, heads, kv_heads, head_dim, kv_capacity, pos_start, pos_dev, theta);
    SKH_CHECK(hipGetLastError());
    return 0;
}
int launch_heads_to_rows(const float* in, float* out, int heads, int tokens, int head_dim) {
    if (tokens <= 0 || heads <= 0 || head_dim <= 0) return 0;
    if (head_dim & 3) return set_error("heads_to_rows: head_dim must be a multiple of 4; got %d", head_dim);
    const int64_t n = (int64_t)heads * tokens * (head_dim / 4);
    heads_to_rows_kernel<<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, current_stream()>>>(in, out, heads, tokens, head_dim);
    SKH_CHECK(hipGetLastError());
    return 0;
}
int launch_i32_store_at(int32_t* dst, const int32_t* index, int32_t offset, const int32_t* src) {
    i32_store_at_kernel<<<dim3(1), dim3(64), 0, current_stream()>>>(dst, index, offset, src);
    SKH_CHECK(hipGetLastError());
    return 0;
}
int launch_i32_increment(int32_t* v, int32_t delta) {
    i32_increment_kernel<<<dim3(1), dim3(64), 0, current_stream()>>>(v, delta);
    SKH_CHECK(hipGetLastError());
    return 0;
}

// Calibration kernel: every thread streams 16-byte loads over a buffer with four independent loads in flight and
// almost no arithmetic. Its rate is what this device sustains for a read-once pass of that size.
__global__ __launch_bounds__(256) void stream_read_kernel(const uint4* __restrict__ p, int64_t n16, uint32_t* __restrict__ sink) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    uint32_t acc = 0;
    for (; i + 3 * stride < n16; i += 4 * stride) {
        const uint4 a = p[i], b = p[i + stride], c = p[i + 2 * stride], d = p[i + 3 * stride];
        acc += a.x ^ b.y ^ c.z ^ d.w;
    }
    for (; i < n16; i += stride) acc += p[i].x;
    if (acc == 0x9E3779B9u) sink[0] = acc;   // keeps the loads alive; practically never true
}

int launch_stream_read(const void* p, int64_t bytes, int grid, uint32_t* sink) {
    if (bytes < 16) return 0;
    stream_read_kernel<<<dim3(grid > 0 ? grid : 2 * num_cus()), dim3(256), 0, current_stream()>>>(static_cast<const uint4*>(p), bytes / 16, sink);
    SKH_CHECK(hipGetLastError());
    return 0;
}

int launch_rms_norm(const float* in, const float* gamma, float* out, int rows, int cols, float eps) {
    if (rows <= 0 || cols <= 0) return 0;
    const bool aligned = ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(gamma)) & 15) == 0;
    if (aligned && (cols & 3) == 0 && cols <= 4 * ROW_THREADS * 8) {
        if (cols <= 4 * ROW_THREADS * 4) rms_norm_cached_kernel<4><<<dim3(rows), dim3(ROW_THREADS), 0, current_stream()>>>(in, gamma, out, cols, eps);
        else rms_norm_cached_kernel<8><<<dim3(rows), dim3(ROW_THREADS), 0, current_stream()>>>(in, gamma, out, cols, eps);
        SKH_CHECK(hipGetLastError());
        return 0;
    }
    rms_norm_kernel<<<dim3(rows), dim3(ROW_THREADS), 0, current_stream()>>>(in, gamma, out, cols, eps);
    SKH_CHECK(hipGetLastError());
    return 0;
}
int launch_layer_norm(const float* in, const float* gamma, const float* beta, float* out, int rows, int cols, float eps) {
    if (rows <= 0 || cols <= 0) return 0;
    layer_norm_kernel<<<dim3(rows), dim3(ROW_THREADS), 0, current_stream()>>>(in, gamma, beta, out, cols, eps);
    SKH_CHECK(hipGetLastError());
    return 0;
}
int launch_softmax_rows(const float* in, float* out, int rows, int cols, int log_form) {
    if (rows <= 0 || cols <= 0) return 0;
    softmax_rows_kernel<<<dim3(rows), dim3(ROW_THREADS), 0, current_stream()>>>(in, out, cols, log_form);
    SKH_CHECK(hipGetLastError());
    return 0;
}
int launch_silu_mul(const float* gate, const float* up, float* out, int64_t n) {
    if (n <= 0) return 0;
    silu_mul_kernel<<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, current_stream()>>>(gate, up, out, n);
    SKH_CHECK(hipGetLastError());
    return 0;
}
int launch_swiglu_pairs(const float* gate_up, float* out, int64_t n) {
    if (n <= 0) return 0;
    swiglu_pairs_kernel<<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, current_stream()>>>(reinterpret_cast<const float2*>(gate_up), out, n);
    SKH_CHECK(hipGetLastError());
    return 0;
}
int launch_add(const float* a, const float* b, float* out, int64_t n) {
    if (n <= 0) return 0;
    add_kernel<<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, current_stream()>>>(a, b, out, n);
    SKH_CHECK(hipGetLastError());
    return 0;
}
int launch_argmax_rows(const float* in, int rows, int cols, int32_t* out) {
    if (rows <= 0 || cols <= 0) return 0;
    if (rows <= ARGMAX_MAX_ROWS && cols >= 16384) {
        ArgmaxScratch* sc = static_cast<ArgmaxScratch*>(sync_scratch(sizeof(ArgmaxScratch)));
        if (!sc) return -1;
        argmax_split_kernel<<<dim3(ARGMAX_SPLIT, rows), dim3(ROW_THREADS), 0, current_stream()>>>(in, cols, out, sc);
        SKH_CHECK(hipGetLastError());
        return 0;
    }
    argmax_rows_kernel<<<dim3(rows), dim3(ROW_THREADS), 0, current_stream()>>>(in, cols, out);
    SKH_CHECK(hipGetLastError());
    return 0;
}
// ---- arg-max for callers that cannot allocate ----
// The same many-workgroups-per-row kernel, with its pairs and counters in a fixed array that is part of the loaded code
// object: every GPU the library runs on holds its own copy until the process ends. In host code the array's name is
// only a handle; the device address comes from hipGetSymbolAddress, once per device, and that address is what the
// kernels are given.
// Everything else in the library is per host thread (stream, scratch), so the array is cut into NOALLOC_SLOTS slots and
// a host thread is handed one on its first call (an atomic counter; kept until the process ends): threads that each use
// their own stream do not share counters. A thread that comes after the slots have run out is refused with a message.
constexpr int NOALLOC_SLOTS = 8;
constexpr size_t NOALLOC_SLOT_BYTES = (sizeof(ArgmaxScratch) + 255) & ~(size_t)255;
static __device__ __align__(256) unsigned char scratch[NOALLOC_SLOTS * NOALLOC_SLOT_BYTES];
static std::atomic<int> g_noalloc_next_slot{0};
static thread_local int t_noalloc_slot = -1;
// this thread's slot (handed out on first use), -1 when every slot is taken; no device call
int argmax_noalloc_slot() {
    if (t_noalloc_slot < 0) {
        int s = g_noalloc_next_slot.load();
        while (s < NOALLOC_SLOTS && !g_noalloc_next_slot.compare_exchange_weak(s, s + 1)) {}
        if (s >= NOALLOC_SLOTS) return -1;
        t_noalloc_slot = s;
    }
    return t_noalloc_slot;
}
constexpr int NOALLOC_MAX_DEVICES = 64;
static void* g_noalloc_scratch[NOALLOC_MAX_DEVICES];    // per device, filled on first use
static std::mutex g_noalloc_mutex;

__global__ void argmax_clear_kernel(ArgmaxScratch* __restrict__ sc, int rows) {
    if ((int)threadIdx.x < rows) sc->done[threadIdx.x] = 0u;
}

static ArgmaxScratch* noalloc_scratch() {
    const int slot = argmax_noalloc_slot();
    if (slot < 0) { set_error("argmax_rows_noalloc: all %d scratch slots are held by other host threads; use skainet_hip_f32_argmax_rows_dev", NOALLOC_SLOTS); return nullptr; }
    int dev = -1;
    if (check_hip(hipGetDevice(&dev), "hipGetDevice") != 0) return nullptr;
    if (dev < 0 || dev >= NOALLOC_MAX_DEVICES) { set_error("argmax_rows_noalloc: device ordinal %d is beyond the %d this entry keeps scratch for", dev, NOALLOC_MAX_DEVICES); return nullptr; }
    std::lock_guard<std::mutex> lock(g_noalloc_mutex);
    if (!g_noalloc_scratch[dev]) {
        void* ptr = nullptr;
        if (check_hip(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)") != 0) return nullptr;
        if (!ptr) { set_error("argmax_rows_noalloc: no device address for the scratch array"); return nullptr; }
        g_noalloc_scratch[dev] = ptr;
    }
    return reinterpret_cast<ArgmaxScratch*>(static_cast<unsigned char*>(g_noalloc_scratch[dev]) + (size_t)slot * NOALLOC_SLOT_BYTES);
}

int launch_argmax_rows_noalloc(const float* in, int rows, int cols, int32_t* out) {
    if (rows <= 0 || cols <= 0) return 0;
    if (rows > ARGMAX_MAX_ROWS)
        return set_error("argmax_rows_noalloc: %d rows exceed the %d rows the fixed scratch holds; use skainet_hip_f32_argmax_rows_dev", rows, ARGMAX_MAX_ROWS);
    ArgmaxScratch* sc = noalloc_scratch();
    if (!sc) return -1;
    // the array keeps what the last call left: the arrival counters must start at zero (a fill kernel, not a memset
    // node, so the pair can be recorded into a graph)
    argmax_clear_kernel<<<dim3(1), dim3(ARGMAX_MAX_ROWS), 0, current_stream()>>>(sc, rows);
    SKH_CHECK(hipGetLastError());
    argmax_split_kernel<<<dim3(ARGMAX_SPLIT, rows), dim3(ROW_THREADS), 0, current_stream()>>>(in, cols, out, sc);
    SKH_CHECK(hipGetLastError());
    return 0;
}

int launch_relayout_to_row_major(const uint8_t* src, uint8_t* dst, int rows, int bpr, int block_bytes) {
    if (rows <= 0 || bpr <= 0) return 0;
    relayout_to_row_major_kernel<<<dim3((unsigned)((int64_t)rows * bpr)), dim3(64), 0, current_stream()>>>(src, dst, rows, bpr, block_bytes);
    SKH_CHECK(hipGetLastError());
    return 0;
}

}  // namespace skh

extern "C" int32_t skainet_hip_f32_argmax_rows_noalloc_slot(void) { return skh::argmax_noalloc_slot(); }

extern "C" int32_t skainet_hip_f32_argmax_rows_noalloc_dev(const float* in, int32_t rows, int32_t cols, int32_t* out) {
    if (skh::ensure_device() != 0) return -1;
    if (rows > 0 && cols > 0 && (!in || !out)) return skh::set_error("argmax_rows_noalloc: null pointer");
    return skh::launch_argmax_rows_noalloc(in, rows, cols, out);
}
