// Fused scaled-dot-product attention, fp32:  out = softmax(q k^T * scale + rules + mask) v
//
// Contract = the reference's skainet_f32_sdpa
//   /root/reference/skainet-backends/skainet-backend-native-cpu/native/src/f32_fused.c:290-396
// with the structural rules of
//   /root/reference/skainet-lang/skainet-lang-core/src/commonMain/kotlin/sk/ainet/lang/tensor/ops/AttentionMask.kt:24-104
//   q [B, H, Sq, D], k / v [B, Hkv, Skv, D], head h reads kv head h / (H / Hkv);
//   absQ = Skv - Sq + qi; causal: ki <= absQ; window w (+ right context r): absQ - w + 1 <= ki <= absQ + r;
//   lengths: ki < lengths[b]; a key outside the set scores -1e30 (finite: a fully masked row is uniform);
//   an additive mask broadcast over [B|1, H|Hkv|1, Sq|1, Skv|1] is added to EVERY score, masked ones included.
//
// sdpa_rows_kernel is the general kernel (every rule, any head_dim <= 256): one workgroup per
// (batch, kv head, query position); its G = H / Hkv waves are the query heads that share that K/V head, so
// a 64-key tile of K, then of V, is staged in LDS once and used by all G rows. Each wave keeps a running
// max / sum (online softmax) and its slice of the output in registers; keys the rules exclude are never
// loaded unless a mask (or an empty key set) makes their -1e30 score matter.
#include "gemv_q4k.h"

namespace skh {

constexpr float SDPA_MASKED = -1.0e30f;
constexpr int SDPA_TILE = 64;        // keys per LDS tile
constexpr int SDPA_MAX_D = 256;
constexpr int SDPA_MAX_GROUP = 16;   // query heads per workgroup

struct SdpaParams {
    const float *q, *k, *v;
    float* out;
    int batch, heads, kv_heads, seq_q, seq_kv, head_dim;
    int kv_capacity;  // key rows of storage per kv head (>= seq_kv): a KV cache holds more rows than are attended
    float scale;
    int causal, window, right_context;
    const int32_t* lengths;
    const float* mask;
    int mask_b, mask_h, mask_q, mask_k;
    int group;        // query heads handled by one workgroup (divides heads / kv_heads)
    int splits;       // key-range splits (gridDim.y); > 1 writes partial results to `part`
    float* part;      // [rows][splits][head_dim + 2]: unnormalised output, running max, running sum
};

__global__ __launch_bounds__(64 * SDPA_MAX_GROUP) void sdpa_rows_kernel(SdpaParams p) {
    extern __shared__ float smem[];
    const int d = p.head_dim, dp = d + 1;
    float* tile = smem;                         // [SDPA_TILE][d + 1]
    float* qs = tile + SDPA_TILE * dp;          // [group][d]
    float* probs = qs + p.group * d;            // [group][SDPA_TILE]

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int per_kv = p.heads / p.kv_heads;
    const int groups_per_kv = per_kv / p.group;
    int idx = blockIdx.x;
    const int qi = idx % p.seq_q; idx /= p.seq_q;
    const int gsel = idx % groups_per_kv; idx /= groups_per_kv;
    const int kvh = idx % p.kv_heads;
    const int b = idx / p.kv_heads;
    const int h = kvh * per_kv + gsel * p.group + wave;

    const float* qrow = p.q + (((int64_t)b * p.heads + h) * p.seq_q + qi) * d;
    const float* kb = p.k + ((int64_t)b * p.kv_heads + kvh) * p.kv_capacity * d;
    const float* vb = p.v + ((int64_t)b * p.kv_heads + kvh) * p.kv_capacity * d;
    float* orow = p.out + (((int64_t)b * p.heads + h) * p.seq_q + qi) * d;

    // Attended key range [first, end) of this query position.
    const int abs_q = p.seq_kv - p.seq_q + qi;
    int first = 0, end = p.seq_kv;
    if (p.window > 0) {
        first = max(first, abs_q - p.window + 1);
        end = min(end, abs_q + p.right_context + 1);
    }
    if (p.causal) end = min(end, abs_q + 1);
    if (p.lengths) end = min(end, p.lengths[b]);
    end = max(end, 0);
    first = min(first, end);
    // Keys that take part in the softmax: the range, or every key when a mask can lift a masked score or the
    // range is empty (uniform row).
    const bool all_keys = p.mask != nullptr || first >= end;
    int lo = all_keys ? 0 : first, hi = all_keys ? p.seq_kv : end;
    if (p.splits > 1) {
        // Split the key range into tile-aligned chunks; a split past the end simply contributes nothing.
        const int chunk = ((hi - lo + p.splits - 1) / p.splits + SDPA_TILE - 1) / SDPA_TILE * SDPA_TILE;
        lo = lo + (int)blockIdx.y * chunk;
        hi = min(hi, lo + chunk);
    }

    const float* mrow = nullptr;
    if (p.mask) {
        const int bi = p.mask_b == 1 ? 0 : b;
        const int hi_ = p.mask_h == 1 ? 0 : (p.mask_h == p.heads ? h : kvh);
        mrow = p.mask + (((int64_t)bi * p.mask_h + hi_) * p.mask_q + (p.mask_q == 1 ? 0 : qi)) * p.mask_k;
    }

    for (int x = lane; x < d; x += 64) qs[wave * d + x] = qrow[x];
    float acc[SDPA_MAX_D / 64];
#pragma unroll
    for (int i = 0; i < SDPA_MAX_D / 64; ++i) acc[i] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;

    for (int k0 = lo; k0 < hi; k0 += SDPA_TILE) {
        const int nk = min(SDPA_TILE, hi - k0);
        __syncthreads();   // previous V tile fully consumed (and qs visible on the first trip)
        for (int t = threadIdx.x; t < nk * d; t += blockDim.x) tile[(t / d) * dp + (t % d)] = kb[(int64_t)k0 * d + t];
        __syncthreads();
        const int ki = k0 + lane;
        float s = -INFINITY;
        if (lane < nk) {
            if (ki >= first && ki < end) {
                float dot = 0.f;
                const float* kr = tile + lane * dp;
                const float* qv = qs + wave * d;
                for (int x = 0; x < d; ++x) dot = fmaf(qv[x], kr[x], dot);
                s = dot * p.scale;
            } else {
                s = SDPA_MASKED;
            }
            if (mrow) s += p.mask_k == 1 ? mrow[0] : mrow[ki];
        }
        const float m_new = fmaxf(m_run, wave_max(s));
        const float alpha = expf(m_run - m_new);          // exp(-inf) = 0 on the first tile
        const float pl = lane < nk ? expf(s - m_new) : 0.f;
        l_run = l_run * alpha + wave_sum(pl);
        m_run = m_new;
        probs[wave * SDPA_TILE + lane] = pl;
        __syncthreads();   // every wave is done with the K tile
        for (int t = threadIdx.x; t < nk * d; t += blockDim.x) tile[(t / d) * dp + (t % d)] = vb[(int64_t)k0 * d + t];
        __syncthreads();
        const float* pw = probs + wave * SDPA_TILE;
#pragma unroll
        for (int i = 0; i < SDPA_MAX_D / 64; ++i) {
            const int x = lane + 64 * i;
            if (x < d) {
                float a = acc[i] * alpha;
                for (int j = 0; j < nk; ++j) a = fmaf(pw[j], tile[j * dp + x], a);
                acc[i] = a;
            }
        }
    }
    if (p.splits > 1) {
        const int64_t row = ((int64_t)b * p.heads + h) * p.seq_q + qi;
        float* dst = p.part + (row * p.splits + blockIdx.y) * (d + 2);
#pragma unroll
        for (int i = 0; i < SDPA_MAX_D / 64; ++i) {
            const int x = lane + 64 * i;
            if (x < d) dst[x] = acc[i];
        }
        if (lane == 0) { dst[d] = m_run; dst[d + 1] = l_run; }
        return;
    }
    const float inv = l_run > 0.f ? 1.0f / l_run : 0.f;
#pragma unroll
    for (int i = 0; i < SDPA_MAX_D / 64; ++i) {
        const int x = lane + 64 * i;
        if (x < d) orow[x] = acc[i] * inv;
    }
}

// Merge the per-split (unnormalised output, max, sum) triples of one query row: one wave per row.
__global__ __launch_bounds__(64) void sdpa_combine_kernel(const float* __restrict__ part, float* __restrict__ out, int splits, int d) {
    const int64_t row = blockIdx.x;
    const float* src = part + row * splits * (d + 2);
    float m = -INFINITY;
    for (int s = 0; s < splits; ++s) m = fmaxf(m, src[s * (d + 2) + d]);
    float l = 0.f;
    for (int s = 0; s < splits; ++s) l += src[s * (d + 2) + d + 1] * expf(src[s * (d + 2) + d] - m);
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    for (int x = threadIdx.x; x < d; x += 64) {
        float a = 0.f;
        for (int s = 0; s < splits; ++s) a = fmaf(src[s * (d + 2) + x], expf(src[s * (d + 2) + d] - m), a);
        out[row * d + x] = a * inv;
    }
}

__global__ __launch_bounds__(256) void zero_kernel(float* out, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = 0.f;
}

float* sdpa_workspace(size_t bytes);   // shim.hip: per-thread scratch, grown on demand
int launch_sdpa_decode(const float* q, const float* k, const float* v, float* out, int batch, int heads, int kv_heads,
                       int seq_kv, int kv_capacity, int head_dim, float scale, int window, int right_context,
                       const int32_t* lengths, AttnMergePrologue* leave);   // sdpa_decode.hip
int launch_sdpa_prefill(const float* q, const float* k, const float* v, float* out, int batch, int heads, int kv_heads,
                        int seq_q, int seq_kv, int kv_capacity, int head_dim, float scale, int causal, int window,
                        int right_context, const int32_t* lengths, const float* mask, int mask_b, int mask_h, int mask_q,
                        int mask_k, int out_rows);   // sdpa_prefill.hip

int launch_sdpa(const float* q, const float* k, const float* v, float* out, int batch, int heads, int kv_heads,
                int seq_q, int seq_kv, int kv_capacity, int head_dim, float scale, int causal, int window, int right_context,
                const int32_t* lengths, const float* mask, int mask_b, int mask_h, int mask_q, int mask_k) {
    if (batch <= 0 || heads <= 0 || kv_heads <= 0 || seq_q <= 0 || head_dim <= 0) return 0;
    if (heads % kv_heads != 0) return set_error("sdpa: heads (%d) must be a multiple of kv_heads (%d)", heads, kv_heads);
    if (window < 0 || right_context < 0) return set_error("sdpa: window and rightContext must be >= 0");
    if (right_context != 0 && window == 0) return set_error("sdpa: rightContext (%d) is only meaningful with window > 0", right_context);
    if (kv_capacity < seq_kv) return set_error("sdpa: kv capacity %d is below seq_kv %d", kv_capacity, seq_kv);
    if (head_dim > SDPA_MAX_D) return set_error("sdpa: head_dim %d exceeds %d", head_dim, SDPA_MAX_D);
    const int64_t rows = (int64_t)batch * heads * seq_q;
    hipStream_t s = current_stream();
    if (seq_kv <= 0) {
        const int64_t n = rows * head_dim;
        zero_kernel<<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s>>>(out, n);
        SKH_CHECK(hipGetLastError());
        return 0;
    }
    if (mask) {
        const bool ok = (mask_b == 1 || mask_b == batch) && (mask_h == 1 || mask_h == heads || mask_h == kv_heads) &&
                        (mask_q == 1 || mask_q == seq_q) && (mask_k == 1 || mask_k == seq_kv);
        if (!ok) return set_error("sdpa: mask dims [%d,%d,%d,%d] do not broadcast over [%d,%d|%d,%d,%d]", mask_b, mask_h,
                                  mask_q, mask_k, batch, heads, kv_heads, seq_q, seq_kv);
    }
    if (seq_q == 1 && !mask) {   // decode shape: the split-K cache-streaming kernel, when the head shape is one it carries
        const int r = launch_sdpa_decode(q, k, v, out, batch, heads, kv_heads, seq_kv, kv_capacity, head_dim, scale, window,
                                         right_context, lengths, nullptr);
        if (r != 0) return r < 0 ? -1 : 0;
    }
    if (seq_q > 1) {   // prompt shape: the matrix-core kernel, when it carries the shape (and the mask's layout)
        const int r = launch_sdpa_prefill(q, k, v, out, batch, heads, kv_heads, seq_q, seq_kv, kv_capacity, head_dim, scale, causal,
                                          window, right_context, lengths, mask, mask_b, mask_h, mask_q, mask_k, 0);
        if (r != 0) return r < 0 ? -1 : 0;
    }
    SdpaParams p{q, k, v, out, batch, heads, kv_heads, seq_q, seq_kv, head_dim, kv_capacity, scale, causal, window, right_context,
                 lengths, mask, mask_b, mask_h, mask_q, mask_k, 1, 1, nullptr};
    const int per_kv = heads / kv_heads;
    int group = per_kv;
    while (group > SDPA_MAX_GROUP || per_kv % group != 0) --group;
    p.group = group;
    const int64_t grid = (int64_t)batch * kv_heads * (per_kv / group) * seq_q;
    if (grid > 0x7FFFFFFFLL) return set_error("sdpa: %lld query rows exceed one launch", (long long)grid);
    // Few query rows (decode): split the keys so the whole chip streams the KV cache, then merge.
    int splits = 1;
    const int64_t want = 2 * (int64_t)num_cus();
    if (grid < want) {
        splits = (int)((want + grid - 1) / grid);
        const int max_splits = (seq_kv + 2 * SDPA_TILE - 1) / (2 * SDPA_TILE);
        if (splits > max_splits) splits = max_splits;
        if (splits < 1) splits = 1;
    }
    if (splits > 1) {
        p.splits = splits;
        p.part = sdpa_workspace(sizeof(float) * (size_t)rows * splits * (head_dim + 2));
        if (!p.part) return -1;
    }
    const size_t smem = sizeof(float) * ((size_t)SDPA_TILE * (head_dim + 1) + (size_t)group * head_dim + (size_t)group * SDPA_TILE);
    note_kernel("sdpa_rows_kernel");
    sdpa_rows_kernel<<<dim3((unsigned)grid, (unsigned)splits), dim3(64 * group), smem, s>>>(p);
    SKH_CHECK(hipGetLastError());
    if (splits > 1) {
        sdpa_combine_kernel<<<dim3((unsigned)rows), dim3(64), 0, s>>>(p.part, out, splits, head_dim);
        SKH_CHECK(hipGetLastError());
    }
    return 0;
}

}  // namespace skh
