// Decode-shape attention (one query position per sequence) over a KV cache: bandwidth-bound split-K.
//
// Same contract as the general kernel in sdpa.hip (reference: skainet_f32_sdpa,
//   /root/reference/skainet-backends/skainet-backend-native-cpu/native/src/f32_fused.c:290-396, rules of
//   /root/reference/skainet-lang/skainet-lang-core/src/commonMain/kotlin/sk/ainet/lang/tensor/ops/AttentionMask.kt:24-104)
// for seq_q == 1 and no additive mask: the attended keys are one range [first, end) per sequence (window, causal
// and key-length rules all cut a range), an empty range means uniform weights over every key.
//
// The K/V rows of a cache are read exactly once, straight from HBM into registers, no LDS staging:
//   * grid (key splits, kv heads x head sub-groups, batch); a workgroup owns one split of the key range of one
//     KV head and GS of the query heads that share it, so a K/V row is loaded once for GS heads;
//   * 16 lanes hold one key row (D / 16 consecutive floats each), a wave covers 4 adjacent keys per load
//     instruction (one contiguous span of 4 rows), the 4 waves interleave groups of 4 keys;
//   * every 16-lane group keeps its own online-softmax state (running max, sum, output slice) for its keys, so
//     the key loop has no cross-lane traffic beyond the 4-step dot-product reduction (DPP rotates inside a row of 16
//     lanes); the 16 states of a workgroup are merged once, through LDS;
//   * splits > 1: each workgroup writes an unnormalised partial (output, max, sum) and a second, small kernel
//     merges them. Merging in the last-arriving workgroup instead was built twice and is slower on this multi-die
//     part: with an agent-scope release / acquire per workgroup (whole L2s written back and invalidated), and with
//     no fence at all -- partials as agent-scope atomic stores / loads that bypass the L2s, one relaxed ticket per
//     workgroup: results identical, but the ticket and the reads behind it are two more trips to memory, about what
//     the second launch costs at 10 splits and far more at 64 (4096 keys: 21.8 us against 12.3).
#include "gemv_q4k.h"

namespace skh {

constexpr float SDPA_DECODE_MASKED = -1.0e30f;
constexpr int SDPA_DECODE_MAX_SPLITS = 64;

struct SdpaDecodeParams {
    const float *q, *k, *v;
    float* out;
    int batch, heads, kv_heads, seq_kv, kv_capacity;
    float scale;
    int window, right_context;
    const int32_t* lengths;
    int splits;
    float* part;          // [batch * heads][splits][D] unnormalised outputs; null: one split, the normalised result goes to out
    float* ml;            // [batch * heads][splits][2] running maximum (in units of ln 2) and sum of each split
};

// Scores are kept in units of ln 2 (the query is scaled by scale * log2(e) once), so every exponential of the softmax is
// one v_exp_f32 of a difference: no range reduction, no multiply. For the differences that carry weight (|x| < 30) the
// rounding of the scaled score moves the result by under 3e-6 relative.
constexpr float SDPA_LOG2E = 1.44269504088896340736f;
__device__ __forceinline__ float exp2_raw(float x) { return __builtin_amdgcn_exp2f(x); }
// 2^(m_old - m_new), 0 for an empty state; the exponential is evaluated unconditionally (a select, not a branch)
__device__ __forceinline__ float exp_diff(float m_old, float m_new) {
    const float e = exp2_raw(m_old - m_new);
    return m_old == -INFINITY ? 0.f : e;
}

template <int GS, int DPL>
__global__ __launch_bounds__(256) void sdpa_decode_kernel(SdpaDecodeParams p) {
    constexpr int D = 16 * DPL;
    constexpr int U = 2;                       // groups of 4 keys a wave has in flight
    __shared__ __attribute__((aligned(16))) float wacc[16][GS][D];
    __shared__ __attribute__((aligned(16))) float cw[GS][16];
    __shared__ float wm[GS][16], wl[GS][16], wmm[GS], wls[GS];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // uniform, and said so: the key loop's exits stay scalar branches
    const int sub = lane & 15, kg = lane >> 4;
    const int split = blockIdx.x, b = blockIdx.z;
    const int per_kv = p.heads / p.kv_heads;
    const int subs = per_kv / GS;
    const int kvh = blockIdx.y / subs;
    const int h0 = kvh * per_kv + (blockIdx.y % subs) * GS;

    // attended key range of this sequence's single query (absolute position seq_kv - 1, so causal cuts nothing)
    int first = 0, end = p.seq_kv;
    if (p.window > 0) {
        first = max(first, p.seq_kv - p.window);
        end = min(end, p.seq_kv + p.right_context);
    }
    if (p.lengths) end = min(end, p.lengths[b]);
    end = max(end, 0);
    const bool uniform = first >= end;         // nothing attended: every key scores the same finite value
    if (uniform) { first = 0; end = p.seq_kv; }
    const int chunk = ((end - first + p.splits - 1) / p.splits + 15) & ~15;
    const int lo = first + split * chunk;
    const int hi = min(end, lo + chunk);

    const float qscale = p.scale * SDPA_LOG2E;
    float qr[GS][DPL];
#pragma unroll
    for (int g = 0; g < GS; ++g) {
        const float* qp = p.q + ((int64_t)b * p.heads + h0 + g) * D + sub * 4;
#pragma unroll
        for (int d = 0; d < DPL; d += 4) {
            const float4 t = *reinterpret_cast<const float4*>(qp + 16 * d);   // float4 number d / 4 of the lane: elements 64 (d / 4) + 4 sub ..
            qr[g][d] = t.x * qscale; qr[g][d + 1] = t.y * qscale; qr[g][d + 2] = t.z * qscale; qr[g][d + 3] = t.w * qscale;
        }
    }
    float m[GS], l[GS], acc[GS][DPL];
#pragma unroll
    for (int g = 0; g < GS; ++g) {
        m[g] = -INFINITY; l[g] = 0.f;
#pragma unroll
        for (int d = 0; d < DPL; ++d) acc[g][d] = 0.f;
    }

    // A lane's DPL elements of a row are float4s 64 elements apart (float4 number j: elements 64 j + 4 sub ..), so that the
    // 16 lanes of a row read 256 consecutive bytes per load instruction and a row's cache lines are each touched once
    // (with DPL consecutive elements per lane every instruction touched every line of the row).
    const float* kb = p.k + ((int64_t)b * p.kv_heads + kvh) * p.kv_capacity * D + sub * 4;
    const float* vb = p.v + ((int64_t)b * p.kv_heads + kvh) * p.kv_capacity * D + sub * 4;
    // The K / V rows of a pass (U groups of 4 keys per wave) are requested one pass ahead of their use, into the other of
    // two register sets: a split of 64 keys is two passes per wave, and both are in flight from the start.
    constexpr int STEP = 16 * U;
    auto request = [&](float (&kr)[U][DPL], float (&vr)[U][DPL], int k0) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int64_t off = (int64_t)min(k0 + 16 * u + kg, hi - 1) * D;   // a lane past the range re-reads the last row
#pragma unroll
            for (int d = 0; d < DPL; d += 4) {
                const float4 a = *reinterpret_cast<const float4*>(kb + off + 16 * d);
                const float4 c = *reinterpret_cast<const float4*>(vb + off + 16 * d);
                kr[u][d] = a.x; kr[u][d + 1] = a.y; kr[u][d + 2] = a.z; kr[u][d + 3] = a.w;
                vr[u][d] = c.x; vr[u][d + 1] = c.y; vr[u][d + 2] = c.z; vr[u][d + 3] = c.w;
            }
        }
    };
    auto consume = [&](const float (&kr)[U][DPL], const float (&vr)[U][DPL], int k0) {
        bool valid[U];
#pragma unroll
        for (int u = 0; u < U; ++u) valid[u] = k0 + 16 * u + kg < hi;
        // Branch-free from here to the end of the body: the U x GS score chains (dot product, row reduction, exponentials)
        // are independent and the compiler interleaves them; behind a per-key branch each ran on its own, one
        // dependent instruction at a time -- with one wave per SIMD that chain, not the memory, set the pace.
        float sc[U][GS];
#pragma unroll
        for (int u = 0; u < U; ++u) {
#pragma unroll
            for (int g = 0; g < GS; ++g) {
                float s = 0.f;
#pragma unroll
                for (int d = 0; d < DPL; ++d) s = fmaf(qr[g][d], kr[u][d], s);
                s = row16_sum(s);
                if (uniform) s = SDPA_DECODE_MASKED;
                sc[u][g] = valid[u] ? s : -INFINITY;
            }
        }
#pragma unroll
        for (int g = 0; g < GS; ++g) {
            // both key groups enter the running state in one update: one rescale of the accumulator per pass
            float m_new = m[g];
#pragma unroll
            for (int u = 0; u < U; ++u) m_new = fmaxf(m_new, sc[u][g]);
            const float alpha = exp_diff(m[g], m_new);
            float pr[U], psum = 0.f;
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const float e = exp2_raw(sc[u][g] - m_new);        // NaN for (-inf) - (-inf): discarded by the select
                pr[u] = valid[u] ? e : 0.f;
                psum += pr[u];
            }
            l[g] = fmaf(l[g], alpha, psum);
#pragma unroll
            for (int d = 0; d < DPL; ++d) {
                float a = acc[g][d] * alpha;
#pragma unroll
                for (int u = 0; u < U; ++u) a = fmaf(pr[u], vr[u][d], a);
                acc[g][d] = a;
            }
            m[g] = m_new;
        }
    };
    // Passes are taken in pairs so that the loop has one exit and one back edge (with an exit between the two halves
    // the compiler's wait-count pass sees a path on which the second set is still in flight at the loop head and makes
    // every request wait for it). The second half of the last pair may lie past the range: none of its keys is valid
    // and it leaves the running state as it is.
    float ka[U][DPL], va[U][DPL], kb2[U][DPL], vb2[U][DPL];
    const int k_first = lo + wave * 4;
    if (k_first < hi) request(ka, va, k_first);                 // wave-uniform
    for (int k0 = k_first; k0 < hi; k0 += 2 * STEP) {
        request(kb2, vb2, k0 + STEP);                           // past the range: clamped re-reads of the last row
        __builtin_amdgcn_sched_barrier(0);                      // requests are issued where they are written, ahead of the arithmetic
        consume(ka, va, k0);
        request(ka, va, k0 + 2 * STEP);
        __builtin_amdgcn_sched_barrier(0);
        consume(kb2, vb2, k0 + STEP);
    }

    // Merge the 16 running states of the workgroup (4 lane groups x 4 waves) through LDS: every lane parks its slice,
    // one 16-lane row per head works out the 16 weights 2^(m_s - max) and the weighted sum of the l_s, then each thread
    // sums its output elements over the states. (Merging lane groups by shuffles first cost 80 crossbar round trips and
    // 16 exponentials per lane.) A lane's float4 number j holds elements 64 j + 4 sub .. of the row, so the 16 lanes of
    // a row store 256 contiguous bytes and a state lies in LDS in the row's own element order.
    const int state = wave * 4 + kg;
#pragma unroll
    for (int g = 0; g < GS; ++g) {
#pragma unroll
        for (int j = 0; j < DPL / 4; ++j)
            *reinterpret_cast<float4*>(&wacc[state][g][j * 64 + sub * 4]) =
                make_float4(acc[g][4 * j], acc[g][4 * j + 1], acc[g][4 * j + 2], acc[g][4 * j + 3]);
        if (sub == 0) { wm[g][state] = m[g]; wl[g][state] = l[g]; }
    }
    __syncthreads();
    if (threadIdx.x < 16 * GS) {
        const int g = threadIdx.x >> 4, st = threadIdx.x & 15;
        const float ms = wm[g][st];
        const float mm = row16_max(ms);
        const float c = exp_diff(ms, mm);
        const float ls = row16_sum(c * wl[g][st]);
        cw[g][st] = c;
        if (st == 0) { wmm[g] = mm; wls[g] = ls; }
    }
    __syncthreads();

    constexpr int EPT = GS * D >= 256 ? GS * D / 256 : 1;       // output elements per thread, adjacent inside one head
    if (threadIdx.x * EPT < GS * D) {
        const int g = threadIdx.x * EPT / D, i0 = threadIdx.x * EPT % D;
        float c[16], o[EPT];
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
            const float4 t = *reinterpret_cast<const float4*>(&cw[g][4 * q4]);
            c[4 * q4] = t.x; c[4 * q4 + 1] = t.y; c[4 * q4 + 2] = t.z; c[4 * q4 + 3] = t.w;
        }
#pragma unroll
        for (int e = 0; e < EPT; ++e) o[e] = 0.f;
#pragma unroll
        for (int st = 0; st < 16; ++st)
#pragma unroll
            for (int e = 0; e < EPT; ++e) o[e] = fmaf(wacc[st][g][i0 + e], c[st], o[e]);
        const float mm = wmm[g], ls = wls[g];
        const int64_t row = (int64_t)b * p.heads + h0 + g;
#pragma unroll
        for (int e = 0; e < EPT; ++e) {
            const int d = i0 + e;                                   // a state's layout in LDS is the row's own element order
            if (!p.part) {
                p.out[row * D + d] = ls > 0.f ? o[e] / ls : 0.f;
            } else {
                p.part[(row * p.splits + split) * D + d] = o[e];
                if (d == 0) *reinterpret_cast<float2*>(p.ml + (row * p.splits + split) * 2) = make_float2(mm, ls);
            }
        }
    }
}

// Merge the per-split (unnormalised output, max, sum) triples of one query row. 4 * D threads: thread (j, d) folds
// splits j, j + 4, ... of output element d (independent loads, all in flight together), LDS folds the four. The
// softmax weights of the splits -- exp(max_s - max) / sum -- are worked out once, by the first wave: one split per
// lane, maximum and sum by wave reductions (splits <= 64), parked in LDS for everyone.
template <int D>
__global__ __launch_bounds__(4 * D) void sdpa_decode_combine_kernel(const float* __restrict__ part, const float* __restrict__ ml,
                                                                    float* __restrict__ out, int splits) {
    __shared__ float sw[SDPA_DECODE_MAX_SPLITS];
    __shared__ float so[4][D];
    const float* src = part + (int64_t)blockIdx.x * splits * D;
    const float2* src_ml = reinterpret_cast<const float2*>(ml) + (int64_t)blockIdx.x * splits;
    const int d = threadIdx.x % D, j = threadIdx.x / D;
    float pv[SDPA_DECODE_MAX_SPLITS / 4];
#pragma unroll
    for (int i = 0; i < SDPA_DECODE_MAX_SPLITS / 4; ++i) {
        const int sp = j + 4 * i;
        pv[i] = src[min(sp, splits - 1) * D + d];               // clamped: a split past the end gets weight zero below
    }
    if (threadIdx.x < 64) {
        const int sp = threadIdx.x;
        const bool live = sp < splits;
        const float2 st = live ? src_ml[sp] : make_float2(-INFINITY, 0.f);
        const float m = st.x, l = st.y;
        float mm = m;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) mm = fmaxf(mm, __shfl_xor(mm, off, 64));
        const float w = exp_diff(m, mm);
        const float ls = wave_sum(l * w);
        if (sp < SDPA_DECODE_MAX_SPLITS) sw[sp] = ls > 0.f ? w / ls : 0.f;
    }
    __syncthreads();
    float o = 0.f;
#pragma unroll
    for (int i = 0; i < SDPA_DECODE_MAX_SPLITS / 4; ++i) {
        const int sp = j + 4 * i;
        o = fmaf(pv[i], sp < splits ? sw[sp] : 0.f, o);
    }
    so[j][d] = o;
    __syncthreads();
    if (j == 0) out[(int64_t)blockIdx.x * D + d] = so[0][d] + so[1][d] + so[2][d] + so[3][d];
}

float* sdpa_workspace(size_t bytes);   // shim.hip: per-thread scratch, grown on demand

static std::atomic<int> g_sdpa_decode_split_keys{64};   // least keys per split (a multiple of 16)
void set_sdpa_decode_split_keys(int v) { if (v >= 16) g_sdpa_decode_split_keys = (v + 15) & ~15; }

template <int GS, int DPL>
static int launch_decode_variant(const SdpaDecodeParams& p, int subs, bool merge) {
    constexpr int D = 16 * DPL;
    note_kernel("sdpa_decode_kernel");
    sdpa_decode_kernel<GS, DPL><<<dim3(p.splits, p.kv_heads * subs, p.batch), dim3(256), 0, current_stream()>>>(p);
    SKH_CHECK(hipGetLastError());
    if (merge) {
        sdpa_decode_combine_kernel<D><<<dim3(p.batch * p.heads), dim3(4 * D), 0, current_stream()>>>(p.part, p.ml, p.out, p.splits);
        SKH_CHECK(hipGetLastError());
    }
    return 1;
}

static std::atomic<int> g_sdpa_decode_gs{0};            // query heads per workgroup: 0 = chosen from the shape, else 1 / 2 / 4
void set_sdpa_decode_gs(int v) { if (v == 0 || v == 1 || v == 2 || v == 4) g_sdpa_decode_gs = v; }
static std::atomic<int> g_attn_merge_max_keys{176};    // most keys per split the unmerged form accepts (a multiple of 16)
void set_attn_merge_max_keys(int v) { if (v >= 16) g_attn_merge_max_keys = (v + 15) & ~15; }
// most splits the unmerged form uses. Measured in a Llama-3-8B decode step at 520 to 650 keys (ms per token): 2 splits 1.637,
// 4: 1.565, 6: 1.540, 8: 1.556; the merge in a launch of its own 1.551 -- every split costs each of the projection's 251
// workgroups another 16 KB of loads, every split less costs the attention workgroups another pass over their keys.
static std::atomic<int> g_attn_merge_splits{6};
void set_attn_merge_splits(int v) { if (v >= 1 && v <= ATTN_MERGE_MAX_SPLITS) g_attn_merge_splits = v; }

// Returns 1 when this kernel took the call, 0 when the shape is outside its range (the caller uses the general
// kernel), -1 on error. With `leave` the per-split results are left unmerged for a consumer that folds the merge into
// its own activation load (at most ATTN_MERGE_MAX_SPLITS splits, one sequence): `out` is not written, *leave describes
// where the partials are; 0 when the key count would need more splits than that.
int launch_sdpa_decode(const float* q, const float* k, const float* v, float* out, int batch, int heads, int kv_heads,
                       int seq_kv, int kv_capacity, int head_dim, float scale, int window, int right_context,
                       const int32_t* lengths, AttnMergePrologue* leave) {
    if (head_dim != 64 && head_dim != 128 && head_dim != 256) return 0;
    if ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(v)) & 15) return 0;
    const int per_kv = heads / kv_heads;
    const int gs_max = head_dim == 256 ? 2 : 4;
    int gs = g_sdpa_decode_gs.load() > 0 ? min(g_sdpa_decode_gs.load(), gs_max) : gs_max;
    while (per_kv % gs != 0) gs >>= 1;
    // Few workgroups (one sequence at a short context, or splits capped for the projection that merges them): two query
    // heads per workgroup instead of four. The K / V rows are then fetched by two workgroups (the second from L2), each
    // with half the arithmetic per pass, and twice as many CUs take part: 1.502 against 1.526 ms per token in a
    // Llama-3-8B decode step at 520 to 650 keys (one head per workgroup: 1.529).
    if (g_sdpa_decode_gs.load() == 0 && gs == 4) {
        const int64_t groups4 = (int64_t)batch * kv_heads * (per_kv / 4);
        const int most = leave ? g_attn_merge_splits.load() : SDPA_DECODE_MAX_SPLITS;
        const int splits4 = min(most, (seq_kv + g_sdpa_decode_split_keys - 1) / g_sdpa_decode_split_keys);
        if (groups4 * splits4 < num_cus()) gs = 2;
    }
    const int subs = per_kv / gs;
    if (batch > 65535) return 0;
    SdpaDecodeParams p{q, k, v, out, batch, heads, kv_heads, seq_kv, kv_capacity, scale, window, right_context, lengths, 1,
                       nullptr, nullptr};
    // enough workgroups to put every CU on the cache, at least 64 keys per split (measured in the decoder at 500 to 650
    // keys: 32 or 48 keys per split 2.5 % slower per token, 96 and 128 keys the same as 64)
    const int64_t groups = (int64_t)batch * kv_heads * subs;
    int splits = (int)((2 * (int64_t)num_cus() + groups - 1) / groups);
    splits = min(splits, min(SDPA_DECODE_MAX_SPLITS, (seq_kv + g_sdpa_decode_split_keys - 1) / g_sdpa_decode_split_keys));
    if (splits < 1) splits = 1;
    if (leave) {
        if (batch != 1) return 0;
        const int most = g_attn_merge_splits;
        if (splits > most) {
            if ((seq_kv + most - 1) / most > g_attn_merge_max_keys) return 0;
            splits = most;
        }
    }
    p.splits = splits;
    if (splits > 1 || leave) {
        const size_t rows = (size_t)batch * heads;
        p.part = sdpa_workspace(sizeof(float) * rows * splits * (head_dim + 2));
        if (!p.part) return -1;
        p.ml = p.part + rows * splits * head_dim;
    }
    if (leave) *leave = AttnMergePrologue{p.part, p.ml, splits, head_dim};
    const bool merge = splits > 1 && !leave;
    if (head_dim == 64) {
        if (gs == 4) return launch_decode_variant<4, 4>(p, subs, merge);
        if (gs == 2) return launch_decode_variant<2, 4>(p, subs, merge);
        return launch_decode_variant<1, 4>(p, subs, merge);
    }
    if (head_dim == 128) {
        if (gs == 4) return launch_decode_variant<4, 8>(p, subs, merge);
        if (gs == 2) return launch_decode_variant<2, 8>(p, subs, merge);
        return launch_decode_variant<1, 8>(p, subs, merge);
    }
    if (gs == 2) return launch_decode_variant<2, 16>(p, subs, merge);
    return launch_decode_variant<1, 16>(p, subs, merge);
}

int launch_q4k_gemv_mfma(const uint8_t* w, const float* x, float* y, int k, int n, const float* gain, float eps,
                         const float* residual, int epilogue, const RopeQkvEpilogue* rope_in,
                         const AttnMergePrologue* merge);   // gemv_q4k_mfma.hip
bool q4k_gemv_mfma_accepts_merge(int k, int n, int head_dim);   // gemv_q4k_mfma.hip

static std::atomic<int> g_attn_merge_enable{1};
void set_attn_merge_enable(int v) { g_attn_merge_enable = v; }

// One decode token's attention over the cache and the Q4_K output projection behind it as two launches: the attention
// kernel leaves its per-split results unmerged and the projection's activation load merges them (the merge launch and its
// round trip through memory disappear). out[n] = (residual ? residual : 0) + Wo[n, heads * head_dim] . attention.
// Returns 1 when the pair took the call, 0 when the shapes are outside its range (nothing launched), -1 on error.
int launch_attn_out_proj_q4k(const uint8_t* wo, int n, int k, const float* q, const float* k_cache, const float* v_cache, int heads,
                             int kv_heads, int head_dim, int seq_kv, int kv_capacity, float scale, int window,
                             const int32_t* lengths, const float* residual, float* out) {
    if (!g_attn_merge_enable || k != heads * head_dim || k > 4096 || (k & 1023)) return 0;
    if (heads % kv_heads != 0 || seq_kv < 1 || kv_capacity < seq_kv) return 0;
    // dry checks of the projection first: once the attention kernel has run without a merge there is no way back
    if ((reinterpret_cast<uintptr_t>(wo) & 15) || !q4k_gemv_mfma_accepts_merge(k, n, head_dim)) return 0;
    if (residual && (reinterpret_cast<uintptr_t>(residual) & 3)) return 0;
    AttnMergePrologue am{};
    const int r = launch_sdpa_decode(q, k_cache, v_cache, nullptr, 1, heads, kv_heads, seq_kv, kv_capacity, head_dim, scale, window, 0,
                                     lengths, &am);
    if (r <= 0) return r;
    const int g = launch_q4k_gemv_mfma(wo, nullptr, out, k, n, nullptr, 0.f, residual, residual ? EPI_RESIDUAL : EPI_NONE, nullptr, &am);
    if (g == 0) return set_error("attn_out_proj: the projection refused a shape its checks had passed (n %d, k %d)", n, k);
    return g;
}

}  // namespace skh
