// Prefill-shape attention on the matrix cores: out = softmax(q k^T * scale + causal rule) v, fp32 in and out,
// bf16 operands on v_mfma_f32_32x32x16_bf16, fp32 accumulation and fp32 online softmax.
//
// Contract: the reference's skainet_f32_sdpa
//   /root/reference/skainet-backends/skainet-backend-native-cpu/native/src/f32_fused.c:290-396
// restricted to what a prompt pass uses: seq_q <= seq_kv, head_dim 64 or 128; causal or full, with or without a
// sliding window (window, rightContext) and per-sequence key lengths, by the rules of
//   /root/reference/skainet-lang/skainet-lang-core/src/commonMain/kotlin/sk/ainet/lang/tensor/ops/AttentionMask.kt:24-104
// and with or without an additive mask broadcast over [B|1, H|Hkv|1, Sq|1, Skv|1] (f32_fused.c:312-331).
// Every other call stays on the general fp32 kernel (sdpa.hip). Without a mask, a query whose rules leave it at least
// one key gives the same result whether excluded keys score -1e30 (the reference) or take no part (here), and a query
// they leave none weighs every key of the sequence equally, as the reference's row of equal scores does. With a mask
// the reference's arithmetic is kept as it stands: every key of the sequence takes part, an excluded one at -1e30
// plus its mask value (the mask is added to every score), so no key block is skipped.
//
// Two launches:
//   1. kv_to_bf16_kernel: K -> bf16 [kv head][key][D], V -> bf16 transposed [kv head][D][key], keys padded with
//      zeros to a multiple of 64. (The PV product contracts over keys, and an MFMA operand wants 8 consecutive
//      contraction values per lane: V has to be read along keys, hence the transpose, done once per call.)
//   2. sdpa_prefill_kernel: one workgroup = two teams of 4 waves; a team = up to 4 query heads that share a KV head x
//      32 query positions (fewer heads per KV head: more query blocks per team). The teams of workgroup i take query
//      group G - 1 - i and query group i of the same KV head (groups 2 i + 1 and 2 i under a sliding window or without
//      the causal rule, where neighbours share their key blocks): under the causal rule a late group (many keys) and an
//      early one (few), so every workgroup carries the same work and one workgroup per CU keeps its SIMDs busy from
//      start to end (with one group per workgroup, which two groups shared a CU was the dispatcher's choice: two late
//      groups on one CU set the kernel's time). Keys in blocks of 64: the K and V^T tiles of a block go
//      global -> registers -> LDS (double-buffered, one barrier per block) and are shared by the 8 waves; a block no
//      wave of either team needs is never loaded. Per wave and block:
//        S^T[key][query] = K_tile . Q^T           16 MFMAs (Q lives in registers, pre-multiplied by scale * log2 e)
//        online softmax per query: a query is one accumulator COLUMN, so its 32 scores per 32-key tile sit in
//          one lane pair (l, l ^ 32): the row statistics need a single cross-lane step
//        O^T[d][query] += V^T_tile . P            16 MFMAs; P is the S^T accumulator converted in place: the MFMA
//          contraction index is a free permutation, so the keys a lane holds (4h + {0..3}, 8 + 4h + {0..3} of each
//          16) are simply declared to be its 8 k-slots and V^T is read in the same order.
//      Blocks wholly above the diagonal are skipped, only blocks that cross it (or the end of the keys) mask.
#include "common.h"

namespace skh {

typedef __bf16 pf_bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 pf_bf16x4 __attribute__((ext_vector_type(4)));
typedef float pf_f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t pf_u32x4 __attribute__((ext_vector_type(4)));   // a native 16-byte vector: staging registers stay registers

constexpr int PF_KB = 64;          // keys per block
constexpr int PF_QW = 32;          // query positions per wave

// K [b][kvh][kv_capacity][D] fp32 -> kb [b*kvh][spad][D] bf16;  V -> vt [b*kvh][D][spad] bf16. One workgroup per
// (64-key block, kv head, batch); keys >= seq_kv are written as zeros.
template <int D>
__global__ __launch_bounds__(256) void kv_to_bf16_kernel(const float* __restrict__ k, const float* __restrict__ v,
                                                         __bf16* __restrict__ kb, __bf16* __restrict__ vt, int kv_heads,
                                                         int seq_kv, int kv_capacity, int spad) {
    __shared__ float tile[PF_KB][D + 1];
    const int k0 = blockIdx.x * PF_KB;
    const int64_t head = (int64_t)blockIdx.z * kv_heads + blockIdx.y;
    const float* ksrc = k + head * kv_capacity * D;
    const float* vsrc = v + head * kv_capacity * D;
    // K: straight conversion, 4 floats per thread-step; every load of the workgroup's 64 KB is requested before the
    // first value is used (keys past the sequence: a clamped address, zeroed afterwards)
    constexpr int STEPS = PF_KB * D / 4 / 256;
    float4 xs[STEPS], ys[STEPS];
#pragma unroll
    for (int i = 0; i < STEPS; ++i) {
        const int t = threadIdx.x + 256 * i, key = t / (D / 4), d4 = t % (D / 4);
        const int64_t off = (int64_t)min(k0 + key, seq_kv - 1) * D + 4 * d4;
        xs[i] = *reinterpret_cast<const float4*>(ksrc + off);
        ys[i] = *reinterpret_cast<const float4*>(vsrc + off);
    }
#pragma unroll
    for (int i = 0; i < STEPS; ++i) {
        const int t = threadIdx.x + 256 * i, key = t / (D / 4), d4 = t % (D / 4);
        const float keep = k0 + key < seq_kv ? 1.0f : 0.0f;
        const float4 x = xs[i], y = ys[i];
        pf_bf16x4 o;
        o[0] = (__bf16)(x.x * keep); o[1] = (__bf16)(x.y * keep); o[2] = (__bf16)(x.z * keep); o[3] = (__bf16)(x.w * keep);
        *reinterpret_cast<pf_bf16x4*>(kb + (head * spad + k0 + key) * D + 4 * d4) = o;
        tile[key][4 * d4] = y.x * keep; tile[key][4 * d4 + 1] = y.y * keep; tile[key][4 * d4 + 2] = y.z * keep; tile[key][4 * d4 + 3] = y.w * keep;
    }
    __syncthreads();
    // V^T: thread-step = (d, 8 consecutive keys)
    for (int t = threadIdx.x; t < D * PF_KB / 8; t += 256) {
        const int d = t / (PF_KB / 8), kc = t % (PF_KB / 8);
        pf_bf16x8 o;
#pragma unroll
        for (int j = 0; j < 8; ++j) o[j] = (__bf16)tile[8 * kc + j][d];
        *reinterpret_cast<pf_bf16x8*>(vt + (head * D + d) * spad + k0 + 8 * kc) = o;
    }
}

struct PrefillParams {
    const float* q;
    const __bf16 *kb, *vt;
    float* out;
    int heads, kv_heads, seq_q, seq_kv, spad;
    float scale_log2e;
    int causal, window, right_context;
    const int32_t* lengths;    // per-sequence key counts on the device, or null
    int heads_per_wg;      // 1, 2 or 4 query heads of one KV head per workgroup
    const float* mask;         // additive mask or null; dims 1 or the full extent (heads: 1, kv_heads or heads)
    int mask_b, mask_h, mask_q, mask_k;
    int out_rows;              // 0: out is [batch, heads, seq_q, D]; 1: [batch, seq_q, heads, D], token rows of a projection's input
};

// One 64-key block of the bf16 K and V^T copies: global -> registers, and registers -> the LDS tiles.
// PF_THREADS threads of a workgroup (one or two teams of four waves) stage a block together
template <int D, int PF_THREADS>
__device__ __forceinline__ void pf_load_block(pf_u32x4 (&kreg)[PF_KB * (D / 8) / PF_THREADS], pf_u32x4 (&vreg)[D * (PF_KB / 8) / PF_THREADS],
                                              const __bf16* kbase, const __bf16* vbase, int spad, int k0, int tid) {
    constexpr int KCH = D / 8;
#pragma unroll
    for (int j = 0; j < PF_KB * KCH / PF_THREADS; ++j) {
        const int c = tid + PF_THREADS * j, key = c / KCH, ch = c % KCH;
        kreg[j] = *reinterpret_cast<const pf_u32x4*>(kbase + (int64_t)(k0 + key) * D + 8 * ch);
    }
#pragma unroll
    for (int j = 0; j < D * (PF_KB / 8) / PF_THREADS; ++j) {
        const int c = tid + PF_THREADS * j, d = c / (PF_KB / 8), ch = c % (PF_KB / 8);
        vreg[j] = *reinterpret_cast<const pf_u32x4*>(vbase + (int64_t)d * spad + k0 + 8 * ch);
    }
}
template <int D, int PF_THREADS>
__device__ __forceinline__ void pf_store_block(const pf_u32x4 (&kreg)[PF_KB * (D / 8) / PF_THREADS], const pf_u32x4 (&vreg)[D * (PF_KB / 8) / PF_THREADS],
                                               __bf16* kt, __bf16* vt, int tid) {
    constexpr int KCH = D / 8, KP = D + 8, VP = PF_KB + 8;
#pragma unroll
    for (int j = 0; j < PF_KB * KCH / PF_THREADS; ++j) {
        const int c = tid + PF_THREADS * j, key = c / KCH, ch = c % KCH;
        *reinterpret_cast<pf_u32x4*>(kt + key * KP + 8 * ch) = kreg[j];
    }
#pragma unroll
    for (int j = 0; j < D * (PF_KB / 8) / PF_THREADS; ++j) {
        const int c = tid + PF_THREADS * j, d = c / (PF_KB / 8), ch = c % (PF_KB / 8);
        *reinterpret_cast<pf_u32x4*>(vt + d * VP + 8 * ch) = vreg[j];
    }
}

// TEAMS 2: the paired form described above. TEAMS 1: one query group per workgroup of four waves (two workgroups per
// CU), for calls whose paired grid would leave CUs without a workgroup.
template <int D, int TEAMS>
__global__ __launch_bounds__(256 * TEAMS, TEAMS == 1 ? 2 : 1) void sdpa_prefill_kernel(PrefillParams p) {
    constexpr int PF_THREADS = 256 * TEAMS;
    constexpr int KP = D + 8;          // K tile row pitch (bf16): 16-byte aligned rows, 16 lanes of a b128 read on distinct banks
    constexpr int VP = PF_KB + 8;      // V^T tile row pitch (bf16)
    constexpr int NT = D / 16;         // MFMA steps along head_dim for S
    constexpr int ND = D / 32;         // 32-row tiles of O^T
    constexpr int KCH = D / 8;         // 16-byte chunks per K row
    constexpr int K_LOADS = PF_KB * KCH / PF_THREADS;       // 16-byte loads per thread for the K tile
    constexpr int V_LOADS = D * (PF_KB / 8) / PF_THREADS;   // and for the V^T tile
    extern __shared__ __attribute__((aligned(16))) uint8_t pf_smem[];       // 2 K tiles, then 2 V^T tiles
    __bf16* const ktile0 = reinterpret_cast<__bf16*>(pf_smem);
    __bf16* const vtile0 = ktile0 + 2 * PF_KB * KP;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave_all = __builtin_amdgcn_readfirstlane(tid >> 6), team = TEAMS == 2 ? wave_all >> 2 : 0, wave = wave_all & 3;
    const int col = lane & 31, h = lane >> 5;
    const int per_kv = p.heads / p.kv_heads;
    const int hpw = p.heads_per_wg;
    const int qblocks_per_wg = 4 / hpw;
    const int head_groups = per_kv / hpw;
    const int kvh = blockIdx.y / head_groups;
    const int head = kvh * per_kv + (blockIdx.y % head_groups) * hpw + wave % hpw;
    const int b = blockIdx.z;
    // query groups (a team's share of the query positions). Causal over the whole prefix: team 0 takes group G - 1 - i,
    // team 1 group i (equal work in every workgroup). Under a sliding window, or without the causal rule, every group
    // has about the same work and neighbours share most of their key blocks: groups 2 i + 1 and 2 i. With an odd number
    // of groups one group is team 0's alone.
    const int q_per_group = qblocks_per_wg * PF_QW;
    const int ngroups = (p.seq_q + q_per_group - 1) / q_per_group;
    const bool adjacent = p.window > 0 || !p.causal;
    int g_early, g_late;
    if (TEAMS == 2) {
        g_early = adjacent ? 2 * (int)blockIdx.x : (int)blockIdx.x;
        g_late = adjacent ? min(g_early + 1, ngroups - 1) : ngroups - 1 - (int)blockIdx.x;
    } else {
        g_late = g_early = p.causal ? ngroups - 1 - (int)blockIdx.x : (int)blockIdx.x;   // the groups with the most keys start first
    }
    const int my_group = team ? g_early : g_late;
    const bool team_active = TEAMS == 1 || !(team == 1 && g_early == g_late);
    const int q0 = my_group * q_per_group + (wave / hpw) * PF_QW;          // first query position of this wave
    auto group_first = [&](int g) { return g * q_per_group; };
    auto group_last = [&](int g) { return min(p.seq_q, (g + 1) * q_per_group) - 1; };
    const int shift = p.seq_kv - p.seq_q;                                   // absolute position of query 0
    const int len = p.lengths ? p.lengths[b] : p.seq_kv;
    // attended keys [first, end) of a query position: both bounds grow with the position
    auto first_of = [&](int qi) { return p.window > 0 ? max(0, qi + shift - p.window + 1) : 0; };
    auto end_of = [&](int qi) {
        int e = p.seq_kv;
        if (p.window > 0) e = min(e, qi + shift + p.right_context + 1);
        if (p.causal) e = min(e, qi + shift + 1);
        return max(min(e, len), 0);
    };
    const int my_q = q0 + col;
    const int my_qc = min(my_q, p.seq_q - 1);
    const bool masked = p.mask != nullptr;                                  // uniform
    const int real_first = first_of(my_qc), real_last = end_of(my_qc) - 1;  // the rules' own range (may be empty)
    // no key left: every key of the sequence, equally (with a mask the -1e30 scores do that by themselves)
    const bool my_uniform = !masked && first_of(my_qc) >= end_of(my_qc);
    const int my_first_key = my_uniform ? 0 : first_of(my_qc);
    const int my_last_key = my_uniform ? p.seq_kv - 1 : end_of(my_qc) - 1;
    const bool wave_uniform = __ballot(my_uniform) != 0;
    const bool wg_uniform = __syncthreads_or(my_uniform) != 0;
    // keys any wave of this workgroup needs: the two teams' ranges (both bounds grow with the query position), whole
    // blocks; between the early team's last block and the late team's first (a sliding window) lie blocks nobody needs
    const bool all_keys = wg_uniform || masked;
    const int e_beg = first_of(group_first(g_early)) / PF_KB, e_end = (end_of(group_last(g_early)) + PF_KB - 1) / PF_KB;
    const int l_beg = first_of(group_first(g_late)) / PF_KB, l_end = (end_of(group_last(g_late)) + PF_KB - 1) / PF_KB;
    const int blk_begin = all_keys ? 0 : min(e_beg, l_beg);
    const int nblocks = all_keys ? (p.seq_kv + PF_KB - 1) / PF_KB : max(max(e_end, l_end), blk_begin);
    auto needed = [&](int blk) { return all_keys || (blk >= e_beg && blk < e_end) || (blk >= l_beg && blk < l_end); };
    auto next_needed = [&](int blk) { int nb = blk + 1; while (nb < nblocks && !needed(nb)) ++nb; return nb; };
    // this wave's 32 positions: the keys any of them attends, and the keys all of them attend
    const int q_wave_last = min(q0 + PF_QW - 1, p.seq_q - 1), q_wave_first = min(q0, p.seq_q - 1);
    const int wave_first_key = (wave_uniform || masked) ? 0 : first_of(q_wave_first);
    const int wave_last_key = !team_active ? -1 : (wave_uniform || masked) ? p.seq_kv - 1 : end_of(q_wave_last) - 1;
    const int wave_common_first = first_of(q_wave_last), wave_common_last = end_of(q_wave_first) - 1;

    // Q fragment: lane (query col, half h) holds q[16 t + 8 h .. + 7] for every t, times scale * log2(e)
    pf_bf16x8 qf[NT];
    {
        const int qrow = min(my_q, p.seq_q - 1);
        const float* qp = p.q + (((int64_t)b * p.heads + head) * p.seq_q + qrow) * D + 8 * h;
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const float4 a = *reinterpret_cast<const float4*>(qp + 16 * t);
            const float4 c = *reinterpret_cast<const float4*>(qp + 16 * t + 4);
            const float f = p.scale_log2e;
            qf[t] = pf_bf16x8{(__bf16)(a.x * f), (__bf16)(a.y * f), (__bf16)(a.z * f), (__bf16)(a.w * f),
                              (__bf16)(c.x * f), (__bf16)(c.y * f), (__bf16)(c.z * f), (__bf16)(c.w * f)};
        }
    }

    // this lane's row of the mask (one query position; the key index is added per score), in units of ln 2 later
    const float* mrow = nullptr;
    if (masked) {
        const int bi = p.mask_b == 1 ? 0 : b;
        const int hi = p.mask_h == 1 ? 0 : (p.mask_h == p.heads ? head : kvh);
        mrow = p.mask + (((int64_t)bi * p.mask_h + hi) * p.mask_q + (p.mask_q == 1 ? 0 : my_qc)) * p.mask_k;
    }
    const int64_t kvhead = (int64_t)b * p.kv_heads + kvh;
    const __bf16* kbase = p.kb + kvhead * p.spad * D;
    const __bf16* vbase = p.vt + kvhead * D * p.spad;
    pf_u32x4 kreg[K_LOADS], vreg[V_LOADS];
    pf_f32x16 oacc[ND];
#pragma unroll
    for (int i = 0; i < ND; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e) oacc[i][e] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;     // per query (column); l_run is this lane's half of the keys

    int blk = blk_begin;
    while (blk < nblocks && !needed(blk)) ++blk;
    if (blk < nblocks) {
        pf_load_block<D, PF_THREADS>(kreg, vreg, kbase, vbase, p.spad, blk * PF_KB, tid);
        pf_store_block<D, PF_THREADS>(kreg, vreg, ktile0, vtile0, tid);
    }
    __syncthreads();

    for (int buf = 0; blk < nblocks; buf ^= 1) {
        const int k0 = blk * PF_KB;
        const int nblk = next_needed(blk);
        if (nblk < nblocks) pf_load_block<D, PF_THREADS>(kreg, vreg, kbase, vbase, p.spad, nblk * PF_KB, tid);
        if (k0 <= wave_last_key && k0 + PF_KB > wave_first_key) {     // wave-uniform: this wave has keys in the block
            // S^T tiles: s[j] covers keys k0 + 32 j .. + 31 (rows) x this wave's 32 queries (columns)
            pf_f32x16 s[2];
#pragma unroll
            for (int j = 0; j < 2; ++j) {
#pragma unroll
                for (int e = 0; e < 16; ++e) s[j][e] = 0.f;
                const __bf16* kt = ktile0 + buf * (PF_KB * KP) + (32 * j + col) * KP + 8 * h;
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    const pf_bf16x8 kf = *reinterpret_cast<const pf_bf16x8*>(kt + 16 * t);
                    s[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[t], s[j], 0, 0, 0);
                }
            }
            if (masked) {
                // the reference's arithmetic: an excluded key scores -1e30, the mask is added to every score; keys past
                // the sequence (padding of the last block) take no part. Four adjacent keys per 16-byte mask load.
                constexpr float LOG2E = 1.4426950408889634f;
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int e4 = 0; e4 < 4; ++e4) {
                        const int key4 = k0 + 32 * j + 8 * e4 + 4 * h;
                        float4 mv;
                        if (p.mask_k == 1) { const float m1 = mrow[0]; mv = make_float4(m1, m1, m1, m1); }
                        else mv = *reinterpret_cast<const float4*>(mrow + min(key4, p.seq_kv - 4));     // seq_kv is a multiple of 4 here
                        const float m4[4] = {mv.x, mv.y, mv.z, mv.w};
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const int key = key4 + i;
                            float sc = (key > real_last || key < real_first) ? -1.0e30f * LOG2E : s[j][4 * e4 + i];
                            sc = fmaf(m4[i], LOG2E, sc);
                            s[j][4 * e4 + i] = key < p.seq_kv ? sc : -INFINITY;
                        }
                    }
            } else
            // keys outside this query's range score -inf (they take no part); a query without a range scores every key 0
            if (wave_uniform || k0 < wave_common_first || k0 + PF_KB - 1 > wave_common_last) {   // wave-uniform: the block crosses a boundary
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        const int key = k0 + 32 * j + 8 * (e >> 2) + 4 * h + (e & 3);
                        if (my_uniform) s[j][e] = 0.f;
                        if (key > my_last_key || key < my_first_key) s[j][e] = -INFINITY;
                    }
            }
            float mx = s[0][0];
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) mx = fmaxf(mx, s[j][e]);
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            // The reference point of the exponentials follows the running maximum lazily: it moves only when a block's
            // maximum exceeds it by more than 8 (in units of ln 2; weights then stay below 2^8, far inside bf16 and fp32
            // range, and the final division by the sum takes the common factor out). So the 64 output accumulators are
            // rescaled in the few blocks where some query of the wave moves its reference -- for most waves the first
            // block only -- instead of in every block.
            const bool move = mx > m_run + 8.0f;                                      // also the first block (m_run = -inf) with any finite score
            const float m_new = move ? mx : m_run;
            // a query of a padded row past seq_q, or a block wholly past a query's keys, can leave m_new at -inf
            const float m_use = m_new == -INFINITY ? 0.f : m_new;
            float psum = 0.f;
            pf_bf16x8 pf[4];                                         // pf[2 j + g]: keys 16 g .. of tile j, this lane's 8 slots
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                float pr[16];
#pragma unroll
                for (int e = 0; e < 16; ++e) { pr[e] = __builtin_amdgcn_exp2f(s[j][e] - m_use); psum += pr[e]; }
                pf[2 * j] = pf_bf16x8{(__bf16)pr[0], (__bf16)pr[1], (__bf16)pr[2], (__bf16)pr[3],
                                      (__bf16)pr[4], (__bf16)pr[5], (__bf16)pr[6], (__bf16)pr[7]};
                pf[2 * j + 1] = pf_bf16x8{(__bf16)pr[8], (__bf16)pr[9], (__bf16)pr[10], (__bf16)pr[11],
                                          (__bf16)pr[12], (__bf16)pr[13], (__bf16)pr[14], (__bf16)pr[15]};
            }
            if (__ballot(move) != 0) {                                               // wave-uniform
                const float alpha = move ? __builtin_amdgcn_exp2f(m_run - m_use) : 1.0f;   // m_run = -inf -> 0
                l_run *= alpha;
#pragma unroll
                for (int i = 0; i < ND; ++i)
#pragma unroll
                    for (int e = 0; e < 16; ++e) oacc[i][e] *= alpha;
            }
            l_run += psum;
            m_run = m_new;
            // O^T += V^T . P : A = V^T rows d, this lane's k-slots are keys 16 g + 4 h + {0..3} and 16 g + 8 + 4 h + {0..3}
#pragma unroll
            for (int g = 0; g < 4; ++g) {
#pragma unroll
                for (int i = 0; i < ND; ++i) {
                    const __bf16* vp = vtile0 + buf * (D * VP) + (32 * i + col) * VP + 16 * g + 4 * h;
                    const pf_bf16x4 lo = *reinterpret_cast<const pf_bf16x4*>(vp);
                    const pf_bf16x4 hi = *reinterpret_cast<const pf_bf16x4*>(vp + 8);
                    const pf_bf16x8 vf = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                    oacc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[g], oacc[i], 0, 0, 0);
                }
            }
        }
        if (nblk < nblocks) pf_store_block<D, PF_THREADS>(kreg, vreg, ktile0 + (buf ^ 1) * (PF_KB * KP), vtile0 + (buf ^ 1) * (D * VP), tid);
        __syncthreads();
        blk = nblk;
    }

    const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
    const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
    if (my_q < p.seq_q && team_active) {
        float* op = p.out + (p.out_rows ? (((int64_t)b * p.seq_q + my_q) * p.heads + head) : (((int64_t)b * p.heads + head) * p.seq_q + my_q)) * D;
#pragma unroll
        for (int i = 0; i < ND; ++i)
#pragma unroll
            for (int e4 = 0; e4 < 4; ++e4) {
                const int d = 32 * i + 8 * e4 + 4 * h;
                *reinterpret_cast<float4*>(op + d) = make_float4(oacc[i][4 * e4] * inv, oacc[i][4 * e4 + 1] * inv,
                                                                 oacc[i][4 * e4 + 2] * inv, oacc[i][4 * e4 + 3] * inv);
            }
    }
}

void* kernel_workspace(size_t bytes);   // shim.hip: per-thread scratch, grown on demand

static std::atomic<int> g_prefill_mfma{1};
void set_sdpa_prefill_mfma(int v) { g_prefill_mfma = v; }
static std::atomic<int> g_prefill_teams{0};   // 0: chosen from the grid, 1: one query group per workgroup, 2: paired groups
void set_sdpa_prefill_teams(int v) { if (v >= 0 && v <= 2) g_prefill_teams = v; }

template <int D>
static int launch_prefill_d(const float* q, const float* k, const float* v, float* out, int batch, int heads, int kv_heads,
                            int seq_q, int seq_kv, int kv_capacity, float scale, int causal, int window, int right_context,
                            const int32_t* lengths, const float* mask, int mask_b, int mask_h, int mask_q, int mask_k, int out_rows) {
    const int spad = (seq_kv + PF_KB - 1) / PF_KB * PF_KB;
    const size_t elems = (size_t)batch * kv_heads * spad * D;
    __bf16* ws = static_cast<__bf16*>(kernel_workspace(2 * elems * sizeof(__bf16)));
    if (!ws) return -1;
    __bf16 *kb = ws, *vt = ws + elems;
    hipStream_t s = current_stream();
    kv_to_bf16_kernel<D><<<dim3(spad / PF_KB, kv_heads, batch), dim3(256), 0, s>>>(k, v, kb, vt, kv_heads, seq_kv, kv_capacity, spad);
    SKH_CHECK(hipGetLastError());
    const int per_kv = heads / kv_heads;
    const int hpw = per_kv % 4 == 0 ? 4 : (per_kv % 2 == 0 ? 2 : 1);
    const int q_per_group = (4 / hpw) * PF_QW;
    const int ngroups = (seq_q + q_per_group - 1) / q_per_group;
    PrefillParams p{q, kb, vt, out, heads, kv_heads, seq_q, seq_kv, spad, scale * 1.4426950408889634f, causal, window, right_context, lengths, hpw,
                    mask, mask_b, mask_h, mask_q, mask_k, out_rows};
    // paired query groups where that still gives every CU a workgroup, else one group per (smaller) workgroup
    const int64_t paired_wgs = (int64_t)((ngroups + 1) / 2) * kv_heads * (per_kv / hpw) * batch;
    const bool paired = g_prefill_teams.load() == 0 ? paired_wgs >= num_cus() : g_prefill_teams.load() == 2;
    const dim3 grid(paired ? (ngroups + 1) / 2 : ngroups, kv_heads * (per_kv / hpw), batch);
    constexpr size_t smem = sizeof(__bf16) * (2 * PF_KB * (D + 8) + 2 * D * (PF_KB + 8));
    note_kernel("sdpa_prefill_kernel");
    if (paired) {
        SKH_SET_MAX_DYNAMIC_LDS_ONCE((&sdpa_prefill_kernel<D, 2>), smem);
        sdpa_prefill_kernel<D, 2><<<grid, dim3(512), smem, s>>>(p);
    } else {
        SKH_SET_MAX_DYNAMIC_LDS_ONCE((&sdpa_prefill_kernel<D, 1>), smem);
        sdpa_prefill_kernel<D, 1><<<grid, dim3(256), smem, s>>>(p);
    }
    SKH_CHECK(hipGetLastError());
    return 1;
}

// Returns 1 when the MFMA path took the call, 0 when the shape is outside its range, -1 on error.
int launch_sdpa_prefill(const float* q, const float* k, const float* v, float* out, int batch, int heads, int kv_heads,
                        int seq_q, int seq_kv, int kv_capacity, int head_dim, float scale, int causal, int window,
                        int right_context, const int32_t* lengths, const float* mask, int mask_b, int mask_h, int mask_q,
                        int mask_k, int out_rows) {
    if (!g_prefill_mfma) return 0;
    // a mask row is read four keys at a time: rows of a multiple of four keys from a 16-byte aligned base (or one value per row)
    if (mask && mask_k != 1 && ((mask_k & 3) || (reinterpret_cast<uintptr_t>(mask) & 15))) return 0;
    if (head_dim != 64 && head_dim != 128) return 0;
    if (seq_q < 16 || seq_q > seq_kv) return 0;          // a handful of rows is the row kernel's business
    if (batch > 65535 || (int64_t)kv_heads * heads > 65535) return 0;
    if ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(v) |
         reinterpret_cast<uintptr_t>(out)) & 15) return 0;
    if (head_dim == 64) return launch_prefill_d<64>(q, k, v, out, batch, heads, kv_heads, seq_q, seq_kv, kv_capacity, scale, causal, window, right_context, lengths, mask, mask_b, mask_h, mask_q, mask_k, out_rows);
    return launch_prefill_d<128>(q, k, v, out, batch, heads, kv_heads, seq_q, seq_kv, kv_capacity, scale, causal, window, right_context, lengths, mask, mask_b, mask_h, mask_q, mask_k, out_rows);
}

}  // namespace skh
