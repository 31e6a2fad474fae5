// Q4_K dequant-GEMV for one activation row on the integer matrix cores, canonical row-major GGUF weight.
//
//   y[o] = sum_j x[j] * dequant(W[o, j]),   W[o, j] = code * (d * sc) - dmin * m  per 32-element sub-block
//
// Same products as the reference's exact-fp32 kernel up to a 22-bit fixed-point rounding of the activations
//   /root/reference/skainet-backends/skainet-backend-cpu/src/commonMain/kotlin/sk/ainet/exec/kernel/ScalarQ4_KMatmulKernel.kt:40-78
// (per sub-block: codeSum * (d * sc) - inputSum * (dmin * m)); the reference's own native kernel rounds the activations to
// 8 bits per 256-element block (native/src/q4k_matmul.c:74-92), this one keeps 22 bits per 64-element group: measured
// 3.6e-5 in the GEMV parity metric against the exact product, bound 1e-3.
//
// What bounds a read-once pass over 25 MB on this device is the shape of the loads, not the arithmetic: a wave load whose
// lanes pick 16-byte pieces out of many cache lines (a lane owning "its" 64 weights of every row) streams at 3.6 TB/s
// with no arithmetic at all, a wave load of 1 KB of consecutive bytes with the non-temporal hint at 5.0 TB/s. So:
//   * Loads are plain consecutive kilobytes. The four waves of a workgroup split K in slices of 1024 elements (576
//     bytes of a row; wave w takes slices w, w + 4, ...); a wave's share of a row quad (4 rows x its slices) is one run of
//     16-byte pieces fetched with full-wave non-temporal loads that write straight into LDS (global_load_lds_dwordx4: no
//     registers are held while the data is in flight), W quads ahead of the one being computed. The loads are inline
//     assembly with explicit wait counts: their issue order is the program order and nothing else waits on them.
//   * The lane that computes is not the lane that loaded: lane 4 * blk + j reads from LDS the header and the 32 code
//     bytes of row j of the quad, 64-weight group blk of the slice (16 groups = 1024 elements).
//   * The dot products run on v_mfma_i32_4x4x4_16b_i8 (16 independent 4x4x4 blocks): as B operand a lane supplies four
//     codes of its row (a nibble mask turns a code dword into two operands: 3 instructions per 8 weights), as A operand
//     four bytes of one "plane" of the activations of its group. The activations of a group are 22-bit fixed point
//     against the group's largest magnitude, split into balanced base-256 digits: planes 0 and 1 are the two low signed
//     digits, plane 2 the top digit + 64 (the byte as it lies in the float x * inv + 1.5 * 2^23 + 0x8080), plane 3 is all
//     ones: the four result registers of a lane are its row's dots with the three digits and its code sum, which takes
//     the + 64 out again. One accumulator per sub-block, scaled by d * sc afterwards; the minima use the exact fp32 sum
//     of the sub-block's activations.
//   * Per quad a lane ends with one partial sum (its row, its group): parked in LDS, summed over the 16 groups and the
//     four waves at the end by 16 lanes per row (one float4 each, a DPP row sum).
//   * Optional fusions as in the row-streaming kernel: RMSNorm prologue (x * gain quantised, outputs scaled by
//     1 / sqrt(mean(x^2) + eps)), epilogue residual / SwiGLU over adjacent (gate, up) rows / RoPE of one token's
//     [q | k | v] rows with the K and V rows written into the cache.
#include "gemv_q4k.h"

#include <type_traits>

namespace skh {

typedef uint32_t u32x4_m __attribute__((ext_vector_type(4)));
typedef int i32x4_m __attribute__((ext_vector_type(4)));
typedef float f32x2_m __attribute__((ext_vector_type(2)));

__device__ __forceinline__ void mfma_plain_load16(u32x4_m& dst, uint32_t off, const void* base) {
    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(dst) : "v"(off), "s"(base) : "memory");
}
__device__ __forceinline__ void mfma_plain_load8(f32x2_m& dst, uint32_t off, const void* base) {
    asm volatile("global_load_dwordx2 %0, %1, %2" : "=v"(dst) : "v"(off), "s"(base) : "memory");
}
__device__ __forceinline__ void mfma_plain_load4(float& dst, uint32_t off, const void* base) {
    asm volatile("global_load_dword %0, %1, %2" : "=v"(dst) : "v"(off), "s"(base) : "memory");
}
// 16 bytes per lane from base + off into LDS at lds_addr + 16 * lane (M0 carries the LDS address)
__device__ __forceinline__ void mfma_stream_to_lds(uint32_t lds_addr, uint32_t off, const uint8_t* base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(lds_addr), "v"(off), "s"(base) : "memory");
}
template <int N> __device__ __forceinline__ void mfma_wait_loads() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }
template <int N, typename T> __device__ __forceinline__ void mfma_wait_loads(T& v) { asm volatile("s_waitcnt vmcnt(%1)" : "+v"(v) : "n"(N) : "memory"); }
__device__ __forceinline__ void mfma_wait_lds() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

template <int I, int N, typename F> __device__ __forceinline__ void mfma_static_for(F&& f) {
    if constexpr (I < N) { f(std::integral_constant<int, I>{}); mfma_static_for<I + 1, N>(f); }
}

// d * sc and dmin * m of the two sub-blocks (2g, 2g + 1) of a lane, ggml get_scale_min_k4 through byte selectors that are
// constant per lane: g < 2 picks bytes 2h, 2h + 1 of the 6-bit fields; g >= 2 the split 4 + 2 bit form.
__device__ __forceinline__ void q4k_lane_scales_sel(const uint4& hdr, uint32_t sel, uint32_t m1, uint32_t sh_min, float& dlo,
                                                    float& dhi, float& mlo, float& mhi) {
    const float d = half_bits_to_float_fast(hdr.x & 0xFFFFu), dmin = half_bits_to_float_fast(hdr.x >> 16);
    const uint32_t A = __builtin_amdgcn_perm(hdr.w, hdr.y, sel), B = __builtin_amdgcn_perm(hdr.w, hdr.z, sel);
    const uint32_t sc = (A & m1) | ((A >> 18) & 0x3030u);
    const uint32_t mn = ((B >> sh_min) & m1) | ((B >> 18) & 0x3030u);
    dlo = d * ubyte0_to_float(sc); dhi = d * ubyte1_to_float(sc);
    mlo = dmin * ubyte0_to_float(mn); mhi = dmin * ubyte1_to_float(mn);
}

constexpr int MFMA_XROW = 20;          // dwords per (group, plane) row of 16 operand dwords, padded against bank conflicts
constexpr int MFMA_MAX_QUADS = 32;     // row quads per workgroup (bounds the final pass: 8 rounds of 256 threads)
constexpr int MFMA_XA_BYTES = 16 * 4 * MFMA_XROW * 4 + 16 * 16 + 16 * ATTN_MERGE_MAX_SPLITS * 4;
// operand planes of 16 groups + {scale, sums} per group + the merge coefficients of up to 16 heads of a slice
constexpr int MFMA_XC_OFFSET = 16 * 4 * MFMA_XROW * 4 + 16 * 16;
// Bytes of a wave's ring: W + 1 quad slots of nli KB. The last slot doubles as the staging area of the activation
// planes (the first W quads go into slots 0 .. W - 1, and the planes are in registers before the main loop asks for quad
// W); where a slot is smaller than that area the ring is that much longer.
__host__ __device__ constexpr uint32_t mfma_ring_bytes(int nli, int window) {
    return (uint32_t)(window + 1) * nli * 1024u > (uint32_t)window * nli * 1024u + MFMA_XA_BYTES
               ? (uint32_t)(window + 1) * nli * 1024u
               : (uint32_t)window * nli * 1024u + MFMA_XA_BYTES;
}

// One wave's pass: K slices wave, wave + NW, ... (NSW of them; NW waves per workgroup), row quads [0, qt) of the workgroup,
// W quads in flight.
// Leaves one partial sum per (quad, lane) in `partials` (index: quad * 64 + (lane % 4) * 16 + lane / 4) and, with the
// RMSNorm prologue, the sum of squares of this wave's activations in *ssq_out.
// PRO: 0 plain activations, 1 RMSNorm prologue (x * gain, sum of squares), 2 activations = merge of attention partials.
// T: teams. With T = 2 (K = 4096, one slice per wave) waves `wave` and `wave + NW` share slice `wave`: each prepares half
// of its activation planes (the staging area is then one per slice, shared, and a workgroup barrier stands between its
// writes and its reads), and team t takes the row quads t, t + 2, ... -- two waves per SIMD, the preparation not doubled.
template <int NSW, int W, int PRO, int NW, int T>
__device__ __forceinline__ void q4k_mfma_wave(const uint8_t* __restrict__ w, const float* __restrict__ x, const float* __restrict__ gain,
                                              const AttnMergePrologue& am, int n, int r0, int qt, uint32_t row_bytes, int wave,
                                              int team, int lane, uint8_t* ring, uint8_t* xa_stage, float* partials, float* ssq_out) {
    constexpr int NPQ = 144 * NSW;                 // 16-byte pieces of a quad in this wave's slices
    constexpr int NLI = (NPQ + 63) / 64;           // wave loads per quad
    constexpr int XI = 4 / T;                      // float4s of a slice this wave prepares per lane
    constexpr int NX = PRO == 2 ? 2 + 4 * ATTN_MERGE_MAX_SPLITS : NSW * XI * (1 + PRO);       // activation (and gain) loads
    static_assert(NX + W * NLI <= 63, "loads in flight must fit the wave's counter");
    static_assert(PRO != 2 || NSW == 1, "the attention-merge prologue serves one slice per wave");
    static_assert(T == 1 || (NSW == 1 && PRO != 2), "two teams: one slice per wave, plain or RMSNorm prologue");
    const int nq = (qt - team + T - 1) / T;        // this wave's quads: team, team + T, ... (uniform; at least one)
    const int blk = lane >> 2, j = lane & 3, g = blk & 3, h = g & 1;
    const uint32_t sel = g < 2 ? (0x0C0C0000u | ((2 * h + 1) << 8) | (2 * h))
                               : (((2 * h + 1) << 24) | ((2 * h) << 16) | ((4 + 2 * h + 1) << 8) | (4 + 2 * h));
    const uint32_t m1 = g < 2 ? 0x3F3Fu : 0x0F0Fu, sh_min = g < 2 ? 0u : 4u;

    // activations (and gains) of this wave's slices first, the first W quads right behind them
    u32x4_m xq[NSW][XI], gq[PRO == 1 ? NSW : 1][XI];
    constexpr int MS = PRO == 2 ? ATTN_MERGE_MAX_SPLITS : 1;
    u32x4_m pq[PRO == 2 ? 4 : 1][MS];              // attention partials of the lane's four float4s, one per split
    f32x2_m mlq[2];                                // (max, sum) of the (head, split) pair this lane weighs, two rounds of 8 heads
    if constexpr (PRO == 2) {
        // lane = (head of the slice, split): 8 heads per round, heads-per-slice = 1024 / head_dim (4, 8 or 16)
        const int hd_shift = __builtin_ctz(am.head_dim), hps = 1024 >> hd_shift, sp = lane & 7;
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            const int hh = r * 8 + (lane >> 3);
            mlq[r] = f32x2_m{-INFINITY, 0.f};
            if (hh < hps && sp < am.splits) mfma_plain_load8(mlq[r], (uint32_t)(((wave * hps + hh) * am.splits + sp) * 2) * 4u, am.ml);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int e = (i * 64 + lane) * 4, hh = e >> hd_shift, d = e - (hh << hd_shift);
#pragma unroll
            for (int sI = 0; sI < MS; ++sI) {
                pq[i][sI] = u32x4_m{0u, 0u, 0u, 0u};
                if (sI < am.splits) mfma_plain_load16(pq[i][sI], (uint32_t)(((wave * hps + hh) * am.splits + sI) * am.head_dim + d) * 4u, am.part);
            }
        }
    } else {
#pragma unroll
        for (int t = 0; t < NSW; ++t)
#pragma unroll
            for (int ii = 0; ii < XI; ++ii) {
                const int i = team * XI + ii;
                const uint32_t off = (uint32_t)((wave + NW * t) * 1024 + (i * 64 + lane) * 4) * 4u;
                mfma_plain_load16(xq[t][ii], off, x);
                if (PRO == 1) mfma_plain_load16(gq[t][ii], off, gain);
            }
    }
    uint32_t loff[NLI];
#pragma unroll
    for (int u = 0; u < NLI; ++u) {
        const uint32_t p = min(64u * u + lane, (uint32_t)(NPQ - 1)), t = (p * 1821u) >> 18;       // p / 144 for p < 2^12
        const uint32_t rem = p - 144u * t, row4 = (rem * 1821u) >> 16, pc = rem - 36u * row4;    // rem / 36
        loff[u] = __umul24(row4, row_bytes) + (wave + (uint32_t)NW * t) * 576u + pc * 16u;
    }
    const uint32_t max_off = (uint32_t)n * row_bytes - 16u;
    const uint32_t ring_addr = (uint32_t)(size_t)(__attribute__((address_space(3))) uint8_t*)ring;
    constexpr uint32_t SLOT = NLI * 1024u;          // bytes of a quad in the ring; W + 1 slots
    // q: index among this wave's quads (the workgroup's quad team + T q), uniform; rows past the weight are clamped
    // (computed, never stored)
    auto issue_quad = [&](int q) {
        const uint32_t base = (uint32_t)(r0 + 4 * (team + T * q)) * row_bytes;
        const uint32_t slot = ring_addr + (uint32_t)(q % (W + 1)) * SLOT;
#pragma unroll
        for (int u = 0; u < NLI; ++u) mfma_stream_to_lds(slot + 1024u * u, min(base + loff[u], max_off), w);
    };
#pragma unroll
    for (int q = 0; q < W; ++q) issue_quad(min(q, nq - 1));
    if constexpr (PRO == 2) {
        mfma_wait_loads<W * NLI>(mlq[0]); mfma_wait_loads<W * NLI>(mlq[1]);
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int sI = 0; sI < MS; ++sI) mfma_wait_loads<W * NLI>(pq[i][sI]);
        // weights of the splits: per head the maximum over its 8 lanes, 2^(m - max), normalised by the weighted sum of l
        float* xc = reinterpret_cast<float*>(xa_stage + MFMA_XC_OFFSET);
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            float mm = mlq[r].x;
            mm = fmaxf(mm, __shfl_xor(mm, 1, 64)); mm = fmaxf(mm, __shfl_xor(mm, 2, 64)); mm = fmaxf(mm, __shfl_xor(mm, 4, 64));
            const float e = __builtin_amdgcn_exp2f(mlq[r].x - mm);
            const float wgt = mlq[r].x == -INFINITY ? 0.f : e;
            float ls = wgt * mlq[r].y;
            ls += __shfl_xor(ls, 1, 64); ls += __shfl_xor(ls, 2, 64); ls += __shfl_xor(ls, 4, 64);
            xc[r * 64 + lane] = ls > 0.f ? wgt / ls : 0.f;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int hh = ((i * 64 + lane) * 4) >> __builtin_ctz(am.head_dim);
            const float4 c0 = *reinterpret_cast<const float4*>(xc + hh * 8), c1 = *reinterpret_cast<const float4*>(xc + hh * 8 + 4);
            const float c[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
            float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int sI = 0; sI < MS; ++sI) {
                a.x = fmaf(c[sI], __uint_as_float(pq[i][sI].x), a.x); a.y = fmaf(c[sI], __uint_as_float(pq[i][sI].y), a.y);
                a.z = fmaf(c[sI], __uint_as_float(pq[i][sI].z), a.z); a.w = fmaf(c[sI], __uint_as_float(pq[i][sI].w), a.w);
            }
            xq[0][i] = u32x4_m{__float_as_uint(a.x), __float_as_uint(a.y), __float_as_uint(a.z), __float_as_uint(a.w)};
        }
    } else {
        mfma_wait_loads<W * NLI>(xq[0][0]);
#pragma unroll
        for (int t = 0; t < NSW; ++t)
#pragma unroll
            for (int i = 0; i < XI; ++i) { mfma_wait_loads<W * NLI>(xq[t][i]); if (PRO == 1) mfma_wait_loads<W * NLI>(gq[t][i]); }
    }

    // activations of a slice: float4 number f = i * 64 + lane belongs to group f / 16 (the 16 lanes of a DPP row share a
    // group); planes go through LDS into operand order
    int xa[NSW][16];
    float s_grp[NSW], xsl[NSW], xsh[NSW];
    float ssq = 0.f;
    uint32_t* xa_lds = reinterpret_cast<uint32_t*>(xa_stage);
    float4* xs_lds = reinterpret_cast<float4*>(xa_stage + 16 * 4 * MFMA_XROW * 4);
#pragma unroll
    for (int t = 0; t < NSW; ++t) {
#pragma unroll
        for (int ii = 0; ii < XI; ++ii) {
            const int i = team * XI + ii;              // float4 number i * 64 + lane of the slice
            float4 v = make_float4(__uint_as_float(xq[t][ii].x), __uint_as_float(xq[t][ii].y), __uint_as_float(xq[t][ii].z), __uint_as_float(xq[t][ii].w));
            if (PRO == 1) {
                ssq = fmaf(v.x, v.x, fmaf(v.y, v.y, fmaf(v.z, v.z, fmaf(v.w, v.w, ssq))));
                v.x *= __uint_as_float(gq[t][ii].x); v.y *= __uint_as_float(gq[t][ii].y);
                v.z *= __uint_as_float(gq[t][ii].z); v.w *= __uint_as_float(gq[t][ii].w);
            }
            const int G = i * 4 + (lane >> 4), tt = lane & 15;
            const float amax = row16_max(fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
            const float inv = 2097151.0f * __builtin_amdgcn_rcpf(fmaxf(amax, 1e-30f));
            float s4 = (v.x + v.y) + (v.z + v.w);                  // summed over the 8 lanes of a half row = a sub-block of 32
            s4 += dpp_row_move<0xB1>(s4); s4 += dpp_row_move<0x4E>(s4); s4 += dpp_row_move<0x141>(s4);
            const uint32_t b0 = __float_as_uint(fmaf(v.x, inv, 12615808.0f)), b1 = __float_as_uint(fmaf(v.y, inv, 12615808.0f));
            const uint32_t b2 = __float_as_uint(fmaf(v.z, inv, 12615808.0f)), b3 = __float_as_uint(fmaf(v.w, inv, 12615808.0f));
            const uint32_t a = __builtin_amdgcn_perm(b1, b0, 0x05010400u), b = __builtin_amdgcn_perm(b3, b2, 0x05010400u);
            const uint32_t c = __builtin_amdgcn_perm(b1, b0, 0x07030602u), d = __builtin_amdgcn_perm(b3, b2, 0x07030602u);
            uint32_t* dst = xa_lds + G * 4 * MFMA_XROW + tt;
            dst[0] = __builtin_amdgcn_perm(b, a, 0x05040100u) ^ 0x80808080u;
            dst[MFMA_XROW] = __builtin_amdgcn_perm(b, a, 0x07060302u) ^ 0x80808080u;
            dst[2 * MFMA_XROW] = __builtin_amdgcn_perm(d, c, 0x05040100u);
            dst[3 * MFMA_XROW] = 0x01010101u;
            float* xs = reinterpret_cast<float*>(xs_lds + G);
            if ((tt & 7) == 0) { xs[0] = amax * (1.0f / 2097151.0f); xs[1 + (tt >> 3)] = s4 * inv; }
        }
        if constexpr (T == 2) __syncthreads();         // the other team's half of the planes (every wave of the workgroup gets here)
        const uint4* src = reinterpret_cast<const uint4*>(xa_lds + (blk * 4 + j) * MFMA_XROW);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const uint4 v4 = src[e];
            xa[t][4 * e] = (int)v4.x; xa[t][4 * e + 1] = (int)v4.y; xa[t][4 * e + 2] = (int)v4.z; xa[t][4 * e + 3] = (int)v4.w;
        }
        const float4 xsv = xs_lds[blk];
        s_grp[t] = xsv.x; xsl[t] = xsv.y; xsh[t] = xsv.z;
    }
    if (PRO == 1) *ssq_out = wave_sum(ssq);

    // lane's read offsets inside a quad slot: header of (row j, super-block blk / 4 of the slice), then its two code pieces
    const uint32_t rd_hdr = (uint32_t)(j * 36 + (blk >> 2) * 9) * 16u, rd_q = rd_hdr + 16u + (uint32_t)g * 32u;
    const int widx = j * 16 + blk;
    auto compute_quad = [&](int q) {                 // q: index among this wave's quads
        const uint8_t* slot = ring + (uint32_t)(q % (W + 1)) * SLOT;
        float total = 0.f;
#pragma unroll
        for (int t = 0; t < NSW; ++t) {
            const uint4 hdr = *reinterpret_cast<const uint4*>(slot + t * 2304 + rd_hdr);
            const uint4 q0 = *reinterpret_cast<const uint4*>(slot + t * 2304 + rd_q);
            const uint4 q1 = *reinterpret_cast<const uint4*>(slot + t * 2304 + rd_q + 16);
            float dlo, dhi, mlo, mhi;
            q4k_lane_scales_sel(hdr, sel, m1, sh_min, dlo, dhi, mlo, mhi);
            const uint32_t qw[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
            i32x4_m dl = {0, 0, 0, 0}, dh = {0, 0, 0, 0};
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int wlo = (int)(qw[u] & 0x0F0F0F0Fu), whi = (int)((qw[u] >> 4) & 0x0F0F0F0Fu);
                dl = __builtin_amdgcn_mfma_i32_4x4x4i8(xa[t][u], wlo, dl, 0, 0, 0);
                dh = __builtin_amdgcn_mfma_i32_4x4x4i8(xa[t][8 + u], whi, dh, 0, 0, 0);
            }
            // digits back together: ((top * 256 + mid) * 256 + low) - 64 * 65536 * (code sum). The top term alone can pass
            // 2^31 (top digit + 64 up to 96, codes up to 15, 32 of them) before the code sum takes the + 64 out again:
            // the sum is formed modulo 2^32 on unsigned values (the true result fits 32 bits) and read as signed at the end.
            const uint32_t ul = (uint32_t)dl[3] * 0xFFC00000u + ((((uint32_t)dl[2] << 8) + (uint32_t)dl[1]) << 8) + (uint32_t)dl[0];
            const uint32_t uh = (uint32_t)dh[3] * 0xFFC00000u + ((((uint32_t)dh[2] << 8) + (uint32_t)dh[1]) << 8) + (uint32_t)dh[0];
            const int tl = (int)ul, th = (int)uh;
            total = fmaf(s_grp[t], fmaf(dlo, (float)tl, fmaf(dhi, (float)th, -fmaf(mlo, xsl[t], mhi * xsh[t]))), total);
        }
        partials[(team + T * q) * 64 + widx] = total;
    };

    // quads [0, base): wait for the quad, ask for the one W ahead, compute; the last W quads without new requests
    const int base = max(nq - W, 0);
    for (int q = 0; q < base; ++q) {
        mfma_wait_loads<(W - 1) * NLI>();
        mfma_wait_lds();                             // the slot about to be refilled has been read
        issue_quad(q + W);
        compute_quad(q);
    }
    mfma_static_for<0, W>([&](auto mc) {
        constexpr int m = decltype(mc)::value;
        mfma_wait_loads<(W - 1 - m) * NLI>();
        if (base + m < nq) compute_quad(base + m);
    });
}

// The epilogue is a template argument, not a run-time switch: what an epilogue reads besides a row's sum (residual
// element, cos / sin pair) is requested at the start of the kernel and held in registers to the end, and with the switch
// at run time every variant paid for those registers (the plain product ran 6.53 us where this form runs 6.15).
// NW: waves that split K, 4 or 8 (eight for long rows: a wave prepares and multiplies half as many slices and two waves
// share a SIMD). T: teams of NW waves that split the workgroup's row quads (two at K = 4096: again two waves per SIMD,
// and each prepares half of its slice's activation planes).
template <int W, int PRO, int EPI, int NW, int T>
__global__ __launch_bounds__(64 * NW * T, (PRO == 2 || NW * T == 8) ? 1 : 2) void q4k_gemv_mfma_kernel(const uint8_t* __restrict__ w, const float* __restrict__ x, float* y,
                                                                            int k, int n, int qt, const float* __restrict__ gain, float eps,
                                                                            const float* residual, RopeQkvEpilogue rope,
                                                                            AttnMergePrologue am) {
    constexpr int epilogue = EPI;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int lane = threadIdx.x & 63, wave_all = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wave = T == 1 ? wave_all : wave_all % NW, team = T == 1 ? 0 : wave_all / NW;
    const int nsl = k >> 10;                                   // slices of 1024 elements
    const int nsw = (nsl - wave + NW - 1) / NW;                // this wave's share (uniform)
    const int ns_max = (nsl + NW - 1) / NW;
    const int nli_max = (144 * ns_max + 63) / 64;
    // One team: the planes' staging area is the ring's last slot (free until the main loop). Two teams: one area per slice,
    // shared by its two waves, behind the rings.
    const uint32_t ring_bytes = T == 1 ? mfma_ring_bytes(nli_max, W) : (uint32_t)(W + 1) * nli_max * 1024u;
    uint8_t* ring = smem + wave_all * ring_bytes;
    uint8_t* xa_stage = T == 1 ? ring + (uint32_t)W * (uint32_t)nli_max * 1024u : smem + NW * T * ring_bytes + wave * MFMA_XA_BYTES;
    float* partials_all = reinterpret_cast<float*>(smem + NW * T * ring_bytes + (T == 1 ? 0 : NW * MFMA_XA_BYTES));   // [NW slices of K][qt][64]
    float* ssq_lds = partials_all + NW * qt * 64;
    float* partials = partials_all + wave * qt * 64;
    const int r0 = blockIdx.x * (4 * qt);
    const uint32_t row_bytes = (uint32_t)(k >> 8) * (uint32_t)Q4K_BYTES;

    // what the final pass will add or rotate with: one output row per 16 threads and round
    constexpr int RPR = 4 * NW * T;                             // rows per round
    constexpr int ROUNDS = MFMA_MAX_QUADS * 4 / RPR;
    float pre_res[EPI == EPI_RESIDUAL ? ROUNDS : 1];
    f32x2_m pre_cs[EPI == EPI_ROPE_QKV ? ROUNDS : 1];
    int pos = 0;
    if constexpr (EPI == EPI_ROPE_QKV) pos = rope.pos_dev[0];
    if constexpr (EPI == EPI_RESIDUAL || EPI == EPI_ROPE_QKV) {
        if (EPI == EPI_RESIDUAL || rope.table) {                                       // uniform
#pragma unroll
            for (int it = 0; it < ROUNDS; ++it) {
                const int row = min(r0 + it * RPR + (threadIdx.x >> 4), n - 1);
                if constexpr (EPI == EPI_RESIDUAL) pre_res[it] = 0.f; else pre_cs[it] = f32x2_m{1.f, 0.f};
                if (it * RPR < 4 * qt) {
                    if constexpr (EPI == EPI_RESIDUAL) mfma_plain_load4(pre_res[it], (uint32_t)row * 4u, residual);
                    else mfma_plain_load8(pre_cs[it], (uint32_t)((row % rope.head_dim) >> 1) * 8u, rope.table);
                }
            }
            mfma_wait_loads<0>();             // a handful of cached loads, before the stream starts
        }
    }

    float ssq = 0.f;
    switch (nsw) {
        case 1: q4k_mfma_wave<1, W, PRO, NW, T>(w, x, gain, am, n, r0, qt, row_bytes, wave, team, lane, ring, xa_stage, partials, &ssq); break;
        case 2: if constexpr (PRO != 2 && T == 1) q4k_mfma_wave<2, W, PRO, NW, T>(w, x, gain, am, n, r0, qt, row_bytes, wave, team, lane, ring, xa_stage, partials, &ssq); break;
        case 3: if constexpr (W <= 2 && PRO != 2 && NW == 4 && T == 1) q4k_mfma_wave<3, W, PRO, NW, T>(w, x, gain, am, n, r0, qt, row_bytes, wave, team, lane, ring, xa_stage, partials, &ssq); break;
        case 4: if constexpr (W <= 2 && PRO != 2 && NW == 4 && T == 1) q4k_mfma_wave<4, W, PRO, NW, T>(w, x, gain, am, n, r0, qt, row_bytes, wave, team, lane, ring, xa_stage, partials, &ssq); break;
        default:                                               // K below NW slices: this wave has none
            for (int i = lane; i < qt * 64; i += 64) partials[i] = 0.f;
    }
    if (PRO == 1 && lane == 0) ssq_lds[wave_all] = ssq;
    __syncthreads();

    float xscale = 1.0f;
    if (PRO == 1) {
        float ss = (ssq_lds[0] + ssq_lds[1]) + (ssq_lds[2] + ssq_lds[3]);
        if (NW * T == 8) ss += (ssq_lds[4] + ssq_lds[5]) + (ssq_lds[6] + ssq_lds[7]);
        xscale = 1.0f / sqrtf(ss * (1.0f / (float)k) + eps);
    }
    const int u = threadIdx.x & 15, pw = u >> 2, pp = u & 3;
#pragma unroll
    for (int it = 0; it < ROUNDS; ++it) {
        if (it * RPR >= 4 * qt) break;                         // uniform
        const int rl = it * RPR + (threadIdx.x >> 4);          // row of the workgroup
        const int rlc = min(rl, 4 * qt - 1);
        float4 p4 = *reinterpret_cast<const float4*>(partials_all + (pw * qt + (rlc >> 2)) * 64 + (rlc & 3) * 16 + pp * 4);
        if (NW == 8) {                                         // waves 4 .. 7: a second float4 per thread
            const float4 p8 = *reinterpret_cast<const float4*>(partials_all + ((pw + 4) * qt + (rlc >> 2)) * 64 + (rlc & 3) * 16 + pp * 4);
            p4.x += p8.x; p4.y += p8.y; p4.z += p8.z; p4.w += p8.w;
        }
        float val = row16_sum((p4.x + p4.y) + (p4.z + p4.w)) * xscale;
        const int row = r0 + rl;
        const bool live = u == 0 && rl < 4 * qt && row < n;
        if constexpr (EPI == EPI_SWIGLU) {
            const float up = __shfl_xor(val, 16, 64);          // rows 2i (gate) and 2i + 1 (up) sit 16 lanes apart
            if (live && !(row & 1)) y[row >> 1] = val * (1.0f / (1.0f + expf(-val))) * up;
        } else if constexpr (EPI == EPI_ROPE_QKV) {
            const float odd = __shfl_xor(val, 16, 64);
            if (live && !(row & 1)) {
                const int slot = row / rope.head_dim, dd = row % rope.head_dim;
                float2 out2 = make_float2(val, odd);
                if (slot < rope.heads + rope.kv_heads) {
                    float sn, cs;
                    if (rope.table) { cs = pre_cs[it].x; sn = pre_cs[it].y; }
                    else sincosf((float)pos * powf(rope.theta, -(float)dd / (float)rope.head_dim), &sn, &cs);
                    out2 = rope_rotate(val, odd, cs, sn);
                }
                const bool in_cache = pos >= 0 && pos < rope.capacity;
                float* dst;
                if (slot < rope.heads) dst = y + (int64_t)slot * rope.head_dim;
                else if (slot < rope.heads + rope.kv_heads) dst = rope.k_cache + ((int64_t)(slot - rope.heads) * rope.capacity + pos) * rope.head_dim;
                else dst = rope.v_cache + ((int64_t)(slot - rope.heads - rope.kv_heads) * rope.capacity + pos) * rope.head_dim;
                if (slot < rope.heads || in_cache) *reinterpret_cast<float2*>(dst + dd) = out2;
            }
        } else if (live) {
            if constexpr (EPI == EPI_RESIDUAL) val += pre_res[it];
            y[row] = val;
        }
    }
}

static std::atomic<int> g_q4k_mfma_enable{1};
void set_q4k_mfma_enable(int v) { g_q4k_mfma_enable = v; }
static size_t mfma_smem_bytes(int k, int qt, int window, int nw, int teams);
// Would launch_q4k_gemv_mfma take a product whose activations are the unmerged results of a one-query attention
// (n outputs, k = heads * head_dim)? Every reason it can refuse that form, without launching anything: a caller that
// leaves attention splits unmerged for it has no way back once the attention kernel has run.
bool q4k_gemv_mfma_accepts_merge(int k, int n, int head_dim) {
    if (!g_q4k_mfma_enable || k < 1024 || (k & 1023) || k > 4096 || n < 4) return false;
    if (head_dim != 64 && head_dim != 128 && head_dim != 256) return false;
    if ((uint64_t)n * (uint64_t)(k >> 8) * Q4K_BYTES >= ((uint64_t)1 << 32)) return false;
    const int quads = (n + 3) / 4;
    int qt = (quads + num_cus() - 1) / num_cus();
    if (qt > MFMA_MAX_QUADS) qt = MFMA_MAX_QUADS;
    return mfma_smem_bytes(k, qt < 1 ? 1 : qt, 3, 4, 1) <= 160 * 1024;
}
static std::atomic<int> g_q4k_mfma_teams{0};       // 0: chosen from the quads a workgroup owns
void set_q4k_mfma_teams(int v) { if (v >= 0 && v <= 2) g_q4k_mfma_teams = v; }
static std::atomic<int> g_q4k_mfma_waves8{1};
void set_q4k_mfma_waves8(int v) { g_q4k_mfma_waves8 = v != 0; }
static std::atomic<int> g_q4k_mfma_window{0};      // 0: chosen from K
void set_q4k_mfma_window(int v) { if (v == 0 || v == 2 || v == 3) g_q4k_mfma_window = v; }

// quads in flight per wave: three while a quad is at most 5 KB per wave, two for the long rows (9 KB per quad and wave)
static int mfma_window(int k) { return (((k >> 10) + 3) >> 2) >= 3 ? 2 : 3; }

static size_t mfma_smem_bytes(int k, int qt, int window, int nw, int teams) {
    const int ns_max = ((k >> 10) + nw - 1) / nw;
    const int nli_max = (144 * ns_max + 63) / 64;
    const size_t rings = teams == 1 ? (size_t)nw * mfma_ring_bytes(nli_max, window)
                                    : (size_t)nw * teams * (window + 1) * nli_max * 1024 + (size_t)nw * MFMA_XA_BYTES;
    return rings + (size_t)nw * qt * 64 * sizeof(float) + 32;
}

template <int W, int PRO, int EPI, int NW = 4, int T = 1>
static int launch_mfma_variant(int grid, size_t smem, hipStream_t s, const uint8_t* w, const float* x, float* y, int k, int n, int qt,
                               const float* gain, float eps, const float* residual, const RopeQkvEpilogue& rope,
                               const AttnMergePrologue& am) {
    SKH_SET_MAX_DYNAMIC_LDS_ONCE((&q4k_gemv_mfma_kernel<W, PRO, EPI, NW, T>), 160 * 1024);
    q4k_gemv_mfma_kernel<W, PRO, EPI, NW, T><<<dim3(grid), dim3(64 * NW * T), smem, s>>>(w, x, y, k, n, qt, gain, eps, residual, rope, am);
    SKH_CHECK(hipGetLastError());
    return 1;
}

// The combinations the entry points use: plain activations with no epilogue or a residual; the RMSNorm prologue with no
// epilogue, SwiGLU or RoPE + cache append; the attention-merge prologue with no epilogue or a residual (K <= 4096: W = 3).
template <int W>
static int launch_mfma(int pro, int grid, size_t smem, hipStream_t s, const uint8_t* w, const float* x, float* y, int k, int n, int qt,
                       const float* gain, float eps, const float* residual, int epilogue, const RopeQkvEpilogue& rope,
                       const AttnMergePrologue& am) {
#define SKH_MFMA_CASE(PRO, EPI) return launch_mfma_variant<W, PRO, EPI>(grid, smem, s, w, x, y, k, n, qt, gain, eps, residual, rope, am)
    if (pro == 2) {
        if constexpr (W == 3) {
            note_kernel("q4k_gemv_mfma_kernel (attention-merge prologue)");
            if (epilogue == EPI_NONE) SKH_MFMA_CASE(2, EPI_NONE);
            if (epilogue == EPI_RESIDUAL) SKH_MFMA_CASE(2, EPI_RESIDUAL);
        }
        return 0;
    }
    note_kernel("q4k_gemv_mfma_kernel");
    if (pro == 1) {
        if (epilogue == EPI_NONE) SKH_MFMA_CASE(1, EPI_NONE);
        if (epilogue == EPI_RESIDUAL) SKH_MFMA_CASE(1, EPI_RESIDUAL);
        if (epilogue == EPI_SWIGLU) SKH_MFMA_CASE(1, EPI_SWIGLU);
        SKH_MFMA_CASE(1, EPI_ROPE_QKV);
    }
    if (epilogue == EPI_NONE) SKH_MFMA_CASE(0, EPI_NONE);
    if (epilogue == EPI_RESIDUAL) SKH_MFMA_CASE(0, EPI_RESIDUAL);
    if (epilogue == EPI_SWIGLU) SKH_MFMA_CASE(0, EPI_SWIGLU);
    SKH_MFMA_CASE(0, EPI_ROPE_QKV);
#undef SKH_MFMA_CASE
}

// Returns 1 when this kernel took the product, 0 when the shape is outside its range (the caller goes on to the
// row-streaming kernel), -1 on a launch error. One activation row; K a multiple of 1024 up to 16384; the weight below
// 4 GiB (32-bit byte offsets); operands 16-byte aligned.
int launch_q4k_gemv_mfma(const uint8_t* w, const float* x, float* y, int k, int n, const float* gain, float eps,
                         const float* residual, int epilogue, const RopeQkvEpilogue* rope_in, const AttnMergePrologue* merge) {
    if (!g_q4k_mfma_enable) return 0;
    if (k < 1024 || (k & 1023) || k > 16384 || n < 4) return 0;
    AttnMergePrologue am{};
    if (merge) {
        // the activations are the merge of attention partials: one slice per wave, heads that tile a slice
        am = *merge;
        if (gain || k > 4096 || am.splits < 1 || am.splits > ATTN_MERGE_MAX_SPLITS) return 0;
        if (am.head_dim != 64 && am.head_dim != 128 && am.head_dim != 256) return 0;
        if ((reinterpret_cast<uintptr_t>(am.part) & 15) || (reinterpret_cast<uintptr_t>(am.ml) & 7)) return 0;
        x = am.part;
    }
    const uint64_t wbytes = (uint64_t)n * (uint64_t)(k >> 8) * Q4K_BYTES;
    if (wbytes >= ((uint64_t)1 << 32) || (uint64_t)n * 4 >= ((uint64_t)1 << 32)) return 0;
    if ((reinterpret_cast<uintptr_t>(w) & 15) || (reinterpret_cast<uintptr_t>(x) & 15)) return 0;
    if (gain && (reinterpret_cast<uintptr_t>(gain) & 15)) return 0;
    RopeQkvEpilogue rope{};
    if (epilogue == EPI_ROPE_QKV) {
        if (!rope_in) return 0;
        rope = *rope_in;
        if ((rope.head_dim & 1) || n != (rope.heads + 2 * rope.kv_heads) * rope.head_dim) return 0;
        if (rope.table && (reinterpret_cast<uintptr_t>(rope.table) & 7)) return 0;
    }
    if (epilogue >= EPI_SWIGLU && (n & 1)) return 0;
    if (epilogue == EPI_RESIDUAL && (!residual || (reinterpret_cast<uintptr_t>(residual) & 3))) return 0;
    // one round of workgroups over the chip: a workgroup's quads are consecutive rows, the last workgroup may own fewer
    const int quads = (n + 3) / 4;
    int qt = (quads + num_cus() - 1) / num_cus();
    if (qt > MFMA_MAX_QUADS) qt = MFMA_MAX_QUADS;
    if (qt < 1) qt = 1;
    const int grid = (quads + qt - 1) / qt;
    // measured on 11008 x 4096 with two / three / four quads in flight: 7.06 / 6.52 / 6.68 us; in a Llama-3-8B decode
    // step (every Q4_K product) 1.617 / 1.564 / 1.568 / 1.578 ms per token with two / three / four / five
    int window = g_q4k_mfma_window.load() > 0 ? g_q4k_mfma_window.load() : mfma_window(k);
    if (mfma_window(k) == 2) window = 2;                       // long rows: the wave's load counter holds 63
    if (merge) window = 3;
    const int pro = merge ? 2 : gain ? 1 : 0;
    // long rows without a prologue (the decoder's down projection): eight waves, K split eight ways
    if (g_q4k_mfma_waves8 && pro == 0 && k >= 8192 && epilogue <= EPI_RESIDUAL) {
        const size_t smem8 = mfma_smem_bytes(k, qt, 2, 8, 1);
        if (smem8 <= 160 * 1024) {
            note_kernel("q4k_gemv_mfma_kernel");
            if (epilogue == EPI_NONE) return launch_mfma_variant<2, 0, EPI_NONE, 8>(grid, smem8, current_stream(), w, x, y, k, n, qt, gain, eps, residual, rope, am);
            return launch_mfma_variant<2, 0, EPI_RESIDUAL, 8>(grid, smem8, current_stream(), w, x, y, k, n, qt, gain, eps, residual, rope, am);
        }
    }
    // K = 4096 with a plain or RMSNorm prologue: two teams of four waves (two waves per SIMD, the planes prepared once)
    // where a workgroup owns enough quads: measured with two teams / one, 28 quads (28672 rows) 11.64 / 12.09 us, 11 quads
    // (11008 rows) 5.98 / 6.23, 6 quads (6144 rows) 4.43 / 4.51, but 4 quads (4096 rows) 3.91 / 3.83 -- the barrier between
    // the halves of the preparation costs more than so short a run of quads gains
    const int teams = g_q4k_mfma_teams.load() != 0 ? g_q4k_mfma_teams.load() : (qt >= 5 ? 2 : 1);
    // (two quads in flight per wave then: with two waves per SIMD 6.14 us at three, 5.98 at two, 6.95 at one)
    if (teams == 2 && pro != 2 && k == 4096 && qt >= 2) {
        const size_t smem2 = mfma_smem_bytes(k, qt, 2, 4, 2);
        if (smem2 <= 160 * 1024) {
            note_kernel("q4k_gemv_mfma_kernel");
#define SKH_MFMA_T2(PRO, EPI) return launch_mfma_variant<2, PRO, EPI, 4, 2>(grid, smem2, current_stream(), w, x, y, k, n, qt, gain, eps, residual, rope, am)
            if (pro == 1) {
                if (epilogue == EPI_NONE) SKH_MFMA_T2(1, EPI_NONE);
                if (epilogue == EPI_RESIDUAL) SKH_MFMA_T2(1, EPI_RESIDUAL);
                if (epilogue == EPI_SWIGLU) SKH_MFMA_T2(1, EPI_SWIGLU);
                SKH_MFMA_T2(1, EPI_ROPE_QKV);
            }
            if (epilogue == EPI_NONE) SKH_MFMA_T2(0, EPI_NONE);
            if (epilogue == EPI_RESIDUAL) SKH_MFMA_T2(0, EPI_RESIDUAL);
            if (epilogue == EPI_SWIGLU) SKH_MFMA_T2(0, EPI_SWIGLU);
            SKH_MFMA_T2(0, EPI_ROPE_QKV);
#undef SKH_MFMA_T2
        }
    }
    const size_t smem = mfma_smem_bytes(k, qt, window, 4, 1);
    if (smem > 160 * 1024) return 0;
    if (window == 2) return launch_mfma<2>(pro, grid, smem, current_stream(), w, x, y, k, n, qt, gain, eps, residual, epilogue, rope, am);
    return launch_mfma<3>(pro, grid, smem, current_stream(), w, x, y, k, n, qt, gain, eps, residual, epilogue, rope, am);
}

}  // namespace skh
