// Q4_K dequant-GEMV for 3 to 8 activation rows on the matrix cores, canonical row-major GGUF weight.
//
//   y[b, o] = sum_j x[b, j] * dequant(W[o, j])
//
// Same products as the reference's exact-fp32 kernel, other summation order
//   /root/reference/skainet-backends/skainet-backend-cpu/src/commonMain/kotlin/sk/ainet/exec/kernel/ScalarQ4_KMatmulKernel.kt:40-78
//
// With one activation row a weight costs a conversion and an FMA per lane; with eight rows it would cost eight FMAs
// and the kernel would be bound by the vector ALU, not by HBM. Here the products run on v_mfma_f32_4x4x4_16b_bf16:
//   * a 4-bit code q is the bf16 value 128 + q after one mask-and-merge (0x4300 | q: bf16 has ulp 1 on [128, 256)), two
//     codes per instruction; the 128 is taken out again by starting each accumulator at -128 * sum(x);
//   * an activation is split into two bf16 values, hi = bf16(x) and lo = bf16(x - hi) (16 to 17 significant bits
//     together, every product exact in fp32); hi and lo run through the same accumulator.
//   (The fp16 form of the same instruction would take the codes as they lie in the code dword, as fp16 subnormals, and
//   22 bits of activation; measured on this device it adds its four products and the accumulator in a truncating
//   adder of about 19 bits below the largest addend, which leaves a one-sided error of 2.5e-5 of the largest output:
//   more than this kernel's whole error with bf16 operands.)
//   * Lane l = 4 * blk + j. As B operand it supplies four weights of output row j of the wave's current row quad; as A
//     operand four activations (hi or lo part) of batch row j of a batch quad; both at the K position of block blk.
//     The four result registers of lane 4 * blk + j are the quad's batch rows against output row j.
//   * Block blk owns one 32-byte nibble group (64 weights: sub-blocks 2g and 2g + 1) of every super-block quartet, so
//     a wave covers 1024 consecutive K elements ("pass") and a lane keeps its 64 activations per batch row in registers
//     (hi and lo: 64 packed dwords) for all the row quads of the workgroup. Per row quad a lane loads its row's block header and
//     its 32 bytes of codes: across the wave, four spans of 576 contiguous bytes.
//   * The four waves of a workgroup take the passes round-robin (K = 4096: one pass each) and all walk the same row
//     quads; per-lane sums are folded across the 16 blocks with a multi-value butterfly and across the waves in LDS.
#include "gemv_q4k.h"

namespace skh {

typedef float f32x4_q __attribute__((ext_vector_type(4)));
constexpr int QD_SLICE = 36;   // dwords per slice: 64 bf16 activations + 4 dwords of padding (16-byte aligned rows that spread over the banks)


// Fold 16 per-lane values across the 16 four-lane blocks of a wave (lane bits 2..5), leaving bits 0..1 apart: on
// return v[0] of lane l is the total, over the lanes with the same l % 4, of value block_fold_index(l).
// The partners 4 and 8 lanes away are inside the lane's row of 16: DPP moves (lane ^ 8 is a rotation by 8; lane ^ 4 is a
// shift left by 4 for the lanes of banks 0 and 2 and a shift right by 4 for banks 1 and 3, two moves under bank masks).
template <int MASK>
__device__ __forceinline__ float block_fold_partner(float v) {
    if constexpr (MASK == 4) {
        const int up = __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x104, 0xF, 0x5, false);      // row_shl:4 -> lane + 4
        return __int_as_float(__builtin_amdgcn_update_dpp(up, __float_as_int(v), 0x114, 0xF, 0xA, false));   // row_shr:4 -> lane - 4
    } else if constexpr (MASK == 8) {
        return dpp_row_move<0x128>(v);                                                                    // row_ror:8
    } else {
        return __shfl_xor(v, MASK, 64);
    }
}
template <int MASK, int HALF>
__device__ __forceinline__ void block_fold_step(float* v, int lane) {
    const uint32_t up = (lane & MASK) ? 0xFFFFFFFFu : 0u;
#pragma unroll
    for (int i = 0; i < HALF; ++i) {
        const uint32_t a = __float_as_uint(v[i]), b = __float_as_uint(v[i + HALF]);
        const float send = __uint_as_float((a & up) | (b & ~up));
        const float keep = __uint_as_float((b & up) | (a & ~up));
        v[i] = keep + block_fold_partner<MASK>(send);
    }
}
__device__ __forceinline__ void block_fold16(float* v, int lane) {
    block_fold_step<4, 8>(v, lane);
    block_fold_step<8, 4>(v, lane);
    block_fold_step<16, 2>(v, lane);
    block_fold_step<32, 1>(v, lane);
}
__device__ __forceinline__ int block_fold_index(int lane) {
    return ((lane & 4) ? 8 : 0) + ((lane & 8) ? 4 : 0) + ((lane & 16) ? 2 : 0) + ((lane & 32) ? 1 : 0);
}

typedef short bf16x4_q __attribute__((ext_vector_type(4)));   // four bf16 bit patterns: one matrix operand of a lane

// NM: batch quads (batch <= 4 * NM). Q: row quads a workgroup owns. R: row quads whose loads are in flight per wave.
// OCC: workgroups per CU the register and LDS budgets are cut for.
template <int NM, int Q, int R, int OCC>
__global__ __launch_bounds__(256, OCC) void q4k_gemv_quads_kernel(const uint8_t* __restrict__ w, const float* __restrict__ x,
                                                             float* __restrict__ y, int k, int n, int batch) {
    constexpr int NBATCH = 4 * NM, NVAL = Q * NBATCH, NG = (NVAL + 15) / 16;
    // [NM batch quads][hi, lo][4 batch rows][64 slices][QD_SLICE dwords]; reused for the wave partials at the end
    extern __shared__ __attribute__((aligned(16))) uint32_t xlds[];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int blk = lane >> 2, j = lane & 3;
    // Every workgroup computes exactly Q row quads: rows past N are clamped to the last row and never stored. With no
    // guard around a quad the pass is one straight-line block, and the compiler's wait counts let every load that has
    // been issued stay in flight (any branch around a load makes it wait for all of them at the join).
    const int r0 = blockIdx.x * (4 * Q);
    const int nrows = min(n, r0 + 4 * Q) - r0;
    const int bpr = k >> 8, npass = (bpr + 3) >> 2;
    const int64_t row_bytes = (int64_t)bpr * Q4K_BYTES;
    const int g = blk & 3;
    const int sh = (g & 1) * 16;
    const uint32_t hi_mask = g >= 2 ? 0xFFFFFFFFu : 0u;
    const int q_off = 16 + g * 32;
    // kept out of the optimiser's sight so that (v & mask) | bias stays one three-operand instruction
    uint32_t code_mask = 0x000F000Fu, code_bias = 0x43004300u;
    asm volatile("" : "+v"(code_bias), "+s"(code_mask));

    float acc[Q][NBATCH];
#pragma unroll
    for (int q = 0; q < Q; ++q)
#pragma unroll
        for (int e = 0; e < NBATCH; ++e) acc[q][e] = 0.f;

    // K is taken in rounds of four passes (4096 elements), one pass per wave. A round's activations are fetched once per
    // workgroup with coalesced 16-byte loads, split into bf16 hi / lo and parked in LDS as slices of 64 activations per
    // batch row and part (32 dwords in operand order, padded to QD_SLICE); a lane then reads its own slices.
    const int nrounds = (npass + 3) >> 2;
    for (int round = 0; round < nrounds; ++round) {
        const int pass = round * 4 + wave;
        const int sb = pass * 4 + (blk >> 2);
        const int sb_c = min(sb, bpr - 1);                 // blocks past K re-read a valid super-block against zero activations
        // this lane's weight row of quad q: r0 + 4 q + j, clamped (rows past N are computed and never stored)
        auto row_ptr = [&](int q) { return w + (int64_t)min(r0 + 4 * q + j, n - 1) * row_bytes + (int64_t)sb_c * Q4K_BYTES; };

        // The round's activations are requested first and the first quads' weights right behind them: loads return in
        // issue order, and the (L2-resident) activations must not queue behind the weight stream.
        Q4KRow raw[R];
        {
            float4 xv[NBATCH][4];
#pragma unroll
            for (int b = 0; b < NBATCH; ++b)
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int e = min(round * 4096 + (threadIdx.x + 256 * u) * 4, k - 4);
                    xv[b][u] = *reinterpret_cast<const float4*>(x + (int64_t)min(b, batch - 1) * k + e);
                }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < R; ++i) {
                const uint8_t* p = row_ptr(i < Q ? i : Q - 1);
                raw[i].hdr = *reinterpret_cast<const uint4*>(p);
                raw[i].q0 = *reinterpret_cast<const uint4*>(p + q_off);
                raw[i].q1 = *reinterpret_cast<const uint4*>(p + q_off + 16);
            }
            __builtin_amdgcn_sched_barrier(0);
            __syncthreads();                               // the previous round's slices have been read
            // float4 number f (of 1024) of batch row b: slice f / 16; inside the slice, sub-block (f % 16) / 8 and code
            // dword f % 8, whose four activations e0..e3 go out as the dword pair (e0, e2), (e1, e3) -- the order in
            // which one mask pulls two codes out of a code dword. Rows past the batch and elements past K become
            // zeros through a mask on the packed values (no branch, no product with what was loaded).
            typedef float f32x2_q __attribute__((ext_vector_type(2)));
            typedef __bf16 bf16x2_q __attribute__((ext_vector_type(2)));
#pragma unroll
            for (int b = 0; b < NBATCH; ++b)
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int f = threadIdx.x + 256 * u;
                    const float4 v4 = xv[b][u];
                    const uint32_t live = (round * 4096 + f * 4 < k && b < batch) ? 0xFFFFFFFFu : 0u;
                    const f32x2_q pr[2] = {f32x2_q{v4.x, v4.z}, f32x2_q{v4.y, v4.w}};
                    uint32_t hi[2], lo[2];
#pragma unroll
                    for (int t = 0; t < 2; ++t) {
                        hi[t] = __builtin_bit_cast(uint32_t, __builtin_convertvector(pr[t], bf16x2_q)) & live;
                        const f32x2_q rest = {pr[t].x - __uint_as_float(hi[t] << 16), pr[t].y - __uint_as_float(hi[t] & 0xFFFF0000u)};
                        lo[t] = __builtin_bit_cast(uint32_t, __builtin_convertvector(rest, bf16x2_q)) & live;
                    }
                    const int pos = ((f >> 3) & 1) * 16 + (f & 7) * 2;
                    uint32_t* dst = &xlds[(((b >> 2) * 8 + (b & 3)) * 64 + (f >> 4)) * QD_SLICE + pos];
                    *reinterpret_cast<uint2*>(dst) = make_uint2(hi[0], hi[1]);
                    *reinterpret_cast<uint2*>(dst + 4 * 64 * QD_SLICE) = make_uint2(lo[0], lo[1]);
                }
            __syncthreads();
        }

        // this lane's operand registers: batch row j of every batch quad at this lane's K group, hi then lo part;
        // [0..7] go with the low nibbles of code dwords 0..7, [8..15] with the high nibbles
        bf16x4_q xs[NM][2][16];
#pragma unroll
        for (int nm = 0; nm < NM; ++nm)
#pragma unroll
            for (int part = 0; part < 2; ++part) {
                const uint32_t* src = &xlds[(((nm * 2 + part) * 4 + j) * 64 + wave * 16 + blk) * QD_SLICE];
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const uint4 v4 = *reinterpret_cast<const uint4*>(src + 4 * i);
                    xs[nm][part][2 * i] = __builtin_bit_cast(bf16x4_q, make_uint2(v4.x, v4.y));
                    xs[nm][part][2 * i + 1] = __builtin_bit_cast(bf16x4_q, make_uint2(v4.z, v4.w));
                }
            }
        // 128 * (sum of the batch row's activations, hi + lo) per sub-block, by the same instruction against a constant
        // operand: negated, the start value of every accumulator; divided by 128, the sum the block minimum multiplies
        f32x4_q tl[NM], th[NM];
        float xlo[NBATCH], xhi[NBATCH];
        {
            const bf16x4_q ones = __builtin_bit_cast(bf16x4_q, make_uint2(code_bias, code_bias));
#pragma unroll
            for (int nm = 0; nm < NM; ++nm) {
                tl[nm] = f32x4_q{0.f, 0.f, 0.f, 0.f}; th[nm] = f32x4_q{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int i = 0; i < 8; ++i)
#pragma unroll
                    for (int part = 0; part < 2; ++part) {
                        tl[nm] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(xs[nm][part][i], ones, tl[nm], 0, 0, 0);
                        th[nm] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(xs[nm][part][8 + i], ones, th[nm], 0, 0, 0);
                    }
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    xlo[4 * nm + e] = tl[nm][e] * 0.0078125f;
                    xhi[4 * nm + e] = th[nm][e] * 0.0078125f;
                }
                tl[nm] = -tl[nm]; th[nm] = -th[nm];
            }
        }

#pragma unroll
        for (int q = 0; q < Q; ++q) {
            const Q4KRow& r = raw[q % R];
            float dlo, dhi, mlo, mhi;
            q4k_lane_scales(r.hdr, sh, hi_mask, dlo, dhi, mlo, mhi);
            const uint32_t qw[8] = {r.q0.x, r.q0.y, r.q0.z, r.q0.w, r.q1.x, r.q1.y, r.q1.z, r.q1.w};
            // a batch row's hi and lo parts run through the same accumulator: their sum costs nothing
            f32x4_q dl[NM], dh[NM];
#pragma unroll
            for (int nm = 0; nm < NM; ++nm) { dl[nm] = tl[nm]; dh[nm] = th[nm]; }
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                // codes of bytes (0, 2) and (1, 3) of the dword as bf16 pairs 128 + q: low nibbles, then high nibbles
                const uint32_t v = qw[i];
                const bf16x4_q wl = __builtin_bit_cast(bf16x4_q, make_uint2((v & code_mask) | code_bias, ((v >> 8) & code_mask) | code_bias));
                const bf16x4_q wh = __builtin_bit_cast(bf16x4_q, make_uint2(((v >> 4) & code_mask) | code_bias, ((v >> 12) & code_mask) | code_bias));
#pragma unroll
                for (int part = 0; part < 2; ++part)
#pragma unroll
                    for (int nm = 0; nm < NM; ++nm) {
                        dl[nm] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(xs[nm][part][i], wl, dl[nm], 0, 0, 0);
                        dh[nm] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(xs[nm][part][8 + i], wh, dh[nm], 0, 0, 0);
                    }
            }
            const float nmlo = -mlo, nmhi = -mhi;
#pragma unroll
            for (int nm = 0; nm < NM; ++nm)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float a = acc[q][4 * nm + e];
                    a = fmaf(nmlo, xlo[4 * nm + e], a);
                    a = fmaf(nmhi, xhi[4 * nm + e], a);
                    a = fmaf(dlo, dl[nm][e], a);
                    acc[q][4 * nm + e] = fmaf(dhi, dh[nm][e], a);
                }
            if (q + R < Q) {                           // compile-time: refill with the quad R ahead
                const uint8_t* p = row_ptr(q + R);
                raw[q % R].hdr = *reinterpret_cast<const uint4*>(p);
                raw[q % R].q0 = *reinterpret_cast<const uint4*>(p + q_off);
                raw[q % R].q1 = *reinterpret_cast<const uint4*>(p + q_off + 16);
            }
        }
    }

    // value v = q * NBATCH + (batch row) of a lane, in groups of 16: fold across the blocks, park per wave, total the waves
    __syncthreads();                                       // every wave is done with the activation slices
    float (*part)[NG][64] = reinterpret_cast<float (*)[NG][64]>(xlds);
#pragma unroll
    for (int grp = 0; grp < NG; ++grp) {
        float v[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int vi = grp * 16 + i;
            v[i] = vi < NVAL ? acc[vi / NBATCH][vi % NBATCH] : 0.f;
        }
        block_fold16(v, lane);
        part[wave][grp][lane] = v[0];
    }
    __syncthreads();
    for (int t = threadIdx.x; t < NG * 64; t += 256) {
        const int grp = t >> 6, ln = t & 63;
        const int vi = grp * 16 + block_fold_index(ln);
        const int q = vi / NBATCH, brow = vi % NBATCH, row = r0 + 4 * q + (ln & 3);
        if (vi < NVAL && brow < batch && row < r0 + nrows)
            y[(int64_t)brow * n + row] = part[0][grp][ln] + part[1][grp][ln] + part[2][grp][ln] + part[3][grp][ln];
    }
}


// ---- K = 4096: the same arithmetic fed from an LDS ring that the loads fill directly ----
// The kernel above fetches a lane's header and code bytes into registers: a load instruction then touches about forty
// cache lines for 1 KB, and with three or four quads in flight per wave the weight streams at 2.4 TB/s (batch 4) where
// the one-row kernel, whose wave loads are consecutive kilobytes written straight into LDS, streams at 4.1. Here wave w
// owns K slice w (1024 elements) of every row quad of the workgroup, as in the one-row kernel: a quad's share (4 rows x
// 576 bytes) arrives by three full-wave global_load_lds_dwordx4 (non-temporal, explicit wait counts), W quads ahead, and
// lane 4 * blk + j reads row j's header and the 32 code bytes of group blk from the ring. Sums of G = 16 / (4 NM) quads
// are folded across the 16 blocks right away (16 values per lane), parked per wave, and totalled over the waves at the end.
typedef uint32_t u32x4_qs __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void qs_load16(u32x4_qs& dst, uint32_t off, const void* base) {
    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(dst) : "v"(off), "s"(base) : "memory");
}
__device__ __forceinline__ void qs_stream_to_lds(uint32_t lds_addr, uint32_t off, const uint8_t* base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(lds_addr), "v"(off), "s"(base) : "memory");
}
template <int N> __device__ __forceinline__ void qs_wait_loads() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }
template <int N> __device__ __forceinline__ void qs_wait_loads(u32x4_qs& v) { asm volatile("s_waitcnt vmcnt(%1)" : "+v"(v) : "n"(N) : "memory"); }
__device__ __forceinline__ void qs_wait_lds() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

constexpr int QS_SLOT = 3 * 1024;      // ring bytes of a quad: 144 pieces of 16 bytes in three wave loads
constexpr int QS_XLDS_BYTES = 8 * 64 * QD_SLICE * 4;   // one batch quad's activation slices (hi and lo part)

template <int NM, int W>
__global__ __launch_bounds__(256, 1) void q4k_gemv_quads_stream_kernel(const uint8_t* __restrict__ w, const float* __restrict__ x,
                                                                       float* __restrict__ y, int n, int batch, int qt) {
    constexpr int K = 4096, NBATCH = 4 * NM, G = 16 / NBATCH, NLI = 3;
    extern __shared__ __attribute__((aligned(16))) uint8_t qsmem[];
    uint32_t* xlds = reinterpret_cast<uint32_t*>(qsmem);                 // activation slices
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    uint8_t* ring = qsmem + QS_XLDS_BYTES + wave * (W + 1) * QS_SLOT;
    const int blk = lane >> 2, j = lane & 3, g = blk & 3;
    const int sh = (g & 1) * 16;
    const uint32_t hi_mask = g >= 2 ? 0xFFFFFFFFu : 0u;
    uint32_t code_mask = 0x000F000Fu, code_bias = 0x43004300u;
    asm volatile("" : "+v"(code_bias), "+s"(code_mask));
    const int r0 = blockIdx.x * (4 * qt);
    const uint32_t row_bytes = (K >> 8) * Q4K_BYTES;
    const int ngroups = (qt + G - 1) / G;                                 // uniform

    // activations first (they come from L2 and must not queue behind the weight stream), the first W quads behind them
    u32x4_qs xv[NBATCH][4];
#pragma unroll
    for (int b = 0; b < NBATCH; ++b)
#pragma unroll
        for (int u = 0; u < 4; ++u)
            qs_load16(xv[b][u], (uint32_t)(min(b, batch - 1) * K + (wave * 256 + lane + 64 * u) * 4) * 4u, x);   // the wave's own K slice
    uint32_t loff[NLI];
#pragma unroll
    for (int u = 0; u < NLI; ++u) {
        const uint32_t p = min(64u * u + lane, 143u), row4 = (p * 1821u) >> 16, pc = p - 36u * row4;   // p / 36 for p < 2^12
        loff[u] = row4 * row_bytes + (uint32_t)wave * 576u + pc * 16u;
    }
    const uint32_t max_off = (uint32_t)n * row_bytes - 16u;
    const uint32_t ring_addr = (uint32_t)(size_t)(__attribute__((address_space(3))) uint8_t*)ring;
    const int last_quad = G * ngroups - 1;
    auto issue_quad = [&](int q) {                  // q uniform; quads past the last one re-read it, rows past N the last bytes
        const uint32_t base = (uint32_t)(r0 + 4 * min(q, last_quad)) * row_bytes;
        const uint32_t slot = ring_addr + (uint32_t)(q % (W + 1)) * QS_SLOT;
#pragma unroll
        for (int u = 0; u < NLI; ++u) qs_stream_to_lds(slot + 1024u * u, min(base + loff[u], max_off), w);
    };
#pragma unroll
    for (int q = 0; q < W; ++q) issue_quad(q);
    qs_wait_loads<W * NLI>();
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int b = 0; b < NBATCH; ++b)
#pragma unroll
        for (int u = 0; u < 4; ++u) qs_wait_loads<W * NLI>(xv[b][u]);

    // bf16 hi / lo parts through LDS into operand order, one batch quad at a time (the slices of one fill the region).
    // A wave prepares exactly the 16 slices it multiplies: no other wave touches them, so there is no workgroup barrier
    // (LDS serves a wave's instructions in order; the fences keep the compiler from reordering them).
    typedef float f32x2_q __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2_q __attribute__((ext_vector_type(2)));
    bf16x4_q xs[NM][2][16];
#pragma unroll
    for (int nm = 0; nm < NM; ++nm) {
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
#pragma unroll
        for (int bb = 0; bb < 4; ++bb)
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int b = 4 * nm + bb, f = wave * 256 + lane + 64 * u;
                const u32x4_qs raw4 = xv[b][u];
                const float4 v4 = make_float4(__uint_as_float(raw4.x), __uint_as_float(raw4.y), __uint_as_float(raw4.z), __uint_as_float(raw4.w));
                const uint32_t live = b < batch ? 0xFFFFFFFFu : 0u;
                const f32x2_q pr[2] = {f32x2_q{v4.x, v4.z}, f32x2_q{v4.y, v4.w}};
                uint32_t hi[2], lo[2];
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    hi[t] = __builtin_bit_cast(uint32_t, __builtin_convertvector(pr[t], bf16x2_q)) & live;
                    const f32x2_q rest = {pr[t].x - __uint_as_float(hi[t] << 16), pr[t].y - __uint_as_float(hi[t] & 0xFFFF0000u)};
                    lo[t] = __builtin_bit_cast(uint32_t, __builtin_convertvector(rest, bf16x2_q)) & live;
                }
                const int pos = ((f >> 3) & 1) * 16 + (f & 7) * 2;
                uint32_t* dst = &xlds[(bb * 64 + (f >> 4)) * QD_SLICE + pos];
                *reinterpret_cast<uint2*>(dst) = make_uint2(hi[0], hi[1]);
                *reinterpret_cast<uint2*>(dst + 4 * 64 * QD_SLICE) = make_uint2(lo[0], lo[1]);
            }
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int part = 0; part < 2; ++part) {
            const uint32_t* src = &xlds[((part * 4 + j) * 64 + wave * 16 + blk) * QD_SLICE];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const uint4 v4 = *reinterpret_cast<const uint4*>(src + 4 * i);
                xs[nm][part][2 * i] = __builtin_bit_cast(bf16x4_q, make_uint2(v4.x, v4.y));
                xs[nm][part][2 * i + 1] = __builtin_bit_cast(bf16x4_q, make_uint2(v4.z, v4.w));
            }
        }
    }

    // 128 * (sum of the batch row's activations) per sub-block: negated, the start value of every accumulator; divided
    // by 128, the sum the block minimum multiplies
    f32x4_q tl[NM], th[NM];
    float xlo[NBATCH], xhi[NBATCH];
    {
        const bf16x4_q ones = __builtin_bit_cast(bf16x4_q, make_uint2(code_bias, code_bias));
#pragma unroll
        for (int nm = 0; nm < NM; ++nm) {
            tl[nm] = f32x4_q{0.f, 0.f, 0.f, 0.f}; th[nm] = f32x4_q{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int i = 0; i < 8; ++i)
#pragma unroll
                for (int part = 0; part < 2; ++part) {
                    tl[nm] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(xs[nm][part][i], ones, tl[nm], 0, 0, 0);
                    th[nm] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(xs[nm][part][8 + i], ones, th[nm], 0, 0, 0);
                }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                xlo[4 * nm + e] = tl[nm][e] * 0.0078125f;
                xhi[4 * nm + e] = th[nm][e] * 0.0078125f;
            }
            tl[nm] = -tl[nm]; th[nm] = -th[nm];
        }
    }

    const uint32_t rd_hdr = (uint32_t)(j * 36 + (blk >> 2) * 9) * 16u, rd_q = rd_hdr + 16u + (uint32_t)g * 32u;
    float* parts = reinterpret_cast<float*>(qsmem + QS_XLDS_BYTES + 4 * (W + 1) * QS_SLOT);   // [4 waves][ngroups][64]
    float* part_out = parts + wave * ngroups * 64;
    for (int grp = 0; grp < ngroups; ++grp) {
        float v[16];
#pragma unroll
        for (int i = 0; i < G; ++i) {
            const int q = grp * G + i;
            qs_wait_loads<(W - 1) * NLI>();
            qs_wait_lds();                         // the slot about to be refilled has been read
            issue_quad(q + W);
            const uint8_t* slot = ring + (uint32_t)(q % (W + 1)) * QS_SLOT;
            const uint4 hdr = *reinterpret_cast<const uint4*>(slot + rd_hdr);
            const uint4 q0 = *reinterpret_cast<const uint4*>(slot + rd_q);
            const uint4 q1 = *reinterpret_cast<const uint4*>(slot + rd_q + 16);
            float dlo, dhi, mlo, mhi;
            q4k_lane_scales(hdr, sh, hi_mask, dlo, dhi, mlo, mhi);
            const uint32_t qw[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
            f32x4_q dl[NM], dh[NM];
#pragma unroll
            for (int nm = 0; nm < NM; ++nm) { dl[nm] = tl[nm]; dh[nm] = th[nm]; }
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                const uint32_t cv = qw[c];
                const bf16x4_q wl = __builtin_bit_cast(bf16x4_q, make_uint2((cv & code_mask) | code_bias, ((cv >> 8) & code_mask) | code_bias));
                const bf16x4_q wh = __builtin_bit_cast(bf16x4_q, make_uint2(((cv >> 4) & code_mask) | code_bias, ((cv >> 12) & code_mask) | code_bias));
#pragma unroll
                for (int part = 0; part < 2; ++part)
#pragma unroll
                    for (int nm = 0; nm < NM; ++nm) {
                        dl[nm] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(xs[nm][part][c], wl, dl[nm], 0, 0, 0);
                        dh[nm] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(xs[nm][part][8 + c], wh, dh[nm], 0, 0, 0);
                    }
            }
            const float nmlo = -mlo, nmhi = -mhi;
#pragma unroll
            for (int nm = 0; nm < NM; ++nm)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float a = nmlo * xlo[4 * nm + e];
                    a = fmaf(nmhi, xhi[4 * nm + e], a);
                    a = fmaf(dlo, dl[nm][e], a);
                    v[i * NBATCH + 4 * nm + e] = fmaf(dhi, dh[nm][e], a);
                }
        }
        block_fold16(v, lane);
        part_out[grp * 64 + lane] = v[0];
    }
    qs_wait_loads<0>();                            // the re-reads past the last quad still write the ring
    __syncthreads();
    for (int t = threadIdx.x; t < ngroups * 64; t += 256) {
        const int grp = t >> 6, ln = t & 63;
        const int vi = block_fold_index(ln);                   // which of the group's 16 values this lane holds
        const int q = grp * G + vi / NBATCH, brow = vi % NBATCH, row = r0 + 4 * q + (ln & 3);
        if (q < qt && brow < batch && row < n)
            y[(int64_t)brow * n + row] = (parts[(0 * ngroups + grp) * 64 + ln] + parts[(1 * ngroups + grp) * 64 + ln]) +
                                         (parts[(2 * ngroups + grp) * 64 + ln] + parts[(3 * ngroups + grp) * 64 + ln]);
    }
}

static std::atomic<int> g_quads_stream_enable{1};
void set_q4k_quads_stream_enable(int v) { g_quads_stream_enable = v != 0; }

template <int NM>
static int launch_quads_stream(hipStream_t s, const uint8_t* w, const float* x, float* y, int n, int batch) {
    constexpr int W = 3;
    constexpr size_t smem = (size_t)QS_XLDS_BYTES + (size_t)4 * (W + 1) * QS_SLOT + (size_t)4 * 16 * 64 * sizeof(float);
    const int quads = (n + 3) / 4;
    int qt = (quads + num_cus() - 1) / num_cus();
    if (qt > 32) qt = 32;                          // more rows than one round of workgroups covers: several rounds
    const int grid = (quads + qt - 1) / qt;
    SKH_SET_MAX_DYNAMIC_LDS_ONCE((&q4k_gemv_quads_stream_kernel<NM, W>), smem);
    note_kernel("q4k_gemv_quads_stream_kernel");
    q4k_gemv_quads_stream_kernel<NM, W><<<dim3(grid), dim3(256), smem, s>>>(w, x, y, n, batch, qt);
    SKH_CHECK(hipGetLastError());
    return 1;
}

template <int NM, int Q, int R, int OCC>
static int launch_quads(hipStream_t s, const uint8_t* w, const float* x, float* y, int k, int n, int batch) {
    constexpr size_t smem = (size_t)(8 * NM * 64 * QD_SLICE) * sizeof(uint32_t);
    static_assert(4 * ((Q * 4 * NM + 15) / 16) * 64 <= 8 * NM * 64 * QD_SLICE, "wave partials must fit in the slices");
    SKH_SET_MAX_DYNAMIC_LDS_ONCE((&q4k_gemv_quads_kernel<NM, Q, R, OCC>), smem);
    const int grid = (n + 4 * Q - 1) / (4 * Q);
    note_kernel("q4k_gemv_quads_kernel");
    q4k_gemv_quads_kernel<NM, Q, R, OCC><<<dim3(grid), dim3(256), smem, s>>>(w, x, y, k, n, batch);
    SKH_CHECK(hipGetLastError());
    return 1;
}

// Returns 1 when this kernel took the product, 0 when the shape is outside its range, -1 on a launch error.
int launch_q4k_gemv_wide(const uint8_t* w, const float* x, float* y, int k, int n, int batch);   // gemv_q4k_wide.hip

int launch_q4k_gemv_quads(const uint8_t* w, const float* x, float* y, int k, int n, int batch) {
    if (batch < 3 || batch > 8) return 0;
    // K = 4096: the kernel on the 16 x 16 x 32 matrix instruction
    if (const int rc = launch_q4k_gemv_wide(w, x, y, k, n, batch)) return rc;
    if ((reinterpret_cast<uintptr_t>(w) & 15) || (reinterpret_cast<uintptr_t>(x) & 15) || (k & 255)) return 0;
    hipStream_t s = current_stream();
    // K = 4096 and offsets that fit 32 bits: the kernel that streams the weight through an LDS ring
    if (g_quads_stream_enable && k == 4096 && n >= 4 && (uint64_t)(n + 256) * (uint64_t)(k >> 8) * Q4K_BYTES < ((uint64_t)1 << 32) &&
        (uint64_t)batch * (uint64_t)k * 4u < ((uint64_t)1 << 32))
        return batch <= 4 ? launch_quads_stream<1>(s, w, x, y, n, batch) : launch_quads_stream<2>(s, w, x, y, n, batch);
    // one round of workgroups over the chip where N allows: two per CU owning up to 6 row quads (one batch quad: 74 KB
    // of activation slices), one per CU owning up to 12 (two batch quads); the quad count is a template parameter
    const int occ = batch <= 4 ? 2 : 1;
    const int q = (n + 4 * occ * num_cus() - 1) / (4 * occ * num_cus());
    if (batch <= 4) {
        switch (q) {
            case 1: return launch_quads<1, 1, 1, 2>(s, w, x, y, k, n, batch);
            case 2: return launch_quads<1, 2, 2, 2>(s, w, x, y, k, n, batch);
            case 3: return launch_quads<1, 3, 3, 2>(s, w, x, y, k, n, batch);
            case 4: return launch_quads<1, 4, 4, 2>(s, w, x, y, k, n, batch);
            case 5: return launch_quads<1, 5, 4, 2>(s, w, x, y, k, n, batch);
            default: return launch_quads<1, 6, 4, 2>(s, w, x, y, k, n, batch);
        }
    }
    if (q <= 2) return launch_quads<2, 2, 2, 1>(s, w, x, y, k, n, batch);
    if (q <= 4) return launch_quads<2, 4, 4, 1>(s, w, x, y, k, n, batch);
    if (q <= 6) return launch_quads<2, 6, 6, 1>(s, w, x, y, k, n, batch);
    if (q <= 8) return launch_quads<2, 8, 6, 1>(s, w, x, y, k, n, batch);
    return launch_quads<2, 12, 6, 1>(s, w, x, y, k, n, batch);
}

}  // namespace skh
