// Q4_K dequant-GEMV for 3 to 8 activation rows on the fp32 matrix instruction, canonical row-major GGUF weight.
//
//   y[b, o] = sum_j x[b, j] * dequant(W[o, j])     exact fp32 products and sums, like the one-row kernel
//
// Same products as the reference's exact-fp32 kernel, other summation order
//   /root/reference/skainet-backends/skainet-backend-cpu/src/commonMain/kotlin/sk/ainet/exec/kernel/ScalarQ4_KMatmulKernel.kt:40-78
//
// With one activation row a weight costs a conversion and an FMA per lane; with eight rows it would cost eight FMAs
// and the kernel would be bound by the vector ALU, not by HBM. v_mfma_f32_4x4x1_16b_f32 multiplies, in each of its 16
// independent blocks of four lanes, the four A values of the block with its four B values: a lane's converted weight
// meets four activation rows in one instruction, at the full fp32 matrix rate and with fp32 operands.
//   * Lane l = 4 * blk + j. As B operand it supplies the weight of output row j of the wave's current row quad; as A
//     operand the activation of batch row j; both at the K position of block blk. The four result registers of lane
//     4 * blk + j are batch rows 0..3 against output row j.
//   * Block blk owns one 32-byte nibble group (64 weights: sub-blocks 2g and 2g + 1) of every super-block quartet, so
//     a wave covers 1024 consecutive K elements ("pass") and a lane keeps its 64 activations per batch quad in
//     registers for all the row quads of the workgroup. Per row quad a lane loads its row's block header and its 32
//     bytes of codes: across the wave, four spans of 576 contiguous bytes.
//   * The four waves of a workgroup take the passes round-robin (K = 4096: one pass each) and all walk the same row
//     quads; per-lane sums are folded across the 16 blocks with a multi-value butterfly and across the waves in LDS.
#include "gemv_q4k.h"

namespace skh {

typedef float f32x4_q __attribute__((ext_vector_type(4)));
constexpr int QD_SLICE = 68;   // 64 activations + 4 floats of padding: 16-byte aligned, bank-conflict free


// Fold 16 per-lane values across the 16 four-lane blocks of a wave (lane bits 2..5), leaving bits 0..1 apart: on
// return v[0] of lane l is the total, over the lanes with the same l % 4, of value block_fold_index(l).
__device__ __forceinline__ void block_fold16(float* v, int lane) {
    int mask = 4;
#pragma unroll
    for (int nv = 16; nv > 1; nv >>= 1, mask <<= 1) {
        const int half = nv >> 1;
        const uint32_t up = (lane & mask) ? 0xFFFFFFFFu : 0u;
#pragma unroll
        for (int i = 0; i < half; ++i) {
            const uint32_t a = __float_as_uint(v[i]), b = __float_as_uint(v[i + half]);
            const float send = __uint_as_float((a & up) | (b & ~up));
            const float keep = __uint_as_float((b & up) | (a & ~up));
            v[i] = keep + __shfl_xor(send, mask, 64);
        }
    }
}
__device__ __forceinline__ int block_fold_index(int lane) {
    return ((lane & 4) ? 8 : 0) + ((lane & 8) ? 4 : 0) + ((lane & 16) ? 2 : 0) + ((lane & 32) ? 1 : 0);
}

// NB: batch quads (batch <= 4 * NB). Q: row quads a workgroup owns. R: row quads whose loads are in flight per wave.
// OCC: workgroups per CU the register budget is cut for (two batch quads keep 128 activations per lane: one per CU).
template <int NB, int Q, int R, int OCC>
__global__ __launch_bounds__(256, OCC) void q4k_gemv_quads_kernel(const uint8_t* __restrict__ w, const float* __restrict__ x,
                                                             float* __restrict__ y, int k, int n, int batch) {
    constexpr int NVAL = Q * 4 * NB, NG = (NVAL + 15) / 16;
    extern __shared__ __attribute__((aligned(16))) float xlds[];   // [4 NB batch rows][64 slices][QD_SLICE]; then the wave partials
    float (*part)[NG][64] = reinterpret_cast<float (*)[NG][64]>(xlds + 4 * NB * 64 * QD_SLICE);
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

    float acc[Q][4 * NB];
#pragma unroll
    for (int q = 0; q < Q; ++q)
#pragma unroll
        for (int e = 0; e < 4 * NB; ++e) acc[q][e] = 0.f;

    // K is taken in rounds of four passes (4096 elements), one pass per wave. A round's activations are fetched once per
    // workgroup with coalesced 16-byte loads and parked in LDS as 64-float slices (one per batch row and K group,
    // padded to 68 floats so the lanes' 16-byte reads spread over the banks); a lane then reads its own slices.
    const int nrounds = (npass + 3) >> 2;
    for (int round = 0; round < nrounds; ++round) {
        const int pass = round * 4 + wave;
        const int sb = pass * 4 + (blk >> 2);
        const bool inside = sb < bpr;
        const int sb_c = min(sb, bpr - 1);                 // blocks past K re-read a valid super-block against zero activations
        // this lane's weight row of quad q: r0 + 4 q + j, clamped (rows past N are computed and never stored)
        auto row_ptr = [&](int q) { return w + (int64_t)min(r0 + 4 * q + j, n - 1) * row_bytes + (int64_t)sb_c * Q4K_BYTES; };

        // The round's activations are requested first and the first quads' weights right behind them: loads return in
        // issue order, and the (L2-resident) activations must not queue behind the weight stream.
        // float4 number f (of 1024) of batch row b goes to slice f / 16 of that row, position f % 16.
        Q4KRow raw[R];
        {
            float4 xv[4 * NB][4];
#pragma unroll
            for (int b = 0; b < 4 * NB; ++b)
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
#pragma unroll
            for (int b = 0; b < 4 * NB; ++b)
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int f = threadIdx.x + 256 * u;
                    float4 v4 = xv[b][u];
                    if (round * 4096 + f * 4 >= k || b >= batch) v4 = make_float4(0.f, 0.f, 0.f, 0.f);
                    *reinterpret_cast<float4*>(&xlds[(b * 64 + (f >> 4)) * QD_SLICE + (f & 15) * 4]) = v4;
                }
            __syncthreads();
        }

        // the 64 activations of this lane's K group, for batch rows j and (NB = 2) 4 + j
        float xs[NB][64], xlo[NB][4], xhi[NB][4];
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            const float* src = &xlds[((nb * 4 + j) * 64 + wave * 16 + blk) * QD_SLICE];
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const float4 v4 = *reinterpret_cast<const float4*>(src + 4 * i);
                xs[nb][4 * i] = v4.x; xs[nb][4 * i + 1] = v4.y; xs[nb][4 * i + 2] = v4.z; xs[nb][4 * i + 3] = v4.w;
            }
            float s0 = 0.f, s1 = 0.f;
#pragma unroll
            for (int i = 0; i < 32; ++i) { s0 += xs[nb][i]; s1 += xs[nb][32 + i]; }
            // the sub-block sums of all four batch rows of the block (a lane holds its own row's)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                xlo[nb][e] = __shfl(s0, (lane & ~3) + e, 64);
                xhi[nb][e] = __shfl(s1, (lane & ~3) + e, 64);
            }
        }
        (void)inside;

#pragma unroll
        for (int q = 0; q < Q; ++q) {
            {
                const Q4KRow& r = raw[q % R];
                float dlo, dhi, mlo, mhi;
                q4k_lane_scales(r.hdr, sh, hi_mask, dlo, dhi, mlo, mhi);
                dhi *= 0.0625f;                            // high nibbles enter as 16 * code
                const uint32_t qw[8] = {r.q0.x, r.q0.y, r.q0.z, r.q0.w, r.q1.x, r.q1.y, r.q1.z, r.q1.w};
                // NCH independent accumulation chains per sub-block and batch quad
                constexpr int NCH = 2;
                f32x4_q dlc[NB][NCH], dhc[NB][NCH];
#pragma unroll
                for (int nb = 0; nb < NB; ++nb)
#pragma unroll
                    for (int c = 0; c < NCH; ++c) { dlc[nb][c] = f32x4_q{0.f, 0.f, 0.f, 0.f}; dhc[nb][c] = f32x4_q{0.f, 0.f, 0.f, 0.f}; }
                // The conversions are plain C so the compiler sees the vector-ALU write of every matrix-instruction
                // operand (an operand written by the instruction just before needs wait states, which the compiler
                // cannot insert for inline assembly: the matrix instruction then reads the register's old value).
                // The empty asm emits nothing: it hides the nibble masks from the optimiser, which otherwise turns
                // each byte conversion into a bit-field extract plus a conversion instead of one v_cvt_f32_ubyteN.
                // Program order is pinned so that the conversions of code dword i + 1 sit between the matrix
                // instructions of dword i: each operand is written a dword ahead of its use.
                float cl[2][4], ch[2][4];
                auto convert = [&](int set, int t, uint32_t l4, uint32_t h4) __attribute__((always_inline)) {
                    cl[set][t] = t == 0 ? (float)(l4 & 0xFFu) : t == 1 ? (float)((l4 >> 8) & 0xFFu) : t == 2 ? (float)((l4 >> 16) & 0xFFu) : (float)(l4 >> 24);
                    ch[set][t] = t == 0 ? (float)(h4 & 0xFFu) : t == 1 ? (float)((h4 >> 8) & 0xFFu) : t == 2 ? (float)((h4 >> 16) & 0xFFu) : (float)(h4 >> 24);
                };
                uint32_t l4 = qw[0] & 0x0F0F0F0Fu, h4 = qw[0] & 0xF0F0F0F0u;
                asm volatile("" : "+v"(l4), "+v"(h4));
#pragma unroll
                for (int t = 0; t < 4; ++t) convert(0, t, l4, h4);
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    if (i < 7) {
                        l4 = qw[i + 1] & 0x0F0F0F0Fu; h4 = qw[i + 1] & 0xF0F0F0F0u;
                        asm volatile("" : "+v"(l4), "+v"(h4));
                    }
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
#pragma unroll
                        for (int nb = 0; nb < NB; ++nb) {
                            dlc[nb][t % NCH] = __builtin_amdgcn_mfma_f32_4x4x1f32(xs[nb][i * 4 + t], cl[i & 1][t], dlc[nb][t % NCH], 0, 0, 0);
                            dhc[nb][t % NCH] = __builtin_amdgcn_mfma_f32_4x4x1f32(xs[nb][32 + i * 4 + t], ch[i & 1][t], dhc[nb][t % NCH], 0, 0, 0);
                        }
                        if (i < 7) convert((i + 1) & 1, t, l4, h4);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
                f32x4_q dl[NB], dh[NB];
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) {
                    dl[nb] = dlc[nb][0]; dh[nb] = dhc[nb][0];
#pragma unroll
                    for (int c = 1; c < NCH; ++c) { dl[nb] += dlc[nb][c]; dh[nb] += dhc[nb][c]; }
                }
#pragma unroll
                for (int nb = 0; nb < NB; ++nb)
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        acc[q][nb * 4 + e] += dlo * dl[nb][e] + dhi * dh[nb][e] - (mlo * xlo[nb][e] + mhi * xhi[nb][e]);
                if (q + R < Q) {                           // compile-time: refill with the quad R ahead
                    const uint8_t* p = row_ptr(q + R);
                    raw[q % R].hdr = *reinterpret_cast<const uint4*>(p);
                    raw[q % R].q0 = *reinterpret_cast<const uint4*>(p + q_off);
                    raw[q % R].q1 = *reinterpret_cast<const uint4*>(p + q_off + 16);
                }
            }
        }
    }

    // value v = q * 4 NB + (batch row) of a lane, in groups of 16: fold across the blocks, park per wave, total the waves
    const int fidx = block_fold_index(lane);
#pragma unroll
    for (int grp = 0; grp < NG; ++grp) {
        float v[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int vi = grp * 16 + i;
            v[i] = vi < NVAL ? acc[vi / (4 * NB)][vi % (4 * NB)] : 0.f;
        }
        block_fold16(v, lane);
        part[wave][grp][lane] = v[0];
    }
    __syncthreads();
    for (int t = threadIdx.x; t < NG * 64; t += 256) {
        const int grp = t >> 6, ln = t & 63;
        const int vi = grp * 16 + block_fold_index(ln);
        const int q = vi / (4 * NB), brow = vi % (4 * NB), row = r0 + 4 * q + (ln & 3);
        if (vi < NVAL && brow < batch && row < r0 + nrows)
            y[(int64_t)brow * n + row] = part[0][grp][ln] + part[1][grp][ln] + part[2][grp][ln] + part[3][grp][ln];
    }
    (void)fidx;
}

template <int NB, int Q, int R, int OCC>
static int launch_quads(hipStream_t s, const uint8_t* w, const float* x, float* y, int k, int n, int batch) {
    constexpr size_t smem = (size_t)(4 * NB * 64 * QD_SLICE + 4 * ((Q * 4 * NB + 15) / 16) * 64) * sizeof(float);
    static bool attr_set = false;
    if (!attr_set) {
        SKH_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&q4k_gemv_quads_kernel<NB, Q, R, OCC>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        attr_set = true;
    }
    const int grid = (n + 4 * Q - 1) / (4 * Q);
    q4k_gemv_quads_kernel<NB, Q, R, OCC><<<dim3(grid), dim3(256), smem, s>>>(w, x, y, k, n, batch);
    SKH_CHECK(hipGetLastError());
    return 1;
}

// Returns 1 when this kernel took the product, 0 when the shape is outside its range, -1 on a launch error.
int launch_q4k_gemv_quads(const uint8_t* w, const float* x, float* y, int k, int n, int batch) {
    if (batch < 3 || batch > 8) return 0;
    if ((reinterpret_cast<uintptr_t>(w) & 15) || (reinterpret_cast<uintptr_t>(x) & 15) || (k & 255)) return 0;
    hipStream_t s = current_stream();
    // one round of workgroups over the chip where N allows: two per CU owning up to 6 row quads (one batch quad), one
    // per CU owning up to 12 (two batch quads); the quad count is a template parameter
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
    if (q <= 6) return launch_quads<2, 6, 4, 1>(s, w, x, y, k, n, batch);
    if (q <= 8) return launch_quads<2, 8, 4, 1>(s, w, x, y, k, n, batch);
    return launch_quads<2, 12, 4, 1>(s, w, x, y, k, n, batch);
}

}  // namespace skh
