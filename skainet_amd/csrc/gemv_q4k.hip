// Q4_K dequant-GEMV, decode shape (1 or 2 activation rows), canonical row-major GGUF weight.
//
//   y[b, o] = sum_j x[b, j] * dequant(W[o, j]),   W[o, j] = code * (d * sc) - dmin * m  per 32-element sub-block
//
// Same products as the reference's exact-fp32 kernel, other summation order
//   /root/reference/skainet-backends/skainet-backend-cpu/src/commonMain/kotlin/sk/ainet/exec/kernel/ScalarQ4_KMatmulKernel.kt:40-78
// (per sub-block: codeSum * (d * sc) - inputSum * (dmin * m)); weight addressing (o * blocksPerRow + b) * 144 as in
//   /root/reference/skainet-backends/skainet-backend-native-cpu/native/src/q4k_matmul.c:294-309.
//
// HBM-bound design (algorithmic bytes = 144 B per 256 weights + 4 B per activation / output element):
//   * One wave owns a contiguous range of output rows and walks K in passes of 16 super-blocks (4096 elements).
//     Lane l owns 32-byte nibble group g = l % 4 of super-block l / 4 of the pass: 64 weights (sub-blocks 2g and
//     2g + 1) whose 64 activations it keeps in registers for all of its rows. A row costs the lane two 16-byte
//     loads of quants and one of the block header; across the wave these are one contiguous 2304-byte span.
//   * The four waves of a workgroup work on the same K pass, so the pass's 4096 activations are fetched once per
//     workgroup with coalesced 16-byte loads, parked in LDS (one padded 64-float slice per lane) and read back by
//     each lane into registers. Weights never touch LDS. Per-row partial sums stay in registers across passes and
//     are folded across the 64 lanes once, at the end, with a multi-value butterfly.
//   * R rows are in flight per wave (loads issued before the arithmetic of the previous rows), rows are spread
//     evenly over all waves of the chip by the host.
//   * Optional fusions, so a decoder block needs no separate row kernels around its products:
//       prologue RMSNorm  y = W . (x * gain / sqrt(mean(x^2) + eps)): every workgroup stages all of x anyway, so it
//                         sums the squares while staging x * gain and scales its outputs at the end;
//       epilogue residual y = residual + W . x  (residual may alias y);
//       epilogue SwiGLU   out[j] = silu(y[2j]) * y[2j + 1] for a weight whose rows alternate gate row, up row;
//       epilogue RoPE     the rows are one token's [q | k | v]: adjacent pairs of q and k rotated by the device-side
//                         position, q written head-major, k and v written into their KV-cache rows.
#include "gemv_q4k.h"

namespace skh {

int launch_q4k_gemv_mfma(const uint8_t* w, const float* x, float* y, int k, int n, const float* gain, float eps,
                         const float* residual, int epilogue, const RopeQkvEpilogue* rope_in,
                         const AttnMergePrologue* merge);   // gemv_q4k_mfma.hip

// One row's 64 weights of a lane against its 64 activations. The 4-bit codes are never converted: a dword of codes is
// masked into pairs of 16-bit fields whose low mantissa bits hold a code (0x000F000F: the low nibbles of bytes 0 and 2;
// 0x00F000F0: their high nibbles, i.e. 16 * code; the same on the dword shifted right by 8 for bytes 1 and 3). Read as
// fp16 such a field is the subnormal code * 2^-24 (or 16 * code * 2^-24), which v_fma_mix_f32 widens to fp32 exactly on
// its way into an fp32 FMA -- five mask / shift operations per eight weights instead of eight conversions, and the
// products and sums are the same fp32 values as with converted codes (the powers of two go into the block scales).
typedef _Float16 q4k_h2 __attribute__((ext_vector_type(2)));
template <int B>
__device__ __forceinline__ void q4k_row_dot(const Q4KRow& r, int sh, uint32_t hi_mask, const float (*x)[64],
                                            const float (*xsum)[2], float* out) {
    float dlo, dhi, mlo, mhi;
    q4k_lane_scales(r.hdr, sh, hi_mask, dlo, dhi, mlo, mhi);
    dlo *= 16777216.0f;                                        // codes enter as code * 2^-24
    dhi *= 1048576.0f;                                         // high nibbles as 16 * code * 2^-24
    const uint32_t q[8] = {r.q0.x, r.q0.y, r.q0.z, r.q0.w, r.q1.x, r.q1.y, r.q1.z, r.q1.w};
    float lo[B], hi[B];
#pragma unroll
    for (int b = 0; b < B; ++b) lo[b] = hi[b] = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const uint32_t q8 = q[i] >> 8;
        const q4k_h2 l02 = __builtin_bit_cast(q4k_h2, q[i] & 0x000F000Fu), h02 = __builtin_bit_cast(q4k_h2, q[i] & 0x00F000F0u);
        const q4k_h2 l13 = __builtin_bit_cast(q4k_h2, q8 & 0x000F000Fu), h13 = __builtin_bit_cast(q4k_h2, q8 & 0x00F000F0u);
#pragma unroll
        for (int b = 0; b < B; ++b) {
            lo[b] = fmaf((float)l02.x, x[b][i * 4 + 0], lo[b]);
            hi[b] = fmaf((float)h02.x, x[b][32 + i * 4 + 0], hi[b]);
            lo[b] = fmaf((float)l13.x, x[b][i * 4 + 1], lo[b]);
            hi[b] = fmaf((float)h13.x, x[b][32 + i * 4 + 1], hi[b]);
            lo[b] = fmaf((float)l02.y, x[b][i * 4 + 2], lo[b]);
            hi[b] = fmaf((float)h02.y, x[b][32 + i * 4 + 2], hi[b]);
            lo[b] = fmaf((float)l13.y, x[b][i * 4 + 3], lo[b]);
            hi[b] = fmaf((float)h13.y, x[b][32 + i * 4 + 3], hi[b]);
        }
    }
#pragma unroll
    for (int b = 0; b < B; ++b) out[b] += dlo * lo[b] + dhi * hi[b] - (mlo * xsum[b][0] + mhi * xsum[b][1]);
}

// Epilogue of a chunk: after the fold lane l < 16 B holds the total of row `row` (of the chunk that starts at output
// row r0) for activation row b. Plain store, `+ residual`, SwiGLU over adjacent (gate, up) rows, or RoPE + scatter of
// one token's [q | k | v] rows.
//
// What the epilogue reads besides the sum -- the residual element, the token position, the (cos, sin) pair -- is
// requested by q4k_epilogue_prefetch at the start of the chunk, ahead of the weight stream: read where it is used it would
// be one more memory round trip at the very end of the kernel.
struct Q4KEpiloguePrefetch { float residual; int pos; float2 cs; };
template <int B>
__device__ __forceinline__ Q4KEpiloguePrefetch q4k_epilogue_prefetch(int lane, int r0, int nrows, int n, const float* x,
                                                                       const float* residual, int epilogue,
                                                                       const RopeQkvEpilogue& rope) {
    constexpr int NV = 16 * B;
    const int idx = wave_fold_index<NV>(lane), row = idx / B, b = idx % B;
    const bool live = lane < NV && row < nrows;
    // lanes (and epilogues) without such an operand read the first activations instead: no branch around a load
    const float* rp = (epilogue == EPI_RESIDUAL && live) ? residual + ((int64_t)b * n + r0 + row) : x;
    const bool rot = epilogue == EPI_ROPE_QKV && live;
    const int32_t* pp = rot ? rope.pos_dev : reinterpret_cast<const int32_t*>(x);
    const int dd = (r0 + row) % max(rope.head_dim, 1);
    const float2* tp = (rot && rope.table) ? rope.table + (dd >> 1) : reinterpret_cast<const float2*>(x);
    Q4KEpiloguePrefetch pre;
    pre.residual = *rp; pre.pos = *pp; pre.cs = *tp;
    return pre;
}
template <int B>
__device__ __forceinline__ void q4k_rows_epilogue(float val, int lane, int row, int b, int r0, int nrows, int n, float* y,
                                                  int epilogue, const RopeQkvEpilogue& rope, const Q4KEpiloguePrefetch& pre) {
    constexpr int NV = 16 * B;
    if (epilogue == EPI_ROPE_QKV) {
        // rows 2i and 2i + 1 of a head are one rotation pair; like the SwiGLU pairs they sit B lanes apart (lane = row * B + b)
        const float odd = __shfl_xor(val, B, 64);
        if (lane < NV && !(row & 1) && row < nrows) {
            const int o = r0 + row, slot = o / rope.head_dim, dd = o % rope.head_dim;
            const int p0 = pre.pos;
            float2 out2 = make_float2(val, odd);
            if (slot < rope.heads + rope.kv_heads) {
                float sn, cs;
                if (rope.table) { cs = pre.cs.x; sn = pre.cs.y; }
                else sincosf((float)p0 * powf(rope.theta, -(float)dd / (float)rope.head_dim), &sn, &cs);
                out2 = rope_rotate(val, odd, cs, sn);
            }
            const bool in_cache = p0 >= 0 && p0 < rope.capacity;   // a device-side position past the cache writes no K / V row
            float* dst;
            if (slot < rope.heads) dst = y + (int64_t)slot * rope.head_dim;
            else if (slot < rope.heads + rope.kv_heads) dst = rope.k_cache + ((int64_t)(slot - rope.heads) * rope.capacity + p0) * rope.head_dim;
            else dst = rope.v_cache + ((int64_t)(slot - rope.heads - rope.kv_heads) * rope.capacity + p0) * rope.head_dim;
            if (slot < rope.heads || in_cache) *reinterpret_cast<float2*>(dst + dd) = out2;
        }
    } else if (epilogue == EPI_SWIGLU) {
        // rows 2j (gate) and 2j + 1 (up) of this wave sit B lanes apart after the fold (lane = row * B + b)
        const float up = __shfl_xor(val, B, 64);
        if (lane < NV && !(row & 1) && row < nrows) y[(int64_t)b * (n >> 1) + ((r0 + row) >> 1)] = val * (1.0f / (1.0f + expf(-val))) * up;
    } else if (lane < NV && row < nrows) {
        const int64_t o = (int64_t)b * n + r0 + row;
        if (epilogue == EPI_RESIDUAL) val += pre.residual;
        y[o] = val;
    }
}

// Two workgroups per CU is the occupancy the register budget is cut for (the row loads in flight, the pass's
// activations and the per-row sums all live in registers); asking for more makes the compiler spill.
//
// NR, the rows a wave owns per chunk, is a template parameter and every wave computes exactly NR rows per chunk (rows
// past N are clamped to the last row and never stored): a pass is then one straight-line block without a guard
// around any load. With a run-time row count every load sits behind a (uniform) branch, and at the join after a
// branch the compiler's wait-count bookkeeping makes the wave wait for loads it has only just issued -- the rows meant
// to be in flight together were fetched one round trip after the other.
template <int B, int R, int NR, int PRO>
__global__ __launch_bounds__(256, 2) void q4k_gemv_rows_kernel(const uint8_t* __restrict__ w, const float* __restrict__ x,
                                                            float* y, int k, int n, int nchunks,
                                                            const float* __restrict__ gain, float eps, const float* residual,
                                                            int epilogue, RopeQkvEpilogue rope) {
    constexpr int NV = 16 * B;   // Q4K_RMAX rows padded to 16, times B
    constexpr int SLICE = 68;    // 64 activations + 4 floats of padding: 16-byte aligned and bank-conflict free
    static_assert(NR >= 1 && NR <= Q4K_RMAX, "rows per chunk");
    __shared__ __attribute__((aligned(16))) float xlds[B][64 * SLICE];
    __shared__ __attribute__((aligned(16))) float ssq_rows[B][16];   // squares of x summed per 16-lane row (RMSNorm prologue)
    const int lane = threadIdx.x & 63;
    // readfirstlane: the wave index is uniform across a wave, and saying so keeps the row addresses scalar
    const int gw = __builtin_amdgcn_readfirstlane(blockIdx.x * 4 + (threadIdx.x >> 6));
    const int wave_r0 = gw * (NR * nchunks);
    const int bpr = k >> 8;
    const int64_t row_bytes = (int64_t)bpr * Q4K_BYTES;
    const int g = lane & 3;
    const int sh = (g & 1) * 16;
    const uint32_t hi_mask = g >= 2 ? 0xFFFFFFFFu : 0u;
    const int q_off = 16 + g * 32;

    float ssq[B], xscale[B];
#pragma unroll
    for (int b = 0; b < B; ++b) { ssq[b] = 0.f; xscale[b] = 1.0f; }

    for (int c0 = 0; c0 < nchunks; ++c0) {
        const int r0 = wave_r0 + c0 * NR;
        const int nrows = max(0, min(n - r0, NR));               // rows of this chunk that exist (the rest are clamped copies)
        const float first = c0 == 0 ? 1.0f : 0.0f;               // the squares are summed during the first chunk only
        const Q4KEpiloguePrefetch pre = q4k_epilogue_prefetch<B>(lane, r0, nrows, n, x, residual, epilogue, rope);

        float acc[16][B];
#pragma unroll
        for (int i = 0; i < 16; ++i)
#pragma unroll
            for (int b = 0; b < B; ++b) acc[i][b] = 0.f;

        for (int blk0 = 0; blk0 < bpr; blk0 += 16) {
            const int blk = blk0 + (lane >> 2);
            const int blk_c = min(blk, bpr - 1);            // lanes past K re-read a valid block and multiply it by zero activations
            auto row_ptr = [&](int i) { return w + (int64_t)min(r0 + i, n - 1) * row_bytes + (int64_t)blk_c * Q4K_BYTES; };

            // This pass's activations are requested first, the first R rows of weights right behind them: loads return in
            // the order they were issued, so the (L2-resident) activations must not queue behind the weight stream --
            // the arithmetic can then start on the first row while the later rows are still arriving.
            // float4 number f of the pass goes to LDS slice f / 16, position f % 16. All loads are issued unconditionally
            // (clamped address, zeroed afterwards) so they overlap.
            float4 xv[B][4], gv[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int e = min(blk0 * 256 + (threadIdx.x + 256 * j) * 4, k - 4);
#pragma unroll
                for (int b = 0; b < B; ++b) xv[b][j] = *reinterpret_cast<const float4*>(x + (int64_t)b * k + e);
                if (PRO) gv[j] = *reinterpret_cast<const float4*>(gain + e);
            }
            __builtin_amdgcn_sched_barrier(0);
            Q4KRow raw[R];
#pragma unroll
            for (int i = 0; i < R; ++i) {
                const uint8_t* p = row_ptr(i < NR ? i : NR - 1);
                raw[i].hdr = *reinterpret_cast<const uint4*>(p);
                raw[i].q0 = *reinterpret_cast<const uint4*>(p + q_off);
                raw[i].q1 = *reinterpret_cast<const uint4*>(p + q_off + 16);
            }
            __builtin_amdgcn_sched_barrier(0);
            __syncthreads();                                // the previous pass's slices have been read
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int f = threadIdx.x + 256 * j;
                const float inside = blk0 * 256 + f * 4 < k ? 1.0f : 0.0f;
#pragma unroll
                for (int b = 0; b < B; ++b) {
                    float4 v4 = xv[b][j];
                    v4.x *= inside; v4.y *= inside; v4.z *= inside; v4.w *= inside;
                    if (PRO) {
                        ssq[b] = fmaf(first, fmaf(v4.x, v4.x, fmaf(v4.y, v4.y, fmaf(v4.z, v4.z, v4.w * v4.w))), ssq[b]);
                        v4.x *= gv[j].x; v4.y *= gv[j].y; v4.z *= gv[j].z; v4.w *= gv[j].w;
                    }
                    *reinterpret_cast<float4*>(&xlds[b][(f >> 4) * SLICE + (f & 15) * 4]) = v4;
                }
            }
            // RMSNorm prologue: once the last pass of the first chunk is staged every thread has its share of the squares.
            // Row sums go to LDS in front of the barrier the staging needs anyway, the total is read behind it -- all in
            // the shadow of the weight loads that are still on their way.
            const bool ssq_done = PRO && c0 == 0 && blk0 + 16 >= bpr;   // uniform
            if (ssq_done) {
#pragma unroll
                for (int b = 0; b < B; ++b) {
                    const float t = row16_sum(ssq[b]);
                    if ((lane & 15) == 0) ssq_rows[b][threadIdx.x >> 4] = t;
                }
            }
            __syncthreads();
            if (ssq_done) {
#pragma unroll
                for (int b = 0; b < B; ++b) {
                    float t = 0.f;
#pragma unroll
                    for (int i = 0; i < 16; i += 4) {
                        const float4 r4 = *reinterpret_cast<const float4*>(&ssq_rows[b][i]);
                        t += (r4.x + r4.y) + (r4.z + r4.w);
                    }
                    xscale[b] = 1.0f / sqrtf(t * (1.0f / (float)k) + eps);
                }
            }

            float xs[B][64], xsum[B][2];
#pragma unroll
            for (int b = 0; b < B; ++b) {
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const float4 v4 = *reinterpret_cast<const float4*>(&xlds[b][lane * SLICE + i * 4]);   // zeros past K
                    xs[b][4 * i] = v4.x; xs[b][4 * i + 1] = v4.y; xs[b][4 * i + 2] = v4.z; xs[b][4 * i + 3] = v4.w;
                }
                float s0 = 0.f, s1 = 0.f;
#pragma unroll
                for (int i = 0; i < 32; ++i) { s0 += xs[b][i]; s1 += xs[b][32 + i]; }
                xsum[b][0] = s0; xsum[b][1] = s1;
            }

#pragma unroll
            for (int c = 0; c < NR; ++c) {
                q4k_row_dot<B>(raw[c % R], sh, hi_mask, xs, xsum, acc[c]);
                if (c + R < NR) {                               // compile-time: refill with the row R ahead
                    const uint8_t* p = row_ptr(c + R);
                    raw[c % R].hdr = *reinterpret_cast<const uint4*>(p);
                    raw[c % R].q0 = *reinterpret_cast<const uint4*>(p + q_off);
                    raw[c % R].q1 = *reinterpret_cast<const uint4*>(p + q_off + 16);
                }
                __builtin_amdgcn_sched_barrier(0);              // a refill is issued where it is written, not later
            }
        }

        float v[NV];
#pragma unroll
        for (int i = 0; i < 16; ++i)
#pragma unroll
            for (int b = 0; b < B; ++b) v[i * B + b] = acc[i][b];
        wave_fold<NV>(v, lane);
        const int idx = wave_fold_index<NV>(lane);
        const int row = idx / B, b = idx % B;
        float val = v[0] * (B == 1 ? xscale[0] : (b == 0 ? xscale[0] : xscale[B - 1]));
        q4k_rows_epilogue<B>(val, lane, row, b, r0, nrows, n, y, epilogue, rope, pre);
    }
}

// Long rows, few of them (the down projection: 4096 rows of 14336): with the shape above a wave would own two rows and
// walk K in several passes, each with its staging barriers, and every workgroup would stage all of x for eight rows.
// Here the four waves of a workgroup own the same NR rows and a quarter of K each: a wave stages only its own quarter,
// through its own LDS region, so the pass loop has no workgroup barrier and (for K <= 16384) a single pass per wave
// with all NR rows streaming behind one staging; the four partial sums per row meet in LDS at the end.
template <int R, int NR>
__global__ __launch_bounds__(256, 2) void q4k_gemv_ksplit_kernel(const uint8_t* __restrict__ w, const float* __restrict__ x,
                                                              float* y, int k, int n, const float* residual, int epilogue) {
    constexpr int NV = 16, SLICE = 68;
    static_assert(NR >= 1 && NR <= Q4K_RMAX && R <= NR, "rows per workgroup");
    __shared__ __attribute__((aligned(16))) float xlds[4][64 * SLICE];
    __shared__ float part[4][NV];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r0 = blockIdx.x * NR;
    const int nrows = min(n - r0, NR);
    const int bpr = k >> 8;
    const int bpw = (bpr + 3) >> 2;                              // super-blocks of a row per wave
    const int wb0 = wave * bpw, wb1 = min(bpr, wb0 + bpw);
    const int64_t row_bytes = (int64_t)bpr * Q4K_BYTES;
    const int g = lane & 3;
    const int sh = (g & 1) * 16;
    const uint32_t hi_mask = g >= 2 ? 0xFFFFFFFFu : 0u;
    const int q_off = 16 + g * 32;
    float* xw = &xlds[wave][0];

    // the residual element a lane will add at the end, requested ahead of the weight stream (a valid address either way)
    const int e_row = wave_fold_index<NV>(lane);
    const float res_pre = *((epilogue == EPI_RESIDUAL && lane < NV && e_row < nrows) ? residual + r0 + e_row : x);

    float acc[16][1];
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i][0] = 0.f;

    for (int blk0 = wb0; blk0 < wb1; blk0 += 16) {
        const int blk_c = min(blk0 + (lane >> 2), wb1 - 1);     // lanes past the quarter re-read a valid block against zero activations
        auto row_ptr = [&](int i) { return w + (int64_t)min(r0 + i, n - 1) * row_bytes + (int64_t)blk_c * Q4K_BYTES; };
        // the pass's activations first (coalesced: float4 number f = lane + 64 j), the first R rows right behind them
        float4 xv[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) xv[j] = *reinterpret_cast<const float4*>(x + min(blk0 * 256 + (lane + 64 * j) * 4, k - 4));
        __builtin_amdgcn_sched_barrier(0);
        Q4KRow raw[R];
#pragma unroll
        for (int i = 0; i < R; ++i) {
            const uint8_t* p = row_ptr(i);
            raw[i].hdr = *reinterpret_cast<const uint4*>(p);
            raw[i].q0 = *reinterpret_cast<const uint4*>(p + q_off);
            raw[i].q1 = *reinterpret_cast<const uint4*>(p + q_off + 16);
        }
        __builtin_amdgcn_sched_barrier(0);
        // through the wave's own LDS region into one 64-float slice per lane; a wave's LDS accesses complete in order,
        // so the region needs no barrier
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const int f = lane + 64 * j;
            const float inside = blk0 * 256 + f * 4 < wb1 * 256 ? 1.0f : 0.0f;
            float4 v4 = xv[j];
            v4.x *= inside; v4.y *= inside; v4.z *= inside; v4.w *= inside;
            *reinterpret_cast<float4*>(&xw[(f >> 4) * SLICE + (f & 15) * 4]) = v4;
        }
        float xs[1][64], xsum[1][2];
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const float4 v4 = *reinterpret_cast<const float4*>(&xw[lane * SLICE + i * 4]);
            xs[0][4 * i] = v4.x; xs[0][4 * i + 1] = v4.y; xs[0][4 * i + 2] = v4.z; xs[0][4 * i + 3] = v4.w;
        }
        float s0 = 0.f, s1 = 0.f;
#pragma unroll
        for (int i = 0; i < 32; ++i) { s0 += xs[0][i]; s1 += xs[0][32 + i]; }
        xsum[0][0] = s0; xsum[0][1] = s1;

#pragma unroll
        for (int c = 0; c < NR; ++c) {
            q4k_row_dot<1>(raw[c % R], sh, hi_mask, xs, xsum, acc[c]);
            if (c + R < NR) {                                   // compile-time: refill with the row R ahead
                const uint8_t* p = row_ptr(c + R);
                raw[c % R].hdr = *reinterpret_cast<const uint4*>(p);
                raw[c % R].q0 = *reinterpret_cast<const uint4*>(p + q_off);
                raw[c % R].q1 = *reinterpret_cast<const uint4*>(p + q_off + 16);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    float v[NV];
#pragma unroll
    for (int i = 0; i < 16; ++i) v[i] = acc[i][0];
    wave_fold<NV>(v, lane);
    if (lane < NV) part[wave][lane] = v[0];
    __syncthreads();
    if (wave == 0 && lane < NV) {
        if (e_row < nrows) {
            float val = (part[0][lane] + part[1][lane]) + (part[2][lane] + part[3][lane]);
            if (epilogue == EPI_RESIDUAL) val += res_pre;
            y[r0 + e_row] = val;
        }
    }
}

static std::atomic<int> g_q4k_rows_waves_per_cu{0};   // 0: chosen from K (below)
void set_q4k_rows_waves_per_cu(int v) { if (v >= 0) g_q4k_rows_waves_per_cu = v; }
int q4k_rows_waves_per_cu() { return g_q4k_rows_waves_per_cu; }
static std::atomic<int> g_q4k_ksplit_enable{1};      // 0: long rows take the plain row shape too
void set_q4k_ksplit_enable(int v) { g_q4k_ksplit_enable = v; }

template <int B, int R, int NR>
static void launch_rows(bool pro, int grid, hipStream_t s, const uint8_t* w, const float* x, float* y, int k, int n, int nchunks,
                        const float* gain, float eps, const float* residual, int epilogue, const RopeQkvEpilogue& rope) {
    note_kernel("q4k_gemv_rows_kernel");
    if (pro) q4k_gemv_rows_kernel<B, R, NR, 1><<<dim3(grid), dim3(256), 0, s>>>(w, x, y, k, n, nchunks, gain, eps, residual, epilogue, rope);
    else q4k_gemv_rows_kernel<B, R, NR, 0><<<dim3(grid), dim3(256), 0, s>>>(w, x, y, k, n, nchunks, gain, eps, residual, epilogue, rope);
}
template <int B, int R>
static void launch_rows_nr(int nr, bool pro, int grid, hipStream_t s, const uint8_t* w, const float* x, float* y, int k, int n,
                           int nchunks, const float* gain, float eps, const float* residual, int epilogue, const RopeQkvEpilogue& rope) {
#define SKH_NR_CASE(N) case N: launch_rows<B, (R < N ? R : N), N>(pro, grid, s, w, x, y, k, n, nchunks, gain, eps, residual, epilogue, rope); break;
    switch (nr) {
        SKH_NR_CASE(1) SKH_NR_CASE(2) SKH_NR_CASE(3) SKH_NR_CASE(4) SKH_NR_CASE(5) SKH_NR_CASE(6)
        SKH_NR_CASE(7) SKH_NR_CASE(8) SKH_NR_CASE(9) SKH_NR_CASE(10) SKH_NR_CASE(11) SKH_NR_CASE(12)
    }
#undef SKH_NR_CASE
}

// Returns 1 when this kernel took the product, 0 when the shape is outside its range (caller falls back to the
// slot kernel), -1 on a launch error.
// y = epilogue(W . prologue(x)); gain != null selects the RMSNorm prologue, epilogue is one of EPI_*.
int launch_q4k_gemv_rows_fused(const uint8_t* w, const float* x, float* y, int k, int n, int batch, const float* gain, float eps,
                               const float* residual, int epilogue, const RopeQkvEpilogue* rope_in) {
    if (batch < 1 || batch > 2) return 0;
    if (epilogue < EPI_NONE || epilogue > EPI_ROPE_QKV) return set_error("q4k gemv: unknown epilogue %d", epilogue);
    RopeQkvEpilogue rope{};
    if (epilogue == EPI_ROPE_QKV) {
        if (!rope_in || batch != 1) return 0;
        rope = *rope_in;
        if ((rope.head_dim & 1) || n != (rope.heads + 2 * rope.kv_heads) * rope.head_dim) return 0;
    }
    if ((reinterpret_cast<uintptr_t>(w) & 15) || (reinterpret_cast<uintptr_t>(x) & 15) || (k & 3)) return 0;
    if (gain && (reinterpret_cast<uintptr_t>(gain) & 15)) return 0;
    if (batch == 1) {
        // one activation row with K in whole slices of 1024: the matrix-core kernel with consecutive-kilobyte loads
        const int r = launch_q4k_gemv_mfma(w, x, y, k, n, gain, eps, residual, epilogue, epilogue == EPI_ROPE_QKV ? &rope : nullptr, nullptr);
        if (r != 0) return r;
    }
    if (g_q4k_ksplit_enable && batch == 1 && !gain && epilogue <= EPI_RESIDUAL && k >= 8192) {
        // long rows: K over the four waves of a workgroup when the plain shape would leave a wave three rows or fewer
        const int nr = (n + 2 * num_cus() - 1) / (2 * num_cus());
        if (nr >= 4 && nr <= Q4K_RMAX && (n + num_cus() * 8 - 1) / (num_cus() * 8) <= 3) {
            const int grid = (n + nr - 1) / nr;
            hipStream_t s = current_stream();
            note_kernel("q4k_gemv_ksplit_kernel");
#define SKH_KS_CASE(N) case N: q4k_gemv_ksplit_kernel<(6 < N ? 6 : N), N><<<dim3(grid), dim3(256), 0, s>>>(w, x, y, k, n, residual, epilogue); break;
            switch (nr) {
                SKH_KS_CASE(4) SKH_KS_CASE(5) SKH_KS_CASE(6) SKH_KS_CASE(7) SKH_KS_CASE(8) SKH_KS_CASE(9)
                SKH_KS_CASE(10) SKH_KS_CASE(11) SKH_KS_CASE(12)
            }
#undef SKH_KS_CASE
            SKH_CHECK(hipGetLastError());
            return 1;
        }
    }
    const bool pairs = epilogue >= EPI_SWIGLU;                   // a (gate, up) or rotation pair never straddles two waves
    if (pairs && (n & 1)) return 0;
    // one round of workgroups over the chip: a wave's rows, taken in equal chunks of at most Q4K_RMAX (the chunk size
    // is a template parameter, so the share is rounded up to a whole number of chunks)
    // (more waves per CU when that keeps a wave's share in one chunk: a second chunk stages the activations again)
    // Measured (2 to 16 waves per CU): a lone product with K of one pass (<= 4096) is fastest at one workgroup per CU
    // -- a wave stages the activations once for up to 12 rows (11008 x 4096: 7.9 us against 8.2 at 8 waves). With
    // several passes the staging and its barriers repeat per pass and a second workgroup per CU hides them (4096 x
    // 14336: 11.7 us at 8 waves against 12.2 at 4), and inside the decoder's chain of fused launches 8 waves measured
    // 0.6 % faster per token than 4 although each launch alone prefers 4.
    const bool lone = !gain && epilogue == EPI_NONE;
    int waves_per_cu = g_q4k_rows_waves_per_cu.load() > 0 ? g_q4k_rows_waves_per_cu.load() : (lone && k <= 4096 ? 4 : 8);
    while (waves_per_cu < 32 && (n + num_cus() * waves_per_cu - 1) / (num_cus() * waves_per_cu) > Q4K_RMAX) waves_per_cu += 4;
    const int total_waves = num_cus() * waves_per_cu;
    const int share = (n + total_waves - 1) / total_waves;
    const int nchunks = (share + Q4K_RMAX - 1) / Q4K_RMAX;
    int nr = (share + nchunks - 1) / nchunks;
    if (pairs) nr = (nr + 1) & ~1;
    const int rows_per_wave = nr * nchunks;
    const int waves = (n + rows_per_wave - 1) / rows_per_wave;
    const int grid = (waves + 3) / 4;
    hipStream_t s = current_stream();
    if (batch == 1) launch_rows_nr<1, 6>(nr, gain != nullptr, grid, s, w, x, y, k, n, nchunks, gain, eps, residual, epilogue, rope);
    else launch_rows_nr<2, 2>(nr, gain != nullptr, grid, s, w, x, y, k, n, nchunks, gain, eps, residual, epilogue, rope);
    SKH_CHECK(hipGetLastError());
    return 1;
}

int launch_q4k_gemv_rows(const uint8_t* w, const float* x, float* y, int k, int n, int batch) {
    return launch_q4k_gemv_rows_fused(w, x, y, k, n, batch, nullptr, 0.f, nullptr, EPI_NONE, nullptr);
}

}  // namespace skh
