// Q8_0 dequant-GEMV for one activation row on the integer matrix cores, canonical row-major GGUF weight, K <= 4096.
//
//   y[o] = sum_b d[o, b] * sum_{j in block b} x[j] * q[o, j],   blocks of 32 int8 codes behind an fp16 scale (34 bytes)
//
// Same products as the reference's exact-fp32 kernel up to a 22-bit fixed-point rounding of the activations
//   /root/reference/skainet-backends/skainet-backend-cpu/src/commonMain/kotlin/sk/ainet/exec/kernel/ScalarQ8_0MatmulKernel.kt:23-65
// (the reference's own native kernel rounds the activations to 8 bits per block, native/src/q8_0_matmul.c).
//
// The int8 codes are the matrix instruction's operand type as they lie in the block: there is no decode at all. The
// kernel is the one-row Q4_K kernel's data path and arithmetic (gemv_q4k_mfma.hip) on this format's geometry:
//   * the four waves of a workgroup split K in slices of 1024 elements (32 blocks = 1088 bytes of a row, one slice per
//     wave); a wave's share of a row quad (4 rows x 1088 bytes = 272 pieces of 16 bytes) is fetched with full-wave
//     non-temporal loads that write straight into LDS (global_load_lds_dwordx4; the fifth load of a quad on 16 lanes), W
//     quads ahead of the one being computed, inline assembly with explicit wait counts;
//   * lane 4 * blk + j reads from LDS the two blocks (68 bytes, dword aligned) of row j of the quad that make up the
//     64-element group blk of the slice; the second block's codes are dwords as they lie, the first block's are re-aligned
//     by two bytes (v_alignbyte_b32);
//   * the dot products run on v_mfma_i32_4x4x4_16b_i8: B operand four codes of the lane's row, A operand four bytes of
//     one plane of the activations of its group -- 22-bit fixed point against the group's largest magnitude, split into
//     balanced base-256 digits (planes: low digit, middle digit, top digit + 64, ones; the ones plane yields the code sum
//     that takes the + 64 out). One accumulator per block. The top digit's sum and the two low digits' sum are converted
//     to fp32 separately (together they can exceed 32 bits with 8-bit codes) and scaled by d;
//   * a group whose activations are not all finite poisons its partial sums with NaN, as the fp32 product would.
#include "gemv_q4k.h"

namespace skh {

typedef uint32_t q8m_u32x4 __attribute__((ext_vector_type(4)));
typedef int q8m_i32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void q8m_plain_load16(q8m_u32x4& dst, uint32_t off, const void* base) {
    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(dst) : "v"(off), "s"(base) : "memory");
}
__device__ __forceinline__ void q8m_stream_to_lds(uint32_t lds_addr, uint32_t off, const uint8_t* base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(lds_addr), "v"(off), "s"(base) : "memory");
}
template <int N> __device__ __forceinline__ void q8m_wait_loads() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }
template <int N> __device__ __forceinline__ void q8m_wait_loads(q8m_u32x4& v) { asm volatile("s_waitcnt vmcnt(%1)" : "+v"(v) : "n"(N) : "memory"); }
__device__ __forceinline__ void q8m_wait_lds() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

constexpr int Q8M_SLICE = 32 * Q80_BYTES;              // 1088 bytes: a row's 1024-element slice
constexpr int Q8M_QUAD = 4 * Q8M_SLICE;                // 4352 bytes = 272 pieces of 16: four full wave loads and one of 16 lanes
constexpr int Q8M_NLI = 5;
constexpr int Q8M_XROW = 20;                           // dwords per (group, plane) row of 16 operand dwords, padded against bank conflicts
constexpr int Q8M_XA_BYTES = 16 * 4 * Q8M_XROW * 4 + 16 * 4;   // operand planes of 16 groups + a scale per group
constexpr int Q8M_MAX_QUADS = 32;                      // row quads per workgroup
__host__ __device__ constexpr uint32_t q8m_ring_bytes(int window) { return (uint32_t)window * Q8M_QUAD + Q8M_XA_BYTES; }   // the planes' staging area behind the W slots

// W: quads in flight per wave (the ring has W slots: a slot is refilled once its quad is used up)
template <int W>
__global__ __launch_bounds__(256, W == 1 ? 4 : W == 2 ? 2 : 1) void q8_0_gemv_mfma_kernel(const uint8_t* __restrict__ w, const float* __restrict__ x,
                                                                float* __restrict__ y, int k, int n, int qt) {
    extern __shared__ __attribute__((aligned(16))) uint8_t q8m_smem[];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int blk = lane >> 2, j = lane & 3;
    const int nsl = k >> 10;                                   // slices of 1024 elements, at most 4
    uint8_t* ring = q8m_smem + wave * q8m_ring_bytes(W);
    uint8_t* xa_stage = ring + W * Q8M_QUAD;
    float* partials_all = reinterpret_cast<float*>(q8m_smem + 4 * q8m_ring_bytes(W));   // [4 slices of K][qt][64]
    float* partials = partials_all + wave * qt * 64;
    const int r0 = blockIdx.x * (4 * qt);
    const int nq = min(qt, (n - r0 + 3) / 4);                  // this workgroup's quads (uniform, at least one)
    const uint32_t row_bytes = (uint32_t)(k >> 5) * (uint32_t)Q80_BYTES;

    if (wave < nsl) {
        // activations of this wave's slice first, the first W quads right behind them
        q8m_u32x4 xq[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) q8m_plain_load16(xq[i], (uint32_t)(wave * 1024 + (i * 64 + lane) * 4) * 4u, x);
        uint32_t loff[Q8M_NLI];
#pragma unroll
        for (int u = 0; u < Q8M_NLI; ++u) {
            const uint32_t p = min(64u * u + lane, 271u), row4 = (p * 964u) >> 16, pc = p - 68u * row4;   // p / 68 for p < 272
            loff[u] = row4 * row_bytes + (uint32_t)wave * Q8M_SLICE + pc * 16u;
        }
        const uint32_t max_off = (uint32_t)n * row_bytes - 16u;                // rows past the weight: the last bytes, never stored
        const uint32_t ring_addr = (uint32_t)(size_t)(__attribute__((address_space(3))) uint8_t*)ring;
        auto issue_quad = [&](int q) {                                         // q uniform, < nq
            const uint32_t base = (uint32_t)(r0 + 4 * q) * row_bytes;
            const uint32_t slot = ring_addr + (uint32_t)(q % W) * Q8M_QUAD;
#pragma unroll
            for (int u = 0; u < 4; ++u) q8m_stream_to_lds(slot + 1024u * u, min(base + loff[u], max_off), w);
            if (lane < 16) q8m_stream_to_lds(slot + 4096u, min(base + loff[4], max_off), w);
        };
        // The wait counts below assume exactly W * 5 weight loads behind the activations: a workgroup with fewer quads
        // makes up the count with loads of the (cached) activations into the unused slots.
#pragma unroll
        for (int q = 0; q < W; ++q) {
            if (q < nq) issue_quad(q);
            else {
#pragma unroll
                for (int u = 0; u < Q8M_NLI; ++u) q8m_stream_to_lds(ring_addr + (uint32_t)q * Q8M_QUAD + 1024u * (u < 4 ? u : 0), 16u * lane, reinterpret_cast<const uint8_t*>(x));
            }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) q8m_wait_loads<W * Q8M_NLI>(xq[i]);

        // Activation planes: float4 number f = i * 64 + lane of the slice belongs to group f / 16 (the 16 lanes of a DPP
        // row share a group). x * inv + 1.5 * 2^23 + 0x8080 carries, in its three low bytes, the balanced base-256 digits
        // of round(x * inv) (top digit + 64); the planes go through LDS into operand order. The largest magnitude is
        // taken on the bit patterns (unsigned order = magnitude order, and an infinity or a NaN is larger than every
        // finite value): a group that holds one gets a NaN scale.
        uint32_t* xa_lds = reinterpret_cast<uint32_t*>(xa_stage);
        float* xs_lds = reinterpret_cast<float*>(xa_stage + 16 * 4 * Q8M_XROW * 4);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float4 v = make_float4(__uint_as_float(xq[i].x), __uint_as_float(xq[i].y), __uint_as_float(xq[i].z), __uint_as_float(xq[i].w));
            const int G = i * 4 + (lane >> 4), tt = lane & 15;
            const uint32_t abits = max(max(xq[i].x & 0x7FFFFFFFu, xq[i].y & 0x7FFFFFFFu), max(xq[i].z & 0x7FFFFFFFu, xq[i].w & 0x7FFFFFFFu));
            const float amax = row16_max(__uint_as_float(abits));      // (fmaxf drops a NaN: the bit patterns below catch it)
            const uint32_t worst = __float_as_uint(row16_max(__uint_as_float(min(abits, 0x7F800000u))));   // clamped to +inf: ordered, never a NaN
            const float inv = 2097151.0f * __builtin_amdgcn_rcpf(fmaxf(amax, 1e-30f));
            const uint32_t b0 = __float_as_uint(fmaf(v.x, inv, 12615808.0f)), b1 = __float_as_uint(fmaf(v.y, inv, 12615808.0f));
            const uint32_t b2 = __float_as_uint(fmaf(v.z, inv, 12615808.0f)), b3 = __float_as_uint(fmaf(v.w, inv, 12615808.0f));
            const uint32_t a = __builtin_amdgcn_perm(b1, b0, 0x05010400u), b = __builtin_amdgcn_perm(b3, b2, 0x05010400u);
            const uint32_t c = __builtin_amdgcn_perm(b1, b0, 0x07030602u), d = __builtin_amdgcn_perm(b3, b2, 0x07030602u);
            uint32_t* dst = xa_lds + G * 4 * Q8M_XROW + tt;
            dst[0] = __builtin_amdgcn_perm(b, a, 0x05040100u) ^ 0x80808080u;
            dst[Q8M_XROW] = __builtin_amdgcn_perm(b, a, 0x07060302u) ^ 0x80808080u;
            dst[2 * Q8M_XROW] = __builtin_amdgcn_perm(d, c, 0x05040100u);
            dst[3 * Q8M_XROW] = 0x01010101u;
            if (tt == 0) xs_lds[G] = worst >= 0x7F800000u ? __uint_as_float(0x7FC00000u) : amax * (1.0f / 2097151.0f);
        }
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
        __builtin_amdgcn_wave_barrier();
        int xa[16];
        {
            const uint4* src = reinterpret_cast<const uint4*>(xa_lds + (blk * 4 + j) * Q8M_XROW);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint4 v4 = src[e];
                xa[4 * e] = (int)v4.x; xa[4 * e + 1] = (int)v4.y; xa[4 * e + 2] = (int)v4.z; xa[4 * e + 3] = (int)v4.w;
            }
        }
        const float s_grp = xs_lds[blk];

        // lane's two blocks inside a quad slot: 17 dwords at row j, group blk
        const uint32_t rd = (uint32_t)j * Q8M_SLICE + (uint32_t)blk * 68u;
        const int widx = j * 16 + blk;
        for (int q = 0; q < nq; ++q) {
            // quad q has landed when at most the loads of the quads requested after it are in flight
            const int behind = min(nq - 1 - q, W - 1);
            if (behind >= 3) q8m_wait_loads<15>();
            else if (behind == 2) q8m_wait_loads<10>();
            else if (behind == 1) q8m_wait_loads<5>();
            else q8m_wait_loads<0>();
            const uint32_t* src = reinterpret_cast<const uint32_t*>(ring + (uint32_t)(q % W) * Q8M_QUAD + rd);
            uint32_t dw[17];
#pragma unroll
            for (int i = 0; i < 17; ++i) dw[i] = src[i];
            const float d0 = half_bits_to_float_fast(dw[0] & 0xFFFFu), d1 = half_bits_to_float_fast(dw[8] >> 16);
            q8m_i32x4 a0 = {0, 0, 0, 0}, a1 = {0, 0, 0, 0};
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int w0 = (int)__builtin_amdgcn_alignbyte(dw[u + 1], dw[u], 2);        // codes 4 u .. 4 u + 3 of the first block
                a0 = __builtin_amdgcn_mfma_i32_4x4x4i8(xa[u], w0, a0, 0, 0, 0);
                a1 = __builtin_amdgcn_mfma_i32_4x4x4i8(xa[8 + u], (int)dw[9 + u], a1, 0, 0, 0);
            }
            // digits back together: (top - 64 * code sum) * 65536 + (mid * 256 + low); the halves go to fp32 apart
            const float t0 = fmaf((float)(a0[2] - 64 * a0[3]), 65536.0f, (float)(a0[1] * 256 + a0[0]));
            const float t1 = fmaf((float)(a1[2] - 64 * a1[3]), 65536.0f, (float)(a1[1] * 256 + a1[0]));
            partials[q * 64 + widx] = s_grp * fmaf(d0, t0, d1 * t1);
            if (q + W < nq) {
                q8m_wait_lds();                        // this quad's slot has been read: refill it
                issue_quad(q + W);
            }
        }
    } else {
        for (int i = lane; i < nq * 64; i += 64) partials[i] = 0.f;            // K below four slices: this wave has none
    }
    __syncthreads();
    // one output row per 16 threads and round: a row's 16 groups x 4 slices are one float4 per thread, a DPP row sum
    const int u = threadIdx.x & 15, pw = u >> 2, pp = u & 3;
    for (int it = 0; it * 16 < 4 * nq; ++it) {
        const int rl = it * 16 + (threadIdx.x >> 4);
        const int rlc = min(rl, 4 * nq - 1);
        const float4 p4 = *reinterpret_cast<const float4*>(partials_all + (pw * qt + (rlc >> 2)) * 64 + (rlc & 3) * 16 + pp * 4);
        const float val = row16_sum((p4.x + p4.y) + (p4.z + p4.w));
        const int row = r0 + rl;
        if (u == 0 && rl < 4 * nq && row < n) y[row] = val;
    }
}

static std::atomic<int> g_q8_0_mfma_enable{1};
void set_q8_0_mfma_enable(int v) { g_q8_0_mfma_enable = v != 0; }
static std::atomic<int> g_q8_0_mfma_per_cu{2};      // workgroups per CU the grid is cut for (4096 x 4096, us per product: 1: 5.33, 2: 4.96, 3: 4.91 with one quad in flight, 4: 5.51)
void set_q8_0_mfma_per_cu(int v) { if (v >= 1 && v <= 4) g_q8_0_mfma_per_cu = v; }

template <int W>
static int launch_q8m(int grid, int qt, hipStream_t s, const uint8_t* w, const float* x, float* y, int k, int n) {
    const size_t smem = (size_t)4 * q8m_ring_bytes(W) + (size_t)4 * qt * 64 * sizeof(float);
    SKH_SET_MAX_DYNAMIC_LDS_ONCE((&q8_0_gemv_mfma_kernel<W>), 160 * 1024);
    if (smem > 160 * 1024) return 0;
    note_kernel("q8_0_gemv_mfma_kernel");
    q8_0_gemv_mfma_kernel<W><<<dim3(grid), dim3(256), smem, s>>>(w, x, y, k, n, qt);
    SKH_CHECK(hipGetLastError());
    return 1;
}

// Returns 1 when this kernel took the product, 0 when the shape is outside its range, -1 on a launch error. One
// activation row; K a multiple of 1024 up to 4096; the weight below 4 GiB; operands 16-byte aligned.
int launch_q8_0_gemv_mfma(const uint8_t* w, const float* x, float* y, int k, int n) {
    if (!g_q8_0_mfma_enable.load() || k < 1024 || (k & 1023) || k > 4096 || n < 1) return 0;
    if ((uint64_t)(n + 4) * (uint64_t)(k >> 5) * Q80_BYTES >= ((uint64_t)1 << 32)) return 0;
    if ((reinterpret_cast<uintptr_t>(w) & 15) || (reinterpret_cast<uintptr_t>(x) & 15)) return 0;
    const int quads = (n + 3) / 4;
    const int per_cu = g_q8_0_mfma_per_cu.load();
    int qt = (quads + per_cu * num_cus() - 1) / (per_cu * num_cus());
    if (qt > Q8M_MAX_QUADS) qt = Q8M_MAX_QUADS;
    const int grid = (quads + qt - 1) / qt;
    if (per_cu >= 3 && qt <= 4) return launch_q8m<1>(grid, qt, current_stream(), w, x, y, k, n);
    if (per_cu == 2 && qt <= 8) return launch_q8m<2>(grid, qt, current_stream(), w, x, y, k, n);
    return launch_q8m<4>(grid, qt, current_stream(), w, x, y, k, n);
}

}  // namespace skh
