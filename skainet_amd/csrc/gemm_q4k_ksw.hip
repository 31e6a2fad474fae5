// Q4_K dequant-GEMM with K split over the waves of a workgroup:  C[m, n] = sum_k A[m, k] * dequant(W[n, k])
//   A bf16 [M, K] (the fp32 activations rounded once by the pass in front, gemm.hip), W packed Q4_K in canonical
//   row-major GGUF order, products bf16 x bf16 on v_mfma_f32_32x32x16_bf16, fp32 accumulation, C fp32 [M, N].
//
// Same contract and arithmetic as dequant_gemm_kernel (gemm.hip): a weight is code * (d * sc) - dmin * m in fp32 (one
// fused multiply-add), rounded to bf16 (nearest even). What differs is who owns what:
//   * workgroup tile 128 (M) x 64 (N): 512 x 4096 outputs are 256 tiles, one per CU, so the chip is full without
//     splitting K across workgroups (no partial tiles parked in memory, no launch that sums them);
//   * every wave owns the WHOLE tile (4 x 2 MFMA tiles of 32 x 32: 128 accumulator registers, each fragment read from
//     LDS feeds two or four matrix instructions) and a quarter of K: in every 64-element step wave w takes the
//     16-element slice w. The four partial tiles meet once, at the end, through LDS;
//   * a 16-element slice of a Q4_K row is one nibble plane (low for slices 0 and 1, high for 2 and 3) of 16 consecutive
//     bytes, and lane (column n, half h) of the matrix instruction's B operand needs 8 of them: so a lane decodes exactly
//     the 8 weights of each of its two columns that its own operand holds, straight into registers. Decoded weights never
//     pass through LDS and nothing is decoded twice. The raw super-blocks (144 bytes per row and 256 elements) are copied
//     into LDS once per four steps with plain coalesced 16-byte loads, so the lanes' 8-byte picks come out of LDS, not out
//     of the cache hierarchy;
//   * the activation tile of a step (128 rows x 64 elements, bf16) goes global -> registers -> LDS as in the other
//     kernel, parked two steps ahead of its use (three LDS stages), so that a step's fragments are read while the
//     previous step multiplies; one barrier per step. A step's weights are decoded during the previous step as well:
//     between the 8 matrix instructions of a step sit, in pinned program order, the reads, the parking and the decode
//     for the steps behind it.
#include "common.h"

#include <type_traits>

namespace skh {

typedef __bf16 ksw_bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 ksw_bf16x2 __attribute__((ext_vector_type(2)));
typedef float ksw_f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t ksw_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t ksw_u32x2 __attribute__((ext_vector_type(2)));

constexpr int KSW_M = 128, KSW_N = 64, KSW_K = 64;
constexpr int KSW_ASTRIDE = KSW_K + 8;                        // bf16 elements per LDS row of the activation tile (144 bytes)
constexpr int KSW_A_BYTES = KSW_M * KSW_ASTRIDE * 2;          // one stage of the activation tile
constexpr int KSW_W_BYTES = 768 * 16;                         // one stage of raw super-blocks: 64 rows x 144 bytes = 576 pieces of 16
                                                              // bytes, padded to three pieces per thread (the padding takes copies)
constexpr int KSW_RED_PITCH = KSW_N + 4;                      // floats per row of a partial tile in the final exchange
constexpr size_t KSW_LOOP_BYTES = 4 * (size_t)KSW_A_BYTES + 2 * (size_t)KSW_W_BYTES;
constexpr size_t KSW_RED_BYTES = (size_t)4 * KSW_M * KSW_RED_PITCH * sizeof(float);
constexpr size_t KSW_SMEM = KSW_RED_BYTES > KSW_LOOP_BYTES ? KSW_RED_BYTES : KSW_LOOP_BYTES;

// The eight 6-bit scales and minima of a super-block header (ggml get_scale_min_k4) as bytes of four dwords: low four
// sub-blocks, high four sub-blocks, each for scales and minima. `pre` shifts a wave's own sub-blocks (even or odd ones:
// the low or the high nibble plane) into bytes 0 and 2.
struct KswScales { float d, dmin; uint32_t sc_lo, sc_hi, mn_lo, mn_hi; };
__device__ __forceinline__ KswScales ksw_unpack(const ksw_u32x4& hdr, int pre, float nib_scale) {
    KswScales r;
    r.d = half_bits_to_float_fast(hdr.x & 0xFFFFu) * nib_scale;
    r.dmin = half_bits_to_float_fast(hdr.x >> 16);
    r.sc_lo = (hdr.y & 0x3F3F3F3Fu) >> pre;
    r.mn_lo = (hdr.z & 0x3F3F3F3Fu) >> pre;
    r.sc_hi = ((hdr.w & 0x0F0F0F0Fu) | ((hdr.y >> 2) & 0x30303030u)) >> pre;
    r.mn_hi = (((hdr.w >> 4) & 0x0F0F0F0Fu) | ((hdr.z >> 2) & 0x30303030u)) >> pre;
    return r;
}
// d * sc and dmin * m of the wave's sub-block in step P (0..3) of the super-block
template <int P>
__device__ __forceinline__ void ksw_step_scale(const KswScales& k, float& scale, float& offset) {
    const uint32_t sc = P < 2 ? k.sc_lo : k.sc_hi, mn = P < 2 ? k.mn_lo : k.mn_hi;
    scale = k.d * ((P & 1) ? ubyte2_to_float(sc) : ubyte0_to_float(sc));
    offset = k.dmin * ((P & 1) ? ubyte2_to_float(mn) : ubyte0_to_float(mn));
}
// four codes of one masked dword (low nibbles, or high nibbles left in place: 16 x code, the 1/16 is in the scale)
__device__ __forceinline__ void ksw_decode4(uint32_t c, float scale, float offset, uint32_t& lo, uint32_t& hi) {
    const float w0 = fmaf(ubyte0_to_float(c), scale, -offset), w1 = fmaf(ubyte1_to_float(c), scale, -offset);
    const float w2 = fmaf(ubyte2_to_float(c), scale, -offset), w3 = fmaf(ubyte3_to_float(c), scale, -offset);
    lo = __builtin_bit_cast(uint32_t, ksw_bf16x2{(__bf16)w0, (__bf16)w1});
    hi = __builtin_bit_cast(uint32_t, ksw_bf16x2{(__bf16)w2, (__bf16)w3});
}

constexpr int KSW_STAGES = 4;                                 // activation stages: parked two steps ahead of their use; four, so
                                                              // that a step's stages are compile-time constants (step % 4)

__global__ __launch_bounds__(256) void q4k_gemm_ksw_kernel(const __bf16* __restrict__ a, const uint8_t* __restrict__ w,
                                                           float* __restrict__ c, int m, int n, int k) {
    extern __shared__ __attribute__((aligned(16))) uint8_t ksw_smem[];
    auto a_stage = [&](int s) { return reinterpret_cast<__bf16*>(ksw_smem + s * KSW_A_BYTES); };
    auto w_stage = [&](int s) { return ksw_smem + KSW_STAGES * KSW_A_BYTES + s * KSW_W_BYTES; };

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col = lane & 31, kh = lane >> 5;
    const int m0 = blockIdx.y * KSW_M, n0 = blockIdx.x * KSW_N;
    const int nsteps = k / KSW_K;                              // k is a multiple of 256: whole super-blocks
    const int nsb = k >> 8;
    const int64_t row_bytes = (int64_t)nsb * 144;

    // activation tile: thread t copies chunks t, t + 256, ... (4 of them): row = chunk / 8, 16-byte piece = chunk % 8
    // Both operands are read through buffer descriptors: a lane's byte offset is a constant register, the step's offset a
    // scalar, so a load costs no address arithmetic (offsets fit 32 bits: the launcher checks the operand sizes).
    const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<__bf16*>(a), 0, (int)0x7FFFFFFF, 0x00020000);
    const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(w), 0, (int)0x7FFFFFFF, 0x00020000);
    uint32_t a_off[4];
    int a_dst[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int p = tid + 256 * j, row = p >> 3, kp = p & 7;
        a_off[j] = ((uint32_t)min(m0 + row, m - 1) * (uint32_t)k + 8u * kp) * 2u;   // bytes; rows past M: a valid copy, never stored
        a_dst[j] = row * KSW_ASTRIDE + 8 * kp;
    }
    // raw super-blocks: 64 rows x 9 pieces of 16 bytes = 576 pieces, thread t copies pieces t, t + 256 and (t < 64) t + 512
    uint32_t w_off[3];
    int w_dst[3];
#pragma unroll
    for (int j = 0; j < 3; ++j) {
        const int p = min(tid + 256 * j, 575), row = p / 9, pc = p - 9 * row;
        w_off[j] = (uint32_t)min(n0 + row, n - 1) * (uint32_t)row_bytes + pc * 16u;   // rows past N: a valid copy, never stored
        w_dst[j] = (tid + 256 * j) * 16;                                             // pieces 576 .. 767: padding
    }

    ksw_u32x4 aring[2][4], wring[3];
    auto load_a_chunk = [&](int slot, int step, int j) __attribute__((always_inline)) {
        const int soff = min(step, nsteps - 1) * (KSW_K * 2);                                              // uniform; past the end: the last step again
        aring[slot][j] = __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, (int)a_off[j], soff, 0);
    };
    auto park_a_chunk = [&](int slot, int stage, int j) __attribute__((always_inline)) {
        *reinterpret_cast<ksw_u32x4*>(a_stage(stage) + a_dst[j]) = aring[slot][j];
    };
    auto load_w = [&](int sb) __attribute__((always_inline)) {
        const int soff = min(sb, nsb - 1) * 144;                             // uniform
#pragma unroll
        for (int j = 0; j < 3; ++j) wring[j] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, (int)w_off[j], soff, 0);
    };
    auto park_w = [&](int stage) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < 3; ++j) *reinterpret_cast<ksw_u32x4*>(w_stage(stage) + w_dst[j]) = wring[j];
    };

    ksw_f32x16 acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    // this lane's picks: rows col and col + 32 of the weight tile; in step p of a super-block the 8 bytes at
    // 16 + 32 p + 16 (wave & 1) + 8 kh of the block, low nibbles for waves 0 and 1, high nibbles for waves 2 and 3
    const int hi_plane = wave >> 1;
    const int w_row0 = col * 144, w_row1 = (col + 32) * 144;
    const int w_pick = 16 + 16 * (wave & 1) + 8 * kh;
    const uint32_t nib_mask = 0x0F0F0F0Fu << (4 * hi_plane);
    const float nib_scale = hi_plane ? 0.0625f : 1.0f;
    const int a_frag = col * KSW_ASTRIDE + 16 * wave + 8 * kh;              // + 32 i rows per MFMA row tile

    auto read_frags = [&](ksw_bf16x8 (&af)[4], int stage) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 4; ++i) af[i] = *reinterpret_cast<const ksw_bf16x8*>(a_stage(stage) + a_frag + 32 * i * KSW_ASTRIDE);
    };
    auto read_raw = [&](ksw_u32x2 (&raw)[2], int wstage, int p) __attribute__((always_inline)) {
        raw[0] = *reinterpret_cast<const ksw_u32x2*>(w_stage(wstage) + w_row0 + w_pick + 32 * p);
        raw[1] = *reinterpret_cast<const ksw_u32x2*>(w_stage(wstage) + w_row1 + w_pick + 32 * p);
    };
    auto read_scales = [&](KswScales (&ks)[2], int wstage) __attribute__((always_inline)) {
        ks[0] = ksw_unpack(*reinterpret_cast<const ksw_u32x4*>(w_stage(wstage) + w_row0), 8 * hi_plane, nib_scale);
        ks[1] = ksw_unpack(*reinterpret_cast<const ksw_u32x4*>(w_stage(wstage) + w_row1), 8 * hi_plane, nib_scale);
    };

    // Prologue: steps 0 and 1 parked, steps 2 and 3 on their way in the ring, super-block 0 parked and 1 on its way;
    // fragments, scales and decoded weights of step 0 in registers.
#pragma unroll
    for (int j = 0; j < 4; ++j) { load_a_chunk(0, 0, j); load_a_chunk(1, 1, j); }
    load_w(0);
#pragma unroll
    for (int j = 0; j < 4; ++j) { park_a_chunk(0, 0, j); park_a_chunk(1, 1, j); }
    park_w(0);
#pragma unroll
    for (int j = 0; j < 4; ++j) { load_a_chunk(0, 2, j); load_a_chunk(1, 3, j); }
    load_w(1);
    __syncthreads();

    ksw_bf16x8 af[2][4];                       // fragments of the step being multiplied and of the next one
    uint32_t bw[2][2][4];                      // [set][column tile][dword]: decoded B operands
    ksw_u32x2 raw[2];
    KswScales ks[2], ks_next[2];
    read_frags(af[0], 0);
    read_raw(raw, 0, 0);
    read_scales(ks, 0);
    {
        float sc, of;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            ksw_step_scale<0>(ks[j], sc, of);
            ksw_decode4(raw[j].x & nib_mask, sc, of, bw[0][j][0], bw[0][j][1]);
            ksw_decode4(raw[j].y & nib_mask, sc, of, bw[0][j][2], bw[0][j][3]);
        }
    }

    // One step: the 8 matrix instructions of step `step` (fragments and weights already in registers, set `P & 1`), and
    // between them, in program order, everything that prepares later steps:
    //   behind MFMA 0   the LDS reads of the next step's fragments and raw codes
    //   behind MFMA 1-2 the activation tile of step + 2 parked (two chunks each), each ring register refilled with step + 4
    //   behind MFMA 3   the next step's scales (and, in step 2 of a super-block, the next super-block's header unpacked)
    //   behind MFMA 4-7 the next step's weights decoded, four at a time
    // then one barrier. sched_barrier(0) pins the order.
    auto step_body = [&](auto pc, int s0) __attribute__((always_inline)) {
        constexpr int P = decltype(pc)::value, SET = P & 1, NP = (P + 1) & 3;
        const int step = s0 + P, sb = s0 >> 2, ws = sb & 1;
        constexpr int st_next = (P + 1) % KSW_STAGES, st_park = (P + 2) % KSW_STAGES;   // s0 is a multiple of 4
        float sc[2], of[2];
        ksw_bf16x8 b[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) b[j] = __builtin_bit_cast(ksw_bf16x8, ksw_u32x4{bw[SET][j][0], bw[SET][j][1], bw[SET][j][2], bw[SET][j][3]});
#pragma clang loop unroll(full)
        for (int q = 0; q < 8; ++q) {
            const int i = q >> 1, j = q & 1;
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[SET][i], b[j], acc[i][j], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            if (q == 0) {
                read_frags(af[SET ^ 1], st_next);
                read_raw(raw, P == 3 ? ws ^ 1 : ws, NP);
                if (P == 2) read_scales(ks_next, ws ^ 1);                   // parked during step 1, behind that step's barrier
            } else if (q == 1 || q == 2) {
                const int j0 = 2 * (q - 1);
                park_a_chunk(P & 1, st_park, j0); park_a_chunk(P & 1, st_park, j0 + 1);
                load_a_chunk(P & 1, step + 4, j0); load_a_chunk(P & 1, step + 4, j0 + 1);
            } else if (q == 3) {
                if (P == 3) { ks[0] = ks_next[0]; ks[1] = ks_next[1]; }
                ksw_step_scale<NP>(ks[0], sc[0], of[0]);
                ksw_step_scale<NP>(ks[1], sc[1], of[1]);
                if (P == 1) park_w(ws ^ 1);                                 // the next super-block's raw bytes, loaded a trip ago
                if (P == 2) load_w(sb + 2);
            } else {
                const int jj = (q - 4) >> 1, half = (q - 4) & 1;
                ksw_decode4((half ? raw[jj].y : raw[jj].x) & nib_mask, sc[jj], of[jj], bw[SET ^ 1][jj][2 * half], bw[SET ^ 1][jj][2 * half + 1]);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        __syncthreads();
    };

    for (int s0 = 0; s0 < nsteps; s0 += 4) {                               // one super-block (four steps) per trip
        step_body(std::integral_constant<int, 0>{}, s0);
        step_body(std::integral_constant<int, 1>{}, s0);
        step_body(std::integral_constant<int, 2>{}, s0);
        step_body(std::integral_constant<int, 3>{}, s0);
    }

    // The four waves hold partial sums of the same 128 x 64 tile: park them, then wave v adds up rows 32 v .. 32 v + 31.
    // Accumulator element e of lane l: row 8 (e / 4) + 4 (l / 32) + e % 4, column l % 32 of its 32 x 32 tile.
    float* red = reinterpret_cast<float*>(ksw_smem);
    float* mine = red + (size_t)wave * KSW_M * KSW_RED_PITCH;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e)
                mine[(32 * i + 8 * (e >> 2) + 4 * kh + (e & 3)) * KSW_RED_PITCH + 32 * j + col] = acc[i][j][e];
    __syncthreads();
    const int c4 = (lane & 15) * 4;
#pragma unroll
    for (int it = 0; it < 8; ++it) {
        const int row = 32 * wave + 4 * it + (lane >> 4);
        float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const float4 t = *reinterpret_cast<const float4*>(red + ((size_t)v * KSW_M + row) * KSW_RED_PITCH + c4);
            sum.x += t.x; sum.y += t.y; sum.z += t.z; sum.w += t.w;
        }
        const int gr = m0 + row, gc = n0 + c4;
        if (gr < m) {
            float* dst = c + (int64_t)gr * n + gc;
            if (gc + 3 < n && (reinterpret_cast<uintptr_t>(dst) & 15) == 0) *reinterpret_cast<float4*>(dst) = sum;
            else {
                if (gc < n) dst[0] = sum.x;
                if (gc + 1 < n) dst[1] = sum.y;
                if (gc + 2 < n) dst[2] = sum.z;
                if (gc + 3 < n) dst[3] = sum.w;
            }
        }
    }
}

static std::atomic<int> g_gemm_ksw{1};      // 0 never, 1 where the launcher's estimate favours it, 2 wherever it fits
void set_gemm_ksw(int v) { if (v >= 0 && v <= 2) g_gemm_ksw = v; }
bool gemm_ksw_enabled() { return g_gemm_ksw.load() != 0; }
bool gemm_ksw_forced() { return g_gemm_ksw.load() == 2; }
bool gemm_ksw_fits(int m, int n, int k) {
    return (uint64_t)m * (uint64_t)k < ((uint64_t)1 << 30) && (uint64_t)n * (uint64_t)(k >> 8) * 144u < ((uint64_t)1 << 31);   // 2 GiB each
}

// C = A . W^T for bf16 activations already in `a`; k a multiple of 256, operands 16-byte aligned, both operands below
// 4 G elements / bytes (the caller checks, see gemm_ksw_fits). 0 on success.
int launch_q4k_gemm_ksw(const __bf16* a, const uint8_t* w, float* c, int m, int n, int k, hipStream_t s) {
    if ((uint64_t)m * (uint64_t)k >= ((uint64_t)1 << 30) || (uint64_t)n * (uint64_t)(k >> 8) * 144u >= ((uint64_t)1 << 31))
        return set_error("gemm: operands of %d x %d x %d exceed the 32-bit offsets of this kernel", m, n, k);
    const dim3 grid((n + KSW_N - 1) / KSW_N, (m + KSW_M - 1) / KSW_M);
    SKH_SET_MAX_DYNAMIC_LDS_ONCE((&q4k_gemm_ksw_kernel), KSW_SMEM);
    note_kernel("q4k_gemm_ksw_kernel");
    q4k_gemm_ksw_kernel<<<grid, dim3(256), KSW_SMEM, s>>>(a, w, c, m, n, k);
    SKH_CHECK(hipGetLastError());
    return 0;
}

}  // namespace skh
