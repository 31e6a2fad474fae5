// Q4_K dequant-GEMM with K split over the waves of a workgroup:  C[m, n] = sum_k A[m, k] * dequant(W[n, k])
//   A bf16 [M, K] (the fp32 activations rounded once by the pass in front, gemm.hip), W packed Q4_K in canonical
//   row-major GGUF order, products bf16 x bf16 on v_mfma_f32_32x32x16_bf16, fp32 accumulation, C fp32 [M, N].
//
// Same contract and arithmetic as dequant_gemm_kernel (gemm.hip): a weight is code * (d * sc) - dmin * m in fp32 (one
// fused multiply-add), rounded to bf16 (nearest even). What differs is who owns what:
//   * workgroup tile 128 (M) x 64 (N): 512 x 4096 outputs are 256 tiles, one per CU, so the chip is full without
//     splitting K across workgroups (no partial tiles parked in memory, no launch that sums them);
//   * every wave owns the WHOLE tile (4 x 2 MFMA tiles of 32 x 32: 128 accumulator registers, each fragment read from
//     LDS feeds two or four matrix instructions) and a share of K: in every 64-element step wave w of a team of four
//     takes the 16-element slice w. The partial tiles meet once, at the end, through LDS;
//   * a 16-element slice of a Q4_K row is one nibble plane (low for slices 0 and 1, high for 2 and 3) of 16 consecutive
//     bytes, and lane (column n, half h) of the matrix instruction's B operand needs 8 of them: so a lane decodes exactly
//     the 8 weights of each of its two columns that its own operand holds, straight into registers. Decoded weights never
//     pass through LDS and nothing is decoded twice;
//   * both operands come in by loads that write LDS directly (global_load_lds_dwordx4: no staging registers, no LDS
//     store instructions; inline assembly with explicit wait counts, since the loads complete in issue order): the raw
//     super-blocks (144 bytes per row and 256 elements, once per four steps) so that the lanes' 8-byte picks come out of
//     LDS, and the activation tile of a step (128 rows x 64 elements, bf16) S - 1 steps ahead of the step that reads it.
//     The lane chooses the source address, so the LDS layout is free: activation rows are 128 bytes with their 16-byte
//     pieces XOR-swizzled by the row, which the fragment reads take without bank conflicts and without padding;
//   * a step's fragments are read, and its weights decoded, during the previous step: between the 8 matrix
//     instructions of a step sit, in pinned program order, the reads, the loads and the decode for the steps behind it;
//     one barrier per step.
// What bounds it (measured by compiling pieces out, 512 x 4096 x 4096, one launch 26 us): the launch, the prologue and
// the final exchange and store 6.5 us; the matrix instructions alone 8.5 us on top; the loads alone 12 us on top (every
// workgroup pulls its whole 1 MB row block of activations through L2: 311 MB per launch, 2/3 of what the L2s deliver);
// decode and matrix instructions do not overlap on a SIMD (a vector instruction issued behind a matrix instruction
// waits for it, also from another wave), so the decode's 44 vector instructions per step add their full time.
#include "common.h"

#include <type_traits>

namespace skh {

typedef __bf16 ksw_bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 ksw_bf16x2 __attribute__((ext_vector_type(2)));
typedef float ksw_f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t ksw_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t ksw_u32x2 __attribute__((ext_vector_type(2)));

constexpr int KSW_M = 128, KSW_N = 64, KSW_K = 64;
constexpr int KSW_A_BYTES = KSW_M * KSW_K * 2;                // one stage of the activation tile: rows of 128 bytes, no padding; the
                                                              // 16-byte piece p of row r sits in slot p ^ ((r >> 1) & 7) of its row
constexpr int KSW_W_BYTES = KSW_N * 144;                      // one stage of raw super-blocks: 64 rows x 144 bytes = 9 wave loads
// Activation stages (template argument S, 3 .. 7): step s multiplies from registers, reads step s + 1 out of LDS and has
// step s + S land in the stage step s has left: S - 2 steps between a load's issue and the barrier it must have landed by.
constexpr int KSW_RED_PITCH = KSW_N + 4;                      // floats per row of a partial tile in the final exchange
constexpr size_t ksw_team_bytes(int stages) { return stages * (size_t)KSW_A_BYTES + 2 * (size_t)KSW_W_BYTES; }   // the loop's LDS of one team of four waves
constexpr size_t KSW_RED_BYTES = (size_t)4 * KSW_M * KSW_RED_PITCH * sizeof(float);
constexpr size_t ksw_smem_bytes(int teams, int stages) { return KSW_RED_BYTES > teams * ksw_team_bytes(stages) ? KSW_RED_BYTES : teams * ksw_team_bytes(stages); }

// 16 bytes per lane from base + off straight into LDS at lds_addr + 16 * lane (M0 carries the LDS address); counted by
// vmcnt like any other load, in issue order
__device__ __forceinline__ void ksw_dma16(uint32_t lds_addr, uint32_t off, const uint8_t* base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(off), "s"(base) : "memory");
}
// of the `steps` steps that end with step p of a super-block, how many are a step 3
constexpr int ksw_count_p3(int p, int steps) {
    int c = 0;
    for (int d = 0; d < steps; ++d) c += (((p - d) % 4 + 4) % 4) == 3;
    return c;
}
template <int N> __device__ __forceinline__ void ksw_wait_loads() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }
// the same, and this wave's LDS reads have returned as well: behind the barrier that follows, another wave's loads may
// overwrite the stage they read
template <int N> __device__ __forceinline__ void ksw_wait_loads_and_reads() { asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(N) : "memory"); }

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

// TEAMS teams of four waves share a workgroup and its tile; team t runs the loop above on its own share of K (whole
// super-blocks, TEAMS equal shares) out of its own part of LDS. With two teams a SIMD holds two waves, so one team's
// decode and LDS traffic issue under the other's matrix instructions; the price is 256 registers per wave instead of 512
// and one more exchange of partial tiles at the end.
template <int TEAMS, int S>
__global__ __launch_bounds__(256 * TEAMS) void q4k_gemm_ksw_kernel(const __bf16* __restrict__ a, const uint8_t* __restrict__ w,
                                                                   float* __restrict__ c, int m, int n, int k) {
    extern __shared__ __attribute__((aligned(16))) uint8_t ksw_smem[];   // the kernel has no other LDS: offsets into it are LDS addresses
    const int lane = threadIdx.x & 63;
    const int wave_all = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int team = TEAMS == 1 ? 0 : wave_all >> 2, wave = wave_all & 3;
    const uint32_t team_lds = (uint32_t)team * (uint32_t)ksw_team_bytes(S);
    auto w_stage_off = [&](int s) { return team_lds + (uint32_t)(S * KSW_A_BYTES + s * KSW_W_BYTES); };

    const int col = lane & 31, kh = lane >> 5;
    const int m0 = blockIdx.y * KSW_M, n0 = blockIdx.x * KSW_N;
    const int nsb = (k >> 8) / TEAMS;                          // this team's super-blocks (the launcher checks divisibility)
    const int nsteps = nsb * 4;
    const uint32_t row_bytes = (uint32_t)(k >> 8) * 144u;
    const uint8_t* const a_team = reinterpret_cast<const uint8_t*>(a) + (size_t)team * nsb * 512;   // the team's first column, bytes
    const uint8_t* const w_team = w + (size_t)team * nsb * 144;

    // Both operands come in by loads that write LDS directly (no registers, no store instruction). A wave load fills
    // 1 KB of consecutive LDS, lane l the 16 bytes at 16 l, from whatever address the lane gives: so the LDS layout is
    // chosen by the lane's source address. Offsets fit 32 bits (the launcher checks the operand sizes).
    //   activation stage: wave load q = 4 j + wave covers rows 8 q .. 8 q + 7 (8 slots of 16 bytes each)
    uint32_t a_voff[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int row = 8 * (4 * j + wave) + (lane >> 3), piece = (lane & 7) ^ ((row >> 1) & 7);
        a_voff[j] = (uint32_t)min(m0 + row, m - 1) * (uint32_t)k * 2u + 16u * piece;   // rows past M: a valid copy, never stored
    }
    //   raw super-blocks: 576 pieces of 16 bytes in row order = 9 wave loads; wave w issues loads w, w + 4 and (all four
    //   waves, so that every wave counts the same number of loads) 8
    uint32_t w_voff[3];
#pragma unroll
    for (int j = 0; j < 3; ++j) {
        const int p = 64 * (j < 2 ? wave + 4 * j : 8) + lane, row = p / 9, pc = p - 9 * row;
        w_voff[j] = (uint32_t)min(n0 + row, n - 1) * row_bytes + 16u * pc;              // rows past N: a valid copy, never stored
    }
    auto dma_a = [&](uint32_t stage_off, int step) __attribute__((always_inline)) {
        const uint8_t* base = a_team + (size_t)min(step, nsteps - 1) * (KSW_K * 2);     // uniform; past the end: the last step again
#pragma unroll
        for (int j = 0; j < 4; ++j) ksw_dma16(stage_off + 1024u * (4 * j + wave), a_voff[j], base);
    };
    auto dma_w = [&](uint32_t stage_off, int sb) __attribute__((always_inline)) {
        const uint8_t* base = w_team + (size_t)min(sb, nsb - 1) * 144;                 // uniform
#pragma unroll
        for (int j = 0; j < 3; ++j) ksw_dma16(stage_off + 1024u * (j < 2 ? wave + 4 * j : 8), w_voff[j], base);
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
    const int w_pick = col * 144 + 16 + 16 * (wave & 1) + 8 * kh;          // row col + 32: 32 * 144 bytes further
    const int w_hdr = col * 144;
    const uint32_t nib_mask = 0x0F0F0F0Fu << (4 * hi_plane);
    const float nib_scale = hi_plane ? 0.0625f : 1.0f;
    // fragment of MFMA row tile i: row col + 32 i, elements 16 wave + 8 kh ..: piece 2 wave + kh, swizzled by the row
    const int a_frag = col * (KSW_K * 2) + 16 * ((2 * wave + kh) ^ ((col >> 1) & 7));

    auto read_frags = [&](ksw_bf16x8 (&af)[4], uint32_t stage_off) __attribute__((always_inline)) {
        const uint8_t* p = ksw_smem + (stage_off + (uint32_t)a_frag);
#pragma unroll
        for (int i = 0; i < 4; ++i) af[i] = *reinterpret_cast<const ksw_bf16x8*>(p + 32 * i * (KSW_K * 2));
    };
    auto read_raw = [&](ksw_u32x2 (&raw)[2], int wstage, int p) __attribute__((always_inline)) {
        const uint8_t* q = ksw_smem + (w_stage_off(wstage) + (uint32_t)w_pick);
        raw[0] = *reinterpret_cast<const ksw_u32x2*>(q + 32 * p);
        raw[1] = *reinterpret_cast<const ksw_u32x2*>(q + 32 * p + 32 * 144);
    };
    auto read_scales = [&](KswScales (&ks)[2], int wstage) __attribute__((always_inline)) {
        const uint8_t* q = ksw_smem + (w_stage_off(wstage) + (uint32_t)w_hdr);
        ks[0] = ksw_unpack(*reinterpret_cast<const ksw_u32x4*>(q), 8 * hi_plane, nib_scale);
        ks[1] = ksw_unpack(*reinterpret_cast<const ksw_u32x4*>(q + 32 * 144), 8 * hi_plane, nib_scale);
    };

    // Prologue: steps 0 .. S - 1 and super-blocks 0 and 1 in LDS; fragments, scales and decoded weights of step 0 in
    // registers. st[i]: the stage of the step i after the current one (they rotate).
    uint32_t st[S];
#pragma unroll
    for (int i = 0; i < S; ++i) { st[i] = team_lds + i * KSW_A_BYTES; dma_a(st[i], i); }
    dma_w(w_stage_off(0), 0); dma_w(w_stage_off(1), 1);
    ksw_wait_loads<0>();
    __syncthreads();

    ksw_bf16x8 af[2][4];                       // fragments of the step being multiplied and of the next one
    uint32_t bw[2][2][4];                      // [set][column tile][dword]: decoded B operands
    ksw_u32x2 raw[2];
    KswScales ks[2];
    read_frags(af[0], st[0]);
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
    __syncthreads();                           // every wave has read stage 0 before step 0 lets step 3 land in it

    // One step: the 8 matrix instructions of step `step` (fragments and weights already in registers, set `P & 1`), and
    // between them, in program order, everything that prepares later steps:
    //   behind MFMA 0   the LDS reads of the next step's fragments and raw codes (in step 3 of a super-block: the next
    //                   super-block's header as well)
    //   behind MFMA 1   the loads of step + S into the stage this step has left (its fragments were read a step ago),
    //                   and in step 3 of a super-block the loads of super-block + 2 into the stage this one has left
    //   behind MFMA 3   the next step's scales
    //   behind MFMA 4-7 the next step's weights decoded, four at a time
    // then a wait for the loads issued a step ago (step + 2 must be readable in the next step) and one barrier.
    // sched_barrier(0) pins the order.
    auto step_body = [&](auto pc, int s0) __attribute__((always_inline)) {
        constexpr int P = decltype(pc)::value, SET = P & 1, NP = (P + 1) & 3;
        const int step = s0 + P, sb = s0 >> 2, ws = sb & 1;
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
                read_frags(af[SET ^ 1], st[1]);
                read_raw(raw, P == 3 ? ws ^ 1 : ws, NP);
                if (P == 3) read_scales(ks, ws ^ 1);                        // this block's last use of ks was in step 2
            } else if (q == 1) {
                dma_a(st[0], step + S);
                if (P == 3) dma_w(w_stage_off(ws), sb + 2);                 // read for the last time a step ago
            } else if (q == 3) {
                ksw_step_scale<NP>(ks[0], sc[0], of[0]);
                ksw_step_scale<NP>(ks[1], sc[1], of[1]);
            } else if (q >= 4) {
                const int jj = (q - 4) >> 1, half = (q - 4) & 1;
                ksw_decode4((half ? raw[jj].y : raw[jj].x) & nib_mask, sc[jj], of[jj], bw[SET ^ 1][jj][2 * half], bw[SET ^ 1][jj][2 * half + 1]);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // Loads complete in issue order: step + 2 (issued S - 2 steps ago) must have landed, so everything issued in the
        // S - 2 steps up to this one may still fly: 4 activation loads a step and the 3 of a super-block in its step 3.
        // The raw super-block requested in step 3 of the previous super-block is read from step 3 of this one on: at the
        // end of step 2 only the 12 activation loads issued since may still fly.
        constexpr int in_flight_a = 4 * (S - 2) + 3 * ksw_count_p3(P, S - 2);
        constexpr int in_flight = P == 2 && in_flight_a > 12 ? 12 : in_flight_a;
        ksw_wait_loads_and_reads<in_flight>();
        __syncthreads();
        const uint32_t t = st[0];
#pragma unroll
        for (int i = 0; i + 1 < S; ++i) st[i] = st[i + 1];
        st[S - 1] = t;
    };

    for (int s0 = 0; s0 < nsteps; s0 += 4) {                               // one super-block (four steps) per trip
        step_body(std::integral_constant<int, 0>{}, s0);
        step_body(std::integral_constant<int, 1>{}, s0);
        step_body(std::integral_constant<int, 2>{}, s0);
        step_body(std::integral_constant<int, 3>{}, s0);
    }
    ksw_wait_loads<0>();                       // the loads past the end still write LDS
    __syncthreads();

    // The waves hold partial sums of the same 128 x 64 tile: park them, then every wave adds up its share of the rows.
    // Accumulator element e of lane l: row 8 (e / 4) + 4 (l / 32) + e % 4, column l % 32 of its 32 x 32 tile.
    // With two teams the second team's tiles go through LDS first, each into the accumulators of the first team's wave
    // of the same number (same lane, same element: the addresses a lane reads are the ones its twin wrote).
    float* red = reinterpret_cast<float*>(ksw_smem);
    float* mine = red + (size_t)wave * KSW_M * KSW_RED_PITCH;
    auto tile_at = [&](int i, int j, int e) -> float& { return mine[(32 * i + 8 * (e >> 2) + 4 * kh + (e & 3)) * KSW_RED_PITCH + 32 * j + col]; };
    if (TEAMS == 2) {
        if (team == 1) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int e = 0; e < 16; ++e) tile_at(i, j, e) = acc[i][j][e];
        }
        __syncthreads();
        if (team == 0) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int e = 0; e < 16; ++e) acc[i][j][e] += tile_at(i, j, e);
        }
        __syncthreads();
    }
    if (team == 0) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) tile_at(i, j, e) = acc[i][j][e];
    }
    __syncthreads();
    const int c4 = (lane & 15) * 4;
    constexpr int ROWS_PER_WAVE = KSW_M / (4 * TEAMS);
#pragma unroll
    for (int it = 0; it < ROWS_PER_WAVE / 4; ++it) {
        const int row = ROWS_PER_WAVE * wave_all + 4 * it + (lane >> 4);
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
static std::atomic<int> g_gemm_ksw_teams{2};   // teams of four waves per workgroup (1 or 2)
void set_gemm_ksw_teams(int v) { if (v == 1 || v == 2) g_gemm_ksw_teams = v; }
static std::atomic<int> g_gemm_ksw_stages{5};  // activation stages of the one-team form (3 .. 7)
void set_gemm_ksw_stages(int v) { if (v >= 3 && v <= 7) g_gemm_ksw_stages = v; }
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
    note_kernel("q4k_gemm_ksw_kernel");
    const int teams = g_gemm_ksw_teams.load(), stages = g_gemm_ksw_stages.load();
#define SKH_KSW_LAUNCH(T, ST)                                                                              \
    do {                                                                                                   \
        SKH_SET_MAX_DYNAMIC_LDS_ONCE((&q4k_gemm_ksw_kernel<T, ST>), ksw_smem_bytes(T, ST));                \
        q4k_gemm_ksw_kernel<T, ST><<<grid, dim3(256 * T), ksw_smem_bytes(T, ST), s>>>(a, w, c, m, n, k);   \
    } while (0)
    if (teams == 2 && ((k >> 8) & 1) == 0) SKH_KSW_LAUNCH(2, 3);   // two teams take half of K each: an even number of super-blocks
    else if (stages <= 3) SKH_KSW_LAUNCH(1, 3);
    else if (stages == 4) SKH_KSW_LAUNCH(1, 4);
    else if (stages == 5) SKH_KSW_LAUNCH(1, 5);
    else if (stages == 6) SKH_KSW_LAUNCH(1, 6);
    else SKH_KSW_LAUNCH(1, 7);
#undef SKH_KSW_LAUNCH
    SKH_CHECK(hipGetLastError());
    return 0;
}

}  // namespace skh
