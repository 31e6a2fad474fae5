// Q4_K dequant-GEMV for 3 to 8 activation rows on the 16 x 16 x 32 matrix instruction, K = 4096, canonical row-major
// GGUF weight.
//
//   y[b, o] = sum_j x[b, j] * dequant(W[o, j])
//
// Same products as the reference's exact-fp32 kernel, other summation order
//   /root/reference/skainet-backends/skainet-backend-cpu/src/commonMain/kotlin/sk/ainet/exec/kernel/ScalarQ4_KMatmulKernel.kt:40-78
// and m rows = m such products (PackedViewMatmulKernel.kt:69-108).
//
// The arithmetic is that of q4k_gemv_quads_stream_kernel (gemv_q4k_quads.hip): a 4-bit code q enters as the bf16 value
// 128 + q (0x4300 | q, exact), an activation as bf16 hi + bf16 lo (16 to 17 significant bits, every product exact in
// fp32). What changes is the instruction: v_mfma_f32_4x4x4_16b_bf16 multiplies 4 weights x 4 rows x 4 columns per block
// and needs 64 instructions per four weight rows of a 1024-element slice; v_mfma_f32_16x16x32_bf16 takes
//   A = activations: 16 "rows" = 8 batch rows x (hi, lo), 32 elements of K = exactly one Q4_K sub-block,
//   B = 16 weight rows x the same 32 elements,
// one instruction per sub-block and 16 weight rows -- an eighth of the matrix cycles per weight. Lane l = 16 kq + r holds,
// as B operand, the 8 weights of row r at bytes 8 kq .. 8 kq + 7 of the sub-block's nibble plane, and receives the sums
// of weight row r against activation columns 4 kq .. 4 kq + 3: so the sub-block's scale d * sc and minimum dmin * m are
// per-lane scalars of the lane's own row, read from the header it has in LDS anyway. The accumulator starts at
// -128 * sum(x) of the sub-block (which takes the 128 out and, divided by 128, is the sum the minimum multiplies).
// Activation columns are ordered (batch row, part) with the part fastest: a lane's four results are two batch rows'
// hi and lo sums, added in the lane.
//
// Data path: eight waves per workgroup (two per SIMD), wave w owns K slice w (512 elements: 288 consecutive bytes of
// every row) of all the workgroup's rows; a unit of 16 rows x 288 bytes arrives by five full-wave
// global_load_lds_dwordx4 (non-temporal, the fifth on 32 lanes) straight into a wave-private LDS ring of W slots (two
// requested up front, the third as soon as the activations it stages are in registers, a slot refilled once its unit
// is used up), explicit wait counts; nothing is requested past the last unit. A wave prepares exactly the activations it multiplies
// (no workgroup barrier before the end); the waves' sums meet once, in LDS.
#include "gemv_q4k.h"

namespace skh {

typedef __bf16 wd_bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 wd_bf16x2 __attribute__((ext_vector_type(2)));
typedef float wd_f32x2 __attribute__((ext_vector_type(2)));
typedef float wd_f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t wd_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t wd_u32x2 __attribute__((ext_vector_type(2)));

constexpr int WD_K = 4096, WD_WAVES = 8, WD_SLICE_BYTES = 288;        // a wave's share of a row: two super-blocks
constexpr int WD_UNIT_ROWS = 16, WD_UNIT_BYTES = WD_UNIT_ROWS * WD_SLICE_BYTES;   // 4608 = 4.5 wave loads
constexpr int WD_W = 3, WD_SLOTS = WD_W;                              // ring slots per wave = units in flight at most (a slot is refilled once its unit is used up)
constexpr int WD_MAX_UNITS = 8;                                       // units (of 16 rows) a workgroup owns at most
constexpr size_t WD_RING_BYTES = (size_t)WD_WAVES * WD_SLOTS * WD_UNIT_BYTES;
constexpr size_t WD_SMEM = WD_RING_BYTES + (size_t)WD_WAVES * WD_MAX_UNITS * 64 * 2 * sizeof(float);

__device__ __forceinline__ void wd_load16(wd_u32x4& dst, uint32_t off, const void* base) {
    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(dst) : "v"(off), "s"(base) : "memory");
}
__device__ __forceinline__ void wd_stream_to_lds(uint32_t lds_addr, uint32_t off, const uint8_t* base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(lds_addr), "v"(off), "s"(base) : "memory");
}
template <int N> __device__ __forceinline__ void wd_wait_loads() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }
// the same, tied to the registers an earlier load writes: their uses cannot move above the wait
template <int N> __device__ __forceinline__ void wd_wait_loads(wd_u32x4& a, wd_u32x4& b, wd_u32x4& c, wd_u32x4& d) {
    asm volatile("s_waitcnt vmcnt(%4)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d) : "n"(N) : "memory");
}
__device__ __forceinline__ void wd_wait_lds() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

__global__ __launch_bounds__(64 * WD_WAVES, 1) void q4k_gemv_wide_kernel(const uint8_t* __restrict__ w, const float* __restrict__ x,
                                                                         float* __restrict__ y, int n, int batch, int rows_per_wg) {
    extern __shared__ __attribute__((aligned(16))) uint8_t wdsmem[];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = lane & 15, kq = lane >> 4;
    const int r0 = blockIdx.x * rows_per_wg;
    const int nrows = min(n - r0, rows_per_wg);
    const int units = (nrows + WD_UNIT_ROWS - 1) / WD_UNIT_ROWS;                   // uniform, 1 .. WD_MAX_UNITS
    const uint32_t row_bytes = (WD_K >> 8) * Q4K_BYTES;
    uint8_t* ring = wdsmem + (size_t)wave * WD_SLOTS * WD_UNIT_BYTES;
    const uint32_t ring_addr = (uint32_t)(size_t)(__attribute__((address_space(3))) uint8_t*)ring;
    uint32_t code_mask = 0x000F000Fu, code_bias = 0x43004300u;
    asm volatile("" : "+v"(code_bias), "+s"(code_mask));       // kept out of the optimiser's sight: (v & mask) | bias stays one instruction

    // Activations first (they come from L2 and must not queue behind the weight stream): the wave's K slice of the 8
    // batch rows, 4096 floats, as 16 coalesced float4 loads per lane. Load i of lane l is float4 number 64 i + l of the
    // rows taken two at a time: rows 2 (i / 4) and 2 (i / 4) + 1, 128 float4s each. (Batch rows past `batch` are copies
    // of the last one: their columns are computed and never stored.)
    wd_u32x4 xr[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int idx = 64 * (i & 3) + lane, b = 2 * (i >> 2) + (idx >> 7), f = idx & 127;
        wd_load16(xr[i], (uint32_t)(min(b, batch - 1) * WD_K + wave * 512 + 4 * f) * 4u, x);
    }
    // the ring: piece p = 64 j + lane of a unit is the 16 bytes at row p / 18, piece p % 18 of the slice. (The 16 rows'
    // copies of a piece side by side -- position p holding piece p / 16 of row p % 16, which takes the four-way bank
    // conflict out of the reads below -- measured 12.7 against 11.7 us: a load then takes 64 bytes out of each of 16
    // lines instead of three rows' worth of consecutive bytes.)
    uint32_t loff[5];
#pragma unroll
    for (int j = 0; j < 5; ++j) {
        const uint32_t p = min(64u * j + lane, 287u), row = (p * 3641u) >> 16, pc = p - 18u * row;     // p / 18 for p < 288
        loff[j] = row * row_bytes + (uint32_t)wave * WD_SLICE_BYTES + pc * 16u;
    }
    const uint32_t max_off = (uint32_t)n * row_bytes - 16u;                        // rows past N: the last bytes, never stored
    auto issue_unit = [&](int u) {                                                 // u uniform, < units
        const uint32_t base = (uint32_t)(r0 + WD_UNIT_ROWS * u) * row_bytes;
        const uint32_t slot = ring_addr + (uint32_t)(u % WD_SLOTS) * WD_UNIT_BYTES;
#pragma unroll
        for (int j = 0; j < 4; ++j) wd_stream_to_lds(slot + 1024u * j, min(base + loff[j], max_off), w);
        if (lane < 32) wd_stream_to_lds(slot + 4096u, min(base + loff[4], max_off), w);
    };
    // Two units are requested up front (the third slot stages the activations first). The wait counts below assume
    // exactly 10 weight loads behind the activations: a workgroup with one unit makes up the count with loads of the
    // (cached) activations into the unused slot.
    issue_unit(0);
    if (units > 1) issue_unit(1);
    else {
#pragma unroll
        for (int j = 0; j < 5; ++j) wd_stream_to_lds(ring_addr + WD_UNIT_BYTES + 1024u * (j < 4 ? j : 0), 16u * lane, reinterpret_cast<const uint8_t*>(x));
    }

    // bf16 hi / lo parts through LDS into operand order, two batch rows at a time (their slices fill 4 KB of the third
    // slot). Every float is split once, by the lane that loaded it: a float4 (v0 .. v3) becomes the pairs (v0, v2) and
    // (v1, v3) -- the B operand's 8 weights come out of two code dwords as bytes 0, 2, 1, 3 of each (one mask-and-merge
    // per pair of codes), so the activations take the same order -- 8 bytes of hi parts and 8 bytes of lo parts, stored
    // at [row][part][float4 number]: the 16 bytes at float4 number 8 sb + 2 kq are then lane (c, kq)'s operand of
    // sub-block sb. A wave prepares exactly the slices it multiplies: no other wave touches them, so there is no
    // workgroup barrier (LDS serves a wave's instructions in order; the fences keep the compiler from reordering them).
    const int col = r, b_of_lane = col >> 1, part = col & 1;
    uint8_t* stage = ring + 2 * WD_UNIT_BYTES;
    wd_bf16x8 act[16];
#pragma unroll
    for (int sb = 0; sb < 16; ++sb) act[sb] = __builtin_bit_cast(wd_bf16x8, wd_u32x4{0u, 0u, 0u, 0u});
#pragma unroll
    for (int round = 0; round < 4; ++round) {
        if (round == 0) wd_wait_loads<22>(xr[0], xr[1], xr[2], xr[3]);
        else if (round == 1) wd_wait_loads<18>(xr[4], xr[5], xr[6], xr[7]);
        else if (round == 2) wd_wait_loads<14>(xr[8], xr[9], xr[10], xr[11]);
        else wd_wait_loads<10>(xr[12], xr[13], xr[14], xr[15]);
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int idx = 64 * i + lane, rb = idx >> 7, f = idx & 127;
            const wd_u32x4 raw = xr[4 * round + i];
            const wd_f32x2 pr[2] = {wd_f32x2{__uint_as_float(raw.x), __uint_as_float(raw.z)}, wd_f32x2{__uint_as_float(raw.y), __uint_as_float(raw.w)}};
            uint32_t hi[2], lo[2];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                hi[t] = __builtin_bit_cast(uint32_t, __builtin_convertvector(pr[t], wd_bf16x2));
                const wd_f32x2 rest = {pr[t].x - __uint_as_float(hi[t] << 16), pr[t].y - __uint_as_float(hi[t] & 0xFFFF0000u)};
                lo[t] = __builtin_bit_cast(uint32_t, __builtin_convertvector(rest, wd_bf16x2));
            }
            *reinterpret_cast<wd_u32x2*>(stage + ((rb * 2 + 0) * 128 + f) * 8) = wd_u32x2{hi[0], hi[1]};
            *reinterpret_cast<wd_u32x2*>(stage + ((rb * 2 + 1) * 128 + f) * 8) = wd_u32x2{lo[0], lo[1]};
        }
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
        __builtin_amdgcn_wave_barrier();
        if ((b_of_lane >> 1) == round) {
            const uint8_t* src = stage + (((b_of_lane & 1) * 2 + part) * 128 + 2 * kq) * 8;
#pragma unroll
            for (int sb = 0; sb < 16; ++sb) act[sb] = __builtin_bit_cast(wd_bf16x8, *reinterpret_cast<const wd_u32x4*>(src + 64 * sb));
        }
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }
    wd_wait_lds();                                 // the staging slot has been read: it takes the third unit
    if (units > 2) issue_unit(2);

    // -128 * (sum of the column's activations over the sub-block), for the lane's four columns: the start value of the
    // sub-block's accumulator; times -1 / 128, the sum its minimum multiplies
    wd_f32x4 neg_x128[16];
    {
        uint32_t minus128 = 0xC300C300u;                       // bf16 -128 twice: the matrix instruction does the negation
        asm volatile("" : "+v"(minus128));
        const wd_bf16x8 m128 = __builtin_bit_cast(wd_bf16x8, wd_u32x4{minus128, minus128, minus128, minus128});
#pragma unroll
        for (int sb = 0; sb < 16; ++sb)
            neg_x128[sb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(act[sb], m128, wd_f32x4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
    }

    float* parts = reinterpret_cast<float*>(wdsmem + WD_RING_BYTES);              // [wave][unit][lane][2]
    float* part_out = parts + (size_t)wave * WD_MAX_UNITS * 128;
    const uint32_t rd_row = (uint32_t)r * WD_SLICE_BYTES, rd_codes = rd_row + 16u + 8u * kq;
    for (int u = 0; u < units; ++u) {
        // unit u has landed when at most the loads of the units requested after it are in flight
        const int behind = min(units - 1 - u, WD_W - 1);
        if (behind >= 2) wd_wait_loads<10>();
        else if (behind == 1) wd_wait_loads<5>();
        else wd_wait_loads<0>();
        const uint8_t* slot = ring + (uint32_t)(u % WD_SLOTS) * WD_UNIT_BYTES;
        wd_f32x4 tot = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            const wd_u32x4 hdr = *reinterpret_cast<const wd_u32x4*>(slot + rd_row + 144 * s);
            const float d = half_bits_to_float_fast(hdr.x & 0xFFFFu), dmin128 = half_bits_to_float_fast(hdr.x >> 16) * 0.0078125f;
            // the eight 6-bit scales and minima (ggml get_scale_min_k4) as bytes: sub-blocks 0..3 and 4..7
            const uint32_t sc4[2] = {hdr.y & 0x3F3F3F3Fu, (hdr.w & 0x0F0F0F0Fu) | ((hdr.y >> 2) & 0x30303030u)};
            const uint32_t mn4[2] = {hdr.z & 0x3F3F3F3Fu, ((hdr.w >> 4) & 0x0F0F0F0Fu) | ((hdr.z >> 2) & 0x30303030u)};
            wd_f32x4 main = {0.f, 0.f, 0.f, 0.f}, mins = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const wd_u32x2 cw = *reinterpret_cast<const wd_u32x2*>(slot + rd_codes + 144 * s + 32 * g);
                const uint32_t scw = sc4[g >> 1], mnw = mn4[g >> 1];
                const float sc_lo = (g & 1) ? ubyte2_to_float(scw) : ubyte0_to_float(scw), sc_hi = (g & 1) ? ubyte3_to_float(scw) : ubyte1_to_float(scw);
                const float mn_lo = (g & 1) ? ubyte2_to_float(mnw) : ubyte0_to_float(mnw), mn_hi = (g & 1) ? ubyte3_to_float(mnw) : ubyte1_to_float(mnw);
                const wd_bf16x8 wlo = __builtin_bit_cast(wd_bf16x8, wd_u32x4{(cw.x & code_mask) | code_bias, ((cw.x >> 8) & code_mask) | code_bias,
                                                                             (cw.y & code_mask) | code_bias, ((cw.y >> 8) & code_mask) | code_bias});
                const wd_bf16x8 whi = __builtin_bit_cast(wd_bf16x8, wd_u32x4{((cw.x >> 4) & code_mask) | code_bias, ((cw.x >> 12) & code_mask) | code_bias,
                                                                             ((cw.y >> 4) & code_mask) | code_bias, ((cw.y >> 12) & code_mask) | code_bias});
                const int sbi = 8 * s + 2 * g;
                const wd_f32x4 dl = __builtin_amdgcn_mfma_f32_16x16x32_bf16(act[sbi], wlo, neg_x128[sbi], 0, 0, 0);
                const wd_f32x4 dh = __builtin_amdgcn_mfma_f32_16x16x32_bf16(act[sbi + 1], whi, neg_x128[sbi + 1], 0, 0, 0);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    main[e] = fmaf(sc_lo, dl[e], main[e]);
                    main[e] = fmaf(sc_hi, dh[e], main[e]);
                    mins[e] = fmaf(mn_lo, neg_x128[sbi][e], mins[e]);
                    mins[e] = fmaf(mn_hi, neg_x128[sbi + 1][e], mins[e]);
                }
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) tot[e] = fmaf(d, main[e], fmaf(dmin128, mins[e], tot[e]));
        }
        // hi + lo of the lane's two batch rows (2 kq and 2 kq + 1), this wave's K slice
        *reinterpret_cast<float2*>(part_out + (u * 64 + lane) * 2) = make_float2(tot[0] + tot[1], tot[2] + tot[3]);
        if (u + WD_W < units) {
            wd_wait_lds();                         // this unit's slot has been read: refill it
            issue_unit(u + WD_W);
        }
    }
    __syncthreads();
    // the waves' slices meet: thread t takes (unit, batch row pair member, kq, r) with r fastest, so that a batch row's
    // outputs leave as runs of 16 consecutive floats
    for (int t = threadIdx.x; t < units * 128; t += 64 * WD_WAVES) {
        const int rr = t & 15, q = (t >> 4) & 3, v = (t >> 6) & 1, u = t >> 7;
        const int row = r0 + WD_UNIT_ROWS * u + rr, b = 2 * q + v;
        if (row < r0 + nrows && b < batch) {
            float sum = 0.f;
#pragma unroll
            for (int wv = 0; wv < WD_WAVES; ++wv) sum += parts[((size_t)wv * WD_MAX_UNITS + u) * 128 + (16 * q + rr) * 2 + v];
            y[(int64_t)b * n + row] = sum;
        }
    }
}

static std::atomic<int> g_q4k_wide_enable{1};
void set_q4k_wide_enable(int v) { g_q4k_wide_enable = v != 0; }
static std::atomic<int> g_q4k_wide_min_batch{5};
void set_q4k_wide_min_batch(int v) { if (v >= 3 && v <= 8) g_q4k_wide_min_batch = v; }

// Returns 1 when this kernel took the product, 0 when the shape is outside its range, -1 on a launch error.
int launch_q4k_gemv_wide(const uint8_t* w, const float* x, float* y, int k, int n, int batch) {
    // 5 rows and more: with 3 and 4 the kernel on the 4 x 4 x 4 instruction is the faster one (it does half the matrix
    // work for them, this one the same vector work as for 8)
    if (!g_q4k_wide_enable.load() || batch < g_q4k_wide_min_batch.load() || batch > 8 || k != WD_K || n < 1) return 0;
    if ((reinterpret_cast<uintptr_t>(w) & 15) || (reinterpret_cast<uintptr_t>(x) & 15)) return 0;
    if ((uint64_t)(n + 256) * (uint64_t)(k >> 8) * Q4K_BYTES >= ((uint64_t)1 << 32)) return 0;     // 32-bit weight offsets
    // one round of workgroups over the chip where the row count allows: every workgroup the same number of rows
    // (so that every CU streams the same number of bytes), at most WD_MAX_UNITS units of 16
    int rows_per_wg = (n + num_cus() - 1) / num_cus();
    if (rows_per_wg > WD_MAX_UNITS * WD_UNIT_ROWS) rows_per_wg = WD_MAX_UNITS * WD_UNIT_ROWS;
    const int grid = (n + rows_per_wg - 1) / rows_per_wg;
    SKH_SET_MAX_DYNAMIC_LDS_ONCE((&q4k_gemv_wide_kernel), WD_SMEM);
    note_kernel("q4k_gemv_wide_kernel");
    q4k_gemv_wide_kernel<<<dim3(grid), dim3(64 * WD_WAVES), WD_SMEM, current_stream()>>>(w, x, y, n, batch, rows_per_wg);
    SKH_CHECK(hipGetLastError());
    return 1;
}

}  // namespace skh
