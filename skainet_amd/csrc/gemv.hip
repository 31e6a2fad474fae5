// Decode-time dequant-GEMV for GGUF Q4_K / Q6_K / Q8_0 weights in canonical row-major block order:
//   y[b, o] = sum_j x[b, j] * dequant(W[o, j])     b < batch <= 4 per launch, fp32 activations and sums.
//
// Semantics follow the reference's exact-fp32 kernels (same products, different summation order):
//   /root/reference/skainet-backends/skainet-backend-cpu/src/commonMain/kotlin/sk/ainet/exec/kernel/
//   ScalarQ4_KMatmulKernel.kt:40-78, ScalarQ6_KMatmulKernel.kt:33-44, ScalarQ8_0MatmulKernel.kt:41-62
// and the row-major weight addressing of the native entries
//   /root/reference/skainet-backends/skainet-backend-native-cpu/native/src/q4k_matmul.c:294-309.
//
// Mapping (HBM-bound, one pass over the weight, nothing staged in LDS):
//   * A weight row is cut into "slots" of SLOT_ELEMS consecutive-in-memory quants (Q4_K: one 16-byte
//     nibble chunk = 16 + 16 elements of two sub-blocks; Q6_K: 4 x 4 elements sharing 12 code bytes;
//     Q8_0: one 34-byte block). Lane l of wave s in a workgroup owns slot s * 64 + l of EVERY row the
//     workgroup processes, so the activation slice that slot needs lives in registers for the whole
//     kernel and each wave-wide load instruction covers one contiguous span of the row.
//   * Rows are streamed R at a time with all loads issued before the arithmetic; the R * B per-lane
//     partial sums are folded across the wave with a multi-value butterfly (log2(R*B) halving steps,
//     then plain xor-shuffles), written to LDS per (wave, row) and summed over the waves in a fixed
//     order, so results are deterministic.
//   * Grid: contiguous row ranges, sized so the whole chip gets an even share (rows_per_wg from the host).
#include "common.h"
#include <type_traits>

#include <cstring>

namespace skh {

constexpr int GEMV_MAX_WAVES = 8;    // waves per workgroup = K segments processed concurrently (2 per SIMD: 256 VGPRs each)
constexpr int GEMV_MAX_ROWS = 64;    // rows per workgroup (bounds the LDS partial-sum buffer)

// ---------------------------------------------------------------------------------------------- Q4_K
struct Q4KSlot {
    static constexpr int BLOCK_BYTES = Q4K_BYTES, SLOTS_PER_BLOCK = 8, SLOT_ELEMS = 32, NX = 32;
    struct Raw { uint4 hdr, qs; };
    struct Lane {
        int blk_off, qs_off;   // byte offsets inside a row
        int sh;                // bit offset of this slot's scale-byte pair inside the header dwords (0 or 16)
        uint32_t hi_mask;      // all ones when the slot's sub-blocks are 4..7 (split 6-bit packing), else 0
    };
    __device__ static void init(Lane& ln, int slot) {
        const int blk = slot >> 3, c = slot & 7;
        ln.blk_off = blk * BLOCK_BYTES;
        ln.qs_off = ln.blk_off + 16 + c * 16;
        ln.sh = ((c >> 1) & 1) * 16;
        ln.hi_mask = (c >> 1) >= 2 ? 0xFFFFFFFFu : 0u;
    }
    // Element index (inside the row) of activation register i for this slot: 16 of sub-block 2g then 16 of 2g+1.
    __device__ static int x_index(int slot, int i) {
        const int blk = slot >> 3, c = slot & 7;
        return blk * 256 + (c >> 1) * 64 + (c & 1) * 16 + (i >> 4) * 32 + (i & 15);
    }
    __device__ static void load(Raw& r, const uint8_t* row, const Lane& ln) {
        r.hdr = *reinterpret_cast<const uint4*>(row + ln.blk_off);
        r.qs = *reinterpret_cast<const uint4*>(row + ln.qs_off);
    }
    // xsum[0] = sum of the 16 low-nibble activations, xsum[1] = sum of the 16 high-nibble activations.
    __device__ static void prep(const float* x, float* xsum) {
        float a = 0.f, b = 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i) { a += x[i]; b += x[16 + i]; }
        xsum[0] = a; xsum[1] = b;
    }
    struct Scales { float dlo, dhi, mlo, mhi; };
    // The 6-bit (scale, min) pairs of sub-blocks 2g and 2g+1 (ggml get_scale_min_k4), folded with d / dmin.
    __device__ static Scales scales(const Raw& r, const Lane& ln) {
        const float d = half_bits_to_float_fast(r.hdr.x & 0xFFFFu), dmin = half_bits_to_float_fast(r.hdr.x >> 16);
        const uint32_t u = r.hdr.y >> ln.sh;   // low 16 bits: scale bytes s[2g'], s[2g'+1]
        const uint32_t v = r.hdr.z >> ln.sh;   // scale bytes s[4+2g'], s[5+2g']
        const uint32_t t = r.hdr.w >> ln.sh;   // scale bytes s[8+2g'], s[9+2g']
        // g < 2: (u & 0x3F3F, v & 0x3F3F); g >= 2: low nibbles of t / high nibbles of t, top two bits from u / v.
        // Both forms are evaluated and picked by the lane-constant mask, so no branch diverges.
        const uint32_t sc = ((u & 0x3F3Fu) & ~ln.hi_mask) | (((t & 0x0F0Fu) | ((u >> 2) & 0x3030u)) & ln.hi_mask);
        const uint32_t mn = ((v & 0x3F3Fu) & ~ln.hi_mask) | ((((t >> 4) & 0x0F0Fu) | ((v >> 2) & 0x3030u)) & ln.hi_mask);
        Scales s;
        s.dlo = d * ubyte0_to_float(sc);
        s.dhi = d * ubyte1_to_float(sc) * 0.0625f;   // high nibbles are accumulated as 16 * code
        s.mlo = dmin * ubyte0_to_float(mn);
        s.mhi = dmin * ubyte1_to_float(mn);
        return s;
    }
    template <int B>
    __device__ static void dot(const Raw& r, const Lane& ln, const float (*x)[NX], const float (*xsum)[2], float* acc) {
        const Scales s = scales(r, ln);
        const uint32_t q[4] = {r.qs.x, r.qs.y, r.qs.z, r.qs.w};
        float lo[B], hi[B];
#pragma unroll
        for (int b = 0; b < B; ++b) lo[b] = hi[b] = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t l4 = q[i] & 0x0F0F0F0Fu, h4 = q[i] & 0xF0F0F0F0u;
            const float cl[4] = {ubyte0_to_float(l4), ubyte1_to_float(l4), ubyte2_to_float(l4), ubyte3_to_float(l4)};
            const float ch[4] = {ubyte0_to_float(h4), ubyte1_to_float(h4), ubyte2_to_float(h4), ubyte3_to_float(h4)};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
#pragma unroll
                for (int b = 0; b < B; ++b) {
                    lo[b] = fmaf(x[b][i * 4 + j], cl[j], lo[b]);
                    hi[b] = fmaf(x[b][16 + i * 4 + j], ch[j], hi[b]);
                }
            }
        }
#pragma unroll
        for (int b = 0; b < B; ++b)
            acc[b] = s.dlo * lo[b] + s.dhi * hi[b] - (s.mlo * xsum[b][0] + s.mhi * xsum[b][1]);
    }
};

// ---------------------------------------------------------------------------------------------- Q6_K
struct Q6KSlot {
    // A slot is 32 weights: 8 consecutive positions l of one half of a super-block, in all four quarters (elements
    // half * 128 + 32 k + l). Their codes sit in three 8-byte runs (two of low / high nibbles, one of the two-bit
    // planes), read with one 8-byte load each; the half's eight scale bytes are a fourth.
    static constexpr int BLOCK_BYTES = Q6K_BYTES, SLOTS_PER_BLOCK = 8, SLOT_ELEMS = 32, NX = 32;
    struct Raw { u32x2_vec qla, qlb, qh, sc; uint32_t d; };
    struct Lane { int blk_off, ql_off, qh_off, sc_off, sc_shift; };
    __device__ static void init(Lane& ln, int slot) {
        const int blk = slot >> 3, t = slot & 7, half = t >> 2, l0 = (t & 3) * 8;
        ln.blk_off = blk * BLOCK_BYTES;
        ln.ql_off = ln.blk_off + half * 64 + l0;
        ln.qh_off = ln.blk_off + 128 + half * 32 + l0;
        ln.sc_off = ln.blk_off + 192 + half * 8;
        ln.sc_shift = (l0 >> 4) * 8;
    }
    // Register i = 8 * k + j pairs with element half*128 + 32*k + l0 + j.
    __device__ static int x_index(int slot, int i) {
        const int blk = slot >> 3, t = slot & 7, half = t >> 2, l0 = (t & 3) * 8;
        return blk * 256 + half * 128 + (i >> 3) * 32 + l0 + (i & 7);
    }
    __device__ static void load(Raw& r, const uint8_t* row, const Lane& ln) {
        r.qla = load_u32x2_a2(row + ln.ql_off);
        r.qlb = load_u32x2_a2(row + ln.ql_off + 32);
        r.qh = load_u32x2_a2(row + ln.qh_off);
        r.sc = load_u32x2_a2(row + ln.sc_off);
        r.d = load_u16(row + ln.blk_off + 208);
    }
    __device__ static void prep(const float* x, float* xsum) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            float s = 0.f;
#pragma unroll
            for (int j = 0; j < 8; ++j) s += x[8 * k + j];
            xsum[k] = 32.f * s;
        }
    }
    template <int B>
    __device__ static void dot(const Raw& r, const Lane& ln, const float (*x)[NX], const float (*xsum)[4], float* acc) {
        const float d = half_bits_to_float_fast(r.d);
        // signed scales of the four quarters: bytes is, is+2, is+4, is+6 of the half's 8 scale bytes
        const uint32_t s0 = r.sc.x >> ln.sc_shift, s1 = r.sc.y >> ln.sc_shift;
        const float sc[4] = {d * (float)(int8_t)(s0), d * (float)(int8_t)(s0 >> 16),
                             d * (float)(int8_t)(s1), d * (float)(int8_t)(s1 >> 16)};
        const uint32_t qla[2] = {r.qla.x, r.qla.y}, qlb[2] = {r.qlb.x, r.qlb.y}, qh[2] = {r.qh.x, r.qh.y};
        float s[4][B];
#pragma unroll
        for (int k = 0; k < 4; ++k)
#pragma unroll
            for (int b = 0; b < B; ++b) s[k][b] = -xsum[b][k];       // the -32 bias of every code, taken out of the loop
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const uint32_t c[4] = {
                (qla[h] & 0x0F0F0F0Fu) | ((qh[h] << 4) & 0x30303030u),
                (qlb[h] & 0x0F0F0F0Fu) | ((qh[h] << 2) & 0x30303030u),
                ((qla[h] >> 4) & 0x0F0F0F0Fu) | (qh[h] & 0x30303030u),
                ((qlb[h] >> 4) & 0x0F0F0F0Fu) | ((qh[h] >> 2) & 0x30303030u)};
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const float cf[4] = {ubyte0_to_float(c[k]), ubyte1_to_float(c[k]), ubyte2_to_float(c[k]), ubyte3_to_float(c[k])};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
#pragma unroll
                    for (int b = 0; b < B; ++b) s[k][b] = fmaf(x[b][8 * k + 4 * h + j], cf[j], s[k][b]);
                }
            }
        }
#pragma unroll
        for (int b = 0; b < B; ++b) {
            float a = 0.f;
#pragma unroll
            for (int k = 0; k < 4; ++k) a = fmaf(sc[k], s[k][b], a);
            acc[b] = a;
        }
    }
};

// Q6_K at batch 1: a slot is 64 weights -- 16 consecutive positions l of one half of a super-block in all four quarters
// (elements half * 128 + 32 k + l) -- so the three code runs are one 16-byte load each (2-byte aligned) instead of two
// slots of 8-byte loads: half the load instructions per weight. Four lanes per super-block; a 4096-wide row is one wave.
struct Q6KSlot64 {
    static constexpr int BLOCK_BYTES = Q6K_BYTES, SLOTS_PER_BLOCK = 4, SLOT_ELEMS = 64, NX = 64;
    struct Raw { u32x4_vec qla, qlb, qh; u32x2_vec sc; uint32_t d; };
    struct Lane { int blk_off, ql_off, qh_off, sc_off, sc_shift; };
    __device__ static void init(Lane& ln, int slot) {
        const int blk = slot >> 2, t = slot & 3, half = t >> 1, l0 = (t & 1) * 16;
        ln.blk_off = blk * BLOCK_BYTES;
        ln.ql_off = ln.blk_off + half * 64 + l0;
        ln.qh_off = ln.blk_off + 128 + half * 32 + l0;
        ln.sc_off = ln.blk_off + 192 + half * 8;
        ln.sc_shift = (l0 >> 4) * 8;
    }
    // Register i = 16 * k + j pairs with element half*128 + 32*k + l0 + j.
    __device__ static int x_index(int slot, int i) {
        const int blk = slot >> 2, t = slot & 3, half = t >> 1, l0 = (t & 1) * 16;
        return blk * 256 + half * 128 + (i >> 4) * 32 + l0 + (i & 15);
    }
    __device__ static void load(Raw& r, const uint8_t* row, const Lane& ln) {
        r.qla = load_u32x4_a2(row + ln.ql_off);
        r.qlb = load_u32x4_a2(row + ln.ql_off + 32);
        r.qh = load_u32x4_a2(row + ln.qh_off);
        r.sc = load_u32x2_a2(row + ln.sc_off);
        r.d = load_u16(row + ln.blk_off + 208);
    }
    __device__ static void prep(const float* x, float* xsum) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            float s = 0.f;
#pragma unroll
            for (int j = 0; j < 16; ++j) s += x[16 * k + j];
            xsum[k] = 32.f * s;
        }
    }
    template <int B>
    __device__ static void dot(const Raw& r, const Lane& ln, const float (*x)[NX], const float (*xsum)[4], float* acc) {
        const float d = half_bits_to_float_fast(r.d);
        const uint32_t s0 = r.sc.x >> ln.sc_shift, s1 = r.sc.y >> ln.sc_shift;
        const float sc[4] = {d * (float)(int8_t)(s0), d * (float)(int8_t)(s0 >> 16),
                             d * (float)(int8_t)(s1), d * (float)(int8_t)(s1 >> 16)};
        const uint32_t qla[4] = {r.qla.x, r.qla.y, r.qla.z, r.qla.w}, qlb[4] = {r.qlb.x, r.qlb.y, r.qlb.z, r.qlb.w},
                       qh[4] = {r.qh.x, r.qh.y, r.qh.z, r.qh.w};
        float s[4][B];
#pragma unroll
        for (int k = 0; k < 4; ++k)
#pragma unroll
            for (int b = 0; b < B; ++b) s[k][b] = -xsum[b][k];       // the -32 bias of every code, taken out of the loop
#pragma unroll
        for (int h = 0; h < 4; ++h) {
            const uint32_t c[4] = {
                (qla[h] & 0x0F0F0F0Fu) | ((qh[h] << 4) & 0x30303030u),
                (qlb[h] & 0x0F0F0F0Fu) | ((qh[h] << 2) & 0x30303030u),
                ((qla[h] >> 4) & 0x0F0F0F0Fu) | (qh[h] & 0x30303030u),
                ((qlb[h] >> 4) & 0x0F0F0F0Fu) | ((qh[h] >> 2) & 0x30303030u)};
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const float cf[4] = {ubyte0_to_float(c[k]), ubyte1_to_float(c[k]), ubyte2_to_float(c[k]), ubyte3_to_float(c[k])};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
#pragma unroll
                    for (int b = 0; b < B; ++b) s[k][b] = fmaf(x[b][16 * k + 4 * h + j], cf[j], s[k][b]);
                }
            }
        }
#pragma unroll
        for (int b = 0; b < B; ++b) {
            float a = 0.f;
#pragma unroll
            for (int k = 0; k < 4; ++k) a = fmaf(sc[k], s[k][b], a);
            acc[b] = a;
        }
    }
};

// ---------------------------------------------------------------------------------------------- Q8_0
struct Q80Slot {
    static constexpr int BLOCK_BYTES = Q80_BYTES, SLOTS_PER_BLOCK = 1, SLOT_ELEMS = 32, NX = 32;
    // A 34-byte block starts 0 or 2 bytes past a dword boundary. Its aligned 32-byte body (bytes 0..31 of the block
    // when it starts on a boundary, bytes 2..33 otherwise) comes in as two 16-byte loads, the two bytes outside the
    // body (the last code pair, or the scale) as one 2-byte load: three loads per block, none outside the block.
    struct Raw { u32x4_vec lo, hi; uint32_t edge; uint32_t odd; };
    struct Lane { int blk_off; };
    __device__ static void init(Lane& ln, int slot) { ln.blk_off = slot * BLOCK_BYTES; }
    __device__ static int x_index(int slot, int i) { return slot * 32 + i; }
    __device__ static void load(Raw& r, const uint8_t* row, const Lane& ln) {
        const uint8_t* p = row + ln.blk_off;
        const uint32_t odd = (uint32_t)(reinterpret_cast<uintptr_t>(p) >> 1) & 1u;   // 1: the block starts 2 bytes past a boundary
        const uint8_t* body = p + 2 * odd;
        r.lo = load_u32x4_a4(body);
        r.hi = load_u32x4_a4(body + 16);
        r.edge = load_u16(p + (odd ? 0 : 32));
        r.odd = odd;
    }
    // The block's scale bits and its eight code dwords from the three loads.
    __device__ static uint32_t unpack(const Raw& r, uint32_t* q) {
        const uint32_t v[9] = {r.lo.x, r.lo.y, r.lo.z, r.lo.w, r.hi.x, r.hi.y, r.hi.z, r.hi.w, r.edge};
        const uint32_t sh = r.odd ? 0u : 2u;                 // bytes to drop in front of the codes
#pragma unroll
        for (int i = 0; i < 8; ++i) q[i] = __builtin_amdgcn_alignbyte(v[i + 1], v[i], sh);
        return r.odd ? r.edge : (r.lo.x & 0xFFFFu);
    }
    __device__ static void prep(const float*, float*) {}
    template <int B>
    __device__ static void dot(const Raw& r, const Lane&, const float (*x)[NX], const float (*)[1], float* acc) {
        uint32_t q[8];
        const float d = half_bits_to_float_fast(unpack(r, q));
        float s[B];
#pragma unroll
        for (int b = 0; b < B; ++b) s[b] = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float cf = (float)(int8_t)(q[i] >> (8 * j));
#pragma unroll
                for (int b = 0; b < B; ++b) s[b] = fmaf(x[b][i * 4 + j], cf, s[b]);
            }
        }
#pragma unroll
        for (int b = 0; b < B; ++b) acc[b] = s[b] * d;
    }
};

// ------------------------------------------------------------------------------- Q4_0 / Q5_0 / Q5_1
// 32-element blocks: fp16 d [fp16 m] [32 fifth bits] 16 bytes of nibbles (low nibbles: elements 0..15, high: 16..31).
// Semantics of ScalarQ4_0MatmulKernel.kt:29-63, ScalarQ5_0MatmulKernel.kt, ScalarQ5_1MatmulKernel.kt (same directory as
// the kernels cited at the top) with the code bias and the Q5_1 minimum taken out of the inner loop:
//   Q4_0  d * (sum code x - 8 sum x)     Q5_0  d * (sum code5 x - 16 sum x)     Q5_1  d * sum code5 x + m * sum x
// The fifth bits of four adjacent elements are spread into bit 4 of the four code bytes with one multiply.
template <int FMT>   // 0 = Q4_0, 1 = Q5_0, 2 = Q5_1
struct Q45Slot {
    static constexpr int BLOCK_BYTES = FMT == 0 ? Q40_BYTES : (FMT == 1 ? Q50_BYTES : Q51_BYTES);
    static constexpr int SLOTS_PER_BLOCK = 1, SLOT_ELEMS = 32, NX = 32;
    static constexpr int QH = FMT == 2 ? 4 : 2, QS = FMT == 0 ? 2 : QH + 4;
    struct Raw { uint32_t d, m, qh, q[4]; };
    struct Lane { int blk_off; };
    __device__ static void init(Lane& ln, int slot) { ln.blk_off = slot * BLOCK_BYTES; }
    __device__ static int x_index(int slot, int i) { return slot * 32 + i; }
    __device__ static void load(Raw& r, const uint8_t* row, const Lane& ln) {
        const uint8_t* p = row + ln.blk_off;                  // 2-byte aligned (Q5_1: 8)
        r.d = load_u16(p);
        r.m = FMT == 2 ? load_u16(p + 2) : 0u;
        r.qh = FMT != 0 ? load_u32_a2(p + QH) : 0u;
        const u32x4_vec q4 = load_u32x4_a2(p + QS);          // the 16 code bytes as one load (2-byte aligned)
        r.q[0] = q4.x; r.q[1] = q4.y; r.q[2] = q4.z; r.q[3] = q4.w;
    }
    __device__ static void prep(const float* x, float* xsum) {
        float a = 0.f;
#pragma unroll
        for (int i = 0; i < 32; ++i) a += x[i];
        xsum[0] = a;
    }
    template <int B>
    __device__ static void dot(const Raw& r, const Lane&, const float (*x)[NX], const float (*xsum)[1], float* acc) {
        const float d = half_bits_to_float_fast(r.d);
        float s[B];
#pragma unroll
        for (int b = 0; b < B; ++b) s[b] = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t l4 = r.q[i] & 0x0F0F0F0Fu, h4 = (r.q[i] >> 4) & 0x0F0F0F0Fu;
            if (FMT != 0) {
                l4 |= ((((r.qh >> (4 * i)) & 0xFu) * 0x00204081u) & 0x01010101u) << 4;
                h4 |= ((((r.qh >> (16 + 4 * i)) & 0xFu) * 0x00204081u) & 0x01010101u) << 4;
            }
            const float cl[4] = {ubyte0_to_float(l4), ubyte1_to_float(l4), ubyte2_to_float(l4), ubyte3_to_float(l4)};
            const float ch[4] = {ubyte0_to_float(h4), ubyte1_to_float(h4), ubyte2_to_float(h4), ubyte3_to_float(h4)};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
#pragma unroll
                for (int b = 0; b < B; ++b) {
                    s[b] = fmaf(x[b][i * 4 + j], cl[j], s[b]);
                    s[b] = fmaf(x[b][16 + i * 4 + j], ch[j], s[b]);
                }
            }
        }
#pragma unroll
        for (int b = 0; b < B; ++b) {
            if (FMT == 0) acc[b] = d * (s[b] - 8.f * xsum[b][0]);
            else if (FMT == 1) acc[b] = d * (s[b] - 16.f * xsum[b][0]);
            else acc[b] = d * s[b] + half_bits_to_float_fast(r.m) * xsum[b][0];
        }
    }
};

// ---------------------------------------------------------------------------------------------- Q5_K
// The Q4_K slot (one 16-byte nibble chunk = 16 + 16 elements of sub-blocks 2g and 2g + 1) plus the matching 16 bytes
// of the fifth-bit plane: bit 2g of byte l belongs to element l of sub-block 2g, bit 2g + 1 to sub-block 2g + 1.
// Block: d, dmin, 12 scale bytes, 32 bytes qh at 16, 128 bytes of nibbles at 48 (176 bytes);
// semantics of ScalarQ5_KMatmulKernel.kt (per sub-block codeSum * (d * sc) - inputSum * (dmin * m)).
struct Q5KSlot {
    static constexpr int BLOCK_BYTES = Q5K_BYTES, SLOTS_PER_BLOCK = 8, SLOT_ELEMS = 32, NX = 32;
    struct Raw { uint4 hdr, qs, qh; };
    struct Lane { int blk_off, qs_off, qh_off, sh, bit; uint32_t hi_mask; };
    __device__ static void init(Lane& ln, int slot) {
        const int blk = slot >> 3, c = slot & 7;
        ln.blk_off = blk * BLOCK_BYTES;
        ln.qs_off = ln.blk_off + 48 + c * 16;
        ln.qh_off = ln.blk_off + 16 + (c & 1) * 16;
        ln.sh = ((c >> 1) & 1) * 16;
        ln.bit = 2 * (c >> 1);
        ln.hi_mask = (c >> 1) >= 2 ? 0xFFFFFFFFu : 0u;
    }
    __device__ static int x_index(int slot, int i) { return Q4KSlot::x_index(slot, i); }
    __device__ static void load(Raw& r, const uint8_t* row, const Lane& ln) {
        r.hdr = *reinterpret_cast<const uint4*>(row + ln.blk_off);
        r.qs = *reinterpret_cast<const uint4*>(row + ln.qs_off);
        r.qh = *reinterpret_cast<const uint4*>(row + ln.qh_off);
    }
    __device__ static void prep(const float* x, float* xsum) { Q4KSlot::prep(x, xsum); }
    template <int B>
    __device__ static void dot(const Raw& r, const Lane& ln, const float (*x)[NX], const float (*xsum)[2], float* acc) {
        Q4KSlot::Raw r4{r.hdr, r.qs};
        Q4KSlot::Lane l4{0, 0, ln.sh, ln.hi_mask};
        const Q4KSlot::Scales s = Q4KSlot::scales(r4, l4);      // dhi carries the 1/16 of a high nibble kept in place
        const uint32_t q[4] = {r.qs.x, r.qs.y, r.qs.z, r.qs.w};
        const uint32_t h[4] = {r.qh.x, r.qh.y, r.qh.z, r.qh.w};
        float lo[B], hi[B];
#pragma unroll
        for (int b = 0; b < B; ++b) lo[b] = hi[b] = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t hb = h[i] >> ln.bit;
            const uint32_t l5 = (q[i] & 0x0F0F0F0Fu) | ((hb & 0x01010101u) << 4);
            const uint32_t h5 = ((q[i] >> 4) & 0x0F0F0F0Fu) | (((hb >> 1) & 0x01010101u) << 4);
            const float cl[4] = {ubyte0_to_float(l5), ubyte1_to_float(l5), ubyte2_to_float(l5), ubyte3_to_float(l5)};
            const float ch[4] = {ubyte0_to_float(h5), ubyte1_to_float(h5), ubyte2_to_float(h5), ubyte3_to_float(h5)};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
#pragma unroll
                for (int b = 0; b < B; ++b) {
                    lo[b] = fmaf(x[b][i * 4 + j], cl[j], lo[b]);
                    hi[b] = fmaf(x[b][16 + i * 4 + j], ch[j], hi[b]);
                }
            }
        }
#pragma unroll
        for (int b = 0; b < B; ++b)
            acc[b] = s.dlo * lo[b] + 16.f * s.dhi * hi[b] - (s.mlo * xsum[b][0] + s.mhi * xsum[b][1]);
    }
};

template <class F> struct XSumCount { static constexpr int N = 1; };
template <> struct XSumCount<Q4KSlot> { static constexpr int N = 2; };
template <> struct XSumCount<Q6KSlot> { static constexpr int N = 4; };
template <> struct XSumCount<Q6KSlot64> { static constexpr int N = 4; };
template <> struct XSumCount<Q5KSlot> { static constexpr int N = 2; };

// F: slot policy, B: activation rows per launch (1, 2 or 4; unused ones are zero), R: weight rows in flight.
template <class F, int B, int R>
__global__ __launch_bounds__(64 * GEMV_MAX_WAVES) void gemv_kernel(
    const uint8_t* __restrict__ w, const float* __restrict__ x, float* __restrict__ y,
    int k, int n, int batch, int64_t row_bytes, int rows_per_wg) {
    constexpr int NX = F::NX, NS = XSumCount<F>::N;
    constexpr int NV = (R * B <= 2) ? 2 : (R * B <= 4) ? 4 : (R * B <= 8) ? 8 : 16;   // fold width: the next power of two, zero padded
    static_assert(R * B <= 16, "at most 16 values per fold");
    __shared__ float partial[GEMV_MAX_WAVES][GEMV_MAX_ROWS][B];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
    const int nslots = k / F::SLOT_ELEMS;
    const int nseg = (nslots + 63) >> 6;
    const int r0 = blockIdx.x * rows_per_wg;
    const int r1 = min(n, r0 + rows_per_wg);
    const int nrows = r1 - r0;
    if (nrows <= 0) return;
    const uint8_t* wbase = w + (int64_t)r0 * row_bytes;
    const int my_value = wave_fold_index<NV>(lane);

    for (int seg = wave, pass = 0; seg < nseg; seg += nwaves, ++pass) {
        const int slot = seg * 64 + lane;
        const bool active = slot < nslots;
        typename F::Lane ln;
        F::init(ln, active ? slot : 0);

        // The activation slice is requested first and unconditionally (clamped address, zeroed afterwards), the first
        // R rows of weights right behind it: loads return in issue order, so the L2-resident activations must not
        // queue behind the weight stream, and a branch around a load would make the wave wait for every load in flight.
        float xs[B][NX], xsum[B][NS];
        const int xslot = active ? slot : 0;
#pragma unroll
        for (int b = 0; b < B; ++b) {
            const float* xb = x + (int64_t)(b < batch ? b : 0) * k;
#pragma unroll
            for (int i = 0; i < NX; i += 4) {
                const float4 v = *reinterpret_cast<const float4*>(xb + F::x_index(xslot, i));
                xs[b][i] = v.x; xs[b][i + 1] = v.y; xs[b][i + 2] = v.z; xs[b][i + 3] = v.w;
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        typename F::Raw raw[R];
#pragma unroll
        for (int i = 0; i < R; ++i) F::load(raw[i], wbase + (int64_t)min(i, nrows - 1) * row_bytes, ln);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int b = 0; b < B; ++b) {
            const float keep = (active && b < batch) ? 1.0f : 0.0f;
#pragma unroll
            for (int i = 0; i < NX; ++i) xs[b][i] *= keep;
            F::prep(xs[b], xsum[b]);
        }

        for (int r = 0; r < nrows; r += R) {
            float acc[NV];
#pragma unroll
            for (int i = R * B; i < NV; ++i) acc[i] = 0.f;
#pragma unroll
            for (int i = 0; i < R; ++i) {
                float a[B];
#pragma unroll
                for (int b = 0; b < B; ++b) a[b] = 0.f;
                if (r + i < nrows) F::template dot<B>(raw[i], ln, xs, xsum, a);   // wave-uniform: no arithmetic on padding rows
#pragma unroll
                for (int b = 0; b < B; ++b) acc[i * B + b] = active ? a[b] : 0.f;
                // refill this register set with the row R ahead (clamped: a repeated last row is discarded)
                F::load(raw[i], wbase + (int64_t)min(r + R + i, nrows - 1) * row_bytes, ln);
            }
            wave_fold<NV>(acc, lane);
            if (lane < NV) {
                const int i = my_value / B, b = my_value % B;
                if (i < R && r + i < nrows) {
                    float* dst = &partial[wave][r + i][b];
                    *dst = pass == 0 ? acc[0] : *dst + acc[0];
                }
            }
        }
    }
    __syncthreads();
    const int used_waves = min(nwaves, nseg);
    for (int t = threadIdx.x; t < nrows * B; t += blockDim.x) {
        const int rr = t / B, b = t % B;
        if (b >= batch) continue;
        float s = 0.f;
        for (int wv = 0; wv < used_waves; ++wv) s += partial[wv][rr][b];
        y[(int64_t)b * n + r0 + rr] = s;
    }
}

template <class F, int B, int R>
static int launch_one(const uint8_t* w, const float* x, float* y, int k, int n, int batch, int waves_per_cu) {
    const int nslots = k / F::SLOT_ELEMS;
    const int nseg = (nslots + 63) / 64;
    const int nwaves = nseg < GEMV_MAX_WAVES ? nseg : GEMV_MAX_WAVES;
    const int64_t row_bytes = (int64_t)(k / (F::SLOT_ELEMS * F::SLOTS_PER_BLOCK)) * F::BLOCK_BYTES;
    // Even contiguous row shares: about waves_per_cu resident waves on every CU.
    int target_wgs = (num_cus() * waves_per_cu) / nwaves;
    if (target_wgs < 1) target_wgs = 1;
    int rows_per_wg = (n + target_wgs - 1) / target_wgs;
    if (rows_per_wg < 1) rows_per_wg = 1;
    if (rows_per_wg > GEMV_MAX_ROWS) rows_per_wg = GEMV_MAX_ROWS;
    const int grid = (n + rows_per_wg - 1) / rows_per_wg;
    note_kernel("gemv_kernel");
    gemv_kernel<F, B, R><<<dim3(grid), dim3(64 * nwaves), 0, current_stream()>>>(w, x, y, k, n, batch, row_bytes, rows_per_wg);
    SKH_CHECK(hipGetLastError());
    return 0;
}

// Weight rows a wave keeps in flight at batch 1, per format (measured over 2 .. 8 on the 11008 x 4096, 32000 x 4096 and
// 4096 x 4096 shapes: the formats with many loads per row are faster with fewer rows requested at once).
template <class F> struct RowsInFlight { static constexpr int B1 = 8; };
template <> struct RowsInFlight<Q80Slot> { static constexpr int B1 = 3; };
template <> struct RowsInFlight<Q6KSlot> { static constexpr int B1 = 2; };
template <> struct RowsInFlight<Q5KSlot> { static constexpr int B1 = 3; };

static std::atomic<int> g_gemv_waves_per_cu{0};   // 0: per encoding (measured best: Q8_0 4, Q6_K at batch 1 6, the others 8)
static std::atomic<int> g_q6k_slot64{1};   // 0: Q6_K at batch 1 stays on the 32-weight slot

template <class F>
static int launch_format(const uint8_t* w, const float* x, float* y, int k, int n, int batch, int waves_per_cu) {
    if (batch == 1) {
        // Q6_K: the 64-weight slot, 2 rows in flight, 6 waves per CU unless the caller set a count (measured on 32000 x 4096
        // over 1 .. 4 rows and 5 .. 16 waves: 23.1 us against 25.5 us for the 32-weight slot at its best, 2 rows and 8 waves)
        if (std::is_same<F, Q6KSlot>::value && g_q6k_slot64)
            return launch_one<Q6KSlot64, 1, 2>(w, x, y, k, n, batch, g_gemv_waves_per_cu.load() > 0 ? g_gemv_waves_per_cu.load() : 6);
        return launch_one<F, 1, RowsInFlight<F>::B1>(w, x, y, k, n, batch, waves_per_cu);
    }
    if (batch == 2) return launch_one<F, 2, 4>(w, x, y, k, n, batch, waves_per_cu);
    return launch_one<F, 4, 2>(w, x, y, k, n, batch, waves_per_cu);
}

static std::atomic<int> g_q4k_rows_enable{1};
void set_q4k_rows_waves_per_cu(int v);
void set_gemm_wide(int v);
void set_gemm_ksplit(int v);
void set_gemm_rows(int v);
void set_gemm_ksw(int v);
void set_gemm_ksw_teams(int v);
void set_gemm_ksw_stages(int v);
void set_sdpa_prefill_mfma(int v);
void set_sdpa_decode_split_keys(int v);
void set_q4k_ksplit_enable(int v);
void set_q4k_mfma_enable(int v);
void set_q4k_mfma_window(int v);
void set_attn_merge_enable(int v);
void set_sdpa_decode_gs(int v);
void set_attn_merge_max_keys(int v);
void set_attn_merge_splits(int v);
int launch_q4k_gemv_rows(const uint8_t* w, const float* x, float* y, int k, int n, int batch);   // gemv_q4k.hip
int launch_q4k_gemv_quads(const uint8_t* w, const float* x, float* y, int k, int n, int batch);  // gemv_q4k_quads.hip

// Experiment knobs (defaults are the measured best): returns 0 when the key is known.
int set_tuning(const char* key, int value) {
    if (!strcmp(key, "gemv_waves_per_cu")) { if (value >= 0) g_gemv_waves_per_cu = value; return 0; }
    if (!strcmp(key, "q4k_rows_waves_per_cu")) { set_q4k_rows_waves_per_cu(value); return 0; }
    if (!strcmp(key, "q6k_slot64")) { g_q6k_slot64 = value != 0; return 0; }
    if (!strcmp(key, "gemm_wide")) { set_gemm_wide(value); return 0; }
    if (!strcmp(key, "q4k_rows_enable")) { g_q4k_rows_enable = value; return 0; }
    if (!strcmp(key, "gemm_ksplit")) { set_gemm_ksplit(value); return 0; }
    if (!strcmp(key, "gemm_rows")) { set_gemm_rows(value); return 0; }
    if (!strcmp(key, "gemm_ksw")) { set_gemm_ksw(value); return 0; }
    if (!strcmp(key, "gemm_ksw_teams")) { set_gemm_ksw_teams(value); return 0; }
    if (!strcmp(key, "gemm_ksw_stages")) { set_gemm_ksw_stages(value); return 0; }
    if (!strcmp(key, "sdpa_prefill_mfma")) { set_sdpa_prefill_mfma(value); return 0; }
    if (!strcmp(key, "q4k_ksplit_enable")) { set_q4k_ksplit_enable(value); return 0; }
    if (!strcmp(key, "q4k_mfma_enable")) { set_q4k_mfma_enable(value); return 0; }
    if (!strcmp(key, "q4k_mfma_window")) { set_q4k_mfma_window(value); return 0; }
    if (!strcmp(key, "sdpa_decode_split_keys")) { set_sdpa_decode_split_keys(value); return 0; }
    if (!strcmp(key, "attn_merge_enable")) { set_attn_merge_enable(value); return 0; }
    if (!strcmp(key, "sdpa_decode_gs")) { set_sdpa_decode_gs(value); return 0; }
    if (!strcmp(key, "attn_merge_max_keys")) { set_attn_merge_max_keys(value); return 0; }
    if (!strcmp(key, "attn_merge_splits")) { set_attn_merge_splits(value); return 0; }
    return -1;
}

// y[m, n] = x[m, k] . W^T for m activation rows, at most 4 per pass over the weight.
int launch_gemv(int enc, const uint8_t* w, const float* x, int m, int k, int n, float* y) {
    if (m <= 0 || n <= 0) return 0;
    if (!is_packed(enc)) return set_error("gemv: unsupported encoding %d", enc);
    if (k <= 0 || k % block_elems(enc) != 0)
        return set_error("gemv: inputDim must be a positive multiple of %d; got %d", block_elems(enc), k);
    const int waves_per_cu = g_gemv_waves_per_cu.load() > 0 ? g_gemv_waves_per_cu.load() : (block_elems(enc) == 32 ? 4 : 8);
    for (int b0 = 0; b0 < m;) {
        const int left = m - b0;
        const float* xb = x + (int64_t)b0 * k;
        float* yb = y + (int64_t)b0 * n;
        int rc;
        if (enc == ENC_Q4_K && g_q4k_rows_enable) {
            // 3 to 8 rows: the fp32 matrix-instruction kernel; 1 or 2: the row-streaming kernel
            const int nq = left < 8 ? left : 8;
            rc = left >= 3 ? launch_q4k_gemv_quads(w, xb, yb, k, n, nq) : launch_q4k_gemv_rows(w, xb, yb, k, n, left);
            if (rc < 0) return rc;
            if (rc == 1) { b0 += left >= 3 ? nq : left; continue; }
        }
        const int nb = left < 4 ? left : 4;
        if (enc == ENC_Q4_K) rc = launch_format<Q4KSlot>(w, xb, yb, k, n, nb, waves_per_cu);
        else if (enc == ENC_Q6_K) rc = launch_format<Q6KSlot>(w, xb, yb, k, n, nb, waves_per_cu);
        else if (enc == ENC_Q5_K) rc = launch_format<Q5KSlot>(w, xb, yb, k, n, nb, waves_per_cu);
        else if (enc == ENC_Q4_0) rc = launch_format<Q45Slot<0>>(w, xb, yb, k, n, nb, waves_per_cu);
        else if (enc == ENC_Q5_0) rc = launch_format<Q45Slot<1>>(w, xb, yb, k, n, nb, waves_per_cu);
        else if (enc == ENC_Q5_1) rc = launch_format<Q45Slot<2>>(w, xb, yb, k, n, nb, waves_per_cu);
        else rc = launch_format<Q80Slot>(w, xb, yb, k, n, nb, waves_per_cu);
        if (rc != 0) return rc;
        b0 += nb;
    }
    return 0;
}

}  // namespace skh
