// Slot policies of the dequant-GEMV kernels: how one lane's share of a weight row ("slot": SLOT_ELEMS consecutive-in-
// memory quants of one block) is addressed, loaded, and multiplied with the activations the lane keeps in registers.
// Shared by the row kernel that reads weights straight from memory (gemv.hip) and the one that streams them through
// LDS (gemv_stream.hip): `load` takes a pointer to the row's first byte in either address space.
//   struct F { BLOCK_BYTES, SLOTS_PER_BLOCK, SLOT_ELEMS, NX (activations per slot);  Raw (a slot's bytes), Lane (offsets);
//              init(Lane&, slot); x_index(slot, i); load(Raw&, row, Lane); prep(x, xsum); dot<B>(Raw, Lane, x, xsum, acc) }
// Semantics follow the reference's exact-fp32 kernels (same products, different summation order):
//   /root/reference/skainet-backends/skainet-backend-cpu/src/commonMain/kotlin/sk/ainet/exec/kernel/
//   ScalarQ4_KMatmulKernel.kt:40-78, ScalarQ6_KMatmulKernel.kt:33-44, ScalarQ8_0MatmulKernel.kt:41-62
#pragma once
#include "common.h"

namespace skh {

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

}  // namespace skh
