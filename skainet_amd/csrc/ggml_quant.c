/*
 * Host-side GGUF block quantizers: fp32 -> Q8_0 / Q4_K / Q6_K bytes in canonical row-major order.
 *
 * These produce the packed weights the device kernels consume (load-time work, never on the
 * per-token path). Q8_0 follows the reference's quantizer
 *   /root/reference/skainet-lang/skainet-lang-core/src/commonMain/kotlin/sk/ainet/lang/tensor/data/Q8_0Quantizer.kt:28-53
 * (d = amax/127 stored as fp16 RNE, inverse taken from the unrounded d, round-half-up, clamp +-127).
 *
 * The reference has no Q4_K / Q6_K quantizer
 *   (.../lang/tensor/data/Requantizers.kt:21-24 supports only Q8_0 and Q4_0),
 * so those two follow the published ggml algorithm (quantize_row_q4_K_ref / quantize_row_q6_K_ref:
 * per-sub-block weighted least-squares scale search, 6-bit scale/min packing, re-quantisation
 * against the decoded scales). Their parity with ggml is unpinned; the tests pin them through the
 * bit-exact decoder instead (valid blocks, round trip within one code step, idempotence).
 *
 * Q4_0 follows the reference's quantizer (.../lang/tensor/data/Q4_0Quantizer.kt:28-66 and its own fp16 rounding, :91-118);
 * Q5_0 / Q5_1 / Q5_K follow ggml's quantize_row_q5_0_ref / q5_1_ref / q5_K_ref (the reference has none): parity with ggml
 * unpinned, pinned through the decoder like the other K-quants.
 *
 * Threads: OpenMP over super-blocks; output is independent of the thread count.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#define QAPI __attribute__((visibility("default")))

static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* fp32 -> fp16 bits, round-to-nearest-even with gradual underflow. */
static uint16_t f2h(float value) {
    const uint32_t bits = f32_bits(value);
    const uint32_t sign = (bits >> 16) & 0x8000u;
    const uint32_t a = bits & 0x7FFFFFFFu;
    if (a >= 0x7F800000u) return (uint16_t)(a == 0x7F800000u ? (sign | 0x7C00u) : (sign | 0x7E00u | ((a >> 13) & 0x3FFu)));
    const int e = (int)(a >> 23) - 127;
    const uint32_t m = a & 0x7FFFFFu;
    if (e >= 16) return (uint16_t)(sign | 0x7C00u);
    if (e >= -14) {
        uint32_t h = ((uint32_t)(e + 15) << 10) | (m >> 13);
        const uint32_t rem = m & 0x1FFFu;
        if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) ++h;
        return (uint16_t)(sign | h);
    }
    if (e < -25) return (uint16_t)sign;
    const uint32_t full = m | 0x800000u;
    const int shift = -1 - e;
    uint32_t q = full >> shift;
    const uint32_t rem = full & ((1u << shift) - 1u), hb = 1u << (shift - 1);
    if (rem > hb || (rem == hb && (q & 1u))) ++q;
    return (uint16_t)(sign | q);
}

static float h2f(uint16_t h) {
    const uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 0x1Fu;
    uint32_t m = h & 0x3FFu;
    if (e == 0) {
        if (m == 0) return bits_f32(sign);
        int ex = -14;
        while (!(m & 0x400u)) { m <<= 1; --ex; }
        return bits_f32(sign | ((uint32_t)(ex + 127) << 23) | ((m & 0x3FFu) << 13));
    }
    if (e == 31) return bits_f32(sign | 0x7F800000u | (m << 13));
    return bits_f32(sign | ((e + 112u) << 23) | (m << 13));
}

/* Round half to even for |f| < 2^22 via the 1.5*2^23 magic constant. */
static inline int nearest_int(float f) {
    const float v = f + 12582912.f;
    return (int)(f32_bits(v) & 0x007FFFFFu) - 0x00400000;
}

/* ---------------------------------------------------------------- Q8_0 */

QAPI void skainet_quantize_q8_0(const float* x, int64_t n, uint8_t* out) {
    const int64_t blocks = n / 32;
#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < blocks; ++b) {
        const float* v = x + b * 32;
        uint8_t* o = out + b * 34;
        float amax = 0.f;
        for (int i = 0; i < 32; ++i) { const float a = fabsf(v[i]); if (a > amax) amax = a; }
        const float d = amax / 127.f;
        const float id = d != 0.f ? 1.f / d : 0.f;
        const uint16_t h = f2h(d);
        o[0] = (uint8_t)(h & 0xFF); o[1] = (uint8_t)(h >> 8);
        for (int i = 0; i < 32; ++i) {
            int q = (int)floor((double)(v[i] * id) + 0.5);
            if (q < -127) q = -127; else if (q > 127) q = 127;
            o[2 + i] = (uint8_t)(int8_t)q;
        }
    }
}

/* ---------------------------------------------------------------- Q4_K */

/* Weighted least-squares (scale, min) for n values quantised to 0..nmax; returns scale, *the_min = -min. */
static float make_qkx2(int n, int nmax, const float* x, const float* w, uint8_t* L, float* the_min,
                       uint8_t* Laux, float rmin, float rdelta, int nstep) {
    float mn = x[0], mx = x[0], sum_w = w[0], sum_x = w[0] * x[0];
    for (int i = 1; i < n; ++i) {
        if (x[i] < mn) mn = x[i];
        if (x[i] > mx) mx = x[i];
        sum_w += w[i]; sum_x += w[i] * x[i];
    }
    if (mn > 0) mn = 0;
    if (mx == mn) { for (int i = 0; i < n; ++i) L[i] = 0; *the_min = -mn; return 0.f; }
    float iscale = nmax / (mx - mn), scale = 1 / iscale, best = 0;
    for (int i = 0; i < n; ++i) {
        int l = nearest_int(iscale * (x[i] - mn));
        l = l < 0 ? 0 : (l > nmax ? nmax : l);
        L[i] = (uint8_t)l;
        const float diff = scale * l + mn - x[i];
        best += w[i] * diff * diff;
    }
    for (int is = 0; is <= nstep; ++is) {
        iscale = (rmin + rdelta * is + nmax) / (mx - mn);
        float sum_l = 0, sum_l2 = 0, sum_xl = 0;
        for (int i = 0; i < n; ++i) {
            int l = nearest_int(iscale * (x[i] - mn));
            l = l < 0 ? 0 : (l > nmax ? nmax : l);
            Laux[i] = (uint8_t)l;
            sum_l += w[i] * l; sum_l2 += w[i] * l * l; sum_xl += w[i] * l * x[i];
        }
        const float D = sum_w * sum_l2 - sum_l * sum_l;
        if (D > 0) {
            float this_scale = (sum_w * sum_xl - sum_x * sum_l) / D;
            float this_min = (sum_l2 * sum_x - sum_l * sum_xl) / D;
            if (this_min > 0) { this_min = 0; this_scale = sum_xl / sum_l2; }
            float err = 0;
            for (int i = 0; i < n; ++i) { const float diff = this_scale * Laux[i] + this_min - x[i]; err += w[i] * diff * diff; }
            if (err < best) { memcpy(L, Laux, (size_t)n); best = err; scale = this_scale; mn = this_min; }
        }
    }
    *the_min = -mn;
    return scale;
}

static inline void scale_min_k4(int j, const uint8_t* q, int* d, int* m) {
    if (j < 4) { *d = q[j] & 63; *m = q[j + 4] & 63; }
    else { *d = (q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4); *m = (q[j + 4] >> 4) | ((q[j] >> 6) << 4); }
}

QAPI void skainet_quantize_q4k(const float* xin, int64_t n, uint8_t* out) {
    const int64_t nb = n / 256;
#pragma omp parallel for schedule(static)
    for (int64_t ib = 0; ib < nb; ++ib) {
        const float* x = xin + ib * 256;
        uint8_t* y = out + ib * 144;
        uint8_t L[256], Laux[32];
        float weights[32], mins[8], scales[8];
        float max_scale = 0, max_min = 0;
        for (int j = 0; j < 8; ++j) {
            float sum_x2 = 0;
            for (int l = 0; l < 32; ++l) sum_x2 += x[32 * j + l] * x[32 * j + l];
            const float av = sqrtf(sum_x2 / 32);
            for (int l = 0; l < 32; ++l) weights[l] = av + fabsf(x[32 * j + l]);
            scales[j] = make_qkx2(32, 15, x + 32 * j, weights, L + 32 * j, &mins[j], Laux, -1.f, 0.1f, 20);
            if (scales[j] > max_scale) max_scale = scales[j];
            if (mins[j] > max_min) max_min = mins[j];
        }
        const float inv_scale = max_scale > 0 ? 63.f / max_scale : 0.f;
        const float inv_min = max_min > 0 ? 63.f / max_min : 0.f;
        uint8_t* sc = y + 4;
        memset(sc, 0, 12);
        for (int j = 0; j < 8; ++j) {
            int ls = nearest_int(inv_scale * scales[j]);
            int lm = nearest_int(inv_min * mins[j]);
            ls = ls > 63 ? 63 : (ls < 0 ? 0 : ls);
            lm = lm > 63 ? 63 : (lm < 0 ? 0 : lm);
            if (j < 4) { sc[j] = (uint8_t)ls; sc[j + 4] = (uint8_t)lm; }
            else {
                sc[j + 4] = (uint8_t)((ls & 0xF) | ((lm & 0xF) << 4));
                sc[j - 4] |= (uint8_t)((ls >> 4) << 6);
                sc[j] |= (uint8_t)((lm >> 4) << 6);
            }
        }
        const uint16_t hd = f2h(max_scale / 63.f), hm = f2h(max_min / 63.f);
        y[0] = (uint8_t)(hd & 0xFF); y[1] = (uint8_t)(hd >> 8);
        y[2] = (uint8_t)(hm & 0xFF); y[3] = (uint8_t)(hm >> 8);
        const float fd = h2f(hd), fm = h2f(hm);
        for (int j = 0; j < 8; ++j) {
            int s, m;
            scale_min_k4(j, sc, &s, &m);
            const float d = fd * s;
            if (d == 0.f) continue;   /* keeps the codes from the search (ggml does the same) */
            const float dm = fm * m;
            for (int ii = 0; ii < 32; ++ii) {
                int l = nearest_int((x[32 * j + ii] + dm) / d);
                l = l < 0 ? 0 : (l > 15 ? 15 : l);
                L[32 * j + ii] = (uint8_t)l;
            }
        }
        uint8_t* q = y + 16;
        for (int j = 0; j < 256; j += 64) {
            for (int l = 0; l < 32; ++l) q[l] = (uint8_t)(L[j + l] | (L[j + l + 32] << 4));
            q += 32;
        }
    }
}

/* ---------------------------------------------------------------- Q6_K */

/* Symmetric scale for n values quantised to -nmax..nmax-1 with weights x^2 (ggml make_qx_quants, rmse_type 1). */
static float make_qx(int n, int nmax, const float* x, int8_t* L) {
    float max = 0, amax = 0;
    for (int i = 0; i < n; ++i) { const float ax = fabsf(x[i]); if (ax > amax) { amax = ax; max = x[i]; } }
    if (amax < 1e-30f) { for (int i = 0; i < n; ++i) L[i] = 0; return 0.f; }
    float iscale = -nmax / max;
    float sumlx = 0, suml2 = 0;
    for (int i = 0; i < n; ++i) {
        int l = nearest_int(iscale * x[i]);
        l = l < -nmax ? -nmax : (l > nmax - 1 ? nmax - 1 : l);
        L[i] = (int8_t)(l + nmax);
        const float w = x[i] * x[i];
        sumlx += w * x[i] * l; suml2 += w * l * l;
    }
    float scale = suml2 ? sumlx / suml2 : 0.f;
    float best = scale * sumlx;
    for (int is = -9; is <= 9; ++is) {
        if (is == 0) continue;
        iscale = -(nmax + 0.1f * is) / max;
        sumlx = suml2 = 0;
        for (int i = 0; i < n; ++i) {
            int l = nearest_int(iscale * x[i]);
            l = l < -nmax ? -nmax : (l > nmax - 1 ? nmax - 1 : l);
            const float w = x[i] * x[i];
            sumlx += w * x[i] * l; suml2 += w * l * l;
        }
        if (suml2 > 0 && sumlx * sumlx > best * suml2) {
            for (int i = 0; i < n; ++i) {
                int l = nearest_int(iscale * x[i]);
                l = l < -nmax ? -nmax : (l > nmax - 1 ? nmax - 1 : l);
                L[i] = (int8_t)(l + nmax);
            }
            scale = sumlx / suml2; best = scale * sumlx;
        }
    }
    return scale;
}

QAPI void skainet_quantize_q6k(const float* xin, int64_t n, uint8_t* out) {
    const int64_t nb = n / 256;
#pragma omp parallel for schedule(static)
    for (int64_t ib = 0; ib < nb; ++ib) {
        const float* x = xin + ib * 256;
        uint8_t* y = out + ib * 210;
        int8_t L[256];
        float scales[16];
        float max_scale = 0, max_abs = 0;
        for (int j = 0; j < 16; ++j) {
            scales[j] = make_qx(16, 32, x + 16 * j, L + 16 * j);
            const float a = fabsf(scales[j]);
            if (a > max_abs) { max_abs = a; max_scale = scales[j]; }
        }
        if (max_abs < 1e-30f) { memset(y, 0, 210); continue; }
        const float iscale = -128.f / max_scale;
        const uint16_t hd = f2h(1 / iscale);
        y[208] = (uint8_t)(hd & 0xFF); y[209] = (uint8_t)(hd >> 8);
        int8_t* sc = (int8_t*)(y + 192);
        for (int j = 0; j < 16; ++j) { int s = nearest_int(iscale * scales[j]); sc[j] = (int8_t)(s > 127 ? 127 : s); }
        const float fd = h2f(hd);
        for (int j = 0; j < 16; ++j) {
            const float d = fd * sc[j];
            if (d == 0.f) continue;
            for (int ii = 0; ii < 16; ++ii) {
                int l = nearest_int(x[16 * j + ii] / d);
                l = l < -32 ? -32 : (l > 31 ? 31 : l);
                L[16 * j + ii] = (int8_t)(l + 32);
            }
        }
        uint8_t* ql = y;
        uint8_t* qh = y + 128;
        for (int j = 0; j < 256; j += 128) {
            for (int l = 0; l < 32; ++l) {
                const uint8_t q1 = L[j + l] & 0xF, q2 = L[j + l + 32] & 0xF, q3 = L[j + l + 64] & 0xF, q4 = L[j + l + 96] & 0xF;
                ql[l] = (uint8_t)(q1 | (q3 << 4));
                ql[l + 32] = (uint8_t)(q2 | (q4 << 4));
                qh[l] = (uint8_t)((L[j + l] >> 4) | ((L[j + l + 32] >> 4) << 2) | ((L[j + l + 64] >> 4) << 4) | ((L[j + l + 96] >> 4) << 6));
            }
            ql += 64; qh += 32;
        }
    }
}

/* ---------------------------------------------------------------- Q4_0, Q5_0, Q5_1 (32-element blocks) */

/* fp32 -> fp16 as Q4_0Quantizer.floatToHalf does it: round on the first dropped bit (no tie rule), truncating subnormals */
static uint16_t q4_0_half(float value) {
    const uint32_t bits = f32_bits(value);
    const uint32_t sign = (bits >> 16) & 0x8000u;
    const int exp = (int)((bits >> 23) & 0xFF) - 127 + 15;
    const uint32_t mant = bits & 0x7FFFFFu;
    if (exp >= 0x1F) return (uint16_t)(sign | 0x7C00u);
    if (exp <= 0) {
        if (exp < -10) return (uint16_t)sign;
        return (uint16_t)(sign | ((mant | 0x800000u) >> (1 - exp + 13)));
    }
    return (uint16_t)((sign | ((uint32_t)exp << 10) | (mant >> 13)) + ((mant >> 12) & 1u));
}

QAPI void skainet_quantize_q4_0(const float* x, int64_t n, uint8_t* out) {
    const int64_t nb = n / 32;
#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < nb; ++b) {
        const float* v = x + b * 32;
        uint8_t* y = out + b * 18;
        float amax = 0.f, max = 0.f;
        for (int i = 0; i < 32; ++i) { const float a = fabsf(v[i]); if (a > amax) { amax = a; max = v[i]; } }
        const float d = max / -8.f;
        const float id = d != 0.f ? 1.f / d : 0.f;
        const uint16_t h = q4_0_half(d);
        y[0] = (uint8_t)(h & 0xFF); y[1] = (uint8_t)(h >> 8);
        for (int j = 0; j < 16; ++j) {
            int lo = (int)(v[j] * id + 8.5f), hi = (int)(v[16 + j] * id + 8.5f);
            lo = lo < 0 ? 0 : (lo > 15 ? 15 : lo);
            hi = hi < 0 ? 0 : (hi > 15 ? 15 : hi);
            y[2 + j] = (uint8_t)((hi << 4) | lo);
        }
    }
}

QAPI void skainet_quantize_q5_0(const float* x, int64_t n, uint8_t* out) {
    const int64_t nb = n / 32;
#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < nb; ++b) {
        const float* v = x + b * 32;
        uint8_t* y = out + b * 22;
        float amax = 0.f, max = 0.f;
        for (int i = 0; i < 32; ++i) { const float a = fabsf(v[i]); if (a > amax) { amax = a; max = v[i]; } }
        const float d = max / -16.f;
        const float id = d != 0.f ? 1.f / d : 0.f;
        const uint16_t h = f2h(d);
        y[0] = (uint8_t)(h & 0xFF); y[1] = (uint8_t)(h >> 8);
        uint32_t qh = 0;
        for (int j = 0; j < 16; ++j) {
            int q0 = (int)(int8_t)(v[j] * id + 16.5f), q1 = (int)(int8_t)(v[16 + j] * id + 16.5f);
            q0 = q0 > 31 ? 31 : (q0 < 0 ? 0 : q0);
            q1 = q1 > 31 ? 31 : (q1 < 0 ? 0 : q1);
            y[6 + j] = (uint8_t)((q0 & 0x0F) | ((q1 & 0x0F) << 4));
            qh |= (uint32_t)((q0 & 0x10) >> 4) << j;
            qh |= (uint32_t)((q1 & 0x10) >> 4) << (j + 16);
        }
        memcpy(y + 2, &qh, 4);
    }
}

QAPI void skainet_quantize_q5_1(const float* x, int64_t n, uint8_t* out) {
    const int64_t nb = n / 32;
#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < nb; ++b) {
        const float* v = x + b * 32;
        uint8_t* y = out + b * 24;
        float mn = v[0], mx = v[0];
        for (int i = 1; i < 32; ++i) { if (v[i] < mn) mn = v[i]; if (v[i] > mx) mx = v[i]; }
        const float d = (mx - mn) / 31.f;
        const float id = d != 0.f ? 1.f / d : 0.f;
        const uint16_t hd = f2h(d), hm = f2h(mn);
        y[0] = (uint8_t)(hd & 0xFF); y[1] = (uint8_t)(hd >> 8);
        y[2] = (uint8_t)(hm & 0xFF); y[3] = (uint8_t)(hm >> 8);
        uint32_t qh = 0;
        for (int j = 0; j < 16; ++j) {
            int q0 = (int)((v[j] - mn) * id + 0.5f), q1 = (int)((v[16 + j] - mn) * id + 0.5f);
            q0 = q0 > 31 ? 31 : (q0 < 0 ? 0 : q0);
            q1 = q1 > 31 ? 31 : (q1 < 0 ? 0 : q1);
            y[8 + j] = (uint8_t)((q0 & 0x0F) | ((q1 & 0x0F) << 4));
            qh |= (uint32_t)((q0 & 0x10) >> 4) << j;
            qh |= (uint32_t)((q1 & 0x10) >> 4) << (j + 16);
        }
        memcpy(y + 4, &qh, 4);
    }
}

/* ---------------------------------------------------------------- Q5_K: the Q4_K search with 32 levels */
QAPI void skainet_quantize_q5k(const float* xin, int64_t n, uint8_t* out) {
    const int64_t nb = n / 256;
#pragma omp parallel for schedule(static)
    for (int64_t ib = 0; ib < nb; ++ib) {
        const float* x = xin + ib * 256;
        uint8_t* y = out + ib * 176;
        uint8_t L[256], Laux[32];
        float weights[32], mins[8], scales[8];
        float max_scale = 0, max_min = 0;
        for (int j = 0; j < 8; ++j) {
            float sum_x2 = 0;
            for (int l = 0; l < 32; ++l) sum_x2 += x[32 * j + l] * x[32 * j + l];
            const float av = sqrtf(sum_x2 / 32);
            for (int l = 0; l < 32; ++l) weights[l] = av + fabsf(x[32 * j + l]);
            scales[j] = make_qkx2(32, 31, x + 32 * j, weights, L + 32 * j, &mins[j], Laux, -0.5f, 0.1f, 15);
            if (scales[j] > max_scale) max_scale = scales[j];
            if (mins[j] > max_min) max_min = mins[j];
        }
        const float inv_scale = max_scale > 0 ? 63.f / max_scale : 0.f;
        const float inv_min = max_min > 0 ? 63.f / max_min : 0.f;
        uint8_t* sc = y + 4;
        memset(sc, 0, 12);
        for (int j = 0; j < 8; ++j) {
            int ls = nearest_int(inv_scale * scales[j]);
            int lm = nearest_int(inv_min * mins[j]);
            ls = ls > 63 ? 63 : (ls < 0 ? 0 : ls);
            lm = lm > 63 ? 63 : (lm < 0 ? 0 : lm);
            if (j < 4) { sc[j] = (uint8_t)ls; sc[j + 4] = (uint8_t)lm; }
            else {
                sc[j + 4] = (uint8_t)((ls & 0xF) | ((lm & 0xF) << 4));
                sc[j - 4] |= (uint8_t)((ls >> 4) << 6);
                sc[j] |= (uint8_t)((lm >> 4) << 6);
            }
        }
        const uint16_t hd = f2h(max_scale / 63.f), hm = f2h(max_min / 63.f);
        y[0] = (uint8_t)(hd & 0xFF); y[1] = (uint8_t)(hd >> 8);
        y[2] = (uint8_t)(hm & 0xFF); y[3] = (uint8_t)(hm >> 8);
        const float fd = h2f(hd), fm = h2f(hm);
        for (int j = 0; j < 8; ++j) {
            int s, m;
            scale_min_k4(j, sc, &s, &m);
            const float d = fd * s;
            if (d == 0.f) continue;
            const float dm = fm * m;
            for (int ii = 0; ii < 32; ++ii) {
                int l = nearest_int((x[32 * j + ii] + dm) / d);
                l = l < 0 ? 0 : (l > 31 ? 31 : l);
                L[32 * j + ii] = (uint8_t)l;
            }
        }
        uint8_t *qh = y + 16, *ql = y + 48;
        memset(qh, 0, 32);
        uint8_t m1 = 1, m2 = 2;
        for (int g = 0; g < 256; g += 64) {
            for (int j = 0; j < 32; ++j) {
                int l1 = L[g + j], l2 = L[g + j + 32];
                if (l1 > 15) { l1 -= 16; qh[j] |= m1; }
                if (l2 > 15) { l2 -= 16; qh[j] |= m2; }
                ql[j] = (uint8_t)(l1 | (l2 << 4));
            }
            m1 <<= 2; m2 <<= 2; ql += 32;
        }
    }
}
