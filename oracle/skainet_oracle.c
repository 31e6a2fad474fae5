/*
 * skainet_oracle.c -- CPU restatement of the SKaiNET kernel semantics this backend must reproduce.
 *
 * THIS FILE IS TEST INFRASTRUCTURE. It is the checker the parity tests compare the HIP path
 * against (and, for the int8-activation "native" section at the bottom, a fallback CPU timing
 * baseline). Nothing in the product path may call it.
 *
 * Build: strict IEEE binary32, no FMA contraction, no reassociation
 *   gcc -O2 -ffp-contract=off -fno-fast-math -fPIC -shared      (see oracle/Makefile)
 * so that every function below rounds exactly where the JVM (strict binary32) reference rounds.
 *
 * Reference files restated here (paths under /root/reference):
 *   [HALF]   skainet-backends/skainet-backend-cpu/src/commonMain/kotlin/sk/ainet/exec/kernel/ScalarHalf.kt:9-31
 *   [Q80D]   skainet-lang/skainet-lang-core/src/commonMain/kotlin/sk/ainet/lang/tensor/data/Q8_0TensorData.kt:80-89
 *   [Q4KD]   .../lang/tensor/data/Q4_KTensorData.kt:120-136 (decode), :184-206 (scale/min index), :215-226 (code)
 *   [Q6KD]   .../lang/tensor/data/Q6_KTensorData.kt:112-165
 *   [Q80M]   skainet-backends/skainet-backend-cpu/src/commonMain/kotlin/sk/ainet/exec/kernel/ScalarQ8_0MatmulKernel.kt:27-66
 *   [Q4KM]   .../exec/kernel/ScalarQ4_KMatmulKernel.kt:21-80
 *   [Q6KM]   .../exec/kernel/ScalarQ6_KMatmulKernel.kt:21-86
 *   [Q40D]   .../lang/tensor/data/Q4_0TensorData.kt:93-107, [Q50D] Q5_0TensorData.kt:68-86, [Q51D] Q5_1TensorData.kt:73-92,
 *   [Q5KD]   Q5_KTensorData.kt:126-142 (decode), :190-219 (scale/min index), :221-236 (code)
 *   [Q40M]   .../exec/kernel/ScalarQ4_0MatmulKernel.kt:29-63, [Q50M] ScalarQ5_0MatmulKernel.kt, [Q51M] ScalarQ5_1MatmulKernel.kt,
 *   [Q5KM]   ScalarQ5_KMatmulKernel.kt (all: one `override fun matmul`)
 *   [NARROW] .../exec/kernel/ScalarBf16MatmulKernel.kt:8-46 and ScalarFp16MatmulKernel.kt (same loop, Fp16Codec.decode)
 *   [Q80Q]   skainet-lang/skainet-lang-core/src/commonMain/kotlin/sk/ainet/lang/tensor/data/Q8_0Quantizer.kt:28-53
 *   [FP16E]  skainet-lang/skainet-lang-core/src/commonMain/kotlin/sk/ainet/lang/types/NarrowFloatCodec.kt:87-130
 *   [SDPA]   skainet-backends/skainet-backend-native-cpu/native/src/f32_fused.c:304-396 and
 *            skainet-lang/skainet-lang-core/src/commonMain/kotlin/sk/ainet/lang/tensor/ops/AttentionMask.kt:24-104
 *   [NORM]   skainet-backends/skainet-backend-native-cpu/native/src/f32_fused.c:232-286
 *   [SGEMM]  skainet-backends/skainet-backend-native-cpu/native/include/skainet_kernels.h:262-276, :495-515
 *   [RELAY]  skainet-backends/skainet-backend-api/src/commonMain/kotlin/sk/ainet/backend/api/kernel/PackedWeights.kt:63-93
 *   [NQ4K]   skainet-backends/skainet-backend-native-cpu/native/src/q4k_matmul.c:74-251
 *   [NQ6K]   skainet-backends/skainet-backend-native-cpu/native/src/q6k_matmul.c:53-213
 *   [NQ80]   skainet-backends/skainet-backend-native-cpu/native/src/q8_0_matmul.c:68-117
 *
 * Pinning (what proves each function, see tests/test_oracle_golden.py):
 *   orc_half_to_float          all 65536 patterns vs numpy float16 (finite + inf), pinned
 *   orc_dequant_{q8_0,q4k,q6k} reference golden digests decode/Q8_0, decode/Q4_K, decode/Q6_K, pinned
 *   orc_{q8_0,q4k,q6k}_matmul  reference golden digests scalar-matmul and dispatch-bridge, pinned
 *   orc_dequant_{q4_0,q5_0,q5_1,q5k} and orc_{q4_0,q5_0,q5_1,q5k}_matmul
 *                              reference golden digests decode/, transpose/, scalar-matmul/, dispatch-bridge/ of
 *                              Q4_0, Q5_0, Q5_1, Q5_K, pinned
 *   orc_bf16_matmul, orc_fp16_matmul  exact on integer-valued operands (every partial sum representable), the reference
 *                              C library's skainet_bf16_matmul / skainet_fp16_matmul (oracle/_ref and recorded vectors), float64, pinned
 *   orc_q8_0_quantize          known answers of the reference's Q8_0QuantizerTest + numpy fp16 RNE, pinned
 *   orc_f32_sdpa, rms_norm,    the reference C library compiled from its own sources (oracle/_ref),
 *   softmax, fp32 matmuls      fp64 closed forms and mask-rule invariants, pinned
 *   orc_native_*               bit-identical to oracle/_ref on seeded inputs, pinned
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_API __attribute__((visibility("default")))

static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

/* ---------------------------------------------------------------- fp16 <-> fp32 */

/* [HALF] binary16 bits -> binary32, subnormals normalised by shifting. */
ORC_API float orc_half_to_float(uint32_t hbits) {
    const uint32_t sign = (hbits & 0x8000u) << 16;
    const uint32_t exp = (hbits & 0x7C00u) >> 10;
    uint32_t mant = hbits & 0x03FFu;
    if (exp == 0) {
        if (mant == 0) return bits_f32(sign);
        int e = -14;
        while ((mant & 0x400u) == 0) { mant <<= 1; --e; }
        mant &= 0x3FFu;
        return bits_f32(sign | ((uint32_t)(e + 127) << 23) | (mant << 13));
    }
    if (exp == 31) return bits_f32(sign | (0xFFu << 23) | (mant << 13));
    return bits_f32(sign | ((exp - 15 + 127) << 23) | (mant << 13));
}

/* [FP16E] binary32 -> binary16 bits, round-to-nearest-even, gradual underflow, overflow to inf. */
ORC_API uint32_t orc_float_to_half(float value) {
    const uint32_t bits = f32_bits(value);
    const uint32_t sign = (bits >> 16) & 0x8000u;
    const uint32_t abs_bits = bits & 0x7FFFFFFFu;
    if (abs_bits >= 0x7F800000u) {
        if (abs_bits == 0x7F800000u) return sign | 0x7C00u;
        return sign | 0x7C00u | 0x0200u | ((abs_bits >> 13) & 0x03FFu);
    }
    const int exp = (int)(abs_bits >> 23) - 127;
    const uint32_t mant = abs_bits & 0x007FFFFFu;
    if (exp >= 16) return sign | 0x7C00u;
    if (exp >= -14) {
        const uint32_t half = ((uint32_t)(exp + 15) << 10) | (mant >> 13);
        const uint32_t rem = mant & 0x1FFFu;
        const int up = rem > 0x1000u || (rem == 0x1000u && (half & 1u));
        return sign | (half + (up ? 1u : 0u));
    }
    if (exp < -25) return sign;
    const uint32_t full = mant | 0x00800000u;
    const int shift = -1 - exp;
    const uint32_t q = full >> shift;
    const uint32_t rem = full & ((1u << shift) - 1u);
    const uint32_t half_bit = 1u << (shift - 1);
    const int up = rem > half_bit || (rem == half_bit && (q & 1u));
    return sign | (q + (up ? 1u : 0u));
}

/* ---------------------------------------------------------------- block decode (bit-exact) */

#define Q80_BS 32
#define Q80_BYTES 34
#define QK_BS 256
#define Q4K_BYTES 144
#define Q6K_BYTES 210
#define Q40_BYTES 18
#define Q50_BYTES 22
#define Q51_BYTES 24
#define Q5K_BYTES 176

static inline uint32_t le16(const uint8_t* p) { return (uint32_t)p[0] | ((uint32_t)p[1] << 8); }

/* [Q80D] w = (float)code * d */
static void q8_0_block(const uint8_t* b, float* out) {
    const float d = orc_half_to_float(le16(b));
    const int8_t* codes = (const int8_t*)(b + 2);
    for (int i = 0; i < Q80_BS; ++i) out[i] = (float)codes[i] * d;
}

/* [Q4KD] get_scale_min_k4 */
static void q4k_scale_min(const uint8_t* s, int* sc, int* mn) {
    for (int j = 0; j < 4; ++j) { sc[j] = s[j] & 0x3F; mn[j] = s[j + 4] & 0x3F; }
    for (int j = 4; j < 8; ++j) {
        sc[j] = (s[j + 4] & 0x0F) | ((s[j - 4] >> 6) << 4);
        mn[j] = (s[j + 4] >> 4) | ((s[j] >> 6) << 4);
    }
}

/* [Q4KD] w = code * (d * scaleIdx) - (dmin * minIdx): two products rounded, then one subtract. */
static void q4k_block(const uint8_t* b, float* out) {
    const float d = orc_half_to_float(le16(b));
    const float dmin = orc_half_to_float(le16(b + 2));
    int sc[8], mn[8];
    q4k_scale_min(b + 4, sc, mn);
    const uint8_t* qs = b + 16;
    for (int sb = 0; sb < 8; ++sb) {
        const float scale = d * (float)sc[sb];
        const float offset = dmin * (float)mn[sb];
        const uint8_t* grp = qs + (sb >> 1) * 32;
        for (int j = 0; j < 32; ++j) {
            const int code = (sb & 1) ? (grp[j] >> 4) : (grp[j] & 0x0F);
            out[sb * 32 + j] = (float)code * scale - offset;
        }
    }
}

/* [Q6KD] w = (d * sc) * q, q = 6-bit code - 32 */
static void q6k_block(const uint8_t* b, float* out) {
    const float d = orc_half_to_float(le16(b + 208));
    const int8_t* scales = (const int8_t*)(b + 192);
    for (int half = 0; half < 2; ++half) {
        const uint8_t* ql = b + half * 64;
        const uint8_t* qh = b + 128 + half * 32;
        const int8_t* sc = scales + half * 8;
        float* o = out + half * 128;
        for (int l = 0; l < 32; ++l) {
            const int is = l / 16;
            const int q1 = ((ql[l] & 0x0F) | ((qh[l] & 0x03) << 4)) - 32;
            const int q2 = ((ql[l + 32] & 0x0F) | (((qh[l] >> 2) & 0x03) << 4)) - 32;
            const int q3 = ((ql[l] >> 4) | (((qh[l] >> 4) & 0x03) << 4)) - 32;
            const int q4 = ((ql[l + 32] >> 4) | (((qh[l] >> 6) & 0x03) << 4)) - 32;
            o[l + 0] = (d * (float)sc[is + 0]) * (float)q1;
            o[l + 32] = (d * (float)sc[is + 2]) * (float)q2;
            o[l + 64] = (d * (float)sc[is + 4]) * (float)q3;
            o[l + 96] = (d * (float)sc[is + 6]) * (float)q4;
        }
    }
}

/* [Q40D] low nibbles are elements 0..15, high nibbles 16..31; w = (float)(code - 8) * d */
static void q4_0_block(const uint8_t* b, float* out) {
    const float d = orc_half_to_float(le16(b));
    for (int j = 0; j < 16; ++j) {
        out[j] = (float)((b[2 + j] & 0x0F) - 8) * d;
        out[16 + j] = (float)((b[2 + j] >> 4) - 8) * d;
    }
}

/* bit j of the 32-bit little-endian high-bit plane at qh */
static inline int q5_bit(const uint8_t* qh, int j) { return (qh[j >> 3] >> (j & 7)) & 1; }

/* [Q50D] w = d * (float)(code5 - 16) */
static void q5_0_block(const uint8_t* b, float* out) {
    const float d = orc_half_to_float(le16(b));
    const uint8_t *qh = b + 2, *qs = b + 6;
    for (int j = 0; j < 16; ++j) {
        out[j] = d * (float)((qs[j] & 0x0F) + (q5_bit(qh, j) << 4) - 16);
        out[16 + j] = d * (float)((qs[j] >> 4) + (q5_bit(qh, j + 16) << 4) - 16);
    }
}

/* [Q51D] w = d * (float)code5 + m: product rounded, then the add */
static void q5_1_block(const uint8_t* b, float* out) {
    const float d = orc_half_to_float(le16(b)), m = orc_half_to_float(le16(b + 2));
    const uint8_t *qh = b + 4, *qs = b + 8;
    for (int j = 0; j < 16; ++j) {
        const float lo = d * (float)((qs[j] & 0x0F) + (q5_bit(qh, j) << 4));
        const float hi = d * (float)((qs[j] >> 4) + (q5_bit(qh, j + 16) << 4));
        out[j] = lo + m;
        out[16 + j] = hi + m;
    }
}

/* [Q5KD] the Q4_K scale/min packing; element e of 64-element group g: low nibble (e < 32) or high nibble of
 * qs[g*32 + e%32], fifth bit = bit (2g or 2g+1) of qh[e%32]; w = (float)code * (d*sc) - (dmin*m) */
static inline int q5k_code(const uint8_t* b, int g, int half, int l) {
    const int byte = b[48 + g * 32 + l];
    const int low = half ? (byte >> 4) : (byte & 0x0F);
    return low | (((b[16 + l] >> (2 * g + half)) & 1) << 4);
}
static void q5k_block(const uint8_t* b, float* out) {
    const float d = orc_half_to_float(le16(b));
    const float dmin = orc_half_to_float(le16(b + 2));
    int sc[8], mn[8];
    q4k_scale_min(b + 4, sc, mn);
    for (int sb = 0; sb < 8; ++sb) {
        const float scale = d * (float)sc[sb];
        const float offset = dmin * (float)mn[sb];
        for (int j = 0; j < 32; ++j) out[sb * 32 + j] = (float)q5k_code(b, sb >> 1, sb & 1, j) * scale - offset;
    }
}

ORC_API void orc_dequant_q4_0(const uint8_t* w, int64_t nblocks, float* out) {
    for (int64_t b = 0; b < nblocks; ++b) q4_0_block(w + b * Q40_BYTES, out + b * 32);
}
ORC_API void orc_dequant_q5_0(const uint8_t* w, int64_t nblocks, float* out) {
    for (int64_t b = 0; b < nblocks; ++b) q5_0_block(w + b * Q50_BYTES, out + b * 32);
}
ORC_API void orc_dequant_q5_1(const uint8_t* w, int64_t nblocks, float* out) {
    for (int64_t b = 0; b < nblocks; ++b) q5_1_block(w + b * Q51_BYTES, out + b * 32);
}
ORC_API void orc_dequant_q5k(const uint8_t* w, int64_t nblocks, float* out) {
    for (int64_t b = 0; b < nblocks; ++b) q5k_block(w + b * Q5K_BYTES, out + b * QK_BS);
}
ORC_API void orc_dequant_q8_0(const uint8_t* w, int64_t nblocks, float* out) {
    for (int64_t b = 0; b < nblocks; ++b) q8_0_block(w + b * Q80_BYTES, out + b * Q80_BS);
}
ORC_API void orc_dequant_q4k(const uint8_t* w, int64_t nblocks, float* out) {
    for (int64_t b = 0; b < nblocks; ++b) q4k_block(w + b * Q4K_BYTES, out + b * QK_BS);
}
ORC_API void orc_dequant_q6k(const uint8_t* w, int64_t nblocks, float* out) {
    for (int64_t b = 0; b < nblocks; ++b) q6k_block(w + b * Q6K_BYTES, out + b * QK_BS);
}

/* ---------------------------------------------------------------- exact fp32 GEMV (parity oracle)
 *
 * row_major == 0: weight is input-block-major, block (b, o) at (b * N + o) * bytes  (the SPI layout)
 * row_major != 0: canonical GGUF order, block (o, b) at (o * bpr + b) * bytes
 * The per-row accumulation order is the scalar kernels' and is identical in both layouts.
 */
static inline const uint8_t* blk(const uint8_t* w, int row_major, int64_t b, int64_t o,
                                 int64_t bpr, int64_t n, int bytes) {
    return w + (row_major ? (o * bpr + b) : (b * n + o)) * bytes;
}

/* [Q80M] acc += (x * code) * d, one element at a time */
ORC_API void orc_q8_0_matmul(const float* input, int32_t input_offset, const uint8_t* weight,
                             int32_t weight_byte_offset, int32_t input_dim, int32_t output_dim,
                             float* output, int32_t output_offset, int32_t row_major) {
    if (output_dim <= 0) return;
    const int64_t bpr = input_dim / Q80_BS;
    const uint8_t* w = weight + weight_byte_offset;
    for (int64_t o = 0; o < output_dim; ++o) {
        float acc = 0.0f;
        for (int64_t b = 0; b < bpr; ++b) {
            const uint8_t* p = blk(w, row_major, b, o, bpr, output_dim, Q80_BYTES);
            const float d = orc_half_to_float(le16(p));
            const int8_t* codes = (const int8_t*)(p + 2);
            const float* x = input + input_offset + b * Q80_BS;
            for (int k = 0; k < Q80_BS; ++k) {
                const float t = x[k] * (float)codes[k];
                acc += t * d;
            }
        }
        output[output_offset + o] = acc;
    }
}

/* [Q40M] per byte j: acc += (x[j] * lo) * d, then acc += (x[16+j] * hi) * d */
ORC_API void orc_q4_0_matmul(const float* input, int32_t input_offset, const uint8_t* weight,
                             int32_t weight_byte_offset, int32_t input_dim, int32_t output_dim,
                             float* output, int32_t output_offset, int32_t row_major) {
    if (output_dim <= 0) return;
    const int64_t bpr = input_dim / 32;
    const uint8_t* w = weight + weight_byte_offset;
    for (int64_t o = 0; o < output_dim; ++o) {
        float acc = 0.0f;
        for (int64_t b = 0; b < bpr; ++b) {
            const uint8_t* p = blk(w, row_major, b, o, bpr, output_dim, Q40_BYTES);
            const float d = orc_half_to_float(le16(p));
            const float* x = input + input_offset + b * 32;
            for (int j = 0; j < 16; ++j) {
                const float lo = (float)((p[2 + j] & 0x0F) - 8), hi = (float)((p[2 + j] >> 4) - 8);
                const float t0 = x[j] * lo;
                acc += t0 * d;
                const float t1 = x[16 + j] * hi;
                acc += t1 * d;
            }
        }
        output[output_offset + o] = acc;
    }
}

/* [Q50M] / [Q51M] per byte j: wLo, wHi decoded as in the block decoders; acc += (x[j]*wLo + x[16+j]*wHi) */
static void q5_01_matmul(const float* input, int32_t input_offset, const uint8_t* weight, int32_t weight_byte_offset,
                         int32_t input_dim, int32_t output_dim, float* output, int32_t output_offset, int32_t row_major,
                         int is_q5_1) {
    if (output_dim <= 0) return;
    const int bytes = is_q5_1 ? Q51_BYTES : Q50_BYTES;
    const int64_t bpr = input_dim / 32;
    const uint8_t* w = weight + weight_byte_offset;
    float dec[32];
    for (int64_t o = 0; o < output_dim; ++o) {
        float acc = 0.0f;
        for (int64_t b = 0; b < bpr; ++b) {
            const uint8_t* p = blk(w, row_major, b, o, bpr, output_dim, bytes);
            if (is_q5_1) q5_1_block(p, dec); else q5_0_block(p, dec);
            const float* x = input + input_offset + b * 32;
            for (int j = 0; j < 16; ++j) {
                const float a = x[j] * dec[j];
                const float c = x[16 + j] * dec[16 + j];
                acc += a + c;
            }
        }
        output[output_offset + o] = acc;
    }
}
ORC_API void orc_q5_0_matmul(const float* input, int32_t input_offset, const uint8_t* weight,
                             int32_t weight_byte_offset, int32_t input_dim, int32_t output_dim,
                             float* output, int32_t output_offset, int32_t row_major) {
    q5_01_matmul(input, input_offset, weight, weight_byte_offset, input_dim, output_dim, output, output_offset, row_major, 0);
}
ORC_API void orc_q5_1_matmul(const float* input, int32_t input_offset, const uint8_t* weight,
                             int32_t weight_byte_offset, int32_t input_dim, int32_t output_dim,
                             float* output, int32_t output_offset, int32_t row_major) {
    q5_01_matmul(input, input_offset, weight, weight_byte_offset, input_dim, output_dim, output, output_offset, row_major, 1);
}

/* [Q5KM] the Q4_K kernel's shape with 5-bit codes: per sub-block codeSum, inputSum; acc += codeSum*(d*sc) - inputSum*(dmin*m) */
ORC_API void orc_q5k_matmul(const float* input, int32_t input_offset, const uint8_t* weight,
                            int32_t weight_byte_offset, int32_t input_dim, int32_t output_dim,
                            float* output, int32_t output_offset, int32_t row_major) {
    if (output_dim <= 0) return;
    const int64_t bpr = input_dim / QK_BS;
    const uint8_t* w = weight + weight_byte_offset;
    for (int64_t o = 0; o < output_dim; ++o) {
        float acc = 0.0f;
        for (int64_t b = 0; b < bpr; ++b) {
            const uint8_t* p = blk(w, row_major, b, o, bpr, output_dim, Q5K_BYTES);
            const float d = orc_half_to_float(le16(p));
            const float dmin = orc_half_to_float(le16(p + 2));
            int sc[8], mn[8];
            q4k_scale_min(p + 4, sc, mn);
            const float* x = input + input_offset + b * QK_BS;
            for (int g = 0; g < 4; ++g) {
                for (int half = 0; half < 2; ++half) {
                    const int sb = 2 * g + half;
                    float code_sum = 0.0f, input_sum = 0.0f;
                    for (int i = 0; i < 32; ++i) {
                        const float v = x[sb * 32 + i];
                        code_sum += v * (float)q5k_code(p, g, half, i);
                        input_sum += v;
                    }
                    const float a = code_sum * (d * (float)sc[sb]);
                    const float c = input_sum * (dmin * (float)mn[sb]);
                    acc += a - c;
                }
            }
        }
        output[output_offset + o] = acc;
    }
}

/* [Q4KM] per sub-block: codeSum = sum x*code, inputSum = sum x; acc += codeSum*(d*sc) - inputSum*(dmin*m) */
ORC_API void orc_q4k_matmul(const float* input, int32_t input_offset, const uint8_t* weight,
                            int32_t weight_byte_offset, int32_t input_dim, int32_t output_dim,
                            float* output, int32_t output_offset, int32_t row_major) {
    if (output_dim <= 0) return;
    const int64_t bpr = input_dim / QK_BS;
    const uint8_t* w = weight + weight_byte_offset;
    for (int64_t o = 0; o < output_dim; ++o) {
        float acc = 0.0f;
        for (int64_t b = 0; b < bpr; ++b) {
            const uint8_t* p = blk(w, row_major, b, o, bpr, output_dim, Q4K_BYTES);
            const float d = orc_half_to_float(le16(p));
            const float dmin = orc_half_to_float(le16(p + 2));
            int sc[8], mn[8];
            q4k_scale_min(p + 4, sc, mn);
            const uint8_t* qs = p + 16;
            const float* x = input + input_offset + b * QK_BS;
            for (int g = 0; g < 4; ++g) {
                for (int half = 0; half < 2; ++half) {
                    const int sb = 2 * g + half;
                    float code_sum = 0.0f, input_sum = 0.0f;
                    for (int i = 0; i < 32; ++i) {
                        const int byte = qs[g * 32 + i];
                        const int code = half ? (byte >> 4) : (byte & 0x0F);
                        const float v = x[sb * 32 + i];
                        code_sum += v * (float)code;
                        input_sum += v;
                    }
                    const float a = code_sum * (d * (float)sc[sb]);
                    const float c = input_sum * (dmin * (float)mn[sb]);
                    acc += a - c;
                }
            }
        }
        output[output_offset + o] = acc;
    }
}

/* [Q6KM] dequantise the block to scratch, then 256 sequential acc += x * w */
ORC_API void orc_q6k_matmul(const float* input, int32_t input_offset, const uint8_t* weight,
                            int32_t weight_byte_offset, int32_t input_dim, int32_t output_dim,
                            float* output, int32_t output_offset, int32_t row_major) {
    if (output_dim <= 0) return;
    const int64_t bpr = input_dim / QK_BS;
    const uint8_t* w = weight + weight_byte_offset;
    float scratch[QK_BS];
    for (int64_t o = 0; o < output_dim; ++o) {
        float acc = 0.0f;
        for (int64_t b = 0; b < bpr; ++b) {
            q6k_block(blk(w, row_major, b, o, bpr, output_dim, Q6K_BYTES), scratch);
            const float* x = input + input_offset + b * QK_BS;
            for (int i = 0; i < QK_BS; ++i) acc += x[i] * scratch[i];
        }
        output[output_offset + o] = acc;
    }
}

/* [RELAY] kernel[(b * rows + o)] = canonical[(o * bpr + b)], block-wise; inverse with to_row_major. */
ORC_API void orc_relayout(const uint8_t* src, uint8_t* dst, int64_t rows, int64_t bpr,
                          int32_t bytes_per_block, int32_t to_row_major) {
    for (int64_t o = 0; o < rows; ++o)
        for (int64_t b = 0; b < bpr; ++b) {
            const int64_t rm = (o * bpr + b) * bytes_per_block;
            const int64_t bm = (b * rows + o) * bytes_per_block;
            if (to_row_major) memcpy(dst + rm, src + bm, (size_t)bytes_per_block);
            else memcpy(dst + bm, src + rm, (size_t)bytes_per_block);
        }
}

/* ---------------------------------------------------------------- Q8_0 quantizer */

/* [Q80Q] d = amax/127 (fp16 RNE stored); id = 1/d from the UNROUNDED d; q = floor(x*id + 0.5) clamped. */
ORC_API void orc_q8_0_quantize(const float* values, int64_t n, uint8_t* out) {
    const int64_t blocks = n / Q80_BS;
    for (int64_t b = 0; b < blocks; ++b) {
        const float* x = values + b * Q80_BS;
        float amax = 0.0f;
        for (int i = 0; i < Q80_BS; ++i) { const float a = fabsf(x[i]); if (a > amax) amax = a; }
        const float d = amax / 127.0f;
        const float id = d != 0.0f ? 1.0f / d : 0.0f;
        uint8_t* o = out + b * Q80_BYTES;
        const uint32_t h = orc_float_to_half(d);
        o[0] = (uint8_t)(h & 0xFF); o[1] = (uint8_t)(h >> 8);
        for (int i = 0; i < Q80_BS; ++i) {
            /* Kotlin Float.roundToInt(): ties toward +inf == floor(v + 0.5) evaluated exactly. */
            const float v = x[i] * id;
            int q = (int)floor((double)v + 0.5);
            if (q < -127) q = -127; else if (q > 127) q = 127;
            o[2 + i] = (uint8_t)(int8_t)q;
        }
    }
}

/* ---------------------------------------------------------------- fused fp32 rows */

#define ORC_MASKED (-1.0e30f)

/* [SDPA] One query row at a time; scores in fp32, sequential ascending-index sums. */
ORC_API void orc_f32_sdpa(const float* q, const float* k, const float* v, float* out,
                          int32_t batch, int32_t heads, int32_t kv_heads, int32_t seq_q, int32_t seq_kv,
                          int32_t head_dim, float scale, int32_t causal, int32_t window,
                          int32_t right_context, const int32_t* lengths, const float* mask,
                          int32_t mask_b, int32_t mask_h, int32_t mask_q, int32_t mask_k) {
    if (batch <= 0 || heads <= 0 || kv_heads <= 0 || seq_q <= 0 || head_dim <= 0) return;
    const int64_t rows = (int64_t)batch * heads * seq_q;
    if (seq_kv <= 0) { for (int64_t i = 0; i < rows * head_dim; ++i) out[i] = 0.0f; return; }
    float* scores = (float*)malloc((size_t)seq_kv * sizeof(float));
    if (!scores) return;
    const int d = head_dim;
    for (int b = 0; b < batch; ++b) for (int h = 0; h < heads; ++h) for (int qi = 0; qi < seq_q; ++qi) {
        const int kvh = h / (heads / kv_heads);
        const float* qr = q + (((size_t)b * heads + h) * seq_q + qi) * d;
        const float* kb = k + ((size_t)b * kv_heads + kvh) * seq_kv * d;
        const float* vb = v + ((size_t)b * kv_heads + kvh) * seq_kv * d;
        float* o = out + (((size_t)b * heads + h) * seq_q + qi) * d;
        const int abs_q = seq_kv - seq_q + qi;
        int first = 0, end = seq_kv;
        if (window > 0) {
            if (abs_q - window + 1 > first) first = abs_q - window + 1;
            if (abs_q + right_context + 1 < end) end = abs_q + right_context + 1;
        }
        if (causal && abs_q + 1 < end) end = abs_q + 1;
        if (lengths && lengths[b] < end) end = lengths[b];
        if (end < 0) end = 0;
        if (first > end) first = end;
        for (int ki = 0; ki < seq_kv; ++ki) {
            if (ki < first || ki >= end) { scores[ki] = ORC_MASKED; continue; }
            float s = 0.0f;
            for (int x = 0; x < d; ++x) s += qr[x] * kb[(size_t)ki * d + x];
            scores[ki] = s * scale;
        }
        if (mask) {
            const int bi = mask_b == 1 ? 0 : b;
            const int hi = mask_h == 1 ? 0 : (mask_h == heads ? h : kvh);
            const size_t row = ((size_t)bi * mask_h + hi) * mask_q + (mask_q == 1 ? 0 : qi);
            const float* m = mask + row * mask_k;
            for (int ki = 0; ki < seq_kv; ++ki) scores[ki] += (mask_k == 1 ? m[0] : m[ki]);
        }
        float mx = scores[0];
        for (int ki = 1; ki < seq_kv; ++ki) if (scores[ki] > mx) mx = scores[ki];
        float sum = 0.0f;
        for (int ki = 0; ki < seq_kv; ++ki) { scores[ki] = expf(scores[ki] - mx); sum += scores[ki]; }
        if (sum > 0.0f) { const float inv = 1.0f / sum; for (int ki = 0; ki < seq_kv; ++ki) scores[ki] *= inv; }
        for (int x = 0; x < d; ++x) o[x] = 0.0f;
        for (int ki = 0; ki < seq_kv; ++ki) {
            const float p = scores[ki];
            if (p == 0.0f) continue;
            for (int x = 0; x < d; ++x) o[x] += p * vb[(size_t)ki * d + x];
        }
    }
    free(scores);
}

/* [NORM] out = x / sqrt(mean(x^2) + eps) * gamma ; gamma may be NULL */
ORC_API void orc_f32_rms_norm(const float* in, const float* gamma, float* out, int32_t rows, int32_t cols, float eps) {
    if (rows <= 0 || cols <= 0) return;
    const float inv_n = 1.0f / (float)cols;
    for (int r = 0; r < rows; ++r) {
        const float* x = in + (size_t)r * cols;
        float* o = out + (size_t)r * cols;
        float s = 0.0f;
        for (int i = 0; i < cols; ++i) s += x[i] * x[i];
        const float sc = 1.0f / sqrtf(s * inv_n + eps);
        for (int i = 0; i < cols; ++i) { float y = x[i] * sc; if (gamma) y *= gamma[i]; o[i] = y; }
    }
}

/* [NORM] softmax rows (max-subtract, exp, divide when sum > 0); log form: x - (log sum + max) */
ORC_API void orc_f32_softmax_rows(const float* in, float* out, int32_t rows, int32_t cols, int32_t log_form) {
    if (rows <= 0 || cols <= 0) return;
    for (int r = 0; r < rows; ++r) {
        const float* x = in + (size_t)r * cols;
        float* o = out + (size_t)r * cols;
        float m = x[0];
        for (int i = 1; i < cols; ++i) if (x[i] > m) m = x[i];
        float sum = 0.0f;
        if (log_form) {
            for (int i = 0; i < cols; ++i) sum += expf(x[i] - m);
            const float lse = logf(sum) + m;
            for (int i = 0; i < cols; ++i) o[i] = x[i] - lse;
            continue;
        }
        for (int i = 0; i < cols; ++i) { o[i] = expf(x[i] - m); sum += o[i]; }
        if (sum > 0.0f) { const float inv = 1.0f / sum; for (int i = 0; i < cols; ++i) o[i] *= inv; }
    }
}

/* [SGEMM] C(m,n) = A(m,k) * B(k,n), float strides, full overwrite, ascending-p sums. */
ORC_API void orc_fp32_matmul(const float* a, int32_t a_offset, int32_t a_stride, const float* b,
                             int32_t b_offset, int32_t b_stride, float* c, int32_t c_offset,
                             int32_t c_stride, int32_t m, int32_t n, int32_t k) {
    if (m <= 0 || n <= 0) return;
    for (int i = 0; i < m; ++i) for (int j = 0; j < n; ++j) {
        float s = 0.0f;
        for (int p = 0; p < k; ++p)
            s += a[a_offset + (size_t)i * a_stride + p] * b[b_offset + (size_t)p * b_stride + j];
        c[c_offset + (size_t)i * c_stride + j] = s;
    }
}

/* [SGEMM] out[i,o] = sum_p in[i,p] * w[o,p] */
ORC_API void orc_fp32_matmul_wt(const float* in, int32_t in_offset, const float* w, int32_t w_offset,
                                float* out, int32_t out_offset, int32_t m, int32_t n, int32_t k) {
    if (m <= 0 || n <= 0 || k < 0) return;
    for (int i = 0; i < m; ++i) for (int o = 0; o < n; ++o) {
        float s = 0.0f;
        for (int p = 0; p < k; ++p) s += in[in_offset + (size_t)i * k + p] * w[w_offset + (size_t)o * k + p];
        out[out_offset + (size_t)i * n + o] = s;
    }
}

/* ---------------------------------------------------------------- int8-activation "native" path
 *
 * A port of the reference's timed C path [NQ4K][NQ6K][NQ80], row-major entries only, single thread.
 * It is NOT the parity oracle (it differs from the exact kernels by the activation quantisation);
 * it exists so a CPU timing baseline is available when oracle/_ref was not built, and as a
 * cross-check of the reference-built library (the integer dots make the two bit-identical).
 */
static float q8_act_block(const float* in, int8_t* q8) {
    float maxabs = 0.0f;
    for (int i = 0; i < QK_BS; ++i) { const float a = fabsf(in[i]); if (a > maxabs) maxabs = a; }
    if (maxabs == 0.0f) { memset(q8, 0, QK_BS); return 0.0f; }
    const float d_in = maxabs / 127.0f;
    const float inv = 127.0f / maxabs;
    for (int i = 0; i < QK_BS; ++i) {
        int v = (int)lrintf(in[i] * inv);
        if (v > 127) v = 127; else if (v < -127) v = -127;
        q8[i] = (int8_t)v;
    }
    return d_in;
}

ORC_API void orc_native_q4k_matmul_rm(const float* input, int32_t input_offset, const uint8_t* weight,
                                      int32_t weight_byte_offset, int32_t input_dim, int32_t output_dim,
                                      float* output, int32_t output_offset) {
    if (output_dim <= 0 || input_dim <= 0) return;
    const int bpr = input_dim / QK_BS;
    int8_t* q8 = (int8_t*)malloc((size_t)input_dim);
    float* d_in = (float*)malloc((size_t)bpr * sizeof(float));
    if (!q8 || !d_in) { free(q8); free(d_in); return; }
    for (int b = 0; b < bpr; ++b) d_in[b] = q8_act_block(input + input_offset + (size_t)b * QK_BS, q8 + (size_t)b * QK_BS);
    const uint8_t* p = weight + weight_byte_offset;
    for (int o = 0; o < output_dim; ++o) {
        float acc = 0.0f;
        for (int b = 0; b < bpr; ++b, p += Q4K_BYTES) {
            const float d = orc_half_to_float(le16(p));
            const float dmin = orc_half_to_float(le16(p + 2));
            int sc[8], mn[8];
            q4k_scale_min(p + 4, sc, mn);
            const int8_t* a = q8 + (size_t)b * QK_BS;
            int64_t sdot = 0, msum = 0;
            for (int g = 0; g < 4; ++g) {
                int32_t dl = 0, sl = 0, dh = 0, sh = 0;
                for (int i = 0; i < 32; ++i) {
                    const int byte = p[16 + g * 32 + i];
                    dl += a[(2 * g) * 32 + i] * (byte & 0x0F); sl += a[(2 * g) * 32 + i];
                    dh += a[(2 * g + 1) * 32 + i] * (byte >> 4); sh += a[(2 * g + 1) * 32 + i];
                }
                sdot += (int64_t)sc[2 * g] * dl + (int64_t)sc[2 * g + 1] * dh;
                msum += (int64_t)mn[2 * g] * sl + (int64_t)mn[2 * g + 1] * sh;
            }
            acc += d_in[b] * (d * (float)sdot - dmin * (float)msum);
        }
        output[output_offset + o] = acc;
    }
    free(q8); free(d_in);
}

ORC_API void orc_native_q6k_matmul_rm(const float* input, int32_t input_offset, const uint8_t* weight,
                                      int32_t weight_byte_offset, int32_t input_dim, int32_t output_dim,
                                      float* output, int32_t output_offset) {
    if (output_dim <= 0 || input_dim <= 0) return;
    const int bpr = input_dim / QK_BS;
    int8_t* q8 = (int8_t*)malloc((size_t)input_dim);
    float* d_in = (float*)malloc((size_t)bpr * sizeof(float));
    if (!q8 || !d_in) { free(q8); free(d_in); return; }
    for (int b = 0; b < bpr; ++b) d_in[b] = q8_act_block(input + input_offset + (size_t)b * QK_BS, q8 + (size_t)b * QK_BS);
    const uint8_t* p = weight + weight_byte_offset;
    int8_t codes[QK_BS];
    for (int o = 0; o < output_dim; ++o) {
        float acc = 0.0f;
        for (int b = 0; b < bpr; ++b, p += Q6K_BYTES) {
            const float d = orc_half_to_float(le16(p + 208));
            const int8_t* sc = (const int8_t*)(p + 192);
            for (int half = 0; half < 2; ++half) for (int l = 0; l < 32; ++l) {
                const int ql0 = p[half * 64 + l], ql32 = p[half * 64 + l + 32], qh = p[128 + half * 32 + l];
                int8_t* c = codes + half * 128;
                c[l] = (int8_t)(((ql0 & 0x0F) | ((qh & 3) << 4)) - 32);
                c[l + 32] = (int8_t)(((ql32 & 0x0F) | (((qh >> 2) & 3) << 4)) - 32);
                c[l + 64] = (int8_t)(((ql0 >> 4) | (((qh >> 4) & 3) << 4)) - 32);
                c[l + 96] = (int8_t)(((ql32 >> 4) | (((qh >> 6) & 3) << 4)) - 32);
            }
            const int8_t* a = q8 + (size_t)b * QK_BS;
            int64_t wdot = 0;
            for (int g = 0; g < 16; ++g) {
                int32_t dot = 0;
                for (int j = 0; j < 16; ++j) dot += (int)a[g * 16 + j] * (int)codes[g * 16 + j];
                /* group g covers elements [16g, 16g+16): half = g/8, k = (g%8)/2, is = g%2 -> sc[half*8 + is + 2k] */
                wdot += (int64_t)sc[(g / 8) * 8 + (g % 2) + 2 * ((g % 8) / 2)] * dot;
            }
            acc += d * d_in[b] * (float)wdot;
        }
        output[output_offset + o] = acc;
    }
    free(q8); free(d_in);
}

ORC_API void orc_native_q8_0_matmul_rm(const float* input, int32_t input_offset, const uint8_t* weight,
                                       int32_t weight_byte_offset, int32_t input_dim, int32_t output_dim,
                                       float* output, int32_t output_offset) {
    if (output_dim <= 0) return;
    if (input_dim <= 0) { for (int o = 0; o < output_dim; ++o) output[output_offset + o] = 0.0f; return; }
    const int bpr = input_dim / Q80_BS;
    const uint8_t* p = weight + weight_byte_offset;
    for (int o = 0; o < output_dim; ++o) {
        float acc = 0.0f;
        for (int b = 0; b < bpr; ++b, p += Q80_BYTES) {
            const float d = orc_half_to_float(le16(p));
            const int8_t* codes = (const int8_t*)(p + 2);
            const float* x = input + input_offset + (size_t)b * Q80_BS;
            float s = 0.0f;
            for (int k = 0; k < Q80_BS; ++k) s += x[k] * (float)codes[k];
            acc += s * d;
        }
        output[output_offset + o] = acc;
    }
}

/* ---------------------------------------------------------------- fp32 x bf16 / fp16 dense matmul [NARROW]
 * C(m, n) = A(m, k) B(k, n): A and C fp32 with float strides, B two bytes per element with a byte row stride;
 * sum in fp32 over ascending p; k == 0 zeroes the block. */
static void narrow_matmul(const float* a, int32_t a_offset, int32_t a_stride, const uint8_t* b, int32_t b_byte_offset,
                          int32_t b_byte_stride, float* out, int32_t out_offset, int32_t out_stride, int32_t m, int32_t n,
                          int32_t k, int is_fp16) {
    if (m <= 0 || n <= 0) return;
    for (int32_t i = 0; i < m; ++i) {
        for (int32_t j = 0; j < n; ++j) {
            float sum = 0.0f;
            for (int32_t p = 0; p < k; ++p) {
                const uint32_t h = le16(b + b_byte_offset + (int64_t)p * b_byte_stride + 2 * j);
                const float bf = is_fp16 ? orc_half_to_float(h) : bits_f32(h << 16);
                sum += a[a_offset + (int64_t)i * a_stride + p] * bf;
            }
            out[out_offset + (int64_t)i * out_stride + j] = sum;
        }
    }
}
ORC_API void orc_bf16_matmul(const float* a, int32_t a_offset, int32_t a_stride, const uint8_t* b, int32_t b_byte_offset,
                             int32_t b_byte_stride, float* out, int32_t out_offset, int32_t out_stride, int32_t m, int32_t n, int32_t k) {
    narrow_matmul(a, a_offset, a_stride, b, b_byte_offset, b_byte_stride, out, out_offset, out_stride, m, n, k, 0);
}
ORC_API void orc_fp16_matmul(const float* a, int32_t a_offset, int32_t a_stride, const uint8_t* b, int32_t b_byte_offset,
                             int32_t b_byte_stride, float* out, int32_t out_offset, int32_t out_stride, int32_t m, int32_t n, int32_t k) {
    narrow_matmul(a, a_offset, a_stride, b, b_byte_offset, b_byte_stride, out, out_offset, out_stride, m, n, k, 1);
}
