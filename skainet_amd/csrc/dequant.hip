// Bit-exact GGUF block decode on the device: packed Q8_0 / Q4_K / Q6_K (and Q4_0 / Q5_0 / Q5_1 / Q5_K) bytes -> fp32.
//
// Every product and difference is rounded exactly where the reference decoders round
// (explicit __fmul_rn / __fsub_rn, never an FMA), so the output bits equal
//   Q8_0: (float)code * d                         Q8_0TensorData.kt:80-89
//   Q4_K: code * (d * scaleIdx) - (dmin * minIdx)  Q4_KTensorData.kt:120-136, :184-206, :215-226
//   Q6_K: (d * sc) * q,  q = 6-bit code - 32       Q6_KTensorData.kt:112-165
//   Q4_0: (float)(code - 8) * d                    Q4_0TensorData.kt:93-107 (low nibbles: elements 0..15, high: 16..31)
//   Q5_0: d * (float)(code5 - 16)                  Q5_0TensorData.kt:68-86  (fifth bit j of the 32-bit plane `qh`)
//   Q5_1: d * (float)code5 + m                     Q5_1TensorData.kt:73-92
//   Q5_K: code5 * (d * scaleIdx) - (dmin * minIdx)  Q5_KTensorData.kt:126-142, :190-236
// (paths under /root/reference/skainet-lang/skainet-lang-core/src/commonMain/kotlin/sk/ainet/lang/tensor/data/).
//
// HBM-bound: one thread decodes 8 (Q8_0: all 32 of a block per 4 threads) consecutive outputs and
// writes them as two float4 stores; algorithmic traffic = packed bytes in + 4 B/element out.
#include "common.h"

namespace skh {

// Output block b reads source block b, or -- for a row gather -- block (b % bpr) of source row row_ids[b / bpr]. A row
// id outside [0, rows) (ids that reach the device unchecked, e.g. a sampled token fed back) is clamped into the weight:
// the read stays inside the allocation; hosts that hold the ids validate them before the call.
__device__ __forceinline__ int64_t source_block(int64_t b, const int32_t* row_ids, int bpr, int rows) {
    return row_ids ? (int64_t)min(max(row_ids[b / bpr], 0), rows - 1) * bpr + (b % bpr) : b;
}

// One thread per 8 output elements; 4 threads per Q8_0 block.
__global__ __launch_bounds__(256) void dequant_q8_0_kernel(const uint8_t* __restrict__ w, float* __restrict__ out,
                                                           int64_t nblocks, const int32_t* __restrict__ row_ids, int bpr, int rows) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t b = t >> 2;
    if (b >= nblocks) return;
    const int part = (int)(t & 3);
    const uint8_t* p = w + source_block(b, row_ids, bpr, rows) * Q80_BYTES;
    const float d = half_bits_to_float(load_u16(p));
    const uint8_t* c = p + 2 + part * 8;
    const uint32_t lo = load_u32_a2(c), hi = load_u32_a2(c + 4);
    float4 a, bq;
    a.x = __fmul_rn((float)(int8_t)(lo), d);
    a.y = __fmul_rn((float)(int8_t)(lo >> 8), d);
    a.z = __fmul_rn((float)(int8_t)(lo >> 16), d);
    a.w = __fmul_rn((float)(int8_t)(lo >> 24), d);
    bq.x = __fmul_rn((float)(int8_t)(hi), d);
    bq.y = __fmul_rn((float)(int8_t)(hi >> 8), d);
    bq.z = __fmul_rn((float)(int8_t)(hi >> 16), d);
    bq.w = __fmul_rn((float)(int8_t)(hi >> 24), d);
    float4* o = reinterpret_cast<float4*>(out + b * Q80_ELEMS + part * 8);
    o[0] = a;
    o[1] = bq;
}

__device__ __forceinline__ void q4k_scale_min(const uint8_t* s, int j, int& sc, int& mn) {
    if (j < 4) {
        sc = s[j] & 63;
        mn = s[j + 4] & 63;
    } else {
        sc = (s[j + 4] & 0x0F) | ((s[j - 4] >> 6) << 4);
        mn = (s[j + 4] >> 4) | ((s[j] >> 6) << 4);
    }
}

// One thread per 8 output elements; 32 threads per Q4_K block. Thread u: sub-block sb = u / 4,
// elements [8 * (u % 4), +8) of it, i.e. 8 consecutive bytes of 32-byte group sb / 2, low or high nibble.
__global__ __launch_bounds__(256) void dequant_q4k_kernel(const uint8_t* __restrict__ w, float* __restrict__ out,
                                                          int64_t nblocks, const int32_t* __restrict__ row_ids, int bpr, int rows) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t b = t >> 5;
    if (b >= nblocks) return;
    const int u = (int)(t & 31), sb = u >> 2, e0 = (u & 3) * 8;
    const uint8_t* p = w + source_block(b, row_ids, bpr, rows) * Q4K_BYTES;
    const uint32_t dd = *reinterpret_cast<const uint32_t*>(p);
    const float d = half_bits_to_float(dd & 0xFFFFu), dmin = half_bits_to_float(dd >> 16);
    int sc, mn;
    q4k_scale_min(p + 4, sb, sc, mn);
    const float scale = __fmul_rn(d, (float)sc);
    const float offset = __fmul_rn(dmin, (float)mn);
    const uint2 q = *reinterpret_cast<const uint2*>(p + 16 + (sb >> 1) * 32 + e0);
    const int shift = (sb & 1) * 4;
    float v[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[i] = __fsub_rn(__fmul_rn((float)((q.x >> (8 * i + shift)) & 0xF), scale), offset);
        v[4 + i] = __fsub_rn(__fmul_rn((float)((q.y >> (8 * i + shift)) & 0xF), scale), offset);
    }
    float4* o = reinterpret_cast<float4*>(out + b * QK_ELEMS + sb * 32 + e0);
    o[0] = make_float4(v[0], v[1], v[2], v[3]);
    o[1] = make_float4(v[4], v[5], v[6], v[7]);
}

// One thread per 8 output elements; 32 threads per Q6_K block. Thread u: half = u / 16, quarter k = (u / 4) % 4
// (output offset 32 * k inside the half), elements l in [8 * (u % 4), +8).
__global__ __launch_bounds__(256) void dequant_q6k_kernel(const uint8_t* __restrict__ w, float* __restrict__ out,
                                                          int64_t nblocks, const int32_t* __restrict__ row_ids, int bpr, int rows) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t b = t >> 5;
    if (b >= nblocks) return;
    const int u = (int)(t & 31), half = u >> 4, k = (u >> 2) & 3, l0 = (u & 3) * 8;
    const uint8_t* p = w + source_block(b, row_ids, bpr, rows) * Q6K_BYTES;
    const float d = half_bits_to_float(load_u16(p + 208));
    const int8_t sc = (int8_t)p[192 + half * 8 + (l0 >> 4) + 2 * k];
    const float ds = __fmul_rn(d, (float)sc);
    const uint8_t* ql = p + half * 64 + (k & 1) * 32 + l0;
    const uint8_t* qh = p + 128 + half * 32 + l0;
    const uint32_t ql0 = load_u32_a2(ql), ql1 = load_u32_a2(ql + 4);
    const uint32_t qh0 = load_u32_a2(qh), qh1 = load_u32_a2(qh + 4);
    const int nib_shift = (k >> 1) * 4, hi_shift = 2 * k;
    float v[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int q0 = (int)(((ql0 >> (8 * i + nib_shift)) & 0xF) | ((((qh0 >> (8 * i)) >> hi_shift) & 3) << 4)) - 32;
        const int q1 = (int)(((ql1 >> (8 * i + nib_shift)) & 0xF) | ((((qh1 >> (8 * i)) >> hi_shift) & 3) << 4)) - 32;
        v[i] = __fmul_rn(ds, (float)q0);
        v[4 + i] = __fmul_rn(ds, (float)q1);
    }
    float4* o = reinterpret_cast<float4*>(out + b * QK_ELEMS + half * 128 + k * 32 + l0);
    o[0] = make_float4(v[0], v[1], v[2], v[3]);
    o[1] = make_float4(v[4], v[5], v[6], v[7]);
}

// Q4_0 / Q5_0 / Q5_1: 32-element blocks of 18 / 22 / 24 bytes (fp16 d [, fp16 m] [, 4 bytes of fifth bits], 16 bytes of
// nibbles). One thread per 8 output elements, 4 threads per block: part p < 2 decodes the low nibbles of bytes
// 8p .. 8p+7, part p >= 2 the high nibbles of bytes 8(p-2) .. 8(p-2)+7. FMT: 0 = Q4_0, 1 = Q5_0, 2 = Q5_1.
template <int FMT>
__global__ __launch_bounds__(256) void dequant_q45_kernel(const uint8_t* __restrict__ w, float* __restrict__ out,
                                                          int64_t nblocks, const int32_t* __restrict__ row_ids, int bpr, int rows) {
    constexpr int BYTES = FMT == 0 ? Q40_BYTES : (FMT == 1 ? Q50_BYTES : Q51_BYTES);
    constexpr int QH = FMT == 2 ? 4 : 2, QS = FMT == 0 ? 2 : QH + 4;
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t b = t >> 2;
    if (b >= nblocks) return;
    const int part = (int)(t & 3), byte0 = (part & 1) * 8, shift = (part >> 1) * 4;
    const uint8_t* p = w + source_block(b, row_ids, bpr, rows) * BYTES;
    const float d = half_bits_to_float(load_u16(p));
    float m = 0.f;
    uint32_t qh = 0;
    if (FMT == 2) m = half_bits_to_float(load_u16(p + 2));
    if (FMT != 0) qh = load_u16(p + QH) | (load_u16(p + QH + 2) << 16);
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int j = byte0 + i;                                  // byte of the block's nibble plane; element j or 16 + j
        int code = (p[QS + j] >> shift) & 0xF;
        if (FMT != 0) code |= (int)((qh >> (part * 8 + i)) & 1u) << 4;
        if (FMT == 0) v[i] = __fmul_rn((float)(code - 8), d);
        else if (FMT == 1) v[i] = __fmul_rn(d, (float)(code - 16));
        else v[i] = __fadd_rn(__fmul_rn(d, (float)code), m);
    }
    float4* o = reinterpret_cast<float4*>(out + b * Q80_ELEMS + part * 8);
    o[0] = make_float4(v[0], v[1], v[2], v[3]);
    o[1] = make_float4(v[4], v[5], v[6], v[7]);
}

// Q5_K: the Q4_K layout with a 32-byte plane of fifth bits at byte 16 and the nibbles at byte 48 (176 bytes). Thread
// u of 32: sub-block sb = u / 4, elements [8 * (u % 4), +8): bytes e0 .. e0+7 of nibble group sb / 2, bit sb of qh[e0 ..].
__global__ __launch_bounds__(256) void dequant_q5k_kernel(const uint8_t* __restrict__ w, float* __restrict__ out,
                                                          int64_t nblocks, const int32_t* __restrict__ row_ids, int bpr, int rows) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t b = t >> 5;
    if (b >= nblocks) return;
    const int u = (int)(t & 31), sb = u >> 2, e0 = (u & 3) * 8;
    const uint8_t* p = w + source_block(b, row_ids, bpr, rows) * Q5K_BYTES;
    const uint32_t dd = *reinterpret_cast<const uint32_t*>(p);
    const float d = half_bits_to_float(dd & 0xFFFFu), dmin = half_bits_to_float(dd >> 16);
    int sc, mn;
    q4k_scale_min(p + 4, sb, sc, mn);
    const float scale = __fmul_rn(d, (float)sc);
    const float offset = __fmul_rn(dmin, (float)mn);
    const uint2 q = *reinterpret_cast<const uint2*>(p + 48 + (sb >> 1) * 32 + e0);
    const uint2 h = *reinterpret_cast<const uint2*>(p + 16 + e0);
    const int shift = (sb & 1) * 4;
    float v[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t c0 = ((q.x >> (8 * i + shift)) & 0xF) | (((h.x >> (8 * i + sb)) & 1u) << 4);
        const uint32_t c1 = ((q.y >> (8 * i + shift)) & 0xF) | (((h.y >> (8 * i + sb)) & 1u) << 4);
        v[i] = __fsub_rn(__fmul_rn((float)c0, scale), offset);
        v[4 + i] = __fsub_rn(__fmul_rn((float)c1, scale), offset);
    }
    float4* o = reinterpret_cast<float4*>(out + b * QK_ELEMS + sb * 32 + e0);
    o[0] = make_float4(v[0], v[1], v[2], v[3]);
    o[1] = make_float4(v[4], v[5], v[6], v[7]);
}

// Decodes `nblocks` consecutive output blocks; with `row_ids` (device int32) output row r is source row row_ids[r]
// of a weight with `bpr` blocks per row.
int launch_dequant(int enc, const uint8_t* w, int64_t nblocks, float* out, const int32_t* row_ids, int bpr, int rows) {
    if (nblocks <= 0) return 0;
    if (!is_packed(enc)) return set_error("dequantize: unsupported encoding %d", enc);
    hipStream_t s = current_stream();
    const int64_t threads = nblocks * (block_elems(enc) / 8);
    const int64_t grid = (threads + 255) / 256;
    if (grid > 0x7FFFFFFFLL) return set_error("dequantize: %lld blocks exceed one launch", (long long)nblocks);
    if (enc == ENC_Q8_0) dequant_q8_0_kernel<<<dim3((unsigned)grid), dim3(256), 0, s>>>(w, out, nblocks, row_ids, bpr, rows);
    else if (enc == ENC_Q4_K) dequant_q4k_kernel<<<dim3((unsigned)grid), dim3(256), 0, s>>>(w, out, nblocks, row_ids, bpr, rows);
    else if (enc == ENC_Q5_K) dequant_q5k_kernel<<<dim3((unsigned)grid), dim3(256), 0, s>>>(w, out, nblocks, row_ids, bpr, rows);
    else if (enc == ENC_Q4_0) dequant_q45_kernel<0><<<dim3((unsigned)grid), dim3(256), 0, s>>>(w, out, nblocks, row_ids, bpr, rows);
    else if (enc == ENC_Q5_0) dequant_q45_kernel<1><<<dim3((unsigned)grid), dim3(256), 0, s>>>(w, out, nblocks, row_ids, bpr, rows);
    else if (enc == ENC_Q5_1) dequant_q45_kernel<2><<<dim3((unsigned)grid), dim3(256), 0, s>>>(w, out, nblocks, row_ids, bpr, rows);
    else dequant_q6k_kernel<<<dim3((unsigned)grid), dim3(256), 0, s>>>(w, out, nblocks, row_ids, bpr, rows);
    SKH_CHECK(hipGetLastError());
    return 0;
}

}  // namespace skh
