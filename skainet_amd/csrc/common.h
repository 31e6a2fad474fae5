// Shared declarations of the gfx950 kernel library: block geometry, error plumbing, small device helpers.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace skh {

// GGUF block geometry (elements per block, bytes per block); see
// /root/reference/skainet-lang/skainet-lang-core/src/commonMain/kotlin/sk/ainet/lang/memory/BlockSpec.kt:84-87
constexpr int Q80_ELEMS = 32, Q80_BYTES = 34;
constexpr int QK_ELEMS = 256, Q4K_BYTES = 144, Q6K_BYTES = 210;
constexpr int Q40_BYTES = 18, Q50_BYTES = 22, Q51_BYTES = 24, Q5K_BYTES = 176;   // Q4_0 / Q5_0 / Q5_1: 32 elements; Q5_K: 256

// Encoding ids are the GGML tensor-type numbers the GGUF reader maps from
// (/root/reference/skainet-io/skainet-io-gguf/src/commonMain/kotlin/sk/ainet/io/gguf/StreamingGGUFReader.kt:190-211).
enum Encoding : int32_t { ENC_F32 = 0, ENC_Q4_0 = 2, ENC_Q5_0 = 6, ENC_Q5_1 = 7, ENC_Q8_0 = 8, ENC_Q4_K = 12, ENC_Q5_K = 13, ENC_Q6_K = 14 };

inline bool is_packed(int enc) {
    return enc == ENC_Q8_0 || enc == ENC_Q4_K || enc == ENC_Q6_K || enc == ENC_Q4_0 || enc == ENC_Q5_0 || enc == ENC_Q5_1 || enc == ENC_Q5_K;
}
inline int block_elems(int enc) { return (enc == ENC_Q4_K || enc == ENC_Q5_K || enc == ENC_Q6_K) ? QK_ELEMS : Q80_ELEMS; }
inline int block_bytes(int enc) {
    switch (enc) {
        case ENC_Q4_0: return Q40_BYTES;
        case ENC_Q5_0: return Q50_BYTES;
        case ENC_Q5_1: return Q51_BYTES;
        case ENC_Q8_0: return Q80_BYTES;
        case ENC_Q4_K: return Q4K_BYTES;
        case ENC_Q5_K: return Q5K_BYTES;
        default: return Q6K_BYTES;
    }
}

// ---- error plumbing (shim.hip owns the storage) ----
int set_error(const char* fmt, ...);          // records a thread-local message, returns -1
int check_hip(hipError_t e, const char* what);  // 0 on success, else records and returns -1
hipStream_t current_stream();                 // the calling thread's launch stream
int ensure_device();                          // lazily initialises the device; 0 when usable
int num_cus();

#define SKH_CHECK(expr)                                     \
    do {                                                    \
        if (skh::check_hip((expr), #expr) != 0) return -1;  \
    } while (0)

#define SKH_LAUNCH_CHECK(name) SKH_CHECK((hipGetLastError()))

// ---- device helpers ----

// IEEE binary16 bits -> binary32, exact for every finite value including subnormals (integer ops only,
// so the result never depends on the FP16 denormal mode).
__device__ __forceinline__ float half_bits_to_float(uint32_t h) {
    const uint32_t sign = (h & 0x8000u) << 16;
    const uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t mant = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (mant == 0) {
            bits = sign;
        } else {
            const int lz = __clz(mant) - 21;  // shifts needed to bring the leading 1 to bit 10
            mant = (mant << lz) & 0x3FFu;
            bits = sign | ((uint32_t)(127 - 14 - lz) << 23) | (mant << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (mant << 13);
    } else {
        bits = sign | ((exp + 112u) << 23) | (mant << 13);
    }
    return __uint_as_float(bits);
}

// RoPE rotation of an adjacent pair by (cos, sin), with the roundings spelled out so that every kernel that rotates
// (prompt scatter, decode epilogue) produces the same bits whatever the compiler contracts elsewhere.
__device__ __forceinline__ float2 rope_rotate(float x0, float x1, float cs, float sn) {
    return make_float2(__fmaf_rn(x0, cs, -__fmul_rn(x1, sn)), __fmaf_rn(x0, sn, __fmul_rn(x1, cs)));
}

// Hardware fp16 -> fp32 (v_cvt_f32_f16): one instruction; used where the result feeds tolerance-checked sums.
__device__ __forceinline__ float half_bits_to_float_fast(uint32_t h) {
    const uint16_t b = (uint16_t)h;
    _Float16 v;
    __builtin_memcpy(&v, &b, 2);
    return (float)v;
}

// Byte N of a dword as float (v_cvt_f32_ubyteN). Written as asm so the compiler keeps one pre-masked dword
// and four conversions instead of re-deriving a shift/mask per byte. The result must pass through another vector-ALU
// instruction before a matrix instruction reads it: an MFMA operand written by the VALU instruction just before needs
// wait states that the compiler only inserts for writes it can see, not for inline assembly (kernels that feed
// conversions straight into an MFMA write them in plain C instead).
__device__ __forceinline__ float ubyte0_to_float(uint32_t v) { float f; asm("v_cvt_f32_ubyte0_e32 %0, %1" : "=v"(f) : "v"(v)); return f; }
__device__ __forceinline__ float ubyte1_to_float(uint32_t v) { float f; asm("v_cvt_f32_ubyte1_e32 %0, %1" : "=v"(f) : "v"(v)); return f; }
__device__ __forceinline__ float ubyte2_to_float(uint32_t v) { float f; asm("v_cvt_f32_ubyte2_e32 %0, %1" : "=v"(f) : "v"(v)); return f; }
__device__ __forceinline__ float ubyte3_to_float(uint32_t v) { float f; asm("v_cvt_f32_ubyte3_e32 %0, %1" : "=v"(f) : "v"(v)); return f; }
template <int J> __device__ __forceinline__ float ubyte_to_float(uint32_t v) {
    if constexpr (J == 0) return ubyte0_to_float(v);
    else if constexpr (J == 1) return ubyte1_to_float(v);
    else if constexpr (J == 2) return ubyte2_to_float(v);
    else return ubyte3_to_float(v);
}

// Loads that tolerate the 2-byte alignment of Q8_0 / Q6_K blocks (34 and 210 bytes per block).
struct __attribute__((packed, aligned(2))) u32_a2 { uint32_t v; };
__device__ __forceinline__ uint32_t load_u32_a2(const uint8_t* p) { return reinterpret_cast<const u32_a2*>(p)->v; }
__device__ __forceinline__ uint32_t load_u16(const uint8_t* p) { return *reinterpret_cast<const uint16_t*>(p); }
// 16 bytes from a 4-byte aligned address as one load (global dwordx4 loads need dword alignment only).
typedef uint32_t u32x4_vec __attribute__((ext_vector_type(4)));
struct __attribute__((packed, aligned(4))) u32x4_a4 { u32x4_vec v; };
__device__ __forceinline__ u32x4_vec load_u32x4_a4(const uint8_t* p) { return reinterpret_cast<const u32x4_a4*>(p)->v; }
// 8 bytes from a 2-byte aligned address as one load.
typedef uint32_t u32x2_vec __attribute__((ext_vector_type(2)));
struct __attribute__((packed, aligned(2))) u32x2_a2 { u32x2_vec v; };
__device__ __forceinline__ u32x2_vec load_u32x2_a2(const uint8_t* p) { return reinterpret_cast<const u32x2_a2*>(p)->v; }
// The same from a 2-byte aligned address (Q6_K code runs): still one global_load_dwordx4, which this device serves.
struct __attribute__((packed, aligned(2))) u32x4_a2 { u32x4_vec v; };
__device__ __forceinline__ u32x4_vec load_u32x4_a2(const uint8_t* p) { return reinterpret_cast<const u32x4_a2*>(p)->v; }

// Sum over the 16 lanes of a DPP row (lanes 16 r .. 16 r + 15), result in every lane: four rotate-and-add steps inside
// the vector ALU instead of four round trips through the LDS crossbar.
template <int CTRL>
__device__ __forceinline__ float dpp_row_move(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ float row16_max(float v) {
    v = fmaxf(v, dpp_row_move<0x128>(v));
    v = fmaxf(v, dpp_row_move<0x124>(v));
    v = fmaxf(v, dpp_row_move<0x122>(v));
    v = fmaxf(v, dpp_row_move<0x121>(v));
    return v;
}
__device__ __forceinline__ float row16_sum(float v) {
    v += dpp_row_move<0x128>(v);   // row_ror:8
    v += dpp_row_move<0x124>(v);   // row_ror:4
    v += dpp_row_move<0x122>(v);   // row_ror:2
    v += dpp_row_move<0x121>(v);   // row_ror:1
    return v;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
    return v;
}
// Fold NV (a power of two, <= 64) per-lane values across the 64 lanes of a wave with a multi-value butterfly:
// each of the first log2(NV) steps halves the number of live values (a lane keeps the half selected by one bit of
// its lane id and hands the other half to its partner), the remaining steps are plain xor-shuffle adds. On return
// v[0] of lane l holds the wave-wide total of value wave_fold_index<NV>(l). The selects are written as bit-field
// inserts on the raw bits so they stay one instruction each (a ?: on array elements is turned into an indexed
// register read, which this target expands into a compare/select chain per element).
template <int NV>
__device__ __forceinline__ void wave_fold(float* v, int lane) {
    static_assert(NV >= 1 && NV <= 64 && (NV & (NV - 1)) == 0, "every halving must pair all values: NV is a power of two");
    int mask = 1;
#pragma unroll
    for (int nv = NV; nv > 1; nv >>= 1, mask <<= 1) {
        const int half = nv >> 1;
        const uint32_t up = (lane & mask) ? 0xFFFFFFFFu : 0u;
#pragma unroll
        for (int i = 0; i < half; ++i) {
            const uint32_t a = __float_as_uint(v[i]), b = __float_as_uint(v[i + half]);
            const float send = __uint_as_float((a & up) | (b & ~up));
            const float keep = __uint_as_float((b & up) | (a & ~up));
            v[i] = keep + __shfl_xor(send, mask, 64);
        }
    }
#pragma unroll
    for (int m = NV; m < 64; m <<= 1) v[0] += __shfl_xor(v[0], m, 64);
}
template <int NV>
__device__ __forceinline__ int wave_fold_index(int lane) {
    int idx = 0, mask = 1;
#pragma unroll
    for (int nv = NV; nv > 1; nv >>= 1, mask <<= 1) idx += (lane & mask) ? (nv >> 1) : 0;
    return idx;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, 64));
    return v;
}

}  // namespace skh
