// Shared declarations of the gfx950 kernel library: block geometry, error plumbing, small device helpers.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <mutex>

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
void note_kernel(const char* family);    // remembers the kernel family this thread launched last (skainet_hip_last_kernel)

#define SKH_CHECK(expr)                                     \
    do {                                                    \
        if (skh::check_hip((expr), #expr) != 0) return -1;  \
    } while (0)

#define SKH_LAUNCH_CHECK(name) SKH_CHECK((hipGetLastError()))

// Raises a kernel's dynamic-LDS limit exactly once per process, whichever thread launches it first (every thread
// passes through the same once-flag; a failure is remembered and reported to every caller).
#define SKH_SET_MAX_DYNAMIC_LDS_ONCE(kernel_ptr, bytes)                                                         \
    do {                                                                                                        \
        static std::once_flag skh_once;                                                                         \
        static int skh_once_rc = 0;                                                                             \
        std::call_once(skh_once, [&] {                                                                          \
            skh_once_rc = skh::check_hip(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel_ptr),        \
                                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)(bytes)), \
                                         "hipFuncSetAttribute(max dynamic LDS)");                               \
        });                                                                                                     \
        if (skh_once_rc != 0) return skh::set_error("kernel attribute could not be set: dynamic LDS of %d bytes refused", (int)(bytes)); \
    } while (0)

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

// Wave-wide sum, result in every lane: the 16 lanes of a row inside the vector ALU, the four rows by two shuffles.
__device__ __forceinline__ float wave_sum(float v) {
    v = row16_sum(v);
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    return v;
}

// The value of the lane that differs from this one in lane-id bit BIT and shares every higher bit: the partner of one
// butterfly step. Inside a row of 16 lanes these are DPP moves (row_mirror = lane ^ 15, row_half_mirror = lane ^ 7,
// quad permutes = lane ^ 2, lane ^ 1: bits below BIT may flip as well, which a step that has not used them yet does not
// mind); across rows a shuffle through the LDS crossbar.
template <int BIT>
__device__ __forceinline__ float fold_partner(float v) {
    if constexpr (BIT == 5) return __shfl_xor(v, 32, 64);
    else if constexpr (BIT == 4) return __shfl_xor(v, 16, 64);
    else if constexpr (BIT == 3) return dpp_row_move<0x140>(v);   // row_mirror
    else if constexpr (BIT == 2) return dpp_row_move<0x141>(v);   // row_half_mirror
    else if constexpr (BIT == 1) return dpp_row_move<0x4E>(v);    // quad_perm:[2,3,0,1]
    else return dpp_row_move<0xB1>(v);                            // quad_perm:[1,0,3,2]
}
// One halving step of wave_fold on lane bit BIT: HALF values stay (the lower or the upper half, by the lane's bit), the
// other HALF go to the partner. The selects are written as bit-field inserts on the raw bits so they stay one
// instruction each (a ?: on array elements is turned into an indexed register read, which this target expands into a
// compare/select chain per element).
template <int BIT, int HALF>
__device__ __forceinline__ void fold_halve(float* v, int lane) {
    const uint32_t up = ((lane >> BIT) & 1) ? 0xFFFFFFFFu : 0u;
#pragma unroll
    for (int i = 0; i < HALF; ++i) {
        const uint32_t a = __float_as_uint(v[i]), b = __float_as_uint(v[i + HALF]);
        const float send = __uint_as_float((a & up) | (b & ~up));
        const float keep = __uint_as_float((b & up) | (a & ~up));
        v[i] = keep + fold_partner<BIT>(send);
    }
}
template <int BIT, int NV>
__device__ __forceinline__ void fold_steps(float* v, int lane) {
    if constexpr ((1 << BIT) < NV) fold_halve<BIT, (1 << BIT)>(v, lane);   // 2 << BIT values are live at this step
    if constexpr (BIT > 0) fold_steps<BIT - 1, NV>(v, lane);
}
// Fold NV (a power of two, <= 64) per-lane values across the 64 lanes of a wave with a multi-value butterfly: the
// log2(NV) low bits of the lane id, taken from the highest down, each halve the number of live values (a lane keeps
// the half its bit selects and hands the other half to its partner); the remaining, higher bits are plain adds of
// v[0] (rotations inside a row, which keep the low bits, then the two cross-row shuffles). On return v[0] of lane l
// holds the wave-wide total of value wave_fold_index<NV>(l) = l mod NV.
template <int NV>
__device__ __forceinline__ void wave_fold(float* v, int lane) {
    static_assert(NV >= 2 && NV <= 64 && (NV & (NV - 1)) == 0, "every halving must pair all values: NV is a power of two");
    fold_steps<5, NV>(v, lane);
    if constexpr (NV <= 8) v[0] += dpp_row_move<0x128>(v[0]);     // row_ror:8
    if constexpr (NV <= 4) v[0] += dpp_row_move<0x124>(v[0]);     // row_ror:4
    if constexpr (NV <= 2) v[0] += dpp_row_move<0x122>(v[0]);     // row_ror:2
    if constexpr (NV <= 16) v[0] += __shfl_xor(v[0], 16, 64);
    if constexpr (NV <= 32) v[0] += __shfl_xor(v[0], 32, 64);
}
template <int NV>
__device__ __forceinline__ int wave_fold_index(int lane) { return lane & (NV - 1); }

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, 64));
    return v;
}

}  // namespace skh
