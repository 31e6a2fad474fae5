// Shared declarations of the gfx950 kernel library: block geometry, error plumbing, small device helpers.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace skh {

// GGUF block geometry (elements per block, bytes per block); see
// /root/reference/skainet-lang/skainet-lang-core/src/commonMain/kotlin/sk/ainet/lang/memory/BlockSpec.kt:84-87
constexpr int Q80_ELEMS = 32, Q80_BYTES = 34;
constexpr int QK_ELEMS = 256, Q4K_BYTES = 144, Q6K_BYTES = 210;

// Encoding ids are the GGML tensor-type numbers the GGUF reader maps from
// (/root/reference/skainet-io/skainet-io-gguf/src/commonMain/kotlin/sk/ainet/io/gguf/StreamingGGUFReader.kt:190-211).
enum Encoding : int32_t { ENC_F32 = 0, ENC_Q8_0 = 8, ENC_Q4_K = 12, ENC_Q6_K = 14 };

inline int block_elems(int enc) { return enc == ENC_Q8_0 ? Q80_ELEMS : QK_ELEMS; }
inline int block_bytes(int enc) { return enc == ENC_Q8_0 ? Q80_BYTES : (enc == ENC_Q4_K ? Q4K_BYTES : Q6K_BYTES); }
inline bool is_packed(int enc) { return enc == ENC_Q8_0 || enc == ENC_Q4_K || enc == ENC_Q6_K; }

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

// Loads that tolerate the 2-byte alignment of Q8_0 / Q6_K blocks (34 and 210 bytes per block).
struct __attribute__((packed, aligned(2))) u32_a2 { uint32_t v; };
__device__ __forceinline__ uint32_t load_u32_a2(const uint8_t* p) { return reinterpret_cast<const u32_a2*>(p)->v; }
__device__ __forceinline__ uint32_t load_u16(const uint8_t* p) { return *reinterpret_cast<const uint16_t*>(p); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, 64));
    return v;
}

}  // namespace skh
