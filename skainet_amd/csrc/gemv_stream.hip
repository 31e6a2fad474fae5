// Dequant-GEMV for one activation row, any block format, with the weight streamed through LDS:
//   y[o] = sum_j x[j] * dequant(W[o, j])      fp32 activations and sums, canonical row-major GGUF blocks.
//
// Same products as the row kernel of gemv.hip (the slot policies of gemv_slots.h do the arithmetic; semantics of the
// reference's exact-fp32 kernels cited there); what differs is how the bytes travel. What bounds a read-once pass over
// 10 .. 30 MB on this device is the shape of the loads: a wave load whose lanes pick their own slot out of every line of
// a row streams far slower than wave loads of consecutive kilobytes with the non-temporal hint. So:
//   * every wave owns a contiguous range of weight rows, i.e. one contiguous run of bytes, and no other wave touches it:
//     no workgroup barrier, no cross-wave sum;
//   * the run is fetched in units of RU rows by full-wave 16-byte-per-lane loads that write LDS directly
//     (global_load_lds_dwordx4 ... nt: 1 KB of consecutive bytes per instruction, no registers held while in flight),
//     two units in flight per wave; inline assembly with explicit wait counts, the loads complete in issue order;
//   * lane l then reads its slots (l and, for rows of more than 64 slots, l + 64) of each row out of LDS and multiplies
//     them with the activations it has held in registers since the start; the RU per-lane sums of a unit are folded
//     over the wave by one multi-value butterfly.
// Used for the formats of 32-element blocks it measured faster on (Q8_0, Q4_0, Q5_0, Q5_1). Rows whose byte length is
// not a multiple of 16, rows of more than 128 slots, and units that do not fit the LDS ring stay on the row kernel (the
// launcher returns 0).
#include "gemv_slots.h"

namespace skh {

constexpr int STREAM_MAX_CHUNKS = 18;          // 1 KB loads per unit: 4 waves x 2 units x 18 KB = 144 KB of LDS

// 16 bytes per lane from base + off into LDS at lds_addr + 16 * lane (M0 carries the LDS address)
__device__ __forceinline__ void stream_dma16(uint32_t lds_addr, uint32_t off, const uint8_t* base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(lds_addr), "v"(off), "s"(base) : "memory");
}
typedef float stream_f32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void stream_load16(stream_f32x4& dst, uint32_t off, const float* base) {
    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(dst) : "v"(off), "s"(base) : "memory");
}
template <int N> __device__ __forceinline__ void stream_wait_imm() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }
template <int N>
__device__ __forceinline__ void stream_wait_case(int n) {
    if constexpr (N >= 0) {
        if (n == N) stream_wait_imm<N>(); else stream_wait_case<N - 1>(n);
    }
}
// wait until at most n (uniform, 0 .. 2 * STREAM_MAX_CHUNKS) loads are in flight: the count is an immediate of the
// instruction, so a chain of scalar compares picks the instruction
__device__ __forceinline__ void stream_wait(int n) { stream_wait_case<2 * STREAM_MAX_CHUNKS>(n); }

// What the kernel needs from a format: the slot policy that addresses and loads a lane's bytes (`Slot`), the lane's
// activations in the form its arithmetic wants (`Act`, built once from the NX floats of the slot), and the product of
// one slot with them. The fp32 form of any slot policy: the activations stay floats, the policy's own dot product.
template <class F>
struct StreamFp32 {
    using Slot = F;
    struct Act { float x[1][F::NX]; float xsum[1][XSumCount<F>::N]; };
    __device__ static void prepare(Act& a, const float* x) {
#pragma unroll
        for (int i = 0; i < F::NX; ++i) a.x[0][i] = x[i];
        F::prep(a.x[0], a.xsum[0]);
    }
    __device__ static float dot(const typename F::Raw& r, const typename F::Lane& ln, const Act& a) {
        float t[1] = {0.f};
        F::template dot<1>(r, ln, a.x, a.xsum, t);
        return t[0];
    }
};

// P: the format's form above, SPL: slots per lane (1 or 2), RU: rows per unit (a power of two)
template <class P, int SPL, int RU>
__global__ __launch_bounds__(256) void gemv_stream_kernel(const uint8_t* __restrict__ w, const float* __restrict__ x, float* __restrict__ y,
                                                          int k, int n, uint32_t row_bytes, int rows_per_wave, int ch) {
    extern __shared__ __attribute__((aligned(16))) uint8_t stream_smem[];   // the kernel has no other LDS: offsets into it are LDS addresses
    using F = typename P::Slot;
    constexpr int NX = F::NX;
    constexpr int NV = RU < 2 ? 2 : RU;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r0 = (blockIdx.x * 4 + wave) * rows_per_wave;
    const int nrows = min(n, r0 + rows_per_wave) - r0;          // uniform
    if (nrows <= 0) return;                                     // the whole wave leaves; nothing in the kernel waits for it
    const int nslots = k / F::SLOT_ELEMS;
    const uint32_t slot_bytes = (uint32_t)ch * 1024u;
    const uint32_t ring = (uint32_t)wave * 2u * slot_bytes;
    const uint8_t* const wbase = w + (int64_t)r0 * row_bytes;
    const uint32_t wave_bytes = (uint32_t)nrows * row_bytes, unit_bytes = RU * row_bytes;
    const int units = (nrows + RU - 1) / RU;

    // the lane's activations: requested first (they come out of L2 and must not queue behind the weight stream)
    typename F::Lane ln[SPL];
    typename P::Act act[SPL];
    bool active[SPL];
    stream_f32x4 xv[SPL][NX / 4];
#pragma unroll
    for (int s = 0; s < SPL; ++s) {
        const int slot = lane + 64 * s;
        active[s] = slot < nslots;
        F::init(ln[s], active[s] ? slot : 0);
#pragma unroll
        for (int i = 0; i < NX; i += 4) stream_load16(xv[s][i / 4], 4u * (uint32_t)F::x_index(active[s] ? slot : 0, i), x);
    }
    // unit u of the wave's run into ring slot u & 1; lanes past the unit's end (the last load of a unit whose length
    // is not a whole number of kilobytes) fetch its last 16 bytes again
    auto issue = [&](int u) __attribute__((always_inline)) {
        const uint32_t lds = ring + (uint32_t)(u & 1) * slot_bytes;
        const uint32_t begin = (uint32_t)u * unit_bytes, last = min(begin + unit_bytes, wave_bytes) - 16u;
        for (int c = 0; c < ch; ++c) stream_dma16(lds + 1024u * c, min(begin + 1024u * c + 16u * lane, last), wbase);
    };
    issue(0);
    if (units > 1) issue(1);
    stream_wait(units > 1 ? 2 * ch : ch);                       // the activations have landed (the units may still fly)
#pragma unroll
    for (int s = 0; s < SPL; ++s) {
        const float keep = active[s] ? 1.0f : 0.0f;
        float xf[NX];
#pragma unroll
        for (int i = 0; i < NX; i += 4) {
            // the asm loads are tied to their registers by the wait above only through program order: name them here
            asm volatile("" : "+v"(xv[s][i / 4]));
            xf[i] = xv[s][i / 4].x * keep; xf[i + 1] = xv[s][i / 4].y * keep;
            xf[i + 2] = xv[s][i / 4].z * keep; xf[i + 3] = xv[s][i / 4].w * keep;
        }
        P::prepare(act[s], xf);
    }

    for (int u = 0; u < units; ++u) {
        stream_wait(u + 1 < units ? ch : 0);                    // unit u has landed; unit u + 1 may still fly
        const uint8_t* unit = stream_smem + (ring + (uint32_t)(u & 1) * slot_bytes);
        float acc[NV];
#pragma unroll
        for (int i = 0; i < NV; ++i) acc[i] = 0.f;
#pragma unroll
        for (int i = 0; i < RU; ++i) {
            if (u * RU + i < nrows) {                           // uniform: no arithmetic on rows past the wave's range
                float a = 0.f;
#pragma unroll
                for (int s = 0; s < SPL; ++s) {
                    typename F::Raw raw;
                    F::load(raw, unit + (uint32_t)i * row_bytes, ln[s]);
                    const float t = P::dot(raw, ln[s], act[s]);
                    a += active[s] ? t : 0.f;
                }
                acc[i] = a;
            }
        }
        wave_fold<NV>(acc, lane);                               // lane l < NV holds the total of value l
        if (lane < RU && u * RU + lane < nrows) y[r0 + u * RU + lane] = acc[0];
        if (u + 2 < units) {
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the slot about to be refilled has been read
            issue(u + 2);
        }
    }
}

static std::atomic<int> g_gemv_stream_enable{1};
void set_gemv_stream_enable(int v) { g_gemv_stream_enable = v != 0; }

template <class P, int SPL>
static int launch_stream_spl(const uint8_t* w, const float* x, float* y, int k, int n, uint32_t row_bytes) {
    const int waves = 4 * num_cus();
    const int rows_per_wave = (n + waves - 1) / waves;
    // rows per unit: as many as fit the ring, but at least two units per wave where it has the rows for them (the second
    // unit is in flight while the first is multiplied)
    int ru = 4;
    while (ru > 1 && ((uint64_t)ru * row_bytes + 1023) / 1024 > (uint64_t)STREAM_MAX_CHUNKS) ru >>= 1;
    while (ru > 1 && rows_per_wave < 2 * ru) ru >>= 1;
    const int ch = (int)(((uint64_t)ru * row_bytes + 1023) / 1024);
    if (ch > STREAM_MAX_CHUNKS || (uint64_t)rows_per_wave * row_bytes >= ((uint64_t)1 << 31)) return 0;
    const int grid = (n + 4 * rows_per_wave - 1) / (4 * rows_per_wave);
    const size_t smem = (size_t)4 * 2 * ch * 1024;
    note_kernel("gemv_stream_kernel");
#define SKH_STREAM_LAUNCH(RU)                                                                                       \
    do {                                                                                                            \
        SKH_SET_MAX_DYNAMIC_LDS_ONCE((&gemv_stream_kernel<P, SPL, RU>), (size_t)4 * 2 * STREAM_MAX_CHUNKS * 1024);  \
        gemv_stream_kernel<P, SPL, RU><<<dim3(grid), dim3(256), smem, current_stream()>>>(w, x, y, k, n, row_bytes, rows_per_wave, ch); \
    } while (0)
    if (ru == 4) SKH_STREAM_LAUNCH(4);
    else if (ru == 2) SKH_STREAM_LAUNCH(2);
    else SKH_STREAM_LAUNCH(1);
#undef SKH_STREAM_LAUNCH
    SKH_CHECK(hipGetLastError());
    return 1;
}

// Returns 1 when the streaming kernel took the product, 0 when its shape is outside the kernel's range (nothing
// launched), -1 on error.
template <class P>
static int launch_stream(const uint8_t* w, const float* x, float* y, int k, int n) {
    using F = typename P::Slot;
    if (!g_gemv_stream_enable) return 0;
    const int nslots = k / F::SLOT_ELEMS;
    const uint64_t row_bytes = (uint64_t)(k / (F::SLOT_ELEMS * F::SLOTS_PER_BLOCK)) * F::BLOCK_BYTES;
    if (nslots < 1 || nslots > 128 || (row_bytes & 15) || row_bytes > (uint64_t)STREAM_MAX_CHUNKS * 1024) return 0;
    if ((reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(x)) & 15) return 0;
    return nslots <= 64 ? launch_stream_spl<P, 1>(w, x, y, k, n, (uint32_t)row_bytes) : launch_stream_spl<P, 2>(w, x, y, k, n, (uint32_t)row_bytes);
}

// The formats this kernel is faster on (one row, MI355X, us per product; row kernel -> this one): Q8_0 4096 x 4096
// 6.97 -> 6.25; Q4_0 / Q5_0 / Q5_1 11008 x 4096 10.95 / 13.31 / 12.90 -> 10.58 / 13.00 / 12.42. Q6_K and Q5_K stay on
// the row kernel: their arithmetic per byte is heavier, and a wave that multiplies a unit while only one more is in
// flight streams slower than six or eight row-kernel waves per CU (Q6_K 128256 x 4096: 101 against 79 us; with two of
// these waves per SIMD 78; Q5_K 11008 x 4096: 12.1 against 9.6). Multiplying Q8_0 on v_dot4_i32_i8 (activations as three
// planes of base-256 digits) was measured slower than the fp32 products (6.9 against 6.25 us).
int launch_gemv_stream(int enc, const uint8_t* w, const float* x, float* y, int k, int n) {
    switch (enc) {
        case ENC_Q8_0: return launch_stream<StreamFp32<Q80Slot>>(w, x, y, k, n);
        case ENC_Q4_0: return launch_stream<StreamFp32<Q45Slot<0>>>(w, x, y, k, n);
        case ENC_Q5_0: return launch_stream<StreamFp32<Q45Slot<1>>>(w, x, y, k, n);
        case ENC_Q5_1: return launch_stream<StreamFp32<Q45Slot<2>>>(w, x, y, k, n);
        default: return 0;
    }
}

}  // namespace skh
