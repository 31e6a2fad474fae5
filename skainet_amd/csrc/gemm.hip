// Prefill dequant-GEMM on the matrix cores:  C[m, n] = sum_k A[m, k] * dequant(W[n, k])
//   A fp32 [M, K] (rounded once to bf16), W packed Q4_K / Q6_K / Q8_0 in canonical row-major GGUF order,
//   products bf16 x bf16 on v_mfma_f32_32x32x16_bf16, fp32 accumulation, C fp32 [M, N].
//
// What it replaces: the reference has no packed GEMM -- a [rows, k] activation is `rows` GEMV calls
//   /root/reference/skainet-backends/skainet-backend-api/src/commonMain/kotlin/sk/ainet/backend/api/kernel/PackedViewMatmulKernel.kt:69-108
//   /root/reference/skainet-backends/skainet-backend-native-cpu/src/jvmMain/kotlin/sk/ainet/exec/kernel/FfmRowMajorKernels.kt:94-104
// so the weight is re-streamed once per row. Here a weight tile is decoded once into LDS and reused by 256 rows.
// The decode is the reference's block arithmetic (code * (d * sc) - dmin * m, (d * sc) * q, code * d) in fp32,
// rounded to bf16 (nearest even) when it is parked in LDS.
//
// Tiling (MFMA-bound): workgroup tile 256 (M) x 128 (N), K step 64, 256 threads = 4 waves in a 2 x 2 grid, each wave
// owning a 128 x 64 patch = 4 x 2 MFMA tiles of 32 x 32 (128 accumulator registers per lane). Per K step a thread
// decodes 32 consecutive weights of one row (one Q4_K sub-block / one Q6_K quarter / one Q8_0 block) and copies
// 8 x 16 bytes of the bf16 activation tile; LDS rows are padded to 144 bytes so the 16-byte fragment reads of 32
// consecutive rows fall on distinct banks. Two LDS stages (108 KB: one workgroup per CU); global loads run two
// steps ahead in a two-slot register ring, one barrier per step. When the tile grid is smaller than the chip, K is split across gridDim.z and
// each split parks its partial tile in a workspace with plain stores and a second launch sums the splits in split order
// (fp32 atomic adds into C cost more than the K loop at these sizes, and their order is not reproducible).
#include "common.h"

namespace skh {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

// The tile comes in two widths, WTN = 2 or 4 32-column MFMA tiles per wave along N (rows: always 4): 256 x 128 and
// 256 x 256. Per K step a CU's LDS moves 144 KB for the narrow tile (1152 cycles at 128 B/clk against the 1024 cycles of
// its MFMAs; measured in isolation, 32 MFMAs take 505 ns, with the 24 fragment reads 688 ns, with the 12 tile stores
// 820 ns: a wave that issues an LDS instruction is held while the LDS moves its 1 KB) and 192 KB for the wide tile with
// twice the MFMAs, so the wide tile is the one that can keep the matrix cores busy; it needs 32 tiles per CU round
// fewer to fill the chip, so it serves the wide weights (N >= 128 rows per CU) and the narrow one the rest.
constexpr int G_WAVES_M = 2, G_WAVES_N = 2;
constexpr int GK = 64;
constexpr int G_THREADS = G_WAVES_M * G_WAVES_N * 64;
constexpr int GSTRIDE = GK + 8;                               // bf16 elements per LDS row (144 bytes)
// A wave owns WTM x WTN MFMA tiles of 32 x 32: WTM = 4 row tiles (workgroup tile 256 rows) for prompts, WTM = 2 (128 rows)
// where at most 128 activation rows exist or where the taller tile would leave most of the chip idle.
constexpr int gemm_gm(int wtm) { return 32 * wtm * G_WAVES_M; }
constexpr int gemm_gn(int wtn) { return 32 * wtn * G_WAVES_N; }
constexpr size_t gemm_smem(int wtm, int wtn) { return 2 * (size_t)(gemm_gm(wtm) + gemm_gn(wtn)) * GSTRIDE * sizeof(__bf16); }   // two stages

void* kernel_workspace(size_t bytes);   // shim.hip
int launch_gemv(int enc, const uint8_t* w, const float* x, int m, int k, int n, float* y);   // gemv.hip
int launch_add(const float* a, const float* b, float* out, int64_t n);                        // rows.hip
int launch_swiglu_pairs(const float* gate_up, float* out, int64_t n);                         // rows.hip

// The pass in front of the GEMM: activations fp32 -> bf16 (nearest even). A thread handles PREPASS_UNROLL float4s a
// whole workgroup stride apart, all loaded before the first is stored (clamped index, guarded store). The pass is a
// launch and one round trip to memory, not bandwidth: one float4 per thread (four times the waves) measured 33.70 us per
// 512 x 4096 x 4096 product where two and four measured 33.9 and 34.0.
constexpr int PREPASS_UNROLL = 1;
__global__ __launch_bounds__(256) void gemm_prepass_kernel(const float* __restrict__ in, __bf16* __restrict__ out, int64_t n4) {
    typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
    const int64_t i0 = (int64_t)blockIdx.x * (256 * PREPASS_UNROLL) + threadIdx.x;
    float4 v[PREPASS_UNROLL];
#pragma unroll
    for (int u = 0; u < PREPASS_UNROLL; ++u) v[u] = reinterpret_cast<const float4*>(in)[min(i0 + 256 * u, n4 - 1)];
#pragma unroll
    for (int u = 0; u < PREPASS_UNROLL; ++u) {
        const int64_t i = i0 + 256 * u;
        if (i < n4) reinterpret_cast<bf16x4*>(out)[i] = bf16x4{(__bf16)v[u].x, (__bf16)v[u].y, (__bf16)v[u].z, (__bf16)v[u].w};
    }
}

// The same pass over rows of interleaved (gate, up) pairs: out[i] = bf16(silu(in[2 i]) * in[2 i + 1]), four per thread.
__global__ __launch_bounds__(256) void gemm_prepass_swiglu_kernel(const float* __restrict__ in, __bf16* __restrict__ out, int64_t n4) {
    typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n4) return;
    const float4 a = reinterpret_cast<const float4*>(in)[2 * i], b = reinterpret_cast<const float4*>(in)[2 * i + 1];
    auto act = [](float g, float u) { return g * (1.0f / (1.0f + expf(-g))) * u; };
    reinterpret_cast<bf16x4*>(out)[i] = bf16x4{(__bf16)act(a.x, a.y), (__bf16)act(a.z, a.w), (__bf16)act(b.x, b.y), (__bf16)act(b.z, b.w)};
}

// The same pass with an RMSNorm folded in: out = bf16(x / sqrt(mean(x^2) + eps) * gain), one workgroup per activation row,
// the row held in registers between the sum of squares and the scaling (k a multiple of 4, at most 256 * 4 * V floats).
template <int V>
__global__ __launch_bounds__(256) void gemm_prepass_rmsnorm_kernel(const float* __restrict__ in, const float* __restrict__ gain,
                                                                   __bf16* __restrict__ out, int k, float eps) {
    typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
    __shared__ float red[4];
    const float4* x = reinterpret_cast<const float4*>(in + (int64_t)blockIdx.x * k);
    const float4* g4 = reinterpret_cast<const float4*>(gain);
    bf16x4* o = reinterpret_cast<bf16x4*>(out + (int64_t)blockIdx.x * k);
    const int k4 = k >> 2;
    float4 xr[V], gr[V];
#pragma unroll
    for (int j = 0; j < V; ++j) {
        const int i = threadIdx.x + 256 * j;
        xr[j] = i < k4 ? x[i] : make_float4(0.f, 0.f, 0.f, 0.f);
        gr[j] = i < k4 ? g4[i] : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < V; ++j) { s = fmaf(xr[j].x, xr[j].x, s); s = fmaf(xr[j].y, xr[j].y, s); s = fmaf(xr[j].z, xr[j].z, s); s = fmaf(xr[j].w, xr[j].w, s); }
    s = wave_sum(s);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
    __syncthreads();
    const float scale = 1.0f / sqrtf((red[0] + red[1] + red[2] + red[3]) * (1.0f / (float)k) + eps);
#pragma unroll
    for (int j = 0; j < V; ++j) {
        const int i = threadIdx.x + 256 * j;
        if (i < k4) o[i] = bf16x4{(__bf16)(xr[j].x * scale * gr[j].x), (__bf16)(xr[j].y * scale * gr[j].y),
                                  (__bf16)(xr[j].z * scale * gr[j].z), (__bf16)(xr[j].w * scale * gr[j].w)};
    }
}

// What happens to a product on its way out, applied by the launch that sums K splits (a GEMM that is not split writes
// the plain product and the row kernels finish it: an epilogue in the tile kernel's own stores measured slower --
// +20 us on 512 x 28672 x 4096 for SwiGLU against 17 us for the separate pass, and it cost the kernels without an
// epilogue 5 % through the register allocation of their main loop):
//   GEMM_EPI_NONE      c[row, col] = p
//   GEMM_EPI_RESIDUAL  c[row, col] = residual[row, col] + p          (residual may be c)
//   GEMM_EPI_SWIGLU    c[row, col / 2] = silu(p[row, col]) * p[row, col + 1] for even col (c has n / 2 columns)
enum { GEMM_EPI_NONE = 0, GEMM_EPI_RESIDUAL = 1, GEMM_EPI_SWIGLU = 2 };
__device__ __forceinline__ float silu_f(float g) { return g * (1.0f / (1.0f + expf(-g))); }

// Split K: C = sum over the splits, in split order, of the partial products parked `stride` floats apart (stride a
// multiple of 4, the buffer 16-byte aligned). Thread i owns elements 4i .. 4i + 3.
__global__ __launch_bounds__(256) void gemm_splitk_sum_kernel(const float* __restrict__ part, int64_t stride, int splits,
                                                              float* c, int64_t total, int c_aligned, const float* residual,
                                                              int epilogue) {
    const int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (i >= total) return;
    float4 acc = *reinterpret_cast<const float4*>(part + i);
    for (int z = 1; z < splits; ++z) {
        const float4 v = *reinterpret_cast<const float4*>(part + z * stride + i);
        acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w;
    }
    float v[4] = {acc.x, acc.y, acc.z, acc.w};
    if (epilogue == GEMM_EPI_SWIGLU) {
        // n is even and elements 4i .. 4i + 3 start at an even column: two (gate, up) pairs, outputs 2i and 2i + 1
        if (i + 1 < total) c[i >> 1] = silu_f(v[0]) * v[1];
        if (i + 3 < total) c[(i >> 1) + 1] = silu_f(v[2]) * v[3];
        return;
    }
    if (epilogue == GEMM_EPI_RESIDUAL) {
#pragma unroll
        for (int j = 0; j < 4; ++j) if (i + j < total) v[j] += residual[i + j];
    }
    if (c_aligned && i + 4 <= total) { *reinterpret_cast<float4*>(c + i) = make_float4(v[0], v[1], v[2], v[3]); return; }
    for (int j = 0; j < 4 && i + j < total; ++j) c[i + j] = v[j];
}

// byte N of a dword as float, N a compile-time index
template <int N>
__device__ __forceinline__ float gemm_byte_to_float(uint32_t v) {
    return N == 0 ? ubyte0_to_float(v) : N == 1 ? ubyte1_to_float(v) : N == 2 ? ubyte2_to_float(v) : ubyte3_to_float(v);
}

// ---- raw bytes a thread needs to decode 32 consecutive weights of one row, per encoding ----
// Per encoding: load_raw (global loads of a thread's 32 weights), decode_prepare (scales of the 32), and the decode of
// part I (0..7, four weights) in two stages the main loop places separately: decode_codes<I> gathers the part's four
// codes into the bytes of one dword, decode_pair<I, H> turns bytes 2 H and 2 H + 1 of it into two fp32 weights.
// What is constant over the four steps of a 256-element super-block is loaded once per super-block into an Sb (load_sb)
// and not with every step's codes: a step's loads are one instruction per 16 bytes and row, each touching as many cache
// lines as the wave has rows, and their number, not their bytes, is what the weight side of the tile costs (Q6_K with
// its two 2-byte loads of scales and d per task and step: 184.7 us per 512 x 32000 x 4096 product, 155 us without them).
struct SbNone {};
struct RawQ4K { uint4 q0, q1; };
struct SbQ4K { uint4 hdr; };
struct RawQ6K { uint32_t ql[8], qh[4]; };
struct SbQ6K { u32x4_vec sc; uint32_t d; };          // the 16 int8 scales, the fp16 d
struct RawQ80 { u32x4_vec lo, hi; uint32_t edge, odd; };   // aligned 32-byte body, the 2 bytes outside it, start parity

// `e` = element offset inside the row, a multiple of 32.
__device__ __forceinline__ void load_raw(RawQ4K& r, const uint8_t* row, int e) {
    const uint8_t* blk = row + (e >> 8) * Q4K_BYTES;
    const int g = (e & 255) >> 6;                     // 32-byte nibble group holding sub-blocks 2g, 2g+1
    r.q0 = *reinterpret_cast<const uint4*>(blk + 16 + g * 32);
    r.q1 = *reinterpret_cast<const uint4*>(blk + 32 + g * 32);
}
__device__ __forceinline__ void load_sb(SbQ4K& sb, const uint8_t* row, int e) {
    sb.hdr = *reinterpret_cast<const uint4*>(row + (e >> 8) * Q4K_BYTES);
}
// The decode of a thread's 32 weights is split into a header part and eight 4-weight parts (one per dword of
// codes) so the main loop can place the parts between its MFMAs.
struct DecQ4K { float scale, offset; int shift; };
// UN: the step's position in its super-block (0..3), known where the K loop is unrolled: sub-block 2 UN + wsub. Which of
// the two packings of the 6-bit scales applies (sub-blocks 0..3 / 4..7) is then decided at compile time; `e` gives wsub.
template <int UN>
__device__ __forceinline__ void decode_prepare_k4(const uint4& hdr, int e, DecQ4K& c) {
    const int wsub = (e >> 5) & 1;
    const float d = half_bits_to_float_fast(hdr.x & 0xFFFFu), dmin = half_bits_to_float_fast(hdr.x >> 16);
    // ggml get_scale_min_k4 on the 12 scale bytes s[0..11] (hdr.y = s[0..3], hdr.z = s[4..7], hdr.w = s[8..11]):
    // byte (2 UN + wsub) % 4 of each
    const int sh = (2 * (UN & 1) + wsub) * 8;
    const uint32_t sa = (hdr.y >> sh) & 0xFFu, sbm = (hdr.z >> sh) & 0xFFu, st = (hdr.w >> sh) & 0xFFu;
    const uint32_t sc = UN < 2 ? (sa & 63u) : ((st & 0xFu) | ((sa >> 6) << 4));
    const uint32_t mn = UN < 2 ? (sbm & 63u) : ((st >> 4) | ((sbm >> 6) << 4));
    c.scale = d * (float)sc;
    c.offset = dmin * (float)mn;
    c.shift = wsub * 4;
}
template <int UN>
__device__ __forceinline__ void decode_prepare(const RawQ4K&, const SbQ4K& sb, int e, DecQ4K& c) { decode_prepare_k4<UN>(sb.hdr, e, c); }
template <int I>
__device__ __forceinline__ uint32_t decode_codes(const RawQ4K& r, const SbQ4K&, const DecQ4K& c) {
    const uint32_t q = I == 0 ? r.q0.x : I == 1 ? r.q0.y : I == 2 ? r.q0.z : I == 3 ? r.q0.w
                     : I == 4 ? r.q1.x : I == 5 ? r.q1.y : I == 6 ? r.q1.z : r.q1.w;
    return (q >> c.shift) & 0x0F0F0F0Fu;
}
template <int I, int H>
__device__ __forceinline__ void decode_pair(uint32_t v, const DecQ4K& c, float& w0, float& w1) {
    w0 = fmaf(gemm_byte_to_float<2 * H>(v), c.scale, -c.offset);
    w1 = fmaf(gemm_byte_to_float<2 * H + 1>(v), c.scale, -c.offset);
}

// Q6_K: the pair of threads that shares a row's 64 elements of a step splits them by position inside the 32-element
// quarters, not by quarter: thread `wsub` decodes positions 16 wsub .. 16 wsub + 15 of both quarters (elements
// E + 16 wsub + .. and E + 32 + 16 wsub + ..). Its codes are then three runs of 16 bytes (low bits of either quarter, the
// shared plane of high bits) that no other thread loads, where a thread that owns a whole quarter needs all 32 bytes of
// the high-bit plane, the same 32 as its neighbour. park_elem gives the position of a thread's weights in the tile row.
__device__ __forceinline__ void load_raw(RawQ6K& r, const uint8_t* row, int e) {
    const uint8_t* blk = row + (e >> 8) * Q6K_BYTES;
    const int half = (e & 255) >> 7, wsub = (e >> 5) & 1;
    const uint8_t* ql = blk + half * 64 + 16 * wsub;
    const u32x4_vec la = load_u32x4_a2(ql), lb = load_u32x4_a2(ql + 32), h4 = load_u32x4_a2(blk + 128 + half * 32 + 16 * wsub);
    r.ql[0] = la.x; r.ql[1] = la.y; r.ql[2] = la.z; r.ql[3] = la.w;
    r.ql[4] = lb.x; r.ql[5] = lb.y; r.ql[6] = lb.z; r.ql[7] = lb.w;
    r.qh[0] = h4.x; r.qh[1] = h4.y; r.qh[2] = h4.z; r.qh[3] = h4.w;
}
__device__ __forceinline__ void load_sb(SbQ6K& sb, const uint8_t* row, int e) {
    const uint8_t* blk = row + (e >> 8) * Q6K_BYTES;
    sb.sc = load_u32x4_a2(blk + 192);
    sb.d = load_u16(blk + 208);
}
struct DecQ6K { float s0, s1, n0, n1; int nib, hs; };   // n = -32 s
template <int UN>
__device__ __forceinline__ void decode_prepare(const RawQ6K&, const SbQ6K& sb, int e, DecQ6K& c) {
    // step UN (0..3) of the super-block: quarters kq and kq + 1 (kq 0 or 2) of half UN / 2; this thread's 16 positions of
    // either lie in one 16-element scale group each: sc[4 UN + wsub] and sc[4 UN + 2 + wsub], bytes wsub and wsub + 2 of
    // dword UN of the 16 scales
    constexpr int kq = 2 * (UN & 1);
    const int wsub = (e >> 5) & 1;
    const float d = half_bits_to_float_fast(sb.d);
    const uint32_t four = (UN == 0 ? sb.sc.x : UN == 1 ? sb.sc.y : UN == 2 ? sb.sc.z : sb.sc.w) >> (8 * wsub);
    c.s0 = d * (float)(int8_t)(four & 0xFF);
    c.s1 = d * (float)(int8_t)((four >> 16) & 0xFF);
    c.n0 = -32.f * c.s0;
    c.n1 = -32.f * c.s1;
    c.nib = (kq >> 1) * 4;
    c.hs = 2 * kq;
}
template <int I>
__device__ __forceinline__ uint32_t decode_codes(const RawQ6K& r, const SbQ6K&, const DecQ6K& c) {
    // parts 0..3: quarter kq (bit pair kq of the high-bit bytes), parts 4..7: quarter kq + 1 (the next bit pair)
    const uint32_t lo = (r.ql[I] >> c.nib) & 0x0F0F0F0Fu;
    const uint32_t hi = ((r.qh[I & 3] >> (c.hs + (I < 4 ? 0 : 2))) & 0x03030303u) << 4;
    return lo | hi;                                          // four 6-bit codes, one per byte
}
template <int I, int H>
__device__ __forceinline__ void decode_pair(uint32_t v, const DecQ6K& c, float& w0, float& w1) {
    // sc * (q - 32) as one FMA: q - 32 is exact and so is 32 * sc, so the single rounding gives the same bits
    const float sc = I < 4 ? c.s0 : c.s1, off = I < 4 ? c.n0 : c.n1;
    w0 = fmaf(gemm_byte_to_float<2 * H>(v), sc, off);
    w1 = fmaf(gemm_byte_to_float<2 * H + 1>(v), sc, off);
}

__device__ __forceinline__ void load_raw(RawQ80& r, const uint8_t* row, int e) {
    // a 34-byte block starts 0 or 2 bytes past a dword boundary: two 16-byte loads of its dword-aligned body and one
    // 2-byte load of what the body leaves out (the last code pair, or the scale)
    const uint8_t* blk = row + (e >> 5) * Q80_BYTES;
    r.odd = (uint32_t)(reinterpret_cast<uintptr_t>(blk) >> 1) & 1u;
    const uint8_t* body = blk + 2 * r.odd;
    r.lo = load_u32x4_a4(body);
    r.hi = load_u32x4_a4(body + 16);
    r.edge = load_u16(blk + (r.odd ? 0 : 32));
}
struct DecQ80 { float d; uint32_t drop; };
template <int UN>
__device__ __forceinline__ void decode_prepare(const RawQ80& r, const SbNone&, int, DecQ80& c) {
    c.d = half_bits_to_float_fast(r.odd ? r.edge : (r.lo.x & 0xFFFFu));
    c.drop = r.odd ? 0u : 2u;                        // bytes in front of the codes in the loaded dwords
}
template <int I>
__device__ __forceinline__ uint32_t decode_codes(const RawQ80& r, const SbNone&, const DecQ80& c) {
    const uint32_t v[9] = {r.lo.x, r.lo.y, r.lo.z, r.lo.w, r.hi.x, r.hi.y, r.hi.z, r.hi.w, r.edge};
    return __builtin_amdgcn_alignbyte(v[I + 1], v[I], c.drop);
}
template <int I, int H>
__device__ __forceinline__ void decode_pair(uint32_t q, const DecQ80& c, float& w0, float& w1) {
    w0 = (float)(int8_t)(q >> (16 * H)) * c.d;
    w1 = (float)(int8_t)(q >> (16 * H + 8)) * c.d;
}

// Q4_0 / Q5_0 / Q5_1 (FMT 0 / 1 / 2): a thread's 32 weights are one block -- fp16 d [fp16 m] [32 fifth bits], then 16 bytes
// whose low nibbles are elements 0..15 and high nibbles elements 16..31. Blocks are 2-byte aligned (Q5_1: 8).
template <int FMT> struct RawQ45 { uint32_t d, m, qh, q[4]; };
template <int FMT>
__device__ __forceinline__ void load_raw(RawQ45<FMT>& r, const uint8_t* row, int e) {
    constexpr int BYTES = FMT == 0 ? Q40_BYTES : (FMT == 1 ? Q50_BYTES : Q51_BYTES);
    constexpr int QH = FMT == 2 ? 4 : 2, QS = FMT == 0 ? 2 : QH + 4;
    const uint8_t* blk = row + (e >> 5) * BYTES;
    r.d = load_u16(blk);
    r.m = FMT == 2 ? load_u16(blk + 2) : 0u;
    r.qh = FMT != 0 ? load_u32_a2(blk + QH) : 0u;
    const u32x4_vec q4 = load_u32x4_a2(blk + QS);           // the 16 code bytes as one load (2-byte aligned)
    r.q[0] = q4.x; r.q[1] = q4.y; r.q[2] = q4.z; r.q[3] = q4.w;
}
struct DecQ45 { float d, add; };
template <int UN, int FMT>
__device__ __forceinline__ void decode_prepare(const RawQ45<FMT>& r, const SbNone&, int, DecQ45& c) {
    c.d = half_bits_to_float_fast(r.d);
    // w = d * code + add:  Q4_0 d * (code - 8),  Q5_0 d * (code5 - 16),  Q5_1 d * code5 + m
    c.add = FMT == 0 ? -8.f * c.d : (FMT == 1 ? -16.f * c.d : half_bits_to_float_fast(r.m));
}
template <int I, int FMT>
__device__ __forceinline__ uint32_t decode_codes(const RawQ45<FMT>& r, const SbNone&, const DecQ45&) {
    // parts 0..3: low nibbles of code dword I (elements 4I ..), parts 4..7: high nibbles of dword I - 4 (elements 16 + ..)
    uint32_t v = (r.q[I & 3] >> (I < 4 ? 0 : 4)) & 0x0F0F0F0Fu;
    if (FMT != 0) v |= ((((r.qh >> (4 * I)) & 0xFu) * 0x00204081u) & 0x01010101u) << 4;   // fifth bits 4I .. 4I + 3
    return v;
}
template <int I, int H>
__device__ __forceinline__ void decode_pair(uint32_t v, const DecQ45& c, float& w0, float& w1) {
    w0 = fmaf(gemm_byte_to_float<2 * H>(v), c.d, c.add);
    w1 = fmaf(gemm_byte_to_float<2 * H + 1>(v), c.d, c.add);
}

// Q5_K: the Q4_K sub-block plus bit sb of the 32-byte fifth-bit plane at byte 16 (nibbles at byte 48).
struct RawQ5K { uint4 q0, q1; };
struct SbQ5K { uint4 hdr, h0, h1; };                // header and the fifth-bit plane: the same for all eight sub-blocks
__device__ __forceinline__ void load_raw(RawQ5K& r, const uint8_t* row, int e) {
    const uint8_t* blk = row + (e >> 8) * Q5K_BYTES;
    const int g = (e & 255) >> 6;
    r.q0 = *reinterpret_cast<const uint4*>(blk + 48 + g * 32);
    r.q1 = *reinterpret_cast<const uint4*>(blk + 64 + g * 32);
}
__device__ __forceinline__ void load_sb(SbQ5K& sb, const uint8_t* row, int e) {
    const uint8_t* blk = row + (e >> 8) * Q5K_BYTES;
    sb.hdr = *reinterpret_cast<const uint4*>(blk);
    sb.h0 = *reinterpret_cast<const uint4*>(blk + 16);
    sb.h1 = *reinterpret_cast<const uint4*>(blk + 32);
}
struct DecQ5K { float scale, offset; int shift, bit; };
template <int UN>
__device__ __forceinline__ void decode_prepare(const RawQ5K&, const SbQ5K& sb, int e, DecQ5K& c) {
    DecQ4K c4;
    decode_prepare_k4<UN>(sb.hdr, e, c4);            // same d / dmin / 6-bit scale and min packing
    c.scale = c4.scale; c.offset = c4.offset; c.shift = c4.shift;
    c.bit = 2 * UN + ((e >> 5) & 1);
}
template <int I>
__device__ __forceinline__ uint32_t decode_codes(const RawQ5K& r, const SbQ5K& sb, const DecQ5K& c) {
    const uint32_t q = I == 0 ? r.q0.x : I == 1 ? r.q0.y : I == 2 ? r.q0.z : I == 3 ? r.q0.w
                     : I == 4 ? r.q1.x : I == 5 ? r.q1.y : I == 6 ? r.q1.z : r.q1.w;
    const uint32_t h = I == 0 ? sb.h0.x : I == 1 ? sb.h0.y : I == 2 ? sb.h0.z : I == 3 ? sb.h0.w
                     : I == 4 ? sb.h1.x : I == 5 ? sb.h1.y : I == 6 ? sb.h1.z : sb.h1.w;
    return ((q >> c.shift) & 0x0F0F0F0Fu) | (((h >> c.bit) & 0x01010101u) << 4);
}
template <int I, int H>
__device__ __forceinline__ void decode_pair(uint32_t v, const DecQ5K& c, float& w0, float& w1) {
    w0 = fmaf(gemm_byte_to_float<2 * H>(v), c.scale, -c.offset);
    w1 = fmaf(gemm_byte_to_float<2 * H + 1>(v), c.scale, -c.offset);
}

__device__ __forceinline__ void load_sb(SbNone&, const uint8_t*, int) {}
template <class Raw> struct SbOf { typedef SbNone type; };
template <> struct SbOf<RawQ4K> { typedef SbQ4K type; };
template <> struct SbOf<RawQ6K> { typedef SbQ6K type; };
template <> struct SbOf<RawQ5K> { typedef SbQ5K type; };
// Steps of 64 elements that one load_raw serves. Q6_K: the two steps of a 128-element half read the same 96 bytes (low
// nibbles and bit pairs 0..3 of the fifth / sixth bit plane in the first, high nibbles and bit pairs 4..7 in the second),
// so they are loaded once per half and decoded twice.
template <class Raw> struct RawSteps { static constexpr int value = 1; };
template <> struct RawSteps<RawQ6K> { static constexpr int value = 2; };
// Element offset, inside a row's 64 elements of a step, of weights 8 i .. 8 i + 7 (i = 0..3) of thread `wsub` of the pair.
template <class Raw> __device__ __forceinline__ int park_elem(int wsub, int i) { return 32 * wsub + 8 * i; }
template <> __device__ __forceinline__ int park_elem<RawQ6K>(int wsub, int i) { return 32 * (i >> 1) + 16 * wsub + 8 * (i & 1); }
template <class Raw> struct DecOf;
template <> struct DecOf<RawQ4K> { typedef DecQ4K type; };
template <> struct DecOf<RawQ6K> { typedef DecQ6K type; };
template <> struct DecOf<RawQ80> { typedef DecQ80 type; };
template <int FMT> struct DecOf<RawQ45<FMT>> { typedef DecQ45 type; };
template <> struct DecOf<RawQ5K> { typedef DecQ5K type; };

typedef __bf16 gemm_bf16x2 __attribute__((ext_vector_type(2)));
// Decode item h (0..15) of a thread's 32 weights: half H = h % 2 of part I = h / 2 -> weights 2 h and 2 h + 1 as one
// packed bf16 pair. The first item of a part gathers its codes into `codes`, the second reuses them: about seven
// vector instructions for the first, five for the second -- what fits between two MFMAs without holding the matrix
// core up.
template <int I, int H, class Raw, class Sb, class Dec>
__device__ __forceinline__ uint32_t decode_item(const Raw& r, const Sb& sb, const Dec& c, uint32_t& codes) {
    if (H == 0) codes = decode_codes<I>(r, sb, c);
    float w0, w1;
    decode_pair<I, H>(codes, c, w0, w1);
    return __builtin_bit_cast(uint32_t, gemm_bf16x2{(__bf16)w0, (__bf16)w1});
}
// item h with h a (constant-folded) loop variable
template <class Raw, class Sb, class Dec>
__device__ __forceinline__ uint32_t decode_item_at(int h, const Raw& r, const Sb& sb, const Dec& c, uint32_t& codes) {
    switch (h) {
        case 0: return decode_item<0, 0>(r, sb, c, codes);
        case 1: return decode_item<0, 1>(r, sb, c, codes);
        case 2: return decode_item<1, 0>(r, sb, c, codes);
        case 3: return decode_item<1, 1>(r, sb, c, codes);
        case 4: return decode_item<2, 0>(r, sb, c, codes);
        case 5: return decode_item<2, 1>(r, sb, c, codes);
        case 6: return decode_item<3, 0>(r, sb, c, codes);
        case 7: return decode_item<3, 1>(r, sb, c, codes);
        case 8: return decode_item<4, 0>(r, sb, c, codes);
        case 9: return decode_item<4, 1>(r, sb, c, codes);
        case 10: return decode_item<5, 0>(r, sb, c, codes);
        case 11: return decode_item<5, 1>(r, sb, c, codes);
        case 12: return decode_item<6, 0>(r, sb, c, codes);
        case 13: return decode_item<6, 1>(r, sb, c, codes);
        case 14: return decode_item<7, 0>(r, sb, c, codes);
        default: return decode_item<7, 1>(r, sb, c, codes);
    }
}

template <class Raw, int BLOCK_ELEMS, int BLOCK_BYTES, int WTM, int WTN>
__global__ __launch_bounds__(G_THREADS) void dequant_gemm_kernel(const __bf16* __restrict__ a, const uint8_t* __restrict__ w,
                                                           float* __restrict__ c, int m, int n, int k, int k_chunk,
                                                           int64_t split_stride) {
    constexpr int G_WTN = WTN, GN = gemm_gn(WTN), GM = gemm_gm(WTM);
    constexpr int G_A_LOADS = GM * (GK / 8) / G_THREADS;      // 16-byte chunks of the activation tile per thread
    constexpr int G_A_ELEMS = GM * GSTRIDE;
    constexpr int G_W_TASKS = GN * 2 / G_THREADS;             // 32-weight decode tasks per thread and step
    constexpr int G_W_ELEMS = GN * GSTRIDE;
    // Register slots of the activation ring. Narrow tile: two (requested two steps ahead, like the weights). Wide tile:
    // one -- the second slot's 32 registers are what the 256 accumulators leave no room for: a step parks the slot in
    // LDS at its end and requests the step after next into it right away, a full step ahead of its own parking.
    constexpr int A_SLOTS = WTM * WTN <= 8 ? 2 : 1;
    extern __shared__ __attribute__((aligned(16))) __bf16 smem[];
    // stage `buf` (0 / 1): activation tile, then weight tile
    auto a_tile = [&](int buf) { return smem + buf * (G_A_ELEMS + G_W_ELEMS); };
    auto w_tile = [&](int buf) { return smem + buf * (G_A_ELEMS + G_W_ELEMS) + G_A_ELEMS; };

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / G_WAVES_N, wn = wave % G_WAVES_N;
    const int m0 = blockIdx.y * GM, n0 = blockIdx.x * GN;
    const int k_begin = blockIdx.z * k_chunk;
    const int k_end = min(k, k_begin + k_chunk);
    const int nsteps = (k_end - k_begin) / GK;
    const int64_t row_bytes = (int64_t)(k / BLOCK_ELEMS) * BLOCK_BYTES;

    // this thread's share of the weight tile: G_W_TASKS times 32 consecutive elements of one row per K step
    const int wrow = tid >> 1, wsub = tid & 1;
    const uint8_t* wrow_ptr[G_W_TASKS];
#pragma unroll
    for (int t = 0; t < G_W_TASKS; ++t)   // rows past N decode a valid row, never stored
        wrow_ptr[t] = w + (int64_t)min(n0 + wrow + (G_THREADS / 2) * t, n - 1) * row_bytes;

    // Staging registers: a two-slot ring of the activation tile chunks and of the raw weight bytes, requested two
    // steps ahead. One workgroup owns a CU (the double-buffered tiles fill its LDS), so the register file is there
    // to be used. Loads are unconditional (clamped rows, never stored) so a step's loads are in flight together.
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    typedef typename DecOf<Raw>::type Dec;
    typedef typename SbOf<Raw>::type Sb;
    u32x4 aring[A_SLOTS][G_A_LOADS];
    Raw wring[2][G_W_TASKS];
    // per-super-block constants of each task's row: those of the super-block being decoded, and those of the one after it,
    // requested in the second of a super-block's four steps and taken over behind the fourth
    Sb sb_cur[G_W_TASKS], sb_next[G_W_TASKS];
    auto step_k = [&](int step) { return k_begin + min(step, nsteps - 1) * GK; };   // loads past the end re-read the last step
    auto load_a_chunk = [&](int slot, int step, int j) __attribute__((always_inline)) {
        const int p = tid + G_THREADS * j, row = p >> 3, kp = p & 7;
        aring[slot][j] = *reinterpret_cast<const u32x4*>(a + (int64_t)min(m0 + row, m - 1) * k + step_k(step) + 8 * kp);
    };
    auto load_a = [&](int slot, int step) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < G_A_LOADS; ++j) load_a_chunk(slot, step, j);
    };
    auto load_w_task = [&](int slot, int step, int t) __attribute__((always_inline)) {
        load_raw(wring[slot][t], wrow_ptr[t], step_k(step) + 32 * wsub);
    };
    auto load_w = [&](int slot, int step) __attribute__((always_inline)) {
#pragma unroll
        for (int t = 0; t < G_W_TASKS; ++t) load_w_task(slot, step, t);
    };
    auto park_a = [&](int slot, int stage, int j) __attribute__((always_inline)) {      // chunk j of a step's activation tile -> LDS stage
        const int p = tid + G_THREADS * j, row = p >> 3, kp = p & 7;
        *reinterpret_cast<u32x4*>(a_tile(stage) + row * GSTRIDE + 8 * kp) = aring[slot][j];
    };
    uint32_t wp[G_W_TASKS][16];                                                         // packed bf16 pairs: weights 2 h, 2 h + 1
    auto park_w = [&](int stage, int t, int i) __attribute__((always_inline)) {         // weights 8 i .. 8 i + 7 of task t's 32
        __bf16* dst = w_tile(stage) + (wrow + (G_THREADS / 2) * t) * GSTRIDE + park_elem<Raw>(wsub, i);
        *reinterpret_cast<u32x4*>(dst) = u32x4{wp[t][4 * i], wp[t][4 * i + 1], wp[t][4 * i + 2], wp[t][4 * i + 3]};
    };

    f32x16 acc[WTM][G_WTN];
#pragma unroll
    for (int i = 0; i < WTM; ++i)
#pragma unroll
        for (int j = 0; j < G_WTN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    const int fr = lane & 31, fk = (lane >> 5) * 8;   // fragment row inside a 32-row tile, first k of this lane's 8

    // One K step of a wave: its MFMAs on LDS stage `stage`, with everything that prepares the steps after it placed
    // between them in program order. A wave issues in order and an MFMA occupies the matrix core for 32 cycles: about
    // seven vector instructions between two MFMAs run for free, what sits in front of the first MFMA or behind the last
    // one is paid for in full -- so nothing but the first fragment reads precedes the first MFMA. sched_barrier(0)
    // pins the order:
    //   behind MFMA t (t < tasks)            the global loads of weight task t for step `load_step` (ring slot `load_slot`)
    //   behind MFMA tasks + t                the scale / offset header of task t of the next step's weights
    //   behind the following MFMAs           the next step's weights, decoded in two-weight items of about seven
    //                                        instructions, evenly spread (a four-weight item behind every third MFMA
    //                                        held the matrix core up each time)
    //                                        (refilling the registers right behind their last use instead, for a load
    //                                        lead of well over a step, changed nothing: the waits are not a lead problem)
    //   behind the slice's first MFMA        the fragment reads of the next 16-wide slice
    //   behind the last N_STORES MFMAs       one LDS store each into the other stage: every weight chunk after its
    //                                        items, the activation chunks as late as possible, each followed by the
    //                                        global load that refills its ring register
    // `uc`: the step's position U in its super-block (0..3), a compile-time constant.
    auto step_body = [&](auto uc, int stage, int slot_next, int step_next, int load_slot, int load_step) __attribute__((always_inline)) {
        constexpr int U = decltype(uc)::value;
        Sb (&sb_dec)[G_W_TASKS] = U == 3 ? sb_next : sb_cur;       // the step decoded during this one is step_next
        // weight ring: a slot per step (requested two steps ahead), or per two steps (requested in the odd steps for the
        // pair that starts three steps on; the slot's last decode was a step ago)
        constexpr int RS = RawSteps<Raw>::value;
        constexpr int w_slot_next = RS == 1 ? (U + 1) & 1 : ((U + 1) >> 1) & 1;
        constexpr int w_load_slot = RS == 1 ? U & 1 : ((U + 3) >> 1) & 1;
        constexpr bool w_load = RS == 1 || (U & 1);
        const int w_load_step = RS == 1 ? load_step : load_step + 1;
        const int a_slot_next = A_SLOTS == 2 ? slot_next : 0;
        const int a_load_slot = A_SLOTS == 2 ? load_slot : 0, a_load_step = A_SLOTS == 2 ? load_step : step_next + 1;
        constexpr int N_MFMA = WTM * G_WTN * (GK / 16), N_HALVES = 16 * G_W_TASKS, N_STORES = G_A_LOADS + 4 * G_W_TASKS;
        constexpr int FIRST_ITEM = 2 * G_W_TASKS;                  // MFMAs whose slots hold the loads and the headers
        constexpr int N_GAPS = N_MFMA - N_STORES - FIRST_ITEM;      // MFMAs with a decode slot behind them
        static_assert(N_GAPS >= 1, "no slot between the MFMAs for the decode");   // the 128-row tiles put several items in a slot
        const __bf16* at = a_tile(stage) + (32 * WTM * wm + fr) * GSTRIDE + fk;
        const __bf16* wt = w_tile(stage) + (32 * G_WTN * wn + fr) * GSTRIDE + fk;
        bf16x8 af[2][WTM], bf[2][G_WTN];
        auto frags = [&](int set, int kk) __attribute__((always_inline)) {
#pragma unroll
            for (int i = 0; i < WTM; ++i) af[set][i] = *reinterpret_cast<const bf16x8*>(at + 32 * i * GSTRIDE + kk);
#pragma unroll
            for (int j = 0; j < G_WTN; ++j) bf[set][j] = *reinterpret_cast<const bf16x8*>(wt + 32 * j * GSTRIDE + kk);
        };
        Dec dc[G_W_TASKS];
        uint32_t codes[G_W_TASKS];                                  // the codes of the part a task's items are working on
        frags(0, 0);
        __builtin_amdgcn_sched_barrier(0);
#pragma clang loop unroll(full)
        for (int q = 0; q < N_MFMA; ++q) {
            const int kk = q / (WTM * G_WTN), r = q % (WTM * G_WTN), i = r / G_WTN, j = r % G_WTN, set = kk & 1;
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[set][i], bf[set][j], acc[i][j], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            if (r == 0 && kk + 1 < GK / 16) {                   // behind the slice's first MFMA: its wait covers only its own reads
                frags(set ^ 1, 16 * (kk + 1));
                __builtin_amdgcn_sched_barrier(0);
            }
            if (q < G_W_TASKS) {
                if (w_load) load_w_task(w_load_slot, w_load_step, q);
                if (U == 1) load_sb(sb_next[q], wrow_ptr[q], step_k(step_next + 2));   // first step of the next super-block
                __builtin_amdgcn_sched_barrier(0);
            } else if (q < FIRST_ITEM) {
                const int t = q - G_W_TASKS;
                decode_prepare<(U + 1) & 3>(wring[w_slot_next][t], sb_dec[t], step_k(step_next) + 32 * wsub, dc[t]);
                __builtin_amdgcn_sched_barrier(0);
            } else if (q < FIRST_ITEM + N_GAPS) {
                // decode item h sits behind MFMA FIRST_ITEM + h * N_GAPS / N_HALVES: evenly spread (the 256-row tiles have
                // more slots than items: at most one per slot)
                const int g = q - FIRST_ITEM;
                const int h0 = (g * N_HALVES + N_GAPS - 1) / N_GAPS, h1 = ((g + 1) * N_HALVES + N_GAPS - 1) / N_GAPS;
#pragma clang loop unroll(full)
                for (int hh = h0; hh < h1 && hh < N_HALVES; ++hh) {
                    wp[hh / 16][hh % 16] = decode_item_at(hh % 16, wring[w_slot_next][hh / 16], sb_dec[hh / 16], dc[hh / 16], codes[hh / 16]);
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else {
                // first the weight chunks of all but the last task, then the activation chunks (their loads are the
                // youngest), then the last task's weight chunks
                const int sidx = q - (N_MFMA - N_STORES);
                constexpr int W_FIRST = 4 * (G_W_TASKS - 1);
                if (sidx < W_FIRST) park_w(stage ^ 1, sidx / 4, sidx % 4);
                else if (sidx < W_FIRST + G_A_LOADS) {
                    park_a(a_slot_next, stage ^ 1, sidx - W_FIRST);
                    if (A_SLOTS == 1) load_a_chunk(0, a_load_step, sidx - W_FIRST);   // the register has just been parked
                } else park_w(stage ^ 1, G_W_TASKS - 1, sidx - W_FIRST - G_A_LOADS);
                if (A_SLOTS == 2 && sidx < G_A_LOADS) load_a_chunk(a_load_slot, a_load_step, sidx);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        if (U == 3) {
#pragma unroll
            for (int t = 0; t < G_W_TASKS; ++t) sb_cur[t] = sb_next[t];
        }
    };

    // nsteps is a multiple of 4 (K chunks are whole 256-element groups) and > 0. The loop body is one straight-line
    // block (no branches), which is what lets the compiler's wait-count bookkeeping leave the newest step's loads in
    // flight while the older ones are parked.
    load_a(0, 0);
#pragma unroll
    for (int t = 0; t < G_W_TASKS; ++t) load_sb(sb_cur[t], wrow_ptr[t], step_k(0));
    load_w(0, 0);
#pragma unroll
    for (int j = 0; j < G_A_LOADS; ++j) park_a(0, 0, j);
#pragma unroll
    for (int t = 0; t < G_W_TASKS; ++t) {
        Dec d0;
        decode_prepare<0>(wring[0][t], sb_cur[t], step_k(0) + 32 * wsub, d0);
        uint32_t codes0 = 0;
#pragma unroll
        for (int h = 0; h < 16; ++h) wp[t][h] = decode_item_at(h, wring[0][t], sb_cur[t], d0, codes0);
#pragma unroll
        for (int i = 0; i < 4; ++i) park_w(0, t, i);
    }
    load_a(A_SLOTS == 2 ? 1 : 0, 1);
    load_w(1, RawSteps<Raw>::value);                             // the ring's second slot: step 1, or steps 2 and 3
    __syncthreads();
    // One trip = the four steps of a super-block. Step s0 + u: MFMAs on stage u % 2; step + 1 (ring slot (u + 1) % 2) is
    // decoded and parked in the other stage meanwhile; ring slot u % 2 held this step's bytes (parked one step ago) and
    // is refilled with the step after next (the wide tile's single activation slot: chunk by chunk behind its parking,
    // with the step after next)
    for (int s0 = 0; s0 < nsteps; s0 += 4) {
        step_body(std::integral_constant<int, 0>{}, 0, 1, s0 + 1, 0, s0 + 2);
        __syncthreads();
        step_body(std::integral_constant<int, 1>{}, 1, 0, s0 + 2, 1, s0 + 3);
        __syncthreads();
        step_body(std::integral_constant<int, 2>{}, 0, 1, s0 + 3, 0, s0 + 4);
        __syncthreads();
        step_body(std::integral_constant<int, 3>{}, 1, 0, s0 + 4, 1, s0 + 5);
        __syncthreads();
    }

    float* cz = c + (int64_t)blockIdx.z * split_stride;      // split K: this split's partial product
    // accumulator element e of lane l sits at row 8 * (e / 4) + 4 * (l / 32) + e % 4, column l % 32 of its 32 x 32 tile.
    // A tile that lies inside C stores without guards: a guard is a branch per store, and at the join after a branch
    // the stores queue one behind the other (the compiler waits for everything in flight there).
    if (m0 + GM <= m && n0 + GN <= n) {
#pragma unroll
        for (int i = 0; i < WTM; ++i)
#pragma unroll
            for (int j = 0; j < G_WTN; ++j) {
                float* dst = cz + (int64_t)(m0 + 32 * WTM * wm + 32 * i + 4 * (lane >> 5)) * n + n0 + 32 * G_WTN * wn + 32 * j + (lane & 31);
#pragma unroll
                for (int e = 0; e < 16; ++e) dst[(int64_t)(8 * (e >> 2) + (e & 3)) * n] = acc[i][j][e];
            }
        return;
    }
#pragma unroll
    for (int i = 0; i < WTM; ++i)
#pragma unroll
        for (int j = 0; j < G_WTN; ++j) {
            const int col = n0 + 32 * G_WTN * wn + 32 * j + (lane & 31);
            if (col >= n) continue;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int row = m0 + 32 * WTM * wm + 32 * i + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
                if (row < m) {
                    cz[(int64_t)row * n + col] = acc[i][j][e];
                }
            }
        }
}

template <class Raw, int BE, int BB, int WTM, int WTN>
static int launch_gemm_tile(const __bf16* a, const uint8_t* w, float* c, int m, int n, int k, dim3 grid, int k_chunk,
                            int64_t split_stride, hipStream_t s) {
    SKH_SET_MAX_DYNAMIC_LDS_ONCE((&dequant_gemm_kernel<Raw, BE, BB, WTM, WTN>), gemm_smem(WTM, WTN));
    note_kernel("dequant_gemm_kernel");
    dequant_gemm_kernel<Raw, BE, BB, WTM, WTN><<<grid, dim3(G_THREADS), gemm_smem(WTM, WTN), s>>>(a, w, c, m, n, k, k_chunk, split_stride);
    SKH_CHECK(hipGetLastError());
    return 0;
}
template <class Raw, int BE, int BB>
static int launch_gemm_enc(int wtm, int wtn, const __bf16* a, const uint8_t* w, float* c, int m, int n, int k, dim3 grid, int k_chunk,
                           int64_t split_stride, hipStream_t s) {
    if (wtm == 2) {
        if (wtn == 4) return launch_gemm_tile<Raw, BE, BB, 2, 4>(a, w, c, m, n, k, grid, k_chunk, split_stride, s);
        return launch_gemm_tile<Raw, BE, BB, 2, 2>(a, w, c, m, n, k, grid, k_chunk, split_stride, s);
    }
    if (wtn == 4) return launch_gemm_tile<Raw, BE, BB, 4, 4>(a, w, c, m, n, k, grid, k_chunk, split_stride, s);
    return launch_gemm_tile<Raw, BE, BB, 4, 2>(a, w, c, m, n, k, grid, k_chunk, split_stride, s);
}

int launch_q4k_gemm_ksw(const __bf16* a, const uint8_t* w, float* c, int m, int n, int k, hipStream_t s);   // gemm_q4k_ksw.hip
bool gemm_ksw_enabled();
bool gemm_ksw_fits(int m, int n, int k);
bool gemm_ksw_forced();
size_t gemm_frag_activation_bytes(int m, int k);                                                              // gemm_q4k_frag.hip
int launch_gemm_frag_prepass(const float* x, const float* gain, float eps, uint8_t* a, int m, int k, const uint8_t* w, int n, hipStream_t s,
                             bool pairs);
int launch_q4k_gemm_frag(const uint8_t* a, const uint8_t* w, float* c, int m, int n, int k, hipStream_t s, const float* residual);
bool gemm_frag_enabled();
bool gemm_frag_fits(int m, int n, int k);
bool gemm_frag_forced();

static std::atomic<int> g_gemm_ksplit{0};   // 0 = choose from the tile count
void set_gemm_ksplit(int v) { g_gemm_ksplit = v; }
static std::atomic<int> g_gemm_wide{-1};    // -1 = choose from the shape, 0 / 1 = narrow / wide tile
void set_gemm_wide(int v) { g_gemm_wide = v; }
static std::atomic<int> g_gemm_rows{0};     // 0 = choose from the shape, 2 / 4 = 128 / 256 activation rows per tile
void set_gemm_rows(int v) { if (v == 0 || v == 2 || v == 4) g_gemm_rows = v; }

// y = epilogue(prologue(x) . W^T): gain != null normalises every activation row first (RMSNorm, folded into the pass that
// rounds the activations to bf16); epilogue is one of GEMM_EPI_* (residual [m, n] may be y; SwiGLU: y is [m, n / 2]).
// `tmp` ([m, n] floats, needed when an epilogue is asked for) takes the plain product when K is not split.
// Returns 1, having launched nothing, when the shape is outside the tile kernel's range and a prologue or epilogue was
// asked for (the caller composes the same arithmetic from separate launches).
// x_pairs: x is [m, 2 k], rows of interleaved (gate, up) pairs, and the product's activation is their SwiGLU, taken in
// the pass that rounds to bf16 (no gain then).
int launch_gemm_fused(int enc, const uint8_t* w, const float* x, int m, int k, int n, float* y, const float* gain, float eps,
                      const float* residual, int epilogue, float* tmp, bool x_pairs) {
    if (m <= 0 || n <= 0) return 0;
    if (!is_packed(enc)) return set_error("gemm: unsupported encoding %d", enc);
    if (k <= 0 || k % block_elems(enc) != 0)
        return set_error("gemm: inputDim must be a positive multiple of %d; got %d", block_elems(enc), k);
    // shapes the tile loader cannot take (a Q8_0 row that is not a whole number of 256-element groups: the K loop
    // runs pairs of 64-element steps over whole groups; unaligned operands) go through the row kernels: same result
    // to fp32 rounding, the weight streamed once per 4 rows
    const bool fused = gain != nullptr || epilogue != GEMM_EPI_NONE || x_pairs;
    if (x_pairs && gain) return set_error("gemm: a SwiGLU prologue takes no RMSNorm gain");
    if (k % 256 != 0 || (reinterpret_cast<uintptr_t>(w) & 15) || (reinterpret_cast<uintptr_t>(x) & 15) ||
        (gain && ((reinterpret_cast<uintptr_t>(gain) & 15) || k > 256 * 4 * 16)) || (epilogue == GEMM_EPI_SWIGLU && (n & 1)) ||
        (epilogue != GEMM_EPI_NONE && !tmp))
        return fused ? 1 : launch_gemv(enc, w, x, m, k, n, y);
    hipStream_t s = current_stream();
    auto round_activations = [&](__bf16* a) -> int {            // fp32 -> bf16, with the RMSNorm of a fused call folded in
        const int64_t n4 = (int64_t)m * k / 4;                  // k is a multiple of 64
        if (x_pairs) gemm_prepass_swiglu_kernel<<<dim3((unsigned)((n4 + 255) / 256)), dim3(256), 0, s>>>(x, a, n4);
        else if (!gain) gemm_prepass_kernel<<<dim3((unsigned)((n4 + 256 * PREPASS_UNROLL - 1) / (256 * PREPASS_UNROLL))), dim3(256), 0, s>>>(x, a, n4);
        else if (k <= 256 * 4 * 4) gemm_prepass_rmsnorm_kernel<4><<<dim3(m), dim3(256), 0, s>>>(x, gain, a, k, eps);
        else gemm_prepass_rmsnorm_kernel<16><<<dim3(m), dim3(256), 0, s>>>(x, gain, a, k, eps);
        SKH_CHECK(hipGetLastError());
        return 0;
    };
    auto finish = [&]() -> int {                                 // the epilogue of a product parked whole in tmp
        if (epilogue == GEMM_EPI_RESIDUAL) return launch_add(residual, tmp, y, (int64_t)m * n);
        if (epilogue == GEMM_EPI_SWIGLU) return launch_swiglu_pairs(tmp, y, (int64_t)m * (n / 2));
        return 0;
    };
    auto run_ksw = [&]() -> int {                                // Q4_K: K split over the waves of a workgroup, 128 x 64 tiles
        __bf16* a = static_cast<__bf16*>(kernel_workspace((size_t)m * k * sizeof(__bf16)));
        if (!a) return -1;
        if (round_activations(a) != 0) return -1;
        if (launch_q4k_gemm_ksw(a, w, epilogue != GEMM_EPI_NONE ? tmp : y, m, n, k, s) != 0) return -1;
        return finish();
    };
    auto run_frag = [&]() -> int {                               // Q4_K: the same tiles, activations in fragment order
        uint8_t* a = static_cast<uint8_t*>(kernel_workspace(gemm_frag_activation_bytes(m, k)));
        if (!a) return -1;
        if (launch_gemm_frag_prepass(x, gain, eps, a, m, k, w, n, s, x_pairs) != 0) return -1;
        // the residual is added where the tile is stored; only SwiGLU still parks the plain product
        if (epilogue == GEMM_EPI_SWIGLU) return launch_q4k_gemm_frag(a, w, tmp, m, n, k, s, nullptr) != 0 ? -1 : finish();
        return launch_q4k_gemm_frag(a, w, y, m, n, k, s, epilogue == GEMM_EPI_RESIDUAL ? residual : nullptr);
    };
    const bool ksw_ok = enc == ENC_Q4_K && gemm_ksw_fits(m, n, k) && g_gemm_wide.load() < 0 && g_gemm_rows.load() == 0;
    const bool frag_ok = ksw_ok && gemm_frag_fits(m, n, k);
    if (frag_ok && gemm_frag_forced()) return run_frag();
    if (ksw_ok && gemm_ksw_forced()) return run_ksw();
    // 128 activation rows per tile where there are no more than that (the weight is then decoded once, and half the
    // matrix work of the taller tile is not spent on rows that do not exist); the wide tile where it alone fills most of
    // the chip in one round
    const int wtm = g_gemm_rows.load() != 0 ? g_gemm_rows.load() : (m <= 128 ? 2 : 4);
    const int tiles_m = (m + gemm_gm(wtm) - 1) / gemm_gm(wtm);
    const int wide_tiles = tiles_m * ((n + gemm_gn(4) - 1) / gemm_gn(4));
    const bool wide = g_gemm_wide.load() >= 0 ? g_gemm_wide.load() != 0 : 4 * wide_tiles >= 3 * num_cus();
    const int wtn = wide ? 4 : 2;
    const int tiles_n = (n + gemm_gn(wtn) - 1) / gemm_gn(wtn);
    const int tiles = tiles_m * tiles_n;
    // K chunks are whole 256-element groups so every encoding's blocks stay intact
    const int kgroups = (k + 255) / 256;
    int ksplit = g_gemm_ksplit;
    double tile_estimate = 0.0;
    if (ksplit <= 0) {
        // One workgroup is resident per CU, so the tile grid runs in rounds of num_cus() workgroups. Measured on this
        // kernel: about 8 us per round outside the K loop, 1.04 us per 64-element K step, and for the launch that sums
        // the splits 2.3 us plus its (splits + 1) * m * n floats at 8 bytes per ns. Take the split with the least estimate.
        const int cus = num_cus();
        double best = 0.0;
        ksplit = 1;
        for (int ks = 1; ks <= 8 && ks <= kgroups; ++ks) {
            const int rounds = (tiles * ks + cus - 1) / cus;
            const int steps = ((kgroups + ks - 1) / ks) * (256 / GK);
            const double step_us = wtm == 4 ? (wide ? 2.0 : 1.04) : (wide ? 1.13 : 0.65);   // measured per tile shape
            double t = rounds * (8.0 + step_us * steps);
            if (ks > 1) t += 2.3 + (double)(ks + 1) * m * n * 4.0 / 8.0e6;
            if (ks == 1 || t < best) { best = t; ksplit = ks; }
        }
        tile_estimate = best;
    }
    if (ksw_ok && gemm_ksw_enabled() && g_gemm_ksplit.load() <= 0) {
        // The kernel that splits K over the waves of a workgroup fills the chip with 128 x 64 tiles and parks no partial
        // products; its step is slower per tile row (0.31 us per 64 elements of K measured, 6.5 us per round outside the loop).
        // It wins where the tile kernel would have to split K across workgroups: 512 x 4096 x 4096 is such a shape.
        const int rounds = (((m + 127) / 128) * ((n + 63) / 64) + num_cus() - 1) / num_cus();
        // the same tiles with the activations in fragment order: measured 8 us per round outside the loop and 0.20 us per
        // 64 elements of K (0.27 on rows longer than two super-blocks per wave, whose weight ring is refilled under way)
        if (frag_ok && gemm_frag_enabled()) {
            if (rounds * (8.0 + (k <= 4096 ? 0.20 : 0.27) * (k / GK)) < tile_estimate) return run_frag();
        } else if (rounds * (6.5 + 0.31 * (k / GK)) < tile_estimate) return run_ksw();
    }
    if (ksplit > kgroups) ksplit = kgroups;
    const int k_chunk = ((kgroups + ksplit - 1) / ksplit) * 256;
    ksplit = (k + k_chunk - 1) / k_chunk;
    // workspace: the bf16 activations, then (split K) one partial product per split
    const size_t a_bytes = (((size_t)m * k * sizeof(__bf16)) + 255) & ~(size_t)255;
    const int64_t split_stride = ksplit > 1 ? (((int64_t)m * n + 3) & ~(int64_t)3) : 0;
    char* ws = static_cast<char*>(kernel_workspace(a_bytes + (size_t)split_stride * ksplit * sizeof(float)));
    if (!ws) return -1;
    __bf16* a = reinterpret_cast<__bf16*>(ws);
    float* part = reinterpret_cast<float*>(ws + a_bytes);
    if (round_activations(a) != 0) return -1;
    const dim3 grid(tiles_n, tiles_m, ksplit);
    float* c = ksplit > 1 ? part : (epilogue != GEMM_EPI_NONE ? tmp : y);
    int rc;
    if (enc == ENC_Q4_K) rc = launch_gemm_enc<RawQ4K, QK_ELEMS, Q4K_BYTES>(wtm, wtn, a, w, c, m, n, k, grid, k_chunk, split_stride, s);
    else if (enc == ENC_Q6_K) rc = launch_gemm_enc<RawQ6K, QK_ELEMS, Q6K_BYTES>(wtm, wtn, a, w, c, m, n, k, grid, k_chunk, split_stride, s);
    else if (enc == ENC_Q5_K) rc = launch_gemm_enc<RawQ5K, QK_ELEMS, Q5K_BYTES>(wtm, wtn, a, w, c, m, n, k, grid, k_chunk, split_stride, s);
    else if (enc == ENC_Q4_0) rc = launch_gemm_enc<RawQ45<0>, Q80_ELEMS, Q40_BYTES>(wtm, wtn, a, w, c, m, n, k, grid, k_chunk, split_stride, s);
    else if (enc == ENC_Q5_0) rc = launch_gemm_enc<RawQ45<1>, Q80_ELEMS, Q50_BYTES>(wtm, wtn, a, w, c, m, n, k, grid, k_chunk, split_stride, s);
    else if (enc == ENC_Q5_1) rc = launch_gemm_enc<RawQ45<2>, Q80_ELEMS, Q51_BYTES>(wtm, wtn, a, w, c, m, n, k, grid, k_chunk, split_stride, s);
    else rc = launch_gemm_enc<RawQ80, Q80_ELEMS, Q80_BYTES>(wtm, wtn, a, w, c, m, n, k, grid, k_chunk, split_stride, s);
    if (rc != 0) return rc;
    if (ksplit == 1) return finish();
    const int64_t total = (int64_t)m * n;
    gemm_splitk_sum_kernel<<<dim3((unsigned)((total / 4 + 256) / 256)), dim3(256), 0, s>>>(
        part, split_stride, ksplit, y, total, (reinterpret_cast<uintptr_t>(y) & 15) == 0, residual, epilogue);
    SKH_CHECK(hipGetLastError());
    return 0;
}

int launch_gemm(int enc, const uint8_t* w, const float* x, int m, int k, int n, float* y) {
    return launch_gemm_fused(enc, w, x, m, k, n, y, nullptr, 0.f, nullptr, GEMM_EPI_NONE, nullptr, false);
}

}  // namespace skh
