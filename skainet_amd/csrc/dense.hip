// Dense fp32 matmul entries of the kernel SPI. No decoder configuration routes through them (every linear layer
// there is packed). Two kernels:
//   sgemm_mfma_kernel  fp32 operands on the fp32 matrix instruction (v_mfma_f32_32x32x2_f32: exact fp32 products, fp32
//                      accumulation), 128 x 128 x 16 tiles, for products of at least 64 rows whose operands are 16-byte
//                      aligned with strides and K (and N, when B is read along its rows) multiples of four;
//   sgemm_kernel       everything else (any stride and alignment, bf16 / fp16 B): an LDS-tiled SGEMM, 64 x 64 output
//                      tile per workgroup, 16-deep K slices, 4 x 4 outputs per thread, fp32 FMA accumulation in
//                      ascending k.
//
//   fp32_matmul     C(m,n) = A(m,k) B(k,n), row strides in floats, full overwrite (k == 0 zeroes C)
//                   /root/reference/skainet-backends/skainet-backend-native-cpu/native/include/skainet_kernels.h:262-276
//   fp32_matmul_wt  out[i,o] = sum_p in[i,p] * w[o,p]
//                   /root/reference/skainet-backends/skainet-backend-native-cpu/native/include/skainet_kernels.h:495-515
//   bf16 / fp16 matmul  C(m,n) = A(m,k) B(k,n) with B two bytes per element, byte row stride (bf16: the high half of
//                   an fp32; fp16: IEEE binary16), same tile kernel with the decode in the tile load
//                   /root/reference/skainet-backends/skainet-backend-native-cpu/native/include/skainet_kernels.h:278-312
#include "common.h"

namespace skh {

constexpr int DT = 64, DK = 16;

// BK 0: B(p, j) = b[p * b_stride + j];  BK 1: B(p, j) = b[j * b_stride + p] (x . W^T);
// BK 2 / 3: B(p, j) = bf16 / fp16 at byte p * b_stride + 2 j of b (b_stride in bytes, any alignment: read bytewise).
template <int BK>
__global__ __launch_bounds__(256) void sgemm_kernel(const float* __restrict__ a, int64_t a_stride, const float* __restrict__ b,
                                                    int64_t b_stride, float* __restrict__ c, int64_t c_stride, int m, int n, int k) {
    constexpr bool BT = BK == 1;
    __shared__ float as[DK][DT + 1];
    __shared__ float bs[DK][DT + 1];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int i0 = blockIdx.y * DT, j0 = blockIdx.x * DT;
    float acc[4][4] = {};
    for (int p0 = 0; p0 < k; p0 += DK) {
        for (int t = threadIdx.x; t < DT * DK; t += 256) {
            // A tile: row i (64) x depth p (16), read along p
            const int ai = t / DK, ap = t % DK;
            as[ap][ai] = (i0 + ai < m && p0 + ap < k) ? a[(int64_t)(i0 + ai) * a_stride + p0 + ap] : 0.f;
            if (BT) {
                const int bj = t / DK, bp = t % DK;
                bs[bp][bj] = (j0 + bj < n && p0 + bp < k) ? b[(int64_t)(j0 + bj) * b_stride + p0 + bp] : 0.f;
            } else if (BK == 0) {
                const int bp = t / DT, bj = t % DT;
                bs[bp][bj] = (j0 + bj < n && p0 + bp < k) ? b[(int64_t)(p0 + bp) * b_stride + j0 + bj] : 0.f;
            } else {
                const int bp = t / DT, bj = t % DT;
                float v = 0.f;
                if (j0 + bj < n && p0 + bp < k) {
                    const uint8_t* e = reinterpret_cast<const uint8_t*>(b) + (int64_t)(p0 + bp) * b_stride + 2 * (j0 + bj);
                    const uint32_t h = (uint32_t)e[0] | ((uint32_t)e[1] << 8);
                    v = BK == 2 ? __uint_as_float(h << 16) : half_bits_to_float(h);
                }
                bs[bp][bj] = v;
            }
        }
        __syncthreads();
#pragma unroll
        for (int p = 0; p < DK; ++p) {
            float av[4], bv[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) { av[r] = as[p][ty * 4 + r]; bv[r] = bs[p][tx * 4 + r]; }
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int s = 0; s < 4; ++s) acc[r][s] = fmaf(av[r], bv[s], acc[r][s]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const int i = i0 + ty * 4 + r, j = j0 + tx * 4 + s;
            if (i < m && j < n) c[(int64_t)i * c_stride + j] = acc[r][s];
        }
}

// fp32 on the matrix cores. Workgroup tile 64 WM x 128 (WM = 2: 128 x 128; WM = 1: 64 x 128, for products whose taller
// tiles would leave CUs idle), K slices of 16; four waves in 2 x 2, each 32 WM x 64 outputs as WM x 2 tiles of 32 x 32. A slice goes global -> registers (requested a slice ahead) -> LDS
// (two stages, one barrier per slice) with K as the slow index of both tiles: the matrix instruction's operands are
// one float per lane -- row (or column) lane % 32 at depth lane / 32 of a two-deep step -- so a wave reads 32
// consecutive floats of two tile rows. BT: B(p, j) = b[j * b_stride + p] (x . W^T), else b[p * b_stride + j].
constexpr int MT = 128, MK = 16, MP = MT + 4;      // tile edge, slice depth, LDS row pitch in floats (16-byte rows)
typedef float dense_f32x16 __attribute__((ext_vector_type(16)));

template <bool BT, int WM>
__global__ __launch_bounds__(256) void sgemm_mfma_kernel(const float* __restrict__ a, int64_t a_stride, const float* __restrict__ b,
                                                         int64_t b_stride, float* __restrict__ c, int64_t c_stride, int m, int n, int k) {
    __shared__ __attribute__((aligned(16))) float as[2][MK][MP];
    __shared__ __attribute__((aligned(16))) float bs[2][MK][MP];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int i0 = blockIdx.y * (64 * WM), j0 = blockIdx.x * MT;
    // loads of a slice: "row-like" operands (A, and B when transposed) 128 rows x 4 float4 along K, two per thread;
    // B read along its rows: 16 depths x 32 float4, two per thread
    const int lr = tid >> 2, lq = tid & 3;            // row (+ 64 j), float4 along K
    const int bp = tid >> 5, bq = tid & 31;           // depth (+ 8 j), float4 along N
    float4 ra[WM], rb[2];
    auto load_slice = [&](int p0) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int row = i0 + lr + 64 * j, p = p0 + 4 * lq;
            if (j < WM) ra[j] = (row < m && p < k) ? *reinterpret_cast<const float4*>(a + (int64_t)row * a_stride + p) : make_float4(0.f, 0.f, 0.f, 0.f);
            if (BT) {
                const int col = j0 + lr + 64 * j;
                rb[j] = (col < n && p < k) ? *reinterpret_cast<const float4*>(b + (int64_t)col * b_stride + p) : make_float4(0.f, 0.f, 0.f, 0.f);
            } else {
                const int pp = p0 + bp + 8 * j, col = j0 + 4 * bq;
                rb[j] = (pp < k && col < n) ? *reinterpret_cast<const float4*>(b + (int64_t)pp * b_stride + col) : make_float4(0.f, 0.f, 0.f, 0.f);
            }
        }
    };
    auto store_slice = [&](int buf) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int r = lr + 64 * j;
            if (j < WM) { as[buf][4 * lq][r] = ra[j].x; as[buf][4 * lq + 1][r] = ra[j].y; as[buf][4 * lq + 2][r] = ra[j].z; as[buf][4 * lq + 3][r] = ra[j].w; }
            if (BT) {
                bs[buf][4 * lq][r] = rb[j].x; bs[buf][4 * lq + 1][r] = rb[j].y; bs[buf][4 * lq + 2][r] = rb[j].z; bs[buf][4 * lq + 3][r] = rb[j].w;
            } else {
                *reinterpret_cast<float4*>(&bs[buf][bp + 8 * j][4 * bq]) = rb[j];
            }
        }
    };
    dense_f32x16 acc[WM][2];
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
    const int nsl = (k + MK - 1) / MK;
    if (nsl > 0) { load_slice(0); store_slice(0); }
    __syncthreads();
    const int col = lane & 31, dh = lane >> 5;
    for (int sl = 0; sl < nsl; ++sl) {
        const int buf = sl & 1;
        if (sl + 1 < nsl) load_slice((sl + 1) * MK);
#pragma unroll
        for (int s2 = 0; s2 < MK / 2; ++s2) {
            float av[WM], bv[2];
#pragma unroll
            for (int i = 0; i < WM; ++i) av[i] = as[buf][2 * s2 + dh][wm * (32 * WM) + 32 * i + col];
#pragma unroll
            for (int i = 0; i < 2; ++i) bv[i] = bs[buf][2 * s2 + dh][wn * 64 + 32 * i + col];
#pragma unroll
            for (int i = 0; i < WM; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[i], bv[j], acc[i][j], 0, 0, 0);
        }
        if (sl + 1 < nsl) store_slice(buf ^ 1);
        __syncthreads();
    }
    // accumulator element e of lane l: row 8 (e / 4) + 4 (l / 32) + e % 4, column l % 32 of its 32 x 32 tile
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int row = i0 + wm * (32 * WM) + 32 * i + 8 * (e >> 2) + 4 * dh + (e & 3), cc = j0 + wn * 64 + 32 * j + col;
                if (row < m && cc < n) c[(int64_t)row * c_stride + cc] = acc[i][j][e];
            }
}

static std::atomic<int> g_dense_mfma{1};
void set_dense_mfma(int v) { g_dense_mfma = v != 0; }

int launch_fp32_matmul(const float* a, int64_t a_stride, const float* b, int64_t b_stride, float* c, int64_t c_stride,
                       int m, int n, int k, bool b_transposed) {
    if (m <= 0 || n <= 0) return 0;
    if (k < 0) k = 0;
    const bool aligned = ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) & 15) == 0 && (a_stride & 3) == 0 &&
                         (b_stride & 3) == 0 && (k & 3) == 0 && (b_transposed || (n & 3) == 0);
    if (g_dense_mfma && aligned && m >= 64 && n >= 32 && k >= 4) {
        // 128-row tiles where they give every CU at least one; else 64-row tiles
        const int tiles128 = ((n + MT - 1) / MT) * ((m + 127) / 128);
        const int wmr = tiles128 >= num_cus() ? 2 : 1;
        const dim3 grid((n + MT - 1) / MT, (m + 64 * wmr - 1) / (64 * wmr));
        note_kernel("sgemm_mfma_kernel");
        if (b_transposed) {
            if (wmr == 2) sgemm_mfma_kernel<true, 2><<<grid, dim3(256), 0, current_stream()>>>(a, a_stride, b, b_stride, c, c_stride, m, n, k);
            else sgemm_mfma_kernel<true, 1><<<grid, dim3(256), 0, current_stream()>>>(a, a_stride, b, b_stride, c, c_stride, m, n, k);
        } else {
            if (wmr == 2) sgemm_mfma_kernel<false, 2><<<grid, dim3(256), 0, current_stream()>>>(a, a_stride, b, b_stride, c, c_stride, m, n, k);
            else sgemm_mfma_kernel<false, 1><<<grid, dim3(256), 0, current_stream()>>>(a, a_stride, b, b_stride, c, c_stride, m, n, k);
        }
        SKH_CHECK(hipGetLastError());
        return 0;
    }
    note_kernel("sgemm_kernel");
    const dim3 grid((n + DT - 1) / DT, (m + DT - 1) / DT);
    if (b_transposed) sgemm_kernel<1><<<grid, dim3(256), 0, current_stream()>>>(a, a_stride, b, b_stride, c, c_stride, m, n, k);
    else sgemm_kernel<0><<<grid, dim3(256), 0, current_stream()>>>(a, a_stride, b, b_stride, c, c_stride, m, n, k);
    SKH_CHECK(hipGetLastError());
    return 0;
}

// C(m, n) = A(m, k) B(k, n), B bf16 (fp16 != 0: IEEE binary16) bytes with a byte row stride.
int launch_narrow_matmul(const float* a, int64_t a_stride, const uint8_t* b, int64_t b_byte_stride, float* c, int64_t c_stride,
                         int m, int n, int k, int fp16) {
    if (m <= 0 || n <= 0) return 0;
    if (k < 0) k = 0;
    const dim3 grid((n + DT - 1) / DT, (m + DT - 1) / DT);
    const float* bf = reinterpret_cast<const float*>(b);
    if (fp16) sgemm_kernel<3><<<grid, dim3(256), 0, current_stream()>>>(a, a_stride, bf, b_byte_stride, c, c_stride, m, n, k);
    else sgemm_kernel<2><<<grid, dim3(256), 0, current_stream()>>>(a, a_stride, bf, b_byte_stride, c, c_stride, m, n, k);
    SKH_CHECK(hipGetLastError());
    return 0;
}

}  // namespace skh
