// Dense fp32 matmul entries of the kernel SPI. No decoder configuration routes through them (every
// linear layer there is packed), so this is a correctness-first LDS-tiled SGEMM: 64 x 64 output tile per
// workgroup, 16-deep K slices, 4 x 4 outputs per thread, fp32 FMA accumulation in ascending k.
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

int launch_fp32_matmul(const float* a, int64_t a_stride, const float* b, int64_t b_stride, float* c, int64_t c_stride,
                       int m, int n, int k, bool b_transposed) {
    if (m <= 0 || n <= 0) return 0;
    if (k < 0) k = 0;
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
