// Dense fp32 elementwise, activation and reduction kernels on device-resident operands: what an ops class that keeps
// activations on the device needs besides the fused row kernels. Contracts of the reference's CPU library
//   /root/reference/skainet-backends/skainet-backend-native-cpu/native/include/skainet_kernels.h:515-546
//   /root/reference/skainet-backends/skainet-backend-native-cpu/native/src/f32_ops.c:130-330
// binary: out[i] = a[ia] op b[ib], op 0 add / 1 sub / 2 mul / 3 div, operand modes 0 full (index i), 1 scalar (index 0),
//         2 bias (index i % inner);
// unary:  0 relu, 1 sigmoid 1 / (1 + exp(-x)), 2 silu x * sigmoid(x), 3 gelu 0.5 x (1 + tanh(0.7978845608 (x + 0.044715 x^3))),
//         4 gelu 0.5 x (1 + erf(x / sqrt 2)) evaluated in double, 5 erf in double, 6 tanh;
// reduce_all: *out = sum (or mean) of n values; reduce_axis: out[o, x] = sum (or mean) over k of in[o, k, x].
// All HBM-bound one-pass kernels: 16-byte accesses where the operands allow, a grid that covers the chip a few times.
#include "common.h"

namespace skh {

void* kernel_workspace(size_t bytes);   // shim.hip: per-thread scratch, grown on demand

__device__ __forceinline__ float ew_apply(int op, float x, float y) {
    switch (op) {
        case 0: return x + y;
        case 1: return x - y;
        case 2: return x * y;
        default: return x / y;
    }
}

template <int OP>
__global__ __launch_bounds__(256) void binary_full_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                          float* __restrict__ out, int64_t n4) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride) {
        const float4 x = reinterpret_cast<const float4*>(a)[i], y = reinterpret_cast<const float4*>(b)[i];
        reinterpret_cast<float4*>(out)[i] = make_float4(ew_apply(OP, x.x, y.x), ew_apply(OP, x.y, y.y), ew_apply(OP, x.z, y.z), ew_apply(OP, x.w, y.w));
    }
}

__global__ __launch_bounds__(256) void binary_modes_kernel(int op, const float* __restrict__ a, int a_mode, const float* __restrict__ b,
                                                           int b_mode, float* __restrict__ out, int64_t n, int inner) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const int64_t x = i % inner;
        const int64_t ia = a_mode == 0 ? i : (a_mode == 1 ? 0 : x), ib = b_mode == 0 ? i : (b_mode == 1 ? 0 : x);
        out[i] = ew_apply(op, a[ia], b[ib]);
    }
}

__device__ __forceinline__ float ew_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float ew_unary(int op, float x) {
    switch (op) {
        case 0: return x < 0.0f ? 0.0f : x;
        case 1: return ew_sigmoid(x);
        case 2: return x * ew_sigmoid(x);
        case 3: return 0.5f * x * (1.0f + tanhf(0.7978845608f * (x + 0.044715f * (x * x * x))));
        case 4: return (float)(0.5 * (double)x * (1.0 + erf((double)x * 0.70710678118654752440)));
        case 5: return (float)erf((double)x);
        default: return tanhf(x);
    }
}

__global__ __launch_bounds__(256) void unary_kernel(int op, const float* __restrict__ in, float* __restrict__ out, int64_t n) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) out[i] = ew_unary(op, in[i]);
}

// Sums: every thread keeps four running sums over a grid-stride walk, a workgroup folds them through a wave sum and LDS.
__device__ __forceinline__ float block_sum_256(float v, float* lds) {
    v = wave_sum(v);
    if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = v;
    __syncthreads();
    return (lds[0] + lds[1]) + (lds[2] + lds[3]);
}

__global__ __launch_bounds__(256) void reduce_partial_kernel(const float* __restrict__ in, int64_t n, float* __restrict__ part) {
    __shared__ float lds[4];
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    for (; i + 3 * stride < n; i += 4 * stride) { s0 += in[i]; s1 += in[i + stride]; s2 += in[i + 2 * stride]; s3 += in[i + 3 * stride]; }
    for (; i < n; i += stride) s0 += in[i];
    const float s = block_sum_256((s0 + s1) + (s2 + s3), lds);
    if (threadIdx.x == 0) part[blockIdx.x] = s;
}

__global__ __launch_bounds__(256) void reduce_final_kernel(const float* __restrict__ part, int count, float scale, float* __restrict__ out) {
    __shared__ float lds[4];
    float s = 0.f;
    for (int i = threadIdx.x; i < count; i += 256) s += part[i];
    s = block_sum_256(s, lds);
    if (threadIdx.x == 0) out[0] = s * scale;
}

// out[o, x] = sum_k in[o, k, x]. Wide inner: one thread per output walks k (a wave reads 256 consecutive bytes per
// step). Narrow inner: one wave per output row o, lanes stride over the red * inner values of the row and fold per x.
__global__ __launch_bounds__(256) void reduce_axis_wide_kernel(const float* __restrict__ in, int outer, int red, int inner, float scale,
                                                               float* __restrict__ out) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (int64_t)outer * inner) return;
    const int64_t o = idx / inner, x = idx % inner;
    const float* p = in + o * red * inner + x;
    float s0 = 0.f, s1 = 0.f;
    int k = 0;
    for (; k + 1 < red; k += 2) { s0 += p[(int64_t)k * inner]; s1 += p[(int64_t)(k + 1) * inner]; }
    if (k < red) s0 += p[(int64_t)k * inner];
    out[idx] = (s0 + s1) * scale;
}

__global__ __launch_bounds__(256) void reduce_axis_narrow_kernel(const float* __restrict__ in, int outer, int red, int inner, float scale,
                                                                 float* __restrict__ out) {
    // one wave per (o, x): lanes stride over k
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= (int64_t)outer * inner) return;
    const int64_t o = row / inner, x = row % inner;
    const float* p = in + o * red * inner + x;
    float s = 0.f;
    for (int k = threadIdx.x & 63; k < red; k += 64) s += p[(int64_t)k * inner];
    s = wave_sum(s);
    if ((threadIdx.x & 63) == 0) out[row] = s * scale;
}

static unsigned ew_grid(int64_t items) {
    const int64_t want = (items + 255) / 256, cap = (int64_t)num_cus() * 8;
    return (unsigned)(want < 1 ? 1 : (want > cap ? cap : want));
}

int launch_f32_binary(int op, const float* a, int a_mode, const float* b, int b_mode, float* out, int64_t n, int inner) {
    if (n <= 0) return 0;
    if (op < 0 || op > 3) return set_error("binary: unknown op %d", op);
    if (a_mode < 0 || a_mode > 2 || b_mode < 0 || b_mode > 2) return set_error("binary: operand modes must be 0 (full), 1 (scalar) or 2 (bias); got %d, %d", a_mode, b_mode);
    if (!a || !b || !out) return set_error("binary: null pointer");
    if (inner <= 0) inner = 1;
    hipStream_t s = current_stream();
    const bool aligned = ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) | reinterpret_cast<uintptr_t>(out)) & 15) == 0;
    if (a_mode == 0 && b_mode == 0 && aligned && (n & 3) == 0) {
        const int64_t n4 = n / 4;
        switch (op) {
            case 0: binary_full_kernel<0><<<dim3(ew_grid(n4)), dim3(256), 0, s>>>(a, b, out, n4); break;
            case 1: binary_full_kernel<1><<<dim3(ew_grid(n4)), dim3(256), 0, s>>>(a, b, out, n4); break;
            case 2: binary_full_kernel<2><<<dim3(ew_grid(n4)), dim3(256), 0, s>>>(a, b, out, n4); break;
            default: binary_full_kernel<3><<<dim3(ew_grid(n4)), dim3(256), 0, s>>>(a, b, out, n4); break;
        }
    } else {
        binary_modes_kernel<<<dim3(ew_grid(n)), dim3(256), 0, s>>>(op, a, a_mode, b, b_mode, out, n, inner);
    }
    SKH_CHECK(hipGetLastError());
    return 0;
}

int launch_f32_unary(int op, const float* in, float* out, int64_t n) {
    if (n <= 0) return 0;
    if (op < 0 || op > 6) return set_error("unary: unknown op %d", op);
    if (!in || !out) return set_error("unary: null pointer");
    unary_kernel<<<dim3(ew_grid(n)), dim3(256), 0, current_stream()>>>(op, in, out, n);
    SKH_CHECK(hipGetLastError());
    return 0;
}

int launch_f32_reduce_all(const float* in, int64_t n, int mean, float* out) {
    if (!out) return set_error("reduce_all: null output");
    if (n > 0 && !in) return set_error("reduce_all: null input");
    hipStream_t s = current_stream();
    const int parts = n > 0 ? (int)ew_grid((n + 3) / 4) : 0;
    float* part = static_cast<float*>(kernel_workspace(sizeof(float) * (size_t)(parts > 0 ? parts : 1)));
    if (!part) return -1;
    if (parts > 0) {
        reduce_partial_kernel<<<dim3(parts), dim3(256), 0, s>>>(in, n, part);
        SKH_CHECK(hipGetLastError());
    }
    reduce_final_kernel<<<dim3(1), dim3(256), 0, s>>>(part, parts, (mean && n > 0) ? 1.0f / (float)n : 1.0f, out);
    SKH_CHECK(hipGetLastError());
    return 0;
}

int launch_f32_reduce_axis(const float* in, int outer, int red, int inner, int mean, float* out) {
    if (outer <= 0 || inner <= 0) return 0;
    if (!out || (red > 0 && !in)) return set_error("reduce_axis: null pointer");
    if (red < 0) return set_error("reduce_axis: negative extent %d", red);
    hipStream_t s = current_stream();
    const float scale = (mean && red > 0) ? 1.0f / (float)red : 1.0f;
    const int64_t outputs = (int64_t)outer * inner;
    if (outputs >= 0x7FFFFFFFLL * 4) return set_error("reduce_axis: %lld outputs exceed one launch", (long long)outputs);
    if (inner >= 64 || red < 128)
        reduce_axis_wide_kernel<<<dim3((unsigned)((outputs + 255) / 256)), dim3(256), 0, s>>>(in, outer, red, inner, scale, out);
    else
        reduce_axis_narrow_kernel<<<dim3((unsigned)((outputs + 3) / 4)), dim3(256), 0, s>>>(in, outer, red, inner, scale, out);
    SKH_CHECK(hipGetLastError());
    return 0;
}

}  // namespace skh
