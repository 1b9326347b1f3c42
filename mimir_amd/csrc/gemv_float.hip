// y = x . W^T for a float32, binary16 or bfloat16 W [N, K] and few rows of
// x: the product a Linear takes when its weight is not block-quantized
// (tensor/quant.go:40-42 -> product, tensor/movement.go:232-243: half operands
// are widened to float32 and multiplied there). Tiny Llama fixtures keep some
// projections in these types; the decode path of a quantized model does not
// come here. One wavefront per row of W.
#include "device_util.h"
#include "kernels.h"

namespace mimir {

template <typename T>
__device__ __forceinline__ float widen(T v);
template <>
__device__ __forceinline__ float widen<float>(float v) { return v; }
struct half_bits { uint16_t v; };
struct bf16_bits { uint16_t v; };
template <>
__device__ __forceinline__ float widen<half_bits>(half_bits v) { return f16_bits_to_f32(v.v); }
template <>
__device__ __forceinline__ float widen<bf16_bits>(bf16_bits v) { return bf16_bits_to_f32(v.v); }

template <typename T>
__global__ __launch_bounds__(256) void gemv_float_kernel(const T* __restrict__ W, const float* __restrict__ x, float* __restrict__ y,
                                                         int N, int K, int64_t x_row_stride) {
    const int lane = threadIdx.x & 63, row = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= N) return;
    const T* w = W + (int64_t)row * K;
    const float* xr = x + (int64_t)blockIdx.y * x_row_stride;
    float acc = 0.f;
    for (int k = lane; k < K; k += 64) acc = fmaf(xr[k], widen<T>(w[k]), acc);
    acc = wave_sum(acc);
    if (lane == 0) y[(int64_t)blockIdx.y * N + row] = acc;
}

hipError_t gemv_float(int dt, const void* W, const float* x, float* y, int64_t M, int64_t N, int64_t K, int64_t x_row_stride,
                      hipStream_t st) {
    if (M == 0 || N == 0) return hipSuccess;
    dim3 grid((unsigned)((N + 3) / 4), (unsigned)M);
    if (dt == kF32)
        hipLaunchKernelGGL(gemv_float_kernel<float>, grid, dim3(256), 0, st, (const float*)W, x, y, (int)N, (int)K, x_row_stride);
    else if (dt == kF16)
        hipLaunchKernelGGL(gemv_float_kernel<half_bits>, grid, dim3(256), 0, st, (const half_bits*)W, x, y, (int)N, (int)K, x_row_stride);
    else
        hipLaunchKernelGGL(gemv_float_kernel<bf16_bits>, grid, dim3(256), 0, st, (const bf16_bits*)W, x, y, (int)N, (int)K, x_row_stride);
    return hipGetLastError();
}

}  // namespace mimir
