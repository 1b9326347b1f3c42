// Shared by the two forms of the prompt-sized Q4_0 product that multiply in binary16 (qgemm_q4_0.hip,
// qgemm_f16_panel.hip): bringing a row of bfloat16 activations to binary16.
#pragma once
#include "device_util.h"

namespace mimir {

// A row of bfloat16 to binary16, scaled by the power of two that brings the row's largest finite magnitude into
// [2^14, 2^15) (clamped to what float32 can hold both ways); scale_back[m] undoes it. One workgroup of 256 threads a row (all of
// them call this with the same m); K in pieces of eight elements.
__device__ __forceinline__ void bf16_row_to_f16_scaled(const uint16_t* __restrict__ x, uint16_t* __restrict__ y, float* __restrict__ scale_back,
                                                       int64_t K, int64_t x_row_stride, int64_t m) {
    __shared__ uint32_t part[4];
    const uint16_t* row = x + m * x_row_stride;
    const int pieces = (int)(K >> 3);
    uint32_t top = 0;  // the largest finite magnitude's bits (bfloat16 magnitudes order as integers)
    for (int p = threadIdx.x; p < pieces; p += 256) {
        u32x4 v;
        __builtin_memcpy(&v, __builtin_assume_aligned(row + 8 * (int64_t)p, 16), 16);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t a = v[i] & 0x7fffu, b = (v[i] >> 16) & 0x7fffu;
            if (a < 0x7f80u && a > top) top = a;
            if (b < 0x7f80u && b > top) top = b;
        }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const uint32_t other = (uint32_t)__shfl_xor((int)top, o, 64);
        top = other > top ? other : top;
    }
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = top;
    __syncthreads();
    top = part[0];
#pragma unroll
    for (int i = 1; i < 4; i++) top = part[i] > top ? part[i] : top;
    int e = 0;
    if (top != 0) {
        const int ex = (int)(top >> 7) - 127;  // floor(log2) of a normal magnitude; subnormals count as 2^-117
        e = 14 - ex;
        e = e > 126 ? 126 : e < -126 ? -126 : e;
    }
    const float up = __uint_as_float((uint32_t)(e + 127) << 23);
    if (threadIdx.x == 0) scale_back[m] = __uint_as_float((uint32_t)(127 - e) << 23);
    uint16_t* out = y + m * K;
    for (int p = threadIdx.x; p < pieces; p += 256) {
        u32x4 v, r;
        __builtin_memcpy(&v, __builtin_assume_aligned(row + 8 * (int64_t)p, 16), 16);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const f16x2 h = {(_Float16)(__uint_as_float(v[i] << 16) * up), (_Float16)(__uint_as_float(v[i] & 0xffff0000u) * up)};
            r[i] = __builtin_bit_cast(uint32_t, h);
        }
        *(u32x4*)(out + 8 * (int64_t)p) = r;
    }
}

}  // namespace mimir
