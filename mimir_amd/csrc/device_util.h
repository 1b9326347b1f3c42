// Device-side helpers shared by the gfx950 kernels: 64-lane wavefront
// reductions over DPP, bit-level half conversions that round exactly as the
// reference's CPU backend does (backend/cpu/half.go:37-102), and unaligned
// loads of ggml blocks.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mimir {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;

// ---- DPP ------------------------------------------------------------------
// update_dpp(old, src, ctrl, row_mask, bank_mask, bound_ctrl): lanes whose row
// is masked off keep `old`; with bound_ctrl a read past the row's edge gives 0.
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ float dpp_f32(float v) {
    int r = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xf, true);
    return __builtin_bit_cast(float, r);
}

// A 4 x 4 transposition within every quad of lanes: lane j's register k and lane k's register j change places.
__device__ __forceinline__ void quad_transpose(float v[4], int lane) {
    const bool odd = lane & 1, upper = lane & 2;
    float got = dpp_f32<0xb1>(odd ? v[0] : v[1]);  // quad_perm [1,0,3,2]: the neighbour in the pair
    if (odd) v[0] = got; else v[1] = got;
    got = dpp_f32<0xb1>(odd ? v[2] : v[3]);
    if (odd) v[2] = got; else v[3] = got;
    got = dpp_f32<0x4e>(upper ? v[0] : v[2]);      // quad_perm [2,3,0,1]: the other pair
    if (upper) v[0] = got; else v[2] = got;
    got = dpp_f32<0x4e>(upper ? v[1] : v[3]);
    if (upper) v[1] = got; else v[3] = got;
}

// Sum of v over the 64 lanes, the same in every call order: an inclusive scan
// of each row of 16 (row_shr 1, 2, 4, 8), then row_bcast:15 and row_bcast:31
// carry the row totals up; lane 63 holds the total, returned to every lane.
__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_f32<0x111>(v);
    v += dpp_f32<0x112>(v);
    v += dpp_f32<0x114>(v);
    v += dpp_f32<0x118>(v);
    v += dpp_f32<0x142, 0xa>(v);
    v += dpp_f32<0x143, 0xc>(v);
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

__device__ __forceinline__ float wave_max(float v) {
    // Butterfly over DPP where it reaches (within rows of 16), then two
    // cross-row steps through the LDS crossbar.
    v = fmaxf(v, dpp_f32<0xb1>(v));   // quad_perm [1,0,3,2]
    v = fmaxf(v, dpp_f32<0x4e>(v));   // quad_perm [2,3,0,1]
    v = fmaxf(v, dpp_f32<0x141>(v));  // row_half_mirror
    v = fmaxf(v, dpp_f32<0x140>(v));  // row_mirror
    v = fmaxf(v, __shfl_xor(v, 16));
    v = fmaxf(v, __shfl_xor(v, 32));
    return v;
}

// Sum and max over each aligned group of 8 lanes, returned to all 8.
__device__ __forceinline__ float group8_sum(float v) {
    v += dpp_f32<0xb1>(v);
    v += dpp_f32<0x4e>(v);
    v += dpp_f32<0x141>(v);
    return v;
}
__device__ __forceinline__ float group8_max(float v) {
    v = fmaxf(v, dpp_f32<0xb1>(v));
    v = fmaxf(v, dpp_f32<0x4e>(v));
    v = fmaxf(v, dpp_f32<0x141>(v));
    return v;
}

// A row's sum of squares as a workgroup of 256 threads adds it: thread t takes x[t], x[t + 256], ...
// in that order (the wavefronts' and the workgroup's sums follow at the caller). The loads go out in
// batches of sixteen (a row of 4096 in one): a loop of unknown length would wait for each before requesting the next.
__device__ __forceinline__ float strided_sum_squares(const float* __restrict__ xr, int d, int t) {
    float ss = 0.f;
    constexpr int kBatch = 16;
    for (int i0 = t; i0 < d; i0 += kBatch * 256) {
        float v[kBatch];
#pragma unroll
        for (int u = 0; u < kBatch; u++) {
            const int i = i0 + 256 * u;
            v[u] = i < d ? xr[i] : 0.f;  // + 0 changes no sum
        }
#pragma unroll
        for (int u = 0; u < kBatch; u++) {
            float sq = v[u] * v[u];
            ss = ss + sq;
        }
    }
    return ss;
}

// ---- half conversions -----------------------------------------------------
// The hardware's cvt instructions round to nearest even and keep subnormals
// (the f16 denormal mode is on), which is what half.go computes for every
// finite input; NaNs are patched to half.go's payload rule.
__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) {
    return (float)__builtin_bit_cast(_Float16, h);
}

__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) {
    uint32_t b = __builtin_bit_cast(uint32_t, f);
    if ((b & 0x7fffffffu) > 0x7f800000u)  // half.go:84-86
        return (uint16_t)((b >> 16) & 0x8000u) | 0x7e00 | (uint16_t)((b >> 13) & 0x1ff);
    return __builtin_bit_cast(uint16_t, (_Float16)f);
}

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t h) {
    return __builtin_bit_cast(float, (uint32_t)h << 16);
}

__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {  // half.go:42-51
    uint32_t b = __builtin_bit_cast(uint32_t, f);
    if ((b & 0x7fffffffu) > 0x7f800000u) return (uint16_t)(b >> 16) | 0x0040;
    b += 0x7fffu + ((b >> 16) & 1u);
    return (uint16_t)(b >> 16);
}

// ---- loads ----------------------------------------------------------------
// ggml blocks are 2-byte aligned. gfx950 serves unaligned dword..dwordx4
// global loads in hardware, so these compile to single wide loads.
__device__ __forceinline__ u32x4 load_u32x4_unaligned(const uint8_t* p) {
    u32x4 v;
    __builtin_memcpy(&v, p, 16);
    return v;
}
__device__ __forceinline__ uint32_t load_u32_unaligned(const uint8_t* p) {
    uint32_t v;
    __builtin_memcpy(&v, p, 4);
    return v;
}
__device__ __forceinline__ uint16_t load_u16(const uint8_t* p) {
    uint16_t v;
    __builtin_memcpy(&v, p, 2);
    return v;
}

__device__ __forceinline__ f16x2 as_f16x2(uint32_t v) { return __builtin_bit_cast(f16x2, v); }

}  // namespace mimir
