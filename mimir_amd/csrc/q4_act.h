// The fixed-point form of activations that the Q4_0 decode kernel reads, and
// the conversion of one item of it, shared by the kernels that produce it
// (the stand-alone conversion, RMSNorm and SwiGLU with a fused conversion).
//
// One row of x with nb blocks, converted (nbp = nb | 1; q4_0_act_bytes(K) bytes):
//   u32x4 plane[6][nbp]  digit plane j of block b at plane[j * nbp + b]: dword i
//                        holds, nibble for nibble as dword i of the block's
//                        weights does (byte k: low nibble element 4i+k, high
//                        nibble element 16+4i+k), digit j of those elements
//   float scale[nb]      x[e] ~ scale * sum_j 16^j digit_j[e]
#pragma once

#include "device_util.h"

namespace mimir {

constexpr int kDigits = 6;
constexpr int kFixMax = 7829367;         // 7 * (16^6 - 1) / 15: the largest balanced 6-digit number
constexpr uint32_t kFixBias = 0x888888;  // 8 in every digit

__host__ __device__ inline size_t q4_0_act_row_bytes(int64_t K) {
    int64_t nb = K / 32;
    return (size_t)(((nb | 1) * kDigits * 16 + nb * 4 + 15) / 16 * 16);
}

// The eight values a thread holds (elements 4i..4i+3 and 16+4i..16+4i+3 of a
// block) to kDigits dwords of digits. Z = (X + kFixBias) ^ kFixBias has the
// two's-complement balanced digit j of X in nibble j.
__device__ __forceinline__ void fix_digits(const float lo[4], const float hi[4], float inv, uint32_t out[kDigits]) {
    uint32_t z[8];
#pragma unroll
    for (int k = 0; k < 4; k++) {
        // x * inv may round half a unit past kFixMax for the block's largest value: clamp
        int a = (int)__builtin_rintf(lo[k] * inv), b = (int)__builtin_rintf(hi[k] * inv);
        a = a > kFixMax ? kFixMax : a < -kFixMax ? -kFixMax : a;
        b = b > kFixMax ? kFixMax : b < -kFixMax ? -kFixMax : b;
        z[2 * k] = ((uint32_t)(a + (int)kFixBias)) ^ kFixBias;      // nibble position 2k
        z[2 * k + 1] = ((uint32_t)(b + (int)kFixBias)) ^ kFixBias;  // nibble position 2k+1
    }
#pragma unroll
    for (int j = 0; j < kDigits; j++) {
        uint32_t w = 0;
#pragma unroll
        for (int p = 0; p < 8; p++) w |= ((z[p] >> (4 * j)) & 15u) << (4 * p);
        out[j] = w;
    }
}

// Converts item (block b, dword d) of a row, whose eight values are lo
// (elements 4d..4d+3 of the block) and hi (16+4d..16+4d+3), and stores its
// digits and, from the item with d == 0, the block's scale. The four items
// of a block must sit in four consecutive lanes, all active: the block's
// largest magnitude is a quad reduction.
__device__ __forceinline__ void q4_convert_item(float lo[4], float hi[4], u32x4* plane, float* xscale, int nbp, int b, int d) {
    float amax = 0.f;
    bool finite = true;
#pragma unroll
    for (int k = 0; k < 4; k++) {
        float a0 = __builtin_fabsf(lo[k]), a1 = __builtin_fabsf(hi[k]);
        finite = finite && a0 < __builtin_inff() && a1 < __builtin_inff();  // false for NaN too
        amax = fmaxf(amax, fmaxf(a0, a1));
    }
    amax = fmaxf(amax, dpp_f32<0xb1>(amax));
    amax = fmaxf(amax, dpp_f32<0x4e>(amax));
    float bad = finite ? 0.f : 1.f;
    bad = fmaxf(bad, dpp_f32<0xb1>(bad));
    bad = fmaxf(bad, dpp_f32<0x4e>(bad));
    float scale, inv;
    if (bad != 0.f) {  // a NaN or an infinity in the block: its products are NaN
        scale = __builtin_nanf("");
        inv = 0.f;
#pragma unroll
        for (int k = 0; k < 4; k++) lo[k] = hi[k] = 0.f;
    } else if (amax < 0x1p-100f) {  // nothing to represent (and 1/amax would overflow)
        scale = 0.f;
        inv = 0.f;
    } else {
        scale = amax / (float)kFixMax;
        inv = (float)kFixMax / amax;
    }
    uint32_t dig[kDigits];
    fix_digits(lo, hi, inv, dig);
#pragma unroll
    for (int j = 0; j < kDigits; j++) ((uint32_t*)(plane + j * nbp + b))[d] = dig[j];
    if (d == 0) xscale[b] = scale;
}

}  // namespace mimir
