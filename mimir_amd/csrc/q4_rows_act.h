// The form of up to eight rows of activations that the Q4_0 product for a few
// rows of x reads (qgemv_q4_0_rows.hip), and the conversion of one item of it,
// shared by the kernels that produce it (the stand-alone conversion, RMSNorm,
// SwiGLU and attention with a fused conversion). The integers and scales are
// those of the one-row form (q4_act.h): the block's largest magnitude maps to
// kFixMax, here cut into three balanced base-256 digits.
//
// Eight rows of x with nb blocks each, together (q4_0_rows_act_bytes(K) bytes):
//   frag[nb][64][16]  block b as the operand of v_mfma_i32_32x32x32_i8: lane 32 h + 8 d + m holds
//                     digit d of elements 16 h .. 16 h + 15 of row m's block (d = 3: unused)
//   tail[nb][16]      float scale[8] of the block in the eight rows, then int32 8 * (sum of its integers)
#pragma once

#include "q4_act.h"

namespace mimir {

constexpr int kRowsFragBytes = 1024;
constexpr int kRowsTailBytes = 64;

__host__ __device__ inline size_t q4_0_rows_act_size(int64_t K) { return (size_t)(K / 32) * (kRowsFragBytes + kRowsTailBytes); }

// Integer a (|a| <= kFixMax) as three balanced base-256 digits, each into byte k of its dword.
__device__ __forceinline__ void rows_digits(int a, int k, uint32_t d[3]) {
    const int d0 = (int)(int8_t)a;  // balanced digits: each in -128..127
    const int a1 = (a - d0) >> 8;
    const int d1 = (int)(int8_t)a1;
    const int d2 = (a1 - d1) >> 8;
    d[0] |= (uint32_t)(d0 & 0xff) << (8 * k);
    d[1] |= (uint32_t)(d1 & 0xff) << (8 * k);
    d[2] |= (uint32_t)(d2 & 0xff) << (8 * k);
}

// Converts item (block b, dword q) of row m, whose eight values are lo (elements 4q..4q+3 of the
// block) and hi (16+4q..16+4q+3), as q4_convert_item does for the one-row form: the four items of a
// block must sit in four consecutive lanes, all active.
__device__ __forceinline__ void rows_convert_item(float lo[4], float hi[4], uint8_t* act, int nb, int m, int b, int q) {
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
    uint32_t dl[3] = {0, 0, 0}, dh[3] = {0, 0, 0};
    int sum = 0;
#pragma unroll
    for (int k = 0; k < 4; k++) {
        int a = (int)__builtin_rintf(lo[k] * inv), c = (int)__builtin_rintf(hi[k] * inv);
        a = a > kFixMax ? kFixMax : a < -kFixMax ? -kFixMax : a;
        c = c > kFixMax ? kFixMax : c < -kFixMax ? -kFixMax : c;
        sum += a + c;
        rows_digits(a, k, dl);
        rows_digits(c, k, dh);
    }
    sum += __builtin_amdgcn_update_dpp(0, sum, 0xb1, 0xf, 0xf, true);  // quad_perm [1,0,3,2]
    sum += __builtin_amdgcn_update_dpp(0, sum, 0x4e, 0xf, 0xf, true);  // quad_perm [2,3,0,1]; below 2^28
    uint32_t* frag = (uint32_t*)(act + (int64_t)b * kRowsFragBytes) + q;
#pragma unroll
    for (int j = 0; j < 3; j++) {
        frag[4 * (8 * j + m)] = dl[j];
        frag[4 * (32 + 8 * j + m)] = dh[j];
    }
    if (q == 0) {
        uint8_t* tail = act + (int64_t)nb * kRowsFragBytes + (int64_t)b * kRowsTailBytes;
        ((float*)tail)[m] = scale;
        ((int32_t*)tail)[8 + m] = 8 * sum;
    }
}

}  // namespace mimir
