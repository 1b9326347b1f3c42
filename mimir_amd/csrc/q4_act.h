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
// two's-complement balanced digit j of X in nibble j, so byte m of Z holds digits
// 2m and 2m+1; dword j of the result wants digit j of the value at position p in
// nibble p (positions 0, 2, 4, 6: lo[0..3]; 1, 3, 5, 7: hi[0..3]). Bytes m of the
// four lo values are gathered into one dword and those of the four hi values into
// another (a 4 x 4 byte transposition: seven v_perm_b32 each), then two
// dwords of digits come out of each such pair by masks and shifts.
__device__ __forceinline__ void fix_digits(const float lo[4], const float hi[4], float inv, uint32_t out[kDigits]) {
    uint32_t ze[4], zo[4];
#pragma unroll
    for (int k = 0; k < 4; k++) {
        // x * inv may round half a unit past kFixMax for the block's largest value: clamp
        int a = (int)__builtin_rintf(lo[k] * inv), b = (int)__builtin_rintf(hi[k] * inv);
        a = a > kFixMax ? kFixMax : a < -kFixMax ? -kFixMax : a;
        b = b > kFixMax ? kFixMax : b < -kFixMax ? -kFixMax : b;
        ze[k] = ((uint32_t)(a + (int)kFixBias)) ^ kFixBias;  // nibble position 2k
        zo[k] = ((uint32_t)(b + (int)kFixBias)) ^ kFixBias;  // nibble position 2k+1
    }
    // v_perm_b32(s0, s1, sel): result byte i is byte sel.byte[i] of the eight bytes {s1 (0..3), s0 (4..7)}
    uint32_t e[3], o[3];
    {
        const uint32_t t01l = __builtin_amdgcn_perm(ze[1], ze[0], 0x05010400u), t01h = __builtin_amdgcn_perm(ze[1], ze[0], 0x07030602u);
        const uint32_t t23l = __builtin_amdgcn_perm(ze[3], ze[2], 0x05010400u), t23h = __builtin_amdgcn_perm(ze[3], ze[2], 0x07030602u);
        e[0] = __builtin_amdgcn_perm(t23l, t01l, 0x05040100u);
        e[1] = __builtin_amdgcn_perm(t23l, t01l, 0x07060302u);
        e[2] = __builtin_amdgcn_perm(t23h, t01h, 0x05040100u);
    }
    {
        const uint32_t t01l = __builtin_amdgcn_perm(zo[1], zo[0], 0x05010400u), t01h = __builtin_amdgcn_perm(zo[1], zo[0], 0x07030602u);
        const uint32_t t23l = __builtin_amdgcn_perm(zo[3], zo[2], 0x05010400u), t23h = __builtin_amdgcn_perm(zo[3], zo[2], 0x07030602u);
        o[0] = __builtin_amdgcn_perm(t23l, t01l, 0x05040100u);
        o[1] = __builtin_amdgcn_perm(t23l, t01l, 0x07060302u);
        o[2] = __builtin_amdgcn_perm(t23h, t01h, 0x05040100u);
    }
#pragma unroll
    for (int m = 0; m < 3; m++) {
        out[2 * m] = (e[m] & 0x0F0F0F0Fu) | ((o[m] << 4) & 0xF0F0F0F0u);
        out[2 * m + 1] = ((e[m] >> 4) & 0x0F0F0F0Fu) | (o[m] & 0xF0F0F0F0u);
    }
}

// Converts item (block b, dword d) of a row, whose eight values are lo
// (elements 4d..4d+3 of the block) and hi (16+4d..16+4d+3), and stores its
// digits and, from the item with d == 0, the block's scale. The four items
// of a block must sit in four consecutive lanes, all active: the block's
// largest magnitude is a quad reduction.
__device__ __forceinline__ void q4_convert_item(float lo[4], float hi[4], u32x4* plane, float* xscale, int nbp, int b, int d) {
    // The largest magnitude as the largest bit pattern without its sign: the order of non-negative floats is that of
    // their bits, and every infinity or NaN lies above every finite value, so one maximum says both how large the block
    // is and whether all of it is finite.
    uint32_t top = 0;
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const uint32_t a0 = __builtin_bit_cast(uint32_t, lo[k]) & 0x7fffffffu, a1 = __builtin_bit_cast(uint32_t, hi[k]) & 0x7fffffffu;
        top = top > a0 ? top : a0;
        top = top > a1 ? top : a1;
    }
    {
        const uint32_t t1 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)top, 0xb1, 0xf, 0xf, true);  // quad_perm [1,0,3,2]
        top = top > t1 ? top : t1;
        const uint32_t t2 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)top, 0x4e, 0xf, 0xf, true);  // quad_perm [2,3,0,1]
        top = top > t2 ? top : t2;
    }
    const float amax = __builtin_bit_cast(float, top);
    float scale, inv;
    if (top >= 0x7f800000u) {  // a NaN or an infinity in the block: its products are NaN
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

// RMSNorm of one row (RMSNorm.Forward, nn/transformer.go:50-61) with the
// conversion behind it, for the first 256 threads of a workgroup: thread t < 256
// holds items t, t + 256, ... (an item is block t / 4, dword t % 4: elements
// 4(t%4).. and 16 + 4(t%4).. of the block), at most kNormItems of them, so the
// row is read once. The stand-alone kernel and the products that take the norm as
// their first phase share these two functions, hence the same sums in the same order.
constexpr int kNormItems = 4;

struct NormRow {
    f32x4 lo[kNormItems], hi[kNormItems];  // x
    f32x4 wl[kNormItems], wh[kNormItems];  // the norm's weights, requested with x so that they are there when the sum is
};

// Loads the thread's items of the row (and of the weights) and returns its share of the sum of squares.
__device__ __forceinline__ float norm_load(NormRow& r, const float* __restrict__ xr, const float* __restrict__ w, int nq, int t0) {
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < kNormItems; i++) {
        int t = t0 + i * 256;
        if (t < nq) {
            int b = t >> 2, q = t & 3;
            __builtin_memcpy(&r.lo[i], xr + 32 * b + 4 * q, 16);
            __builtin_memcpy(&r.hi[i], xr + 32 * b + 16 + 4 * q, 16);
            __builtin_memcpy(&r.wl[i], w + 32 * b + 4 * q, 16);
            __builtin_memcpy(&r.wh[i], w + 32 * b + 16 + 4 * q, 16);
#pragma unroll
            for (int k = 0; k < 4; k++) {
                float a = r.lo[i][k] * r.lo[i][k], c = r.hi[i][k] * r.hi[i][k];
                ss = ss + a;
                ss = ss + c;
            }
        }
    }
    return ss;
}

// part: the four wavefronts' sums. Scales, multiplies by the norm's weights,
// writes y (if not null) and the converted items.
__device__ __forceinline__ void norm_convert(const NormRow& r, const float* part, float* yr, u32x4* plane, float* xscale, int nbp, int nq,
                                             int t0, float inv_d, float eps) {
    float total = (part[0] + part[1]) + (part[2] + part[3]);
    float ms = total * inv_d;
    float scale = 1.0f / __builtin_sqrtf(ms + eps);
#pragma unroll
    for (int i = 0; i < kNormItems; i++) {
        int t = t0 + i * 256;
        if (t < nq) {
            int b = t >> 2, q = t & 3;
            float l4[4], h4[4];
#pragma unroll
            for (int k = 0; k < 4; k++) {
                float a = r.lo[i][k] * scale, c = r.hi[i][k] * scale;
                l4[k] = a * r.wl[i][k];
                h4[k] = c * r.wh[i][k];
            }
            if (yr) {
                f32x4 ol = {l4[0], l4[1], l4[2], l4[3]}, oh = {h4[0], h4[1], h4[2], h4[3]};
                __builtin_memcpy(yr + 32 * b + 4 * q, &ol, 16);
                __builtin_memcpy(yr + 32 * b + 16 + 4 * q, &oh, 16);
            }
            q4_convert_item(l4, h4, plane, xscale, nbp, b, q);
        }
    }
}

}  // namespace mimir
