// The int8 form of a row of x for the Q4_K / Q6_K products (quantizeRow with the sums of 16,
// backend/cpu/qmatmul.go: per super-block of 256 a float32 scale amax / 127, quants round(x * 127 / amax)
// to even, sixteen int16 sums), as device code shared by the kernels that leave their results in it.
// A converted row with nsb super-blocks (kq_act_bytes(K) bytes):
//   u32x4 q[nsb][16]     the 256 int8 quants
//   uint32 sums[nsb][8]  sixteen int16 sums of 16 quants, packed in pairs
//   float d[nsb]
#pragma once
#include "device_util.h"

namespace mimir {

__device__ __forceinline__ int dpp_i32_quad_sum(int v) {
    v += __builtin_amdgcn_update_dpp(0, v, 0xb1, 0xf, 0xf, true);
    v += __builtin_amdgcn_update_dpp(0, v, 0x4e, 0xf, 0xf, true);
    return v;
}

// quantizeRow for one super-block of 256 with its sums: one wavefront, lane i holding values 4i..4i+3.
// q: the super-block's 64 dwords of quants; sums: its 16 sums; d: its scale.
__device__ __forceinline__ void kq_convert_superblock_to(const f32x4 v, int lane, uint32_t* q, uint16_t* sums, float* d_out) {
    float amax = 0.f;
    bool finite = true;
#pragma unroll
    for (int k = 0; k < 4; k++) {
        float a = __builtin_fabsf(v[k]);
        finite = finite && a < __builtin_inff();
        if (a > amax) amax = a;
    }
    amax = wave_max(amax);
    float bad = wave_max(finite ? 0.f : 1.f);
    float d = 0.f;
    uint32_t packed = 0;
    int local = 0;
    if (bad != 0.f) {
        d = __builtin_nanf("");
    } else if (amax != 0.f) {
        d = amax / 127.0f;
        float id = 127.0f / amax;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            int r = (int)__builtin_rintf(v[k] * id);
            r = r > 127 ? 127 : r < -127 ? -127 : r;
            packed |= (uint32_t)(r & 0xff) << (8 * k);
            local += r;
        }
    }
    q[lane] = packed;
    int s16 = dpp_i32_quad_sum(local);  // 16 quants = 4 consecutive lanes
    if ((lane & 3) == 0) sums[lane >> 2] = (uint16_t)(int16_t)s16;
    if (lane == 0) *d_out = d;
}

// Into a converted row in global memory (kq_act_bytes' layout).
__device__ __forceinline__ void kq_convert_superblock(const f32x4 v, int sb, int lane, int nsb, uint8_t* __restrict__ row) {
    kq_convert_superblock_to(v, lane, (uint32_t*)row + (int64_t)sb * 64, (uint16_t*)(row + (int64_t)nsb * 256) + sb * 16,
                             (float*)(row + (int64_t)nsb * 288) + sb);
}

}  // namespace mimir
