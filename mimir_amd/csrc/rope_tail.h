// The rotation and cache writes of a decoding step as the tail of the product that computes q, k and v
// (rope_kv's arithmetic): shared by the kernels whose wavefronts own pairs of output rows.
#pragma once

#include "device_util.h"
#include "kernels.h"

namespace mimir {

// Whether rows (row, row + 1) are a pair that turns, and if so its cosine and sine at position pos: requested apart
// from the store below by kernels that want the two loads under way before their weights'.
__device__ __forceinline__ bool q4_rope_coeffs(const Q4RopeTail& t, int pos, int row, float* c, float* sn) {
    const int head = row / t.dim, f = row - head * t.dim;
    *c = 1.f;
    *sn = 0.f;
    if (head >= t.H + t.HK || f >= t.rope_dim) return false;
    const int half = t.rope_dim >> 1, i = f >> 1;
    *c = t.cosv[(int64_t)pos * half + i];
    *sn = t.sinv[(int64_t)pos * half + i];
    return true;
}

// Rows (row, row + 1) of sequence m: features (f, f + 1) of one head, f even; turns says whether they rotate, by (c, sn).
__device__ __forceinline__ void q4_rope_store_with(const Q4RopeTail& t, int pos, int m, int row, float a, float b, bool turns, float c, float sn, float* yr) {
    const int head = row / t.dim, f = row - head * t.dim;
    float va = a, vb = b;
    if (turns) {
        const float ac = a * c, bs = b * sn, as = a * sn, bc = b * c;  // four products, then one subtraction and one addition
        va = ac - bs;
        vb = as + bc;
    }
    if (head < t.H) {
        yr[row] = va;
        yr[row + 1] = vb;
        return;
    }
    const bool is_k = head < t.H + t.HK;
    const int kh = is_k ? head - t.H : head - t.H - t.HK;
    void* cache = is_k ? t.kcache : t.vcache;
    const int64_t at = (((int64_t)m * t.HK + kh) * t.cap + pos) * t.dim + f;
    if (t.cache_dt == kF32) {
        ((float*)cache)[at] = va;
        ((float*)cache)[at + 1] = vb;
    } else {
        ((uint16_t*)cache)[at] = f32_to_f16_bits(va);
        ((uint16_t*)cache)[at + 1] = f32_to_f16_bits(vb);
    }
}

__device__ __forceinline__ void q4_rope_store(const Q4RopeTail& t, int pos, int m, int row, float a, float b, float* yr) {
    float c, sn;
    const bool turns = q4_rope_coeffs(t, pos, row, &c, &sn);
    q4_rope_store_with(t, pos, m, row, a, b, turns, c, sn, yr);
}

}  // namespace mimir
