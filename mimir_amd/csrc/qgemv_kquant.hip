// Decode products by Q4_K and Q6_K weights, y = x . W^T with few rows of x,
// for gfx950, computing what the reference's CPU backend computes
// (backend/cpu/qmatmul.go:141-200): activations rounded to int8 in
// super-blocks of 256 with the int16 sums of each 16 quants (quantizeRow,
// qmatmul.go:208-254), integer dot products weighted by the 6-bit (Q4_K) or
// int8 (Q6_K) sub-block scales, one float32 multiply-add pair per super-block
// (multiply, then add: never fused), Q4_K's mins applied through the sums.
// The integers are exact; only the order in which a row's super-blocks are
// added differs from the CPU's.
//
// One wavefront per row of W, read in place in ggml's layout; the lanes split
// each super-block (4 lanes of 64 weights for Q4_K, 8 lanes of 32 for Q6_K)
// and walk the row 16 or 8 super-blocks at a time. These are the formats real
// Llama files use for a minority of tensors; they are written for
// correctness first.
#include "device_util.h"
#include "kernels.h"

namespace mimir {

#pragma clang fp contract(off)

// One row of x with nsb super-blocks, converted:
//   u32x4 q[nsb][16]     the 256 int8 quants
//   uint32 sums[nsb][8]  sixteen int16 sums of 16 quants, packed in pairs
//   float d[nsb]
size_t kq_act_bytes(int64_t K) {
    int64_t nsb = K / 256;
    return (size_t)((nsb * (256 + 32 + 4) + 15) / 16 * 16);
}

__device__ __forceinline__ int dpp_i32_quad_sum(int v) {
    v += __builtin_amdgcn_update_dpp(0, v, 0xb1, 0xf, 0xf, true);
    v += __builtin_amdgcn_update_dpp(0, v, 0x4e, 0xf, 0xf, true);
    return v;
}
__device__ __forceinline__ int dpp_i32_group8_sum(int v) {
    v = dpp_i32_quad_sum(v);
    v += __builtin_amdgcn_update_dpp(0, v, 0x141, 0xf, 0xf, true);
    return v;
}

// quantizeRow for super-blocks of 256 with sums: one wavefront per
// super-block, lane i taking values 4i..4i+3.
__global__ __launch_bounds__(64) void kq_convert_act_kernel(const float* __restrict__ x, int64_t x_row_stride, int nsb,
                                                            uint8_t* __restrict__ act, int64_t act_row_bytes) {
    const int sb = blockIdx.x, lane = threadIdx.x;
    const float* xr = x + (int64_t)blockIdx.y * x_row_stride + 256 * (int64_t)sb;
    uint8_t* row = act + (int64_t)blockIdx.y * act_row_bytes;
    uint32_t* q = (uint32_t*)row + (int64_t)sb * 64;
    uint16_t* sums = (uint16_t*)(row + (int64_t)nsb * 256) + sb * 16;
    float* dscale = (float*)(row + (int64_t)nsb * 288);
    f32x4 v;
    __builtin_memcpy(&v, xr + 4 * lane, 16);
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
    if (lane == 0) dscale[sb] = d;
}

hipError_t kq_convert_act(const float* x, int64_t M, int64_t K, int64_t x_row_stride, void* act, hipStream_t st) {
    int nsb = (int)(K / 256);
    hipLaunchKernelGGL(kq_convert_act_kernel, dim3((unsigned)nsb, (unsigned)M), dim3(64), 0, st, x, x_row_stride, nsb,
                       (uint8_t*)act, (int64_t)kq_act_bytes(K));
    return hipGetLastError();
}

// backend/cpu/quant.go:129-134
__device__ __forceinline__ void scale_min_k4(int j, const uint8_t* s, int& sc, int& m) {
    if (j < 4) {
        sc = s[j] & 63;
        m = s[j + 4] & 63;
    } else {
        sc = (s[j + 4] & 0xf) | ((s[j - 4] >> 6) << 4);
        m = (s[j + 4] >> 4) | ((s[j] >> 6) << 4);
    }
}

__device__ __forceinline__ int i16_at(const uint16_t* p, int i) { return (int)(int16_t)p[i]; }

// qdotQ4KGo (backend/cpu/qmatmul.go:148-172): lane (sb, j) takes the 64
// weights of nibble group j of super-block sb.
__global__ __launch_bounds__(256) void qgemv_q4k_kernel(const uint8_t* __restrict__ W, const uint8_t* __restrict__ act,
                                                        float* __restrict__ y, int N, int nsb, int64_t act_row_bytes) {
    const int lane = threadIdx.x & 63, row = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= N) return;
    const uint8_t* arow = act + (int64_t)blockIdx.y * act_row_bytes;
    const uint32_t* xq = (const uint32_t*)arow;
    const uint16_t* xsums = (const uint16_t*)(arow + (int64_t)nsb * 256);
    const float* xd = (const float*)(arow + (int64_t)nsb * 288);
    const uint8_t* wrow = W + (int64_t)row * nsb * 144;
    float acc = 0.f, accm = 0.f;
    const int j = lane & 3;
    for (int sb0 = 0; sb0 < nsb; sb0 += 16) {
        int sb = sb0 + (lane >> 2);
        const bool live = sb < nsb;
        sb = live ? sb : nsb - 1;
        const uint8_t* wb = wrow + (int64_t)sb * 144;
        uint8_t scales[12];
#pragma unroll
        for (int k = 0; k < 3; k++) {
            uint32_t t = load_u32_unaligned(wb + 4 + 4 * k);
            __builtin_memcpy(scales + 4 * k, &t, 4);
        }
        int lo = 0, hi = 0;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            uint32_t w = load_u32_unaligned(wb + 16 + 32 * j + 4 * i);
            lo = __builtin_amdgcn_sdot4((int)(w & 0x0F0F0F0Fu), (int)xq[sb * 64 + 16 * j + i], lo, false);
            hi = __builtin_amdgcn_sdot4((int)((w >> 4) & 0x0F0F0F0Fu), (int)xq[sb * 64 + 16 * j + 8 + i], hi, false);
        }
        int sc0, m0, sc1, m1;
        scale_min_k4(2 * j, scales, sc0, m0);
        scale_min_k4(2 * j + 1, scales, sc1, m1);
        const uint16_t* s = xsums + sb * 16 + 4 * j;
        int sumi = sc0 * lo + sc1 * hi;
        int summ = m0 * (i16_at(s, 0) + i16_at(s, 1)) + m1 * (i16_at(s, 2) + i16_at(s, 3));
        sumi = dpp_i32_quad_sum(live ? sumi : 0);
        summ = dpp_i32_quad_sum(live ? summ : 0);
        if (j == 0 && live) {
            float xdv = xd[sb];
            float dd = f16_bits_to_f32(load_u16(wb)) * xdv, dm = f16_bits_to_f32(load_u16(wb + 2)) * xdv;
            float t = dd * (float)sumi;
            acc = acc + t;
            float u = dm * (float)summ;
            accm = accm + u;
        }
    }
    acc = wave_sum(acc);
    accm = wave_sum(accm);
    if (lane == 0) y[(int64_t)blockIdx.y * N + row] = acc - accm;
}

// qdotQ6KGo (backend/cpu/qmatmul.go:180-200): lane (sb, n, k) takes the 32
// weights of quarter k of half n of super-block sb, groups 8n+2k and 8n+2k+1.
__global__ __launch_bounds__(256) void qgemv_q6k_kernel(const uint8_t* __restrict__ W, const uint8_t* __restrict__ act,
                                                        float* __restrict__ y, int N, int nsb, int64_t act_row_bytes) {
    const int lane = threadIdx.x & 63, row = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= N) return;
    const uint8_t* arow = act + (int64_t)blockIdx.y * act_row_bytes;
    const uint32_t* xq = (const uint32_t*)arow;
    const uint16_t* xsums = (const uint16_t*)(arow + (int64_t)nsb * 256);
    const float* xd = (const float*)(arow + (int64_t)nsb * 288);
    const uint8_t* wrow = W + (int64_t)row * nsb * 210;
    float acc = 0.f;
    const int part = lane & 7, n = part >> 2, k = part & 3;
    for (int sb0 = 0; sb0 < nsb; sb0 += 8) {
        int sb = sb0 + (lane >> 3);
        const bool live = sb < nsb;
        sb = live ? sb : nsb - 1;
        const uint8_t* wb = wrow + (int64_t)sb * 210;
        const uint8_t* ql = wb + 64 * n + 32 * (k & 1);
        const uint8_t* qh = wb + 128 + 32 * n;
        int s[2] = {0, 0};
#pragma unroll
        for (int i = 0; i < 8; i++) {
            uint32_t lw = load_u16(ql + 4 * i) | ((uint32_t)load_u16(ql + 4 * i + 2) << 16);
            uint32_t hw = load_u16(qh + 4 * i) | ((uint32_t)load_u16(qh + 4 * i + 2) << 16);
            if (k >= 2) lw >>= 4;
            uint32_t v = (lw & 0x0F0F0F0Fu) | (((hw >> (2 * k)) & 0x03030303u) << 4);  // 0..63 per byte
            s[i >> 2] = __builtin_amdgcn_sdot4((int)v, (int)xq[sb * 64 + 32 * n + 8 * k + i], s[i >> 2], false);
        }
        int g0 = 8 * n + 2 * k;
        int sc0 = (int)(int8_t)wb[192 + g0], sc1 = (int)(int8_t)wb[192 + g0 + 1];
        const uint16_t* xs = xsums + sb * 16 + g0;
        int sumi = sc0 * s[0] - 32 * sc0 * i16_at(xs, 0) + sc1 * s[1] - 32 * sc1 * i16_at(xs, 1);
        sumi = dpp_i32_group8_sum(live ? sumi : 0);
        if (part == 0 && live) {
            float dd = f16_bits_to_f32(load_u16(wb + 208)) * xd[sb];
            float t = dd * (float)sumi;
            acc = acc + t;
        }
    }
    acc = wave_sum(acc);
    if (lane == 0) y[(int64_t)blockIdx.y * N + row] = acc;
}

hipError_t qgemv_kquant_act(int dt, const QGemvArgs& a, hipStream_t st) {
    int nsb = (int)(a.K / 256);
    const int waves = 4;
    dim3 grid((unsigned)((a.N + waves - 1) / waves), (unsigned)a.M);
    if (dt == kQ4_K)
        hipLaunchKernelGGL(qgemv_q4k_kernel, grid, dim3(64 * waves), 0, st, (const uint8_t*)a.W, (const uint8_t*)a.act, a.y,
                           (int)a.N, nsb, (int64_t)kq_act_bytes(a.K));
    else
        hipLaunchKernelGGL(qgemv_q6k_kernel, grid, dim3(64 * waves), 0, st, (const uint8_t*)a.W, (const uint8_t*)a.act, a.y,
                           (int)a.N, nsb, (int64_t)kq_act_bytes(a.K));
    return hipGetLastError();
}

}  // namespace mimir
