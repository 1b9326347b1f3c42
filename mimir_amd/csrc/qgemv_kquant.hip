// Decode products by Q4_K and Q6_K weights, y = x . W^T with few rows of x,
// for gfx950, computing what the reference's CPU backend computes
// (backend/cpu/qmatmul.go:141-200): activations rounded to int8 in
// super-blocks of 256 with the int16 sums of each 16 quants (quantizeRow,
// qmatmul.go:208-254), integer dot products weighted by the 6-bit (Q4_K) or
// int8 (Q6_K) sub-block scales, one float32 multiply-add pair per super-block
// (multiply, then add: never fused), Q4_K's mins applied through the sums.
// The integers are exact and a row's super-blocks are added in the CPU's
// order: the results are the CPU's bit for bit.
//
// W is read in place in ggml's layout. The kernels that serve ordinary shapes
// stage the converted row of x in LDS once per workgroup; a wavefront owns R
// rows of W and walks them 16 (Q4_K) or 8 (Q6_K) super-blocks at a time, a
// lane taking 16 bytes of nibbles per load so that a super-block is fetched
// with a few 128-bit loads per lane (the texture addresser issues one
// wavefront load in the same time whatever its width, and it, not HBM, bounds
// a kernel built from dword loads). The loads of the next pass are requested
// before the current pass is multiplied. A second pair of kernels, one
// wavefront per row with x read from global memory, serves rows of x too long
// for the LDS.
#include "device_util.h"
#include "kernels.h"
#include "kq_act.h"
#include "rope_tail.h"

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

__device__ __forceinline__ int dpp_i32_group8_sum(int v) {
    v = dpp_i32_quad_sum(v);
    v += __builtin_amdgcn_update_dpp(0, v, 0x141, 0xf, 0xf, true);
    return v;
}

// Every STRIDE-th lane holds the term of one super-block, in the order of the
// super-blocks; they are added to acc one after the other, the order in which the
// CPU adds its super-blocks (qmatmul.go:148-200), so the float32 sum is the CPU's
// bit for bit. A lane without a term holds +0, which changes no sum that began at +0.
template <int STRIDE>
__device__ __forceinline__ float add_in_order(float acc, float term) {
#pragma unroll
    for (int q = 0; q < 64 / STRIDE; q++)
        acc = acc + __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, term), q * STRIDE));
    return acc;
}

// One wavefront per super-block.
template <bool BF16>  // x float32, or bfloat16 (widened exactly, as the cast in front of the product does: tensor/quant.go:45-48)
__global__ __launch_bounds__(64) void kq_convert_act_kernel(const void* __restrict__ xv, int64_t x_row_stride, int nsb,
                                                            uint8_t* __restrict__ act, int64_t act_row_bytes) {
    const int sb = blockIdx.x, lane = threadIdx.x;
    const int64_t at = (int64_t)blockIdx.y * x_row_stride + 256 * (int64_t)sb + 4 * lane;
    f32x4 v;
    if (BF16) {
        u32x2 h;
        __builtin_memcpy(&h, (const uint16_t*)xv + at, 8);
        v[0] = __builtin_bit_cast(float, h[0] << 16);
        v[1] = __builtin_bit_cast(float, h[0] & 0xffff0000u);
        v[2] = __builtin_bit_cast(float, h[1] << 16);
        v[3] = __builtin_bit_cast(float, h[1] & 0xffff0000u);
    } else {
        __builtin_memcpy(&v, (const float*)xv + at, 16);
    }
    kq_convert_superblock(v, sb, lane, nsb, act + (int64_t)blockIdx.y * act_row_bytes);
}

// RMSNorm (rmsnorm_kernel's arithmetic, operation for operation: nn/transformer.go:50-61) and the
// conversion of its result in one launch: a workgroup of four wavefronts sums the row's squares as
// rmsnorm_kernel does (each workgroup of a row for itself), then each wavefront converts one super-block.
__global__ __launch_bounds__(256) void rmsnorm_kq_act_kernel(const float* __restrict__ x, const float* __restrict__ w, int d, float inv_d,
                                                             float eps, uint8_t* __restrict__ act, int64_t act_row_bytes) {
    __shared__ float part[4];
    const float* xr = x + (int64_t)blockIdx.y * d;
    const int lane = threadIdx.x & 63, nsb = d >> 8;
    const int sb = blockIdx.x * 4 + (threadIdx.x >> 6);
    f32x4 v = {0.f, 0.f, 0.f, 0.f}, wv = {0.f, 0.f, 0.f, 0.f};
    if (sb < nsb) {  // requested with the loads of the sum
        __builtin_memcpy(&v, xr + 256 * sb + 4 * lane, 16);
        __builtin_memcpy(&wv, w + 256 * sb + 4 * lane, 16);
    }
    float ss = wave_sum(strided_sum_squares(xr, d, threadIdx.x));
    if (lane == 0) part[threadIdx.x >> 6] = ss;
    __syncthreads();
    float total = (part[0] + part[1]) + (part[2] + part[3]);
    float ms = total * inv_d;
    float scale = 1.0f / __builtin_sqrtf(ms + eps);
    if (sb < nsb) {
#pragma unroll
        for (int k = 0; k < 4; k++) {
            float t = v[k] * scale;
            v[k] = t * wv[k];
        }
        kq_convert_superblock(v, sb, lane, nsb, act + (int64_t)blockIdx.y * act_row_bytes);
    }
}

hipError_t rmsnorm_kq_act(const float* x, const float* w, void* act, int64_t rows, int64_t d, double eps, hipStream_t st) {
    if (rows == 0) return hipSuccess;
    hipLaunchKernelGGL(rmsnorm_kq_act_kernel, dim3((unsigned)((d / 256 + 3) / 4), (unsigned)rows), dim3(256), 0, st, x, w, (int)d,
                       (float)(1.0 / (double)d), (float)eps, (uint8_t*)act, (int64_t)kq_act_bytes(d));
    return hipGetLastError();
}

// SiLU(g) * u (swiglu_kernel's arithmetic: llm/model.go:446-448) and the conversion of the result in one
// launch, one wavefront per super-block; rows of g and u are `stride` floats apart.
__global__ __launch_bounds__(64) void swiglu_kq_act_kernel(const float* __restrict__ g, const float* __restrict__ u, int64_t stride, int nsb,
                                                           uint8_t* __restrict__ act, int64_t act_row_bytes) {
    const int sb = blockIdx.x, lane = threadIdx.x;
    const int64_t at = (int64_t)blockIdx.y * stride + 256 * (int64_t)sb + 4 * lane;
    const float nl2e = (float)(-1.4426950408889634);
    f32x4 gv, uv, v;
    __builtin_memcpy(&gv, g + at, 16);
    __builtin_memcpy(&uv, u + at, 16);
#pragma unroll
    for (int k = 0; k < 4; k++) {
        float e = __builtin_exp2f(gv[k] * nl2e);
        float sg = 1.0f / (1.0f + e);
        float a = gv[k] * sg;
        v[k] = a * uv[k];
    }
    kq_convert_superblock(v, sb, lane, nsb, act + (int64_t)blockIdx.y * act_row_bytes);
}

hipError_t swiglu_kq_act(const float* g, const float* u, void* act, int64_t rows, int64_t n, int64_t stride, hipStream_t st) {
    if (rows == 0) return hipSuccess;
    int nsb = (int)(n / 256);
    hipLaunchKernelGGL(swiglu_kq_act_kernel, dim3((unsigned)nsb, (unsigned)rows), dim3(64), 0, st, g, u, stride, nsb, (uint8_t*)act,
                       (int64_t)kq_act_bytes(n));
    return hipGetLastError();
}

hipError_t kq_convert_act(const float* x, int64_t M, int64_t K, int64_t x_row_stride, void* act, hipStream_t st) {
    int nsb = (int)(K / 256);
    hipLaunchKernelGGL(kq_convert_act_kernel<false>, dim3((unsigned)nsb, (unsigned)M), dim3(64), 0, st, (const void*)x, x_row_stride,
                       nsb, (uint8_t*)act, (int64_t)kq_act_bytes(K));
    return hipGetLastError();
}

hipError_t kq_convert_act_bf16(const void* x, int64_t M, int64_t K, int64_t x_row_stride, void* act, hipStream_t st) {
    int nsb = (int)(K / 256);
    hipLaunchKernelGGL(kq_convert_act_kernel<true>, dim3((unsigned)nsb, (unsigned)M), dim3(64), 0, st, x, x_row_stride, nsb,
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
__global__ __launch_bounds__(256) void qgemv_q4k_plain_kernel(const uint8_t* __restrict__ W, const uint8_t* __restrict__ act, float* y,
                                                              const float* resid, int N, int nsb, int64_t act_row_bytes) {
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
        float t = 0.f, u = 0.f;
        if (j == 0 && live) {
            float xdv = xd[sb];
            float dd = f16_bits_to_f32(load_u16(wb)) * xdv, dm = f16_bits_to_f32(load_u16(wb + 2)) * xdv;
            t = dd * (float)sumi;
            u = dm * (float)summ;
        }
        acc = add_in_order<4>(acc, t);
        accm = add_in_order<4>(accm, u);
    }
    if (lane == 0) {
        const int64_t at = (int64_t)blockIdx.y * N + row;
        const float v = acc - accm;
        y[at] = resid ? v + resid[at] : v;
    }
}

// qdotQ6KGo (backend/cpu/qmatmul.go:180-200): lane (sb, n, k) takes the 32
// weights of quarter k of half n of super-block sb, groups 8n+2k and 8n+2k+1.
__global__ __launch_bounds__(256) void qgemv_q6k_plain_kernel(const uint8_t* __restrict__ W, const uint8_t* __restrict__ act, float* y,
                                                              const float* resid, int N, int nsb, int64_t act_row_bytes) {
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
        float t = 0.f;
        if (part == 0 && live) {
            float dd = f16_bits_to_f32(load_u16(wb + 208)) * xd[sb];
            t = dd * (float)sumi;
        }
        acc = add_in_order<8>(acc, t);
    }
    if (lane == 0) {
        const int64_t at = (int64_t)blockIdx.y * N + row;
        y[at] = resid ? acc + resid[at] : acc;
    }
}

// ---- the LDS kernels ----------------------------------------------------------
//
// LDS copy of one converted row: the quants of super-block sb at sb * kKqStride
// (16 bytes of padding keep the lanes of neighbouring super-blocks off one
// bank), then the sums and the scales as in global memory.
constexpr int kKqStride = 256 + 16;
constexpr int kKqThreads = 256;
constexpr size_t kKqMaxLds = 160 * 1024;
static size_t kq_lds_bytes(int nsb) { return (size_t)nsb * (kKqStride + 32 + 4); }

__device__ __forceinline__ void kq_stage_act(const uint8_t* __restrict__ arow, int nsb, uint8_t* lds, int tid) {
    const u32x4* src = (const u32x4*)arow;
    for (int c = tid; c < nsb * 16; c += kKqThreads) *(u32x4*)(lds + (c >> 4) * kKqStride + (c & 15) * 16) = src[c];
    const uint32_t* tail = (const uint32_t*)(arow + (int64_t)nsb * 256);
    uint32_t* dst = (uint32_t*)(lds + nsb * kKqStride);
    for (int c = tid; c < nsb * 9; c += kKqThreads) dst[c] = tail[c];
}

// The same row from float32 x, rounded by the workgroup itself (quantizeRow, as kq_convert_act_kernel):
// wavefront w takes super-blocks w, w + 4, ...
__device__ __forceinline__ void kq_convert_into_lds(const float* __restrict__ xr, int nsb, uint8_t* lds, int tid) {
    const int lane = tid & 63;
    constexpr int kWaves = kKqThreads / 64, kBatch = 4;  // loads requested kBatch at a time: a loop of unknown length waits for each
    for (int sb0 = tid >> 6; sb0 < nsb; sb0 += kWaves * kBatch) {
        f32x4 v[kBatch];
#pragma unroll
        for (int j = 0; j < kBatch; ++j) {
            const int sb = min(sb0 + kWaves * j, nsb - 1);
            __builtin_memcpy(&v[j], xr + 256 * sb + 4 * lane, 16);
        }
#pragma unroll
        for (int j = 0; j < kBatch; ++j) {
            const int sb = sb0 + kWaves * j;
            if (sb < nsb)
                kq_convert_superblock_to(v[j], lane, (uint32_t*)(lds + sb * kKqStride), (uint16_t*)(lds + nsb * kKqStride) + sb * 16,
                                         (float*)(lds + nsb * (kKqStride + 32)) + sb);
        }
    }
}

__device__ __forceinline__ u32x4 lds_u32x4(const uint8_t* p) { return *(const u32x4*)p; }

struct Q4KTile {
    u32x4 hdr, q0, q1;  // d, dmin and the 12 scale bytes; bytes 16j.. and 64+16j.. of the nibbles
};

// qdotQ4KGo (backend/cpu/qmatmul.go:148-172). Lane (sb, j): nibble bytes
// 16j..16j+15 and 64+16j..64+16j+15 of super-block sb, which are 16 weights
// each of sub-blocks 2g, 2g+1, 2g+4 and 2g+5 (g = j/2), the 16-weight chunks
// 4g+h, 4g+2+h, 4g+8+h, 4g+10+h of the super-block (h = j%2); the sums kept
// with x are per chunk.
template <int R>
__global__ __launch_bounds__(kKqThreads) void qgemv_q4k_kernel(const uint8_t* __restrict__ W, const uint8_t* __restrict__ act, float* y,
                                                               const float* resid, int N, int nsb, int64_t act_row_bytes, Q4RopeTail rope,
                                                               int rope_on, int x_is_f32) {
    extern __shared__ __align__(16) uint8_t kq_lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int row0 = (blockIdx.x * (kKqThreads / 64) + wave) * R;
    const int j = lane & 3, g = j >> 1, h = j & 1, sbl = lane >> 2;
    const int64_t row_bytes = (int64_t)nsb * 144;
    Q4KTile next[R];
    auto fetch = [&](int sb0) {
        int sb = sb0 + sbl;
        sb = sb < nsb ? sb : nsb - 1;
#pragma unroll
        for (int r = 0; r < R; r++) {
            int row = row0 + r;
            row = row < N ? row : N - 1;
            const uint8_t* wb = W + (int64_t)row * row_bytes + (int64_t)sb * 144;
            next[r].hdr = *(const u32x4*)wb;
            next[r].q0 = *(const u32x4*)(wb + 16 + 16 * j);
            next[r].q1 = *(const u32x4*)(wb + 80 + 16 * j);
        }
    };
    fetch(0);
    // act: rows converted beforehand, or (x_is_f32) rows of float32 x, act_row_bytes apart, which the workgroup rounds itself
    if (x_is_f32) kq_convert_into_lds((const float*)(act + (int64_t)blockIdx.y * act_row_bytes), nsb, kq_lds, tid);
    else kq_stage_act(act + (int64_t)blockIdx.y * act_row_bytes, nsb, kq_lds, tid);
    __syncthreads();
    const int16_t* sums = (const int16_t*)(kq_lds + nsb * kKqStride);
    const float* xd = (const float*)(kq_lds + nsb * (kKqStride + 32));
    const int ca = 4 * g + h, sh = 16 * g;
    float acc[R], accm[R];
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = accm[r] = 0.f;
    for (int sb0 = 0; sb0 < nsb; sb0 += 16) {
        int sb = sb0 + sbl;
        const bool live = sb < nsb;
        sb = live ? sb : nsb - 1;
        Q4KTile cur[R];
#pragma unroll
        for (int r = 0; r < R; r++) cur[r] = next[r];
        if (sb0 + 16 < nsb) fetch(sb0 + 16);
        const uint8_t* xq = kq_lds + sb * kKqStride + 16 * ca;
        const u32x4 xa = lds_u32x4(xq), xb = lds_u32x4(xq + 32), xc = lds_u32x4(xq + 128), xe = lds_u32x4(xq + 160);
        const int16_t* s16 = sums + sb * 16 + ca;
        const int sa = s16[0], sb_ = s16[2], sc_ = s16[8], se = s16[10];
        const float xscale = xd[sb];
#pragma unroll
        for (int r = 0; r < R; r++) {
            const uint32_t s0 = cur[r].hdr[1], s1 = cur[r].hdr[2], s2 = cur[r].hdr[3];
            // scale_min_k4 (backend/cpu/quant.go:129-134) for sub-blocks 2g, 2g+1 (< 4) and 2g+4, 2g+5
            const int sc_a = (s0 >> sh) & 63, sc_b = (s0 >> (sh + 8)) & 63;
            const int m_a = (s1 >> sh) & 63, m_b = (s1 >> (sh + 8)) & 63;
            const int sc_c = ((s2 >> sh) & 0xf) | (((s0 >> (sh + 6)) & 3) << 4);
            const int sc_e = ((s2 >> (sh + 8)) & 0xf) | (((s0 >> (sh + 14)) & 3) << 4);
            const int m_c = ((s2 >> (sh + 4)) & 0xf) | (((s1 >> (sh + 6)) & 3) << 4);
            const int m_e = ((s2 >> (sh + 12)) & 0xf) | (((s1 >> (sh + 14)) & 3) << 4);
            int lo0 = 0, hi0 = 0, lo1 = 0, hi1 = 0;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t w0 = cur[r].q0[i], w1 = cur[r].q1[i];
                lo0 = __builtin_amdgcn_sdot4((int)(w0 & 0x0F0F0F0Fu), (int)xa[i], lo0, false);
                hi0 = __builtin_amdgcn_sdot4((int)((w0 >> 4) & 0x0F0F0F0Fu), (int)xb[i], hi0, false);
                lo1 = __builtin_amdgcn_sdot4((int)(w1 & 0x0F0F0F0Fu), (int)xc[i], lo1, false);
                hi1 = __builtin_amdgcn_sdot4((int)((w1 >> 4) & 0x0F0F0F0Fu), (int)xe[i], hi1, false);
            }
            // 24-bit multiplies (full rate; a 32-bit one takes four times as long): scales and mins below 64, sums within 16 * 15 * 127
            int sumi = __mul24(sc_a, lo0) + __mul24(sc_b, hi0) + __mul24(sc_c, lo1) + __mul24(sc_e, hi1);
            int summ = __mul24(m_a, sa) + __mul24(m_b, sb_) + __mul24(m_c, sc_) + __mul24(m_e, se);
            sumi = dpp_i32_quad_sum(live ? sumi : 0);
            summ = dpp_i32_quad_sum(live ? summ : 0);
            float t = 0.f, u = 0.f;
            if (j == 0 && live) {
                const uint32_t dw = cur[r].hdr[0];
                float dd = f16_bits_to_f32((uint16_t)dw) * xscale, dm = f16_bits_to_f32((uint16_t)(dw >> 16)) * xscale;
                t = dd * (float)sumi;
                u = dm * (float)summ;
            }
            acc[r] = add_in_order<4>(acc[r], t);
            accm[r] = add_in_order<4>(accm[r], u);
        }
    }
    if (rope_on) {  // R even: the wavefront's rows are pairs of features; rotation and cache writes as rope_kv does them
        if (R >= 2) {
            const int pos = *rope.pos;
#pragma unroll
            for (int r = 0; r + 1 < R; r += 2)
                if (lane == 0 && row0 + r < N)
                    q4_rope_store(rope, pos, blockIdx.y, row0 + r, acc[r] - accm[r], acc[r + 1] - accm[r + 1], y + (int64_t)blockIdx.y * N);
        }
        return;
    }
#pragma unroll
    for (int r = 0; r < R; r++)
        if (lane == 0 && row0 + r < N) {
            const int64_t at = (int64_t)blockIdx.y * N + row0 + r;
            const float v = acc[r] - accm[r];
            y[at] = resid ? v + resid[at] : v;
        }
}

// Sixteen bytes at a 2-byte aligned address as five aligned dwords; take(i)
// shifts dword i of the sixteen out of them.
struct Bytes16 {
    u32x4 lo;
    uint32_t top;
    __device__ __forceinline__ uint32_t take(int i, uint32_t mis) const {
        return __builtin_amdgcn_alignbyte(i == 3 ? top : lo[i + 1 > 3 ? 3 : i + 1], lo[i], mis);
    }
};
// The dword after the sixteen bytes is read only where the address is off by
// two; `last` says that nothing readable follows an aligned sixteen.
__device__ __forceinline__ Bytes16 load_bytes16(const uint8_t* p, uint32_t mis) {
    Bytes16 b;
    const uint8_t* base = p - mis;
    __builtin_memcpy(&b.lo, __builtin_assume_aligned(base, 4), 16);
    __builtin_memcpy(&b.top, __builtin_assume_aligned(base + (mis ? 16 : 12), 4), 4);
    return b;
}

struct Q6KTile {
    Bytes16 ql, qh, sc;  // 16 bytes of low nibbles, the 16 bytes of high bits that go with them, the 16 scales
    uint16_t d;
};

// qdotQ6KGo (backend/cpu/qmatmul.go:180-200). Lane (sb, n, c): bytes
// 64n+16c..64n+16c+15 of ql, whose low nibbles are chunk 8n+c of the
// super-block and whose high nibbles are chunk 8n+c+4, with bytes
// 32n+16(c%2).. of qh holding their upper two bits at bit 2(c/2) and
// 2(c/2)+4; Q6_K's scales are per chunk.
template <int R>
__global__ __launch_bounds__(kKqThreads) void qgemv_q6k_kernel(const uint8_t* __restrict__ W, const uint8_t* __restrict__ act, float* y,
                                                               const float* resid, int N, int nsb, int64_t act_row_bytes, Q4RopeTail rope,
                                                               int rope_on, int x_is_f32) {
    extern __shared__ __align__(16) uint8_t kq_lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int row0 = (blockIdx.x * (kKqThreads / 64) + wave) * R;
    const int part = lane & 7, n = part >> 2, c = part & 3, sbl = lane >> 3;
    const int64_t row_bytes = (int64_t)nsb * 210;
    Q6KTile next[R];
    auto fetch = [&](int sb0) {
        int sb = sb0 + sbl;
        sb = sb < nsb ? sb : nsb - 1;
#pragma unroll
        for (int r = 0; r < R; r++) {
            int row = row0 + r;
            row = row < N ? row : N - 1;
            const uint8_t* wb = W + (int64_t)row * row_bytes + (int64_t)sb * 210;
            const uint32_t mis = (uint32_t)(uintptr_t)wb & 3;  // 0 or 2, the same for every part of a block
            next[r].ql = load_bytes16(wb + 64 * n + 16 * c, mis);
            next[r].qh = load_bytes16(wb + 128 + 32 * n + 16 * (c & 1), mis);
            next[r].sc = load_bytes16(wb + 192, mis);
            next[r].d = load_u16(wb + 208);
        }
    };
    fetch(0);
    // act: rows converted beforehand, or (x_is_f32) rows of float32 x, act_row_bytes apart, which the workgroup rounds itself
    if (x_is_f32) kq_convert_into_lds((const float*)(act + (int64_t)blockIdx.y * act_row_bytes), nsb, kq_lds, tid);
    else kq_stage_act(act + (int64_t)blockIdx.y * act_row_bytes, nsb, kq_lds, tid);
    __syncthreads();
    const int16_t* sums = (const int16_t*)(kq_lds + nsb * kKqStride);
    const float* xd = (const float*)(kq_lds + nsb * (kKqStride + 32));
    const int chunk = 8 * n + c, shl = c & 2;
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = 0.f;
    for (int sb0 = 0; sb0 < nsb; sb0 += 8) {
        int sb = sb0 + sbl;
        const bool live = sb < nsb;
        sb = live ? sb : nsb - 1;
        Q6KTile cur[R];
        uint32_t mis[R];
#pragma unroll
        for (int r = 0; r < R; r++) {
            cur[r] = next[r];
            int row = row0 + r;
            row = row < N ? row : N - 1;
            mis[r] = (uint32_t)(uintptr_t)(W + (int64_t)row * row_bytes + (int64_t)sb * 210) & 3;
        }
        if (sb0 + 8 < nsb) fetch(sb0 + 8);
        const uint8_t* xq = kq_lds + sb * kKqStride + 16 * chunk;
        const u32x4 xl = lds_u32x4(xq), xh = lds_u32x4(xq + 64);
        const int sl = sums[sb * 16 + chunk], sh_ = sums[sb * 16 + chunk + 4];
        const float xscale = xd[sb];
#pragma unroll
        for (int r = 0; r < R; r++) {
            int dl = 0, dh = 0;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t a = cur[r].ql.take(i, mis[r]), b = cur[r].qh.take(i, mis[r]) >> shl;
                const uint32_t vl = (a & 0x0F0F0F0Fu) | ((b & 0x03030303u) << 4);  // 0..63 per byte
                const uint32_t vh = ((a >> 4) & 0x0F0F0F0Fu) | (((b >> 4) & 0x03030303u) << 4);
                dl = __builtin_amdgcn_sdot4((int)vl, (int)xl[i], dl, false);
                dh = __builtin_amdgcn_sdot4((int)vh, (int)xh[i], dh, false);
            }
            const uint32_t pair = n ? cur[r].sc.take(2, mis[r]) : cur[r].sc.take(0, mis[r]);
            const uint32_t pair4 = n ? cur[r].sc.take(3, mis[r]) : cur[r].sc.take(1, mis[r]);
            const int sc_l = (int)(int8_t)(pair >> (8 * c)), sc_h = (int)(int8_t)(pair4 >> (8 * c));
            int sumi = __mul24(sc_l, dl - 32 * sl) + __mul24(sc_h, dh - 32 * sh_);  // int8 scales, |dl - 32 sl| below 2^18: 24-bit multiplies
            sumi = dpp_i32_group8_sum(live ? sumi : 0);
            float t = 0.f;
            if (part == 0 && live) {
                float dd = f16_bits_to_f32(cur[r].d) * xscale;
                t = dd * (float)sumi;
            }
            acc[r] = add_in_order<8>(acc[r], t);
        }
    }
    if (rope_on) {
        if (R >= 2) {
            const int pos = *rope.pos;
#pragma unroll
            for (int r = 0; r + 1 < R; r += 2)
                if (lane == 0 && row0 + r < N) q4_rope_store(rope, pos, blockIdx.y, row0 + r, acc[r], acc[r + 1], y + (int64_t)blockIdx.y * N);
        }
        return;
    }
#pragma unroll
    for (int r = 0; r < R; r++)
        if (lane == 0 && row0 + r < N) {
            const int64_t at = (int64_t)blockIdx.y * N + row0 + r;
            y[at] = resid ? acc[r] + resid[at] : acc[r];
        }
}

// [0] rows per wavefront (0: by shape). [1] 1: always the kernels without LDS, 2: never the
// matrix-core kernel, 3: the matrix-core kernel for any number of rows.
static std::atomic<int> g_kq_tune[2] = {{0}, {0}};
void set_kquant_tune(int which, int value) {
    if (which >= 0 && which < 2) g_kq_tune[which] = value;
}

template <int R>
static hipError_t launch_kq(int dt, const QGemvArgs& a, int nsb, const Q4RopeTail* rope, hipStream_t st) {
    static std::atomic<bool> raised[2];  // zero at start; threads may race here: both then set the same attribute
    const size_t lds = kq_lds_bytes(nsb);
    const int rows_per_wg = kKqThreads / 64 * R;
    dim3 grid((unsigned)((a.N + rows_per_wg - 1) / rows_per_wg), (unsigned)a.M);
    const void* fn = dt == kQ4_K ? (const void*)qgemv_q4k_kernel<R> : (const void*)qgemv_q6k_kernel<R>;
    if (lds > 48 * 1024 && !raised[dt == kQ4_K]) {
        hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kKqMaxLds);
        if (e != hipSuccess) return e;
        raised[dt == kQ4_K] = true;
    }
    const Q4RopeTail tail = rope ? *rope : Q4RopeTail{};
    // without converted activations the kernel reads float32 x and rounds it per workgroup
    const uint8_t* in = a.act ? (const uint8_t*)a.act : (const uint8_t*)a.x;
    const int64_t in_row = a.act ? (int64_t)kq_act_bytes(a.K) : a.x_row_stride * 4;
    if (dt == kQ4_K)
        hipLaunchKernelGGL(qgemv_q4k_kernel<R>, grid, dim3(kKqThreads), lds, st, (const uint8_t*)a.W, in, a.y, a.resid, (int)a.N, nsb, in_row,
                           tail, rope ? 1 : 0, a.act ? 0 : 1);
    else
        hipLaunchKernelGGL(qgemv_q6k_kernel<R>, grid, dim3(kKqThreads), lds, st, (const uint8_t*)a.W, in, a.y, a.resid, (int)a.N, nsb, in_row,
                           tail, rope ? 1 : 0, a.act ? 0 : 1);
    return hipGetLastError();
}

// Whether qgemv_kquant_act_rope takes the product: the kernels that own pairs of rows.
bool qgemv_kquant_rope_ok(int dt, const QGemvArgs& a) {
    const int nsb = (int)(a.K / 256);
    return (dt == kQ4_K || dt == kQ6_K) && a.K % 256 == 0 && kq_lds_bytes(nsb) <= kKqMaxLds && ((uintptr_t)a.W & (dt == kQ4_K ? 15 : 1)) == 0;
}

// The q|k|v product of a decoding step with the rotation and the cache writes as its tail: y receives
// the rotated queries only (see Q4RopeTail; interleaved pairs, even widths).
hipError_t qgemv_kquant_act_rope(int dt, const QGemvArgs& a, const Q4RopeTail& rope, hipStream_t st) {
    return launch_kq<2>(dt, a, (int)(a.K / 256), &rope, st);
}

hipError_t qgemv_kquant_act(int dt, const QGemvArgs& a, hipStream_t st) {
    int nsb = (int)(a.K / 256);
    // Float32 x in place of converted rows (a.act null): only the kernels that stage the row in LDS round it themselves.
    if (!a.act) {
        if (!qgemv_kquant_rope_ok(dt, a) || ((uintptr_t)a.x & 15) || a.x_row_stride % 4) return hipErrorInvalidValue;
        return a.N * a.M >= 2048 ? launch_kq<2>(dt, a, nsb, nullptr, st) : launch_kq<1>(dt, a, nsb, nullptr, st);
    }
    // A few rows of x: W read once per eight of them.
    if (g_kq_tune[0] == 0 && g_kq_tune[1] == 0 && qgemv_kquant_rows_pays(dt, a)) return qgemv_kquant_rows(dt, a, st);
    // From a few rows of x on, the matrix cores (whose results are the CPU's bit for bit).
    if (!a.resid && (g_kq_tune[1] == 3 || (g_kq_tune[1] == 0 && qgemm_kquant_pays(dt, a))) && qgemm_kquant_ok(dt, a)) return qgemm_kquant(dt, a, st);
    // Q4_K blocks are read with aligned 128-bit loads: 144-byte blocks keep a 16-byte aligned W aligned.
    // Q6_K's 210-byte blocks are read as aligned dwords around a 2-byte aligned start.
    const bool lds_ok = kq_lds_bytes(nsb) <= kKqMaxLds && ((uintptr_t)a.W & (dt == kQ4_K ? 15 : 1)) == 0;
    if (g_kq_tune[1] != 1 && lds_ok) {
        int R = g_kq_tune[0];
        if (R != 1 && R != 2 && R != 4) R = a.N * a.M >= 2048 ? 2 : 1;  // measured: see the sweep keys of mi355x_tune
        return R == 4 ? launch_kq<4>(dt, a, nsb, nullptr, st) : R == 2 ? launch_kq<2>(dt, a, nsb, nullptr, st) : launch_kq<1>(dt, a, nsb, nullptr, st);
    }
    const int waves = 4;
    dim3 grid((unsigned)((a.N + waves - 1) / waves), (unsigned)a.M);
    if (dt == kQ4_K)
        hipLaunchKernelGGL(qgemv_q4k_plain_kernel, grid, dim3(64 * waves), 0, st, (const uint8_t*)a.W, (const uint8_t*)a.act,
                           a.y, a.resid, (int)a.N, nsb, (int64_t)kq_act_bytes(a.K));
    else
        hipLaunchKernelGGL(qgemv_q6k_plain_kernel, grid, dim3(64 * waves), 0, st, (const uint8_t*)a.W, (const uint8_t*)a.act,
                           a.y, a.resid, (int)a.N, nsb, (int64_t)kq_act_bytes(a.K));
    return hipGetLastError();
}

}  // namespace mimir
