// The small kernels of a decoding step, for gfx950: RMSNorm, rotary
// embedding, the KV-cache write, SwiGLU, the residual add and greedy argmax.
// On the reference's ROCm backend these arrive as runs of generated
// elementwise and reduction kernels (backend/internal/gen/gen.go:556+); here
// each is one launch, so that a whole step is queued with no host round trip.
// The arithmetic follows the reference operation by operation (each product
// rounded to float32 on its own, no fused multiply-adds) except for the order
// of RMSNorm's sum of squares, which a parallel reduction fixes differently.
#include "device_util.h"
#include "kernels.h"
#include "q4_act.h"

namespace mimir {

#pragma clang fp contract(off)

// ---- RMSNorm: nn/transformer.go:50-61; llm/decode.go:376-385 -----------------
// y = (x * recip(sqrt(mean(x^2) + eps))) * w, one workgroup per row. mean is
// sum * float32(1/d); eps is added as a float32; the reciprocal and the square
// root are correctly rounded.
__global__ __launch_bounds__(256) void rmsnorm_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                      float* __restrict__ y, int d, float inv_d, float eps) {
    __shared__ float part[4];
    const float* xr = x + (int64_t)blockIdx.x * d;
    float* yr = y + (int64_t)blockIdx.x * d;
    float ss = wave_sum(strided_sum_squares(xr, d, threadIdx.x));
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
    __syncthreads();
    float total = (part[0] + part[1]) + (part[2] + part[3]);
    float ms = total * inv_d;
    float scale = 1.0f / __builtin_sqrtf(ms + eps);
    for (int i0 = threadIdx.x; i0 < d; i0 += 8 * 256) {  // loads in batches, as above
        float xv[8], wv[8];
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const int i = i0 + 256 * u;
            xv[u] = i < d ? xr[i] : 0.f;
            wv[u] = w && i < d ? w[i] : 1.f;
        }
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const int i = i0 + 256 * u;
            float v = xv[u] * scale;
            if (i < d) yr[i] = w ? v * wv[u] : v;
        }
    }
}

hipError_t rmsnorm(const float* x, const float* w, float* y, int64_t rows, int64_t d, double eps, hipStream_t st) {
    if (rows == 0 || d == 0) return hipSuccess;
    hipLaunchKernelGGL(rmsnorm_kernel, dim3((unsigned)rows), dim3(256), 0, st, x, w, y, (int)d, (float)(1.0 / (double)d), (float)eps);
    return hipGetLastError();
}

// RMSNorm with the Q4_0 kernel's activation conversion fused in: the row is
// held in registers between the sum of squares and the conversion, so x is
// read once. Writes y (if not null) and the converted row. d a multiple of
// 64 and at most 256 * 4 * 8 * kNormItems floats.
__global__ __launch_bounds__(256) void rmsnorm_q4act_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                            float* __restrict__ y, uint8_t* __restrict__ act, int d, float inv_d,
                                                            float eps, int64_t act_row_bytes) {
    __shared__ float part[4];
    const float* xr = x + (int64_t)blockIdx.x * d;
    const int nb = d >> 5, nbp = nb | 1, nq = nb * 4;
    u32x4* plane = (u32x4*)(act + (int64_t)blockIdx.x * act_row_bytes);
    NormRow row;
    float ss = wave_sum(norm_load(row, xr, w, nq, threadIdx.x));
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
    __syncthreads();
    norm_convert(row, part, y ? y + (int64_t)blockIdx.x * d : nullptr, plane, (float*)(plane + kDigits * nbp), nbp, nq, threadIdx.x,
                 inv_d, eps);
}

bool rmsnorm_q4act_ok(int64_t d) { return d > 0 && d % 64 == 0 && d / 32 * 4 <= 256 * kNormItems; }

hipError_t rmsnorm_q4act(const float* x, const float* w, float* y, void* act, int64_t rows, int64_t d, double eps, hipStream_t st) {
    if (rows == 0) return hipSuccess;
    hipLaunchKernelGGL(rmsnorm_q4act_kernel, dim3((unsigned)rows), dim3(256), 0, st, x, w, y, (uint8_t*)act, (int)d,
                       (float)(1.0 / (double)d), (float)eps, (int64_t)q4_0_act_row_bytes(d));
    return hipGetLastError();
}

// ---- RoPE: nn/transformer.go:225-257 -------------------------------------------
// x is [rows, S, head_dim] with explicit strides; position s of every row
// turns by the angles of table row offset + s (cos and sin are [len, dim/2],
// computed on the host in float64 as the reference does, transformer.go:146-164).
// a' = a*cos - b*sin, b' = a*sin + b*cos for interleaved pairs (2i, 2i+1), and
// for halves (i, i + dim/2) a' = a*cos - b*sin, b' = b*cos + a*sin.
__global__ __launch_bounds__(256) void rope_kernel(const float* __restrict__ x, float* __restrict__ y, int64_t rows, int s,
                                                   int head_dim, int dim, int interleaved, int64_t x_row_stride,
                                                   int64_t x_pos_stride, int64_t y_row_stride, int64_t y_pos_stride,
                                                   const float* __restrict__ cosv, const float* __restrict__ sinv, int offset, int period) {
    const int half = dim >> 1, per = half + (head_dim - dim);  // work items per (row, position)
    int64_t total = rows * s * per;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (int64_t)gridDim.x * blockDim.x) {
        int i = (int)(t % per);
        int64_t rp = t / per;
        int q = (int)(rp % s);
        int64_t r = rp / s;
        const float* xi = x + r * x_row_stride + q * x_pos_stride;
        float* yo = y + r * y_row_stride + q * y_pos_stride;
        if (i >= half) {  // features past dim pass through
            int f = dim + (i - half);
            yo[f] = xi[f];
            continue;
        }
        int ia = interleaved ? 2 * i : i, ib = interleaved ? 2 * i + 1 : i + half;
        float a = xi[ia], b = xi[ib];
        const int64_t at = offset + q % period;  // several sequences' positions in a row: each counts from the offset
        float c = cosv[at * half + i], sn = sinv[at * half + i];
        float ac = a * c, bs = b * sn, as = a * sn, bc = b * c;
        yo[ia] = ac - bs;
        yo[ib] = interleaved ? as + bc : bc + as;
    }
}

hipError_t rope(const float* x, float* y, int64_t rows, int64_t s, int head_dim, int dim, int interleaved, int64_t x_row_stride,
                int64_t x_pos_stride, int64_t y_row_stride, int64_t y_pos_stride, const float* cosv, const float* sinv,
                int64_t offset, hipStream_t st, int64_t period) {
    int64_t total = rows * s * (dim / 2 + head_dim - dim);
    if (total == 0) return hipSuccess;
    int64_t groups = (total + 255) / 256;
    if (groups > 65536) groups = 65536;
    hipLaunchKernelGGL(rope_kernel, dim3((unsigned)groups), dim3(256), 0, st, x, y, rows, (int)s, head_dim, dim, interleaved,
                       x_row_stride, x_pos_stride, y_row_stride, y_pos_stride, cosv, sinv, (int)offset, (int)(period > 0 ? period : s));
    return hipGetLastError();
}

// ---- KV cache write: nn/transformer.go:397-423 (Append) ---------------------------
// src is [B, heads, S, dim] read with strides; it lands at positions
// [pos, pos + S) of a cache [B, heads, cap, dim], cast to the cache's dtype
// (float32 kept, binary16 rounded to nearest even).
__global__ __launch_bounds__(256) void kv_write_kernel(const float* __restrict__ src, void* __restrict__ cache, int cache_dt,
                                                       int64_t total, int heads, int s, int dim, int64_t cap, int64_t pos,
                                                       int64_t src_b, int64_t src_h, int64_t src_p) {
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (int64_t)gridDim.x * blockDim.x) {
        int d = (int)(t % dim);
        int64_t r = t / dim;
        int q = (int)(r % s);
        r /= s;
        int h = (int)(r % heads);
        int64_t b = r / heads;
        float v = src[b * src_b + h * src_h + q * src_p + d];
        int64_t at = ((b * heads + h) * cap + pos + q) * dim + d;
        if (cache_dt == kF32)
            ((float*)cache)[at] = v;
        else
            ((uint16_t*)cache)[at] = f32_to_f16_bits(v);
    }
}

hipError_t kv_write(const float* src, void* cache, int cache_dt, int64_t B, int heads, int64_t s, int dim, int64_t cap,
                    int64_t pos, int64_t src_b, int64_t src_h, int64_t src_p, hipStream_t st) {
    int64_t total = B * heads * s * dim;
    if (total == 0) return hipSuccess;
    int64_t groups = (total + 255) / 256;
    if (groups > 65536) groups = 65536;
    hipLaunchKernelGGL(kv_write_kernel, dim3((unsigned)groups), dim3(256), 0, st, src, cache, cache_dt, total, heads, (int)s, dim,
                       cap, pos, src_b, src_h, src_p);
    return hipGetLastError();
}

// One position of a decoding step in one launch: qkv is [B, (H + 2 HK) * dim],
// the rows of a fused q|k|v product. The query heads are rotated in place, the
// key heads are rotated and written to the keys cache at the position *pos_dev
// holds, the value heads are written to the values cache, each cast to the
// cache's dtype. The position is read on the device so that a captured step
// can be replayed at every position (the reference's recorded step takes the
// position as a tensor for the same reason, llm/decode.go:27-41,166-183).
__global__ __launch_bounds__(256) void rope_kv_kernel(float* __restrict__ q, const float* __restrict__ k, const float* __restrict__ v,
                                                      int64_t q_row, int64_t k_row, int64_t v_row, void* __restrict__ kcache,
                                                      void* __restrict__ vcache, int cache_dt, int B, int H, int HK, int dim, int rope_dim,
                                                      int interleaved, int64_t cap, const float* __restrict__ cosv,
                                                      const float* __restrict__ sinv, const int32_t* __restrict__ pos_dev,
                                                      const float* __restrict__ bias) {
    // bias: null, or [(H + 2 HK) dim] added to every sequence's heads before anything else happens to them: Linear.Forward's
    // bias behind the product (nn/layers.go:49-55), for models whose q, k and v have one (llm/model.go:251-258)
    const int pos = *pos_dev;
    const int half = rope_dim >> 1, hd2 = dim >> 1;  // work items: pairs of features
    const int64_t total = (int64_t)B * (H + 2 * HK) * hd2;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (int64_t)gridDim.x * blockDim.x) {
        int i = (int)(t % hd2);
        int64_t r = t / hd2;
        int head = (int)(r % (H + 2 * HK));
        int64_t b = r / (H + 2 * HK);
        // sequence b's heads: H of queries at q, HK of keys at k, HK of values at v, rows q_row, k_row, v_row floats apart
        const float* hp = head < H ? q + b * q_row + (int64_t)head * dim
                                   : head < H + HK ? k + b * k_row + (int64_t)(head - H) * dim : v + b * v_row + (int64_t)(head - H - HK) * dim;
        const float* bp = bias ? bias + (int64_t)head * dim : nullptr;
        int ia, ib;
        float va, vb;
        if (head < H + HK && i < half) {
            ia = interleaved ? 2 * i : i;
            ib = interleaved ? 2 * i + 1 : i + half;
            float a = hp[ia], c2 = hp[ib];
            if (bp) {
                a = a + bp[ia];
                c2 = c2 + bp[ib];
            }
            float c = cosv[(int64_t)pos * half + i], sn = sinv[(int64_t)pos * half + i];
            float ac = a * c, bs = c2 * sn, as = a * sn, bc = c2 * c;
            va = ac - bs;
            vb = interleaved ? as + bc : bc + as;
        } else {  // values, and features past rope_dim: pass through (two at a time)
            int j = head < H + HK ? i - half : i;
            ia = head < H + HK ? rope_dim + 2 * j : 2 * j;
            ib = ia + 1;
            va = hp[ia];
            vb = hp[ib];
            if (bp) {
                va = va + bp[ia];
                vb = vb + bp[ib];
            }
        }
        if (head < H) {
            float* qp = q + b * q_row + (int64_t)head * dim;
            qp[ia] = va;
            qp[ib] = vb;
        } else {
            const bool is_k = head < H + HK;
            const int kh = is_k ? head - H : head - H - HK;
            void* cache = is_k ? kcache : vcache;
            const int64_t at = ((b * HK + kh) * cap + pos) * dim;
            if (cache_dt == kF32) {
                ((float*)cache)[at + ia] = va;
                ((float*)cache)[at + ib] = vb;
            } else {
                ((uint16_t*)cache)[at + ia] = f32_to_f16_bits(va);
                ((uint16_t*)cache)[at + ib] = f32_to_f16_bits(vb);
            }
        }
    }
}

static hipError_t rope_kv_launch(float* q, const float* k, const float* v, int64_t q_row, int64_t k_row, int64_t v_row, void* kcache,
                                 void* vcache, int cache_dt, int64_t B, int H, int HK, int dim, int rope_dim, int interleaved, int64_t cap,
                                 const float* cosv, const float* sinv, const int32_t* pos_dev, const float* bias, hipStream_t st) {
    int64_t total = B * (H + 2 * HK) * (dim / 2);
    if (total == 0) return hipSuccess;
    int64_t groups = (total + 255) / 256;
    if (groups > 65536) groups = 65536;
    hipLaunchKernelGGL(rope_kv_kernel, dim3((unsigned)groups), dim3(256), 0, st, q, k, v, q_row, k_row, v_row, kcache, vcache, cache_dt,
                       (int)B, H, HK, dim, rope_dim, interleaved, cap, cosv, sinv, pos_dev, bias);
    return hipGetLastError();
}

// qkv [B, (H + 2 HK) dim]: each sequence's query, key and value heads in one row. bias: null, or [(H + 2 HK) dim] added first.
hipError_t rope_kv(float* qkv, void* kcache, void* vcache, int cache_dt, int64_t B, int H, int HK, int dim, int rope_dim,
                   int interleaved, int64_t cap, const float* cosv, const float* sinv, const int32_t* pos_dev, hipStream_t st, const float* bias) {
    const int64_t row = (int64_t)(H + 2 * HK) * dim;
    return rope_kv_launch(qkv, qkv + (int64_t)H * dim, qkv + (int64_t)(H + HK) * dim, row, row, row, kcache, vcache, cache_dt, B, H, HK, dim,
                          rope_dim, interleaved, cap, cosv, sinv, pos_dev, bias, st);
}

// q [B, H dim], k and v [B, HK dim], each contiguous.
hipError_t rope_kv_split(float* q, const float* k, const float* v, void* kcache, void* vcache, int cache_dt, int64_t B, int H, int HK, int dim,
                         int rope_dim, int interleaved, int64_t cap, const float* cosv, const float* sinv, const int32_t* pos_dev,
                         hipStream_t st, const float* bias) {
    return rope_kv_launch(q, k, v, (int64_t)H * dim, (int64_t)HK * dim, (int64_t)HK * dim, kcache, vcache, cache_dt, B, H, HK, dim, rope_dim,
                          interleaved, cap, cosv, sinv, pos_dev, bias, st);
}

// After a step: appends the chosen tokens to the record and moves on one
// position. state = {position, steps taken}.
__global__ void advance_kernel(int32_t* __restrict__ state, const int32_t* __restrict__ next_tok, int32_t* __restrict__ record, int B,
                               int pos_inc) {
    int step = state[1];
    if ((int)threadIdx.x < B) record[(int64_t)step * B + threadIdx.x] = next_tok[threadIdx.x];
    __syncthreads();
    if (threadIdx.x == 0) {
        state[0] += pos_inc;
        state[1] = step + 1;
    }
}

hipError_t advance(int32_t* state, const int32_t* next_tok, int32_t* record, int B, int pos_inc, hipStream_t st) {
    hipLaunchKernelGGL(advance_kernel, dim3(1), dim3(B < 64 ? 64 : ((B + 63) / 64) * 64), 0, st, state, next_tok, record, B, pos_inc);
    return hipGetLastError();
}

__global__ void set_state_kernel(int32_t* __restrict__ state, int pos, int step) {
    state[0] = pos;
    state[1] = step;
}

hipError_t set_state(int32_t* state, int pos, int step, hipStream_t st) {
    hipLaunchKernelGGL(set_state_kernel, dim3(1), dim3(1), 0, st, state, pos, step);
    return hipGetLastError();
}

// ---- SwiGLU: llm/model.go:446-448; tensor/elementwise.go:520-525,583-585 ----------
// out = (g * recip(1 + exp2(g * -log2e))) * u, each step a float32. Rows of g
// and u are `stride` floats apart (they may be the halves of one fused
// product); out is contiguous.
__global__ __launch_bounds__(256) void swiglu_kernel(const float* __restrict__ g, const float* __restrict__ u,
                                                     float* __restrict__ out, int64_t rows, int64_t n, int64_t stride) {
    const float nl2e = (float)(-1.4426950408889634);
    int64_t total = rows * n;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (int64_t)gridDim.x * blockDim.x) {
        int64_t r = t / n, i = t % n;
        float gv = g[r * stride + i];
        float e = __builtin_exp2f(gv * nl2e);
        float s = 1.0f / (1.0f + e);
        float a = gv * s;
        out[t] = a * u[r * stride + i];
    }
}

hipError_t swiglu(const float* g, const float* u, float* out, int64_t rows, int64_t n, int64_t stride, hipStream_t st) {
    if (rows * n == 0) return hipSuccess;
    int64_t groups = (rows * n + 255) / 256;
    if (groups > 65536) groups = 65536;
    hipLaunchKernelGGL(swiglu_kernel, dim3((unsigned)groups), dim3(256), 0, st, g, u, out, rows, n, stride);
    return hipGetLastError();
}

// ---- residual add ------------------------------------------------------------
__global__ __launch_bounds__(256) void add_kernel(const float* __restrict__ a, const float* __restrict__ b, float* __restrict__ out,
                                                  int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) out[i] = a[i] + b[i];
}

// y[r, j] += bias[j]: Linear.Forward's bias (nn/layers.go:49-55), one float32 addition per element behind the product.
__global__ __launch_bounds__(256) void add_bias_kernel(float* __restrict__ y, const float* __restrict__ bias, int64_t rows, int64_t n) {
    const int64_t total = rows * n;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) y[i] = y[i] + bias[i % n];
}

hipError_t add_bias(float* y, const float* bias, int64_t rows, int64_t n, hipStream_t st) {
    if (rows * n == 0) return hipSuccess;
    int64_t groups = (rows * n + 255) / 256;
    if (groups > 65536) groups = 65536;
    hipLaunchKernelGGL(add_bias_kernel, dim3((unsigned)groups), dim3(256), 0, st, y, bias, rows, n);
    return hipGetLastError();
}

hipError_t add(const float* a, const float* b, float* out, int64_t n, hipStream_t st) {
    if (n == 0) return hipSuccess;
    int64_t groups = (n + 255) / 256;
    if (groups > 65536) groups = 65536;
    hipLaunchKernelGGL(add_kernel, dim3((unsigned)groups), dim3(256), 0, st, a, b, out, n);
    return hipGetLastError();
}

// ---- greedy argmax: examples/llama/generate.go:44-53 -----------------------------
// The first index of the largest value per row. The reference scans with
// `v > logits[best]` from best = 0, so a NaN never wins, and a NaN at index 0
// is never beaten.
__global__ __launch_bounds__(1024) void argmax_kernel(const float* __restrict__ logits, int64_t n, int32_t* __restrict__ out) {
    __shared__ float bv[16];
    __shared__ int bi[16];
    const float* row = logits + (int64_t)blockIdx.x * n;
    float best = -__builtin_inff();
    int at = 0x7fffffff;
    for (int64_t i = threadIdx.x; i < n; i += blockDim.x) {
        float v = row[i];
        if (v > best || (v == best && (int)i < at)) {
            best = v;
            at = (int)i;
        }
    }
    // over the wavefront, then over the wavefronts: larger value, then smaller index
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        float ov = __shfl_xor(best, off);
        int oi = __shfl_xor(at, off);
        if (ov > best || (ov == best && oi < at)) {
            best = ov;
            at = oi;
        }
    }
    if ((threadIdx.x & 63) == 0) {
        bv[threadIdx.x >> 6] = best;
        bi[threadIdx.x >> 6] = at;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < (int)(blockDim.x >> 6); w++)
            if (bv[w] > best || (bv[w] == best && bi[w] < at)) {
                best = bv[w];
                at = bi[w];
            }
        float first = row[0];
        if (first != first || at == 0x7fffffff) at = 0;  // NaN at 0, or nothing but NaNs
        out[blockIdx.x] = at;
    }
}

// The same over many workgroups per row: each scans a span of the row and
// leaves its candidate; the last one of a row to finish (a ticket per row)
// picks among the candidates. tickets: one zeroed word per row, which the last
// workgroup zeroes again.
constexpr int kArgmaxBlocks = 64;  // at most, per row

__device__ __forceinline__ void argmax_better(float& best, int& at, float v, int i) {
    if (v > best || (v == best && i < at)) {
        best = v;
        at = i;
    }
}

__global__ __launch_bounds__(256) void argmax_split_kernel(const float* __restrict__ logits, int64_t n, int span, int32_t* __restrict__ out,
                                                           uint32_t* __restrict__ tickets, float* __restrict__ cand_v,
                                                           int* __restrict__ cand_i) {
    __shared__ float bv[4];
    __shared__ int bi[4];
    __shared__ int s_last;
    const int r = blockIdx.y, nblk = gridDim.x;
    const float* row = logits + (int64_t)r * n;
    const int64_t lo = (int64_t)blockIdx.x * span, hi = lo + span < n ? lo + span : n;
    float best = -__builtin_inff();
    int at = 0x7fffffff;
    for (int64_t i0 = lo + threadIdx.x; i0 < hi; i0 += 4 * 256) {
        float v[4];
#pragma unroll
        for (int u = 0; u < 4; u++) v[u] = i0 + 256 * u < hi ? row[i0 + 256 * u] : -__builtin_inff();
#pragma unroll
        for (int u = 0; u < 4; u++)
            if (i0 + 256 * u < hi) argmax_better(best, at, v[u], (int)(i0 + 256 * u));
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        float ov = __shfl_xor(best, off);
        int oi = __shfl_xor(at, off);
        argmax_better(best, at, ov, oi);
    }
    if ((threadIdx.x & 63) == 0) {
        bv[threadIdx.x >> 6] = best;
        bi[threadIdx.x >> 6] = at;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 4; w++) argmax_better(best, at, bv[w], bi[w]);
        // candidates cross between workgroups through stores and loads that are
        // coherent at device scope on their own; the stores have completed
        // before the ticket is taken
        __hip_atomic_store(&cand_v[r * kArgmaxBlocks + blockIdx.x], best, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(&cand_i[r * kArgmaxBlocks + blockIdx.x], at, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __builtin_amdgcn_s_waitcnt(0);
        // release-acquire at device scope: the candidates stored above happen before it, the loads of the last workgroup after it
        uint32_t ticket = __hip_atomic_fetch_add(&tickets[r], 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
        s_last = ticket == (uint32_t)(nblk - 1);
        if (s_last) __hip_atomic_store(&tickets[r], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!s_last || threadIdx.x >= 64) return;
    best = -__builtin_inff();
    at = 0x7fffffff;
    if ((int)threadIdx.x < nblk) {
        best = __hip_atomic_load(&cand_v[r * kArgmaxBlocks + threadIdx.x], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        at = __hip_atomic_load(&cand_i[r * kArgmaxBlocks + threadIdx.x], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        float ov = __shfl_xor(best, off);
        int oi = __shfl_xor(at, off);
        argmax_better(best, at, ov, oi);
    }
    if (threadIdx.x == 0) {
        float first = row[0];
        if (first != first || at == 0x7fffffff) at = 0;  // NaN at 0, or nothing but NaNs
        out[r] = at;
    }
}

size_t argmax_workspace_bytes(int64_t rows) { return kArgmaxTicketBytes + (size_t)rows * kArgmaxBlocks * 8; }

// workspace: argmax_workspace_bytes(rows) bytes whose first kArgmaxTicketBytes were
// zero before the first launch, or null for the one-workgroup kernel.
hipError_t argmax(const float* logits, int64_t rows, int64_t n, int32_t* out, void* workspace, hipStream_t st) {
    if (rows == 0) return hipSuccess;
    if (!workspace || rows > (int64_t)(kArgmaxTicketBytes / 4) || n < 8192) {
        hipLaunchKernelGGL(argmax_kernel, dim3((unsigned)rows), dim3(1024), 0, st, logits, n, out);
        return hipGetLastError();
    }
    int64_t nblk = (n + 4095) / 4096;
    nblk = nblk > kArgmaxBlocks ? kArgmaxBlocks : nblk;
    int64_t span = ((n + nblk - 1) / nblk + 255) / 256 * 256;
    nblk = (n + span - 1) / span;
    uint32_t* tickets = (uint32_t*)workspace;
    float* cand_v = (float*)((uint8_t*)workspace + kArgmaxTicketBytes);
    int* cand_i = (int*)(cand_v + rows * kArgmaxBlocks);
    hipLaunchKernelGGL(argmax_split_kernel, dim3((unsigned)nblk, (unsigned)rows), dim3(256), 0, st, logits, n, (int)span, out, tickets,
                       cand_v, cand_i);
    return hipGetLastError();
}

}  // namespace mimir
