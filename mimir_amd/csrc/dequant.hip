// Dequantizing casts and gathers of block-quantized buffers for gfx950:
// OpCast and OpGather of the reference (backend/cpu/quant.go:113-327; the
// replaced generated kernels are backend/internal/gen/quant.go:41-150).
// Every value is computed operation by operation as ggml's dequantize_row
// functions do, each product and difference rounded to float32 on its own
// (never fused), so the bits match the CPU backend's.
#include "device_util.h"
#include "kernels.h"

namespace mimir {

#pragma clang fp contract(off)

// backend/cpu/quant.go:129-134
__device__ __forceinline__ void scale_min_k4(int j, const uint8_t* s, uint8_t& sc, uint8_t& m) {
    if (j < 4) {
        sc = s[j] & 63;
        m = s[j + 4] & 63;
    } else {
        sc = (uint8_t)((s[j + 4] & 0xf) | ((s[j - 4] >> 6) << 4));
        m = (uint8_t)((s[j + 4] >> 4) | ((s[j] >> 6) << 4));
    }
}

// Element i of the blocks at data: backend/cpu/quant.go:198-218, with Q4_0 as
// ggml's block_q4_0 (element j < 16 is the low nibble of byte j, element
// j + 16 its high nibble, value (n - 8) * d).
__device__ float dequant_at(int dt, const uint8_t* __restrict__ data, int64_t i) {
    switch (dt) {
    case kQ8_0: {
        const uint8_t* b = data + i / 32 * 34;
        int j = (int)(i % 32);
        return (float)(int8_t)b[2 + j] * f16_bits_to_f32(load_u16(b));
    }
    case kQ4_0: {
        const uint8_t* b = data + i / 32 * 18;
        int j = (int)(i % 32);
        int n = j < 16 ? (b[2 + j] & 0xf) : (b[2 + j - 16] >> 4);
        return (float)(n - 8) * f16_bits_to_f32(load_u16(b));
    }
    case kQ4_K: {
        const uint8_t* b = data + i / 256 * 144;
        int j = (int)(i % 256);
        float d = f16_bits_to_f32(load_u16(b)), dmin = f16_bits_to_f32(load_u16(b + 2));
        int sub = j / 32, l = j % 32;
        uint8_t sc, m;
        scale_min_k4(sub, b + 4, sc, m);
        uint8_t v = b[16 + 32 * (sub / 2) + l];
        if (sub & 1) v >>= 4;
        float t = d * (float)sc;
        t = t * (float)(v & 0xf);
        float mm = dmin * (float)m;
        return t - mm;
    }
    default: {  // kQ6_K
        const uint8_t* b = data + i / 256 * 210;
        int j = (int)(i % 256);
        int n = j / 128, k = j % 128 / 32, l = j % 32;
        const uint8_t *ql = b + 64 * n, *qh = b + 128 + 32 * n;
        uint8_t lo = ql[l + 32 * (k & 1)];
        if (k >= 2) lo >>= 4;
        int q = (int)((lo & 0xf) | (((qh[l] >> (2 * k)) & 3) << 4));
        float s = f16_bits_to_f32(load_u16(b + 208)) * (float)(int8_t)b[192 + 8 * n + l / 16 + 2 * k];
        return s * (float)(q - 32);
    }
    }
}

template <typename T>
__device__ __forceinline__ void store_as(T* out, int64_t i, float v, int out_dt);
template <>
__device__ __forceinline__ void store_as<float>(float* out, int64_t i, float v, int) { out[i] = v; }
template <>
__device__ __forceinline__ void store_as<uint16_t>(uint16_t* out, int64_t i, float v, int out_dt) {
    out[i] = out_dt == kBF16 ? f32_to_bf16_bits(v) : f32_to_f16_bits(v);
}

// out[i] = value of element first + i, i < n, rounded to out_dt.
template <typename T>
__global__ __launch_bounds__(256) void dequant_kernel(int dt, const uint8_t* __restrict__ data, int64_t first, int64_t n,
                                                      T* __restrict__ out, int out_dt) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) store_as<T>(out, i, dequant_at(dt, data, first + i), out_dt);
}

hipError_t dequantize(int dt, const void* data, int64_t first, int64_t n, void* out, int out_dt, hipStream_t st) {
    if (n == 0) return hipSuccess;
    int64_t groups = (n + 255) / 256;
    if (groups > 65536) groups = 65536;
    if (out_dt == kF32)
        hipLaunchKernelGGL(dequant_kernel<float>, dim3((unsigned)groups), dim3(256), 0, st, dt, (const uint8_t*)data, first, n,
                           (float*)out, out_dt);
    else
        hipLaunchKernelGGL(dequant_kernel<uint16_t>, dim3((unsigned)groups), dim3(256), 0, st, dt, (const uint8_t*)data, first,
                           n, (uint16_t*)out, out_dt);
    return hipGetLastError();
}

// Embedding lookup: out[r, c] = value of table[idx[r], c] for r < n, c < k;
// an index outside [0, rows) sets bit kErrIndex of *err and writes zeros
// (backend/cpu/quant.go:296-327 fails the kernel with ErrIndex).
__global__ __launch_bounds__(256) void gather_rows_kernel(int dt, const uint8_t* __restrict__ table, int64_t rows, int64_t k,
                                                          const int32_t* __restrict__ idx, int64_t n, float* __restrict__ out,
                                                          uint32_t* err) {
    int64_t r = blockIdx.y;
    int64_t j = idx[r];
    bool bad = j < 0 || j >= rows;
    if (bad && threadIdx.x == 0 && blockIdx.x == 0 && err) atomicOr(err, kErrIndex);
    for (int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; c < k; c += (int64_t)gridDim.x * blockDim.x)
        out[r * k + c] = bad ? 0.f : dequant_at(dt, table, j * k + c);
}

hipError_t gather_rows(int dt, const void* table, int64_t rows, int64_t k, const int32_t* idx, int64_t n, float* out,
                       uint32_t* err, hipStream_t st) {
    if (n == 0 || k == 0) return hipSuccess;
    int64_t gx = (k + 255) / 256;
    if (gx > 64) gx = 64;
    hipLaunchKernelGGL(gather_rows_kernel, dim3((unsigned)gx, (unsigned)n), dim3(256), 0, st, dt, (const uint8_t*)table, rows, k,
                       idx, n, out, err);
    return hipGetLastError();
}

// ---- reads through views (backend/view.go): element i of the contiguous
// output is element offset + sum_d coord_d * stride_d of the buffer ---------------
__device__ __forceinline__ int64_t view_element(const ViewArg& v, int64_t i) {
    int64_t at = v.offset;
    for (int d = v.rank - 1; d >= 0; d--) {
        at += (i % v.shape[d]) * v.strides[d];
        i /= v.shape[d];
    }
    return at;
}

// OpCast of a block-quantized input read through any view (dequantAt,
// backend/cpu/quant.go:236-256).
template <typename T>
__global__ __launch_bounds__(256) void dequant_view_kernel(int dt, const uint8_t* __restrict__ data, ViewArg v, int64_t n,
                                                           T* __restrict__ out, int out_dt) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        store_as<T>(out, i, dequant_at(dt, data, view_element(v, i)), out_dt);
}

hipError_t dequantize_view(int dt, const void* data, const ViewArg& v, int64_t n, void* out, int out_dt, hipStream_t st) {
    if (n == 0) return hipSuccess;
    int64_t groups = (n + 255) / 256;
    if (groups > 65536) groups = 65536;
    if (out_dt == kF32)
        hipLaunchKernelGGL(dequant_view_kernel<float>, dim3((unsigned)groups), dim3(256), 0, st, dt, (const uint8_t*)data, v, n, (float*)out,
                           out_dt);
    else
        hipLaunchKernelGGL(dequant_view_kernel<uint16_t>, dim3((unsigned)groups), dim3(256), 0, st, dt, (const uint8_t*)data, v, n,
                           (uint16_t*)out, out_dt);
    return hipGetLastError();
}

// OpGather of a block-quantized table through views (gatherQuant,
// backend/cpu/quant.go:296-327): out[m] = table[m with m[axis] = idx[m]]; an
// index outside the axis sets bit kErrIndex of *err and writes zero.
__global__ __launch_bounds__(256) void gather_view_kernel(int dt, const uint8_t* __restrict__ table, ViewArg tv, const int32_t* __restrict__ idx,
                                                          ViewArg iv, int axis, int64_t n, float* __restrict__ out, uint32_t* err) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        // coordinates of i in the output, whose shape is the index view's
        int64_t rem = i, at = tv.offset;
        const int64_t j = idx[view_element(iv, i)];
        bool bad = j < 0 || j >= tv.shape[axis];
        for (int d = iv.rank - 1; d >= 0; d--) {
            int64_t c = rem % iv.shape[d];
            rem /= iv.shape[d];
            at += (d == axis ? (bad ? 0 : j) : c) * tv.strides[d];
        }
        if (bad && err) atomicOr(err, kErrIndex);
        out[i] = bad ? 0.f : dequant_at(dt, table, at);
    }
}

hipError_t gather_view(int dt, const void* table, const ViewArg& tv, const int32_t* idx, const ViewArg& iv, int axis, int64_t n, float* out,
                       uint32_t* err, hipStream_t st) {
    if (n == 0) return hipSuccess;
    int64_t groups = (n + 255) / 256;
    if (groups > 65536) groups = 65536;
    hipLaunchKernelGGL(gather_view_kernel, dim3((unsigned)groups), dim3(256), 0, st, dt, (const uint8_t*)table, tv, idx, iv, axis, n, out, err);
    return hipGetLastError();
}

// A view of 32-bit elements copied into a contiguous buffer (OpContiguous).
__global__ __launch_bounds__(256) void copy_view32_kernel(const uint32_t* __restrict__ src, ViewArg v, int64_t n, uint32_t* __restrict__ out) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) out[i] = src[view_element(v, i)];
}

hipError_t copy_view32(const void* src, const ViewArg& v, int64_t n, void* out, hipStream_t st) {
    if (n == 0) return hipSuccess;
    int64_t groups = (n + 255) / 256;
    if (groups > 65536) groups = 65536;
    hipLaunchKernelGGL(copy_view32_kernel, dim3((unsigned)groups), dim3(256), 0, st, (const uint32_t*)src, v, n, (uint32_t*)out);
    return hipGetLastError();
}

// ---- fill (a kernel, not a memset node, so callers may capture it) ---------
__global__ __launch_bounds__(256) void fill_u32_kernel(uint32_t* __restrict__ p, uint32_t v, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) p[i] = v;
}

hipError_t fill_u32(void* p, uint32_t v, int64_t n, hipStream_t st) {
    if (n == 0) return hipSuccess;
    int64_t groups = (n + 255) / 256;
    if (groups > 4096) groups = 4096;
    hipLaunchKernelGGL(fill_u32_kernel, dim3((unsigned)groups), dim3(256), 0, st, (uint32_t*)p, v, n);
    return hipGetLastError();
}

// ---- streaming read ---------------------------------------------------------
__global__ __launch_bounds__(1024) void stream_read_kernel(const u32x4* __restrict__ p, int64_t n16, float* __restrict__ out) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    uint32_t acc = 0;
#pragma unroll 8
    for (; i < n16; i += stride) {
        u32x4 v = p[i];
        acc ^= v[0] ^ v[1] ^ v[2] ^ v[3];
    }
    float s = wave_sum((float)(acc & 0xff));
    if ((threadIdx.x & 63) == 0) out[blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)] = s;
}

int stream_read_out_len(int grid, int threads) { return grid * (threads / 64); }

hipError_t stream_read(const void* p, size_t bytes, float* out, int grid, int threads, hipStream_t st) {
    hipLaunchKernelGGL(stream_read_kernel, dim3(grid), dim3(threads), 0, st, (const u32x4*)p, (int64_t)(bytes / 16), out);
    return hipGetLastError();
}

}  // namespace mimir
