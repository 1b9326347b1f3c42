// Prompt-sized product of binary16-brain activations with Q4_0 weights on the
// matrix cores of gfx950: Y[M, N] = X[M, K] . W[N, K]^T, X and Y bfloat16, W in
// ggml Q4_0 blocks, float32 accumulation (Tensor.MatMulT with a half x and a
// block-quantized w, tensor/quant.go:45-48: x is cast to float32, multiplied,
// and the result rounded once to x's dtype).
//
// The arithmetic is exact up to float32 accumulation, not a product with
// weights rounded to 16 bits. A weight is (n - 8) * d with a 4-bit n and a
// binary16 d, 15 significant bits, which no 16-bit float holds. So the matrix
// cores multiply x by the integer 128 + n, which bfloat16 holds exactly and
// which costs one mask-or per pair of nibbles to form (0x4300 | n), one Q4_0
// block (32 of K) at a time:
//     S[m, n] = -136 * sum_k x[m, k]  +  sum_k x[m, k] * (128 + n[n, k])
// with the first term, the same for every column, entering as the
// accumulator the MFMA starts from (a small kernel sums the blocks of x
// beforehand). Every product there is exact in float32 (8 x 8 significant
// bits). The block's binary16 scale then multiplies in float32 on the vector
// unit: Y[m, n] += d[n, block] * S[m, n], one FMA per output per block, which
// the compiler interleaves with the MFMAs of the next block.
//
// A workgroup of four wavefronts computes a 64 or 128 x 128 tile over steps of
// 64 of K (two blocks): X rows and unpacked weights are staged through LDS
// (rows padded by 16 bytes, which makes the 128-bit fragment reads
// conflict-free), double-buffered, one barrier a step. v_mfma_f32_32x32x16_bf16
// takes, per lane, eight consecutive k of row (lane % 32), the lane's half
// (lane / 32) choosing which eight of the sixteen; its result holds column
// (lane % 32) and rows 8 (i / 4) + 4 (lane / 32) + i % 4 in register i, so one
// scale per lane serves all sixteen registers.
#include "device_util.h"
#include "kernels.h"

namespace mimir {

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kBN = 128;        // columns of Y (rows of W) per workgroup
constexpr int kKS = 64;         // K per step: two Q4_0 blocks
constexpr int kLd = kKS + 8;    // bfloat16 elements per LDS row
constexpr float kOffset = 136;  // (128 + n) - (n - 8)

constexpr size_t stage_bytes(int BM) { return (size_t)(BM + kBN) * kLd * 2 + 2 * kBN * 4 + 2 * BM * 4; }

// xs[m, b] = -136 * sum of block b of row m of X.
__global__ __launch_bounds__(256) void qgemm_xsum_kernel(const uint16_t* __restrict__ X, float* __restrict__ xs, int64_t items, int nb,
                                                         int64_t x_row_stride) {
    int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= items) return;
    int64_t m = t / nb;
    int b = (int)(t % nb);
    const uint16_t* p = X + m * x_row_stride + 32 * b;
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        u32x4 v;
        __builtin_memcpy(&v, __builtin_assume_aligned(p + 8 * i, 16), 16);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            s += __uint_as_float(v[j] << 16);
            s += __uint_as_float(v[j] & 0xffff0000u);
        }
    }
    xs[t] = -kOffset * s;
}

template <int MT, bool OUT_F32>  // MT 32-row tiles per wavefront: the workgroup's tile is (64 MT) x 128
__global__ __launch_bounds__(256) void qgemm_q4_0_kernel(const uint16_t* __restrict__ X, const uint8_t* __restrict__ W,
                                                         const float* __restrict__ xs, void* __restrict__ Yv, int M, int N, int K,
                                                         int64_t x_row_stride, int tiles_m, int ntiles) {
    constexpr int BM = 64 * MT;
    constexpr int TPR = 256 / BM;         // threads per row of the X tile
    constexpr int AV = 8 / TPR;           // 16-byte pieces per thread (4 or 2)
    extern __shared__ __align__(16) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1, l32 = lane & 31, lh = lane >> 5;

    // consecutive workgroup ids go round the chip's eight dies; give each die a
    // run of tiles that share their columns of W (tiles of one column strip are
    // consecutive), so that a strip is fetched into one L2
    const int per = (ntiles + 7) >> 3;
    const int tile = ((int)blockIdx.x & 7) * per + ((int)blockIdx.x >> 3);
    if (tile >= ntiles) return;
    const int m0 = (tile % tiles_m) * BM, n0 = (tile / tiles_m) * kBN;
    const int nb = K >> 5, nk = K / kKS;
    const int64_t w_row_bytes = (int64_t)nb * 18;

    // what this thread stages: a piece of a row of X, one block of one row of W, one start value
    const int a_row = tid / TPR, a_part = tid % TPR;
    const int a_m = m0 + a_row < M ? m0 + a_row : M - 1;
    const uint16_t* a_src = X + (int64_t)a_m * x_row_stride + a_part * (kKS / TPR);
    const int w_col = tid >> 1, w_blk = tid & 1;
    const int w_n = n0 + w_col < N ? n0 + w_col : N - 1;
    const uint8_t* w_src = W + (int64_t)w_n * w_row_bytes + w_blk * 18;
    const bool c_live = tid < 2 * BM;
    const int c_blk = tid / BM, c_row = tid % BM;
    const int c_m = m0 + c_row < M ? m0 + c_row : M - 1;
    const float* c_src = xs + (int64_t)c_m * nb + c_blk;

    u32x4 ra[AV], rq;
    uint16_t rd;
    float rc;
    auto fetch = [&](int kb) {
#pragma unroll
        for (int i = 0; i < AV; i++) __builtin_memcpy(&ra[i], __builtin_assume_aligned(a_src + (int64_t)kb * kKS + 8 * i, 16), 16);
        const uint8_t* wp = w_src + (int64_t)kb * 36;
        rd = *(const uint16_t*)wp;
        rq = load_u32x4_unaligned(wp + 2);
        rc = c_live ? c_src[2 * kb] : 0.f;
    };
    auto stage = [&](int buf) {
        uint8_t* base = smem + (size_t)buf * stage_bytes(BM);
        uint16_t* As = (uint16_t*)base;
        uint16_t* Bs = As + BM * kLd;
        float* dsc = (float*)(Bs + kBN * kLd);
        float* cs = dsc + 2 * kBN;
#pragma unroll
        for (int i = 0; i < AV; i++) *(u32x4*)(As + a_row * kLd + a_part * (kKS / TPR) + 8 * i) = ra[i];
        // dword i of a block: byte k holds element 4i + k (low nibble) and 16 + 4i + k (high nibble)
        u32x4 lo[2], hi[2];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t l = rq[i] & 0x0f0f0f0fu, h = (rq[i] >> 4) & 0x0f0f0f0fu;
            // bytes {l.b0, 0x43, l.b1, 0x43} and {l.b2, 0x43, l.b3, 0x43}: 0x4300 | n = bfloat16(128 + n)
            lo[i >> 1][2 * (i & 1)] = __builtin_amdgcn_perm(0x43434343u, l, 0x04010400u);
            lo[i >> 1][2 * (i & 1) + 1] = __builtin_amdgcn_perm(0x43434343u, l, 0x04030402u);
            hi[i >> 1][2 * (i & 1)] = __builtin_amdgcn_perm(0x43434343u, h, 0x04010400u);
            hi[i >> 1][2 * (i & 1) + 1] = __builtin_amdgcn_perm(0x43434343u, h, 0x04030402u);
        }
        uint16_t* brow = Bs + w_col * kLd + w_blk * 32;
        *(u32x4*)(brow) = lo[0];
        *(u32x4*)(brow + 8) = lo[1];
        *(u32x4*)(brow + 16) = hi[0];
        *(u32x4*)(brow + 24) = hi[1];
        dsc[w_blk * kBN + w_col] = f16_bits_to_f32(rd);
        if (c_live) cs[c_blk * BM + c_row] = rc;
    };

    f32x16 total[MT][2];
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int nt = 0; nt < 2; nt++)
#pragma unroll
            for (int i = 0; i < 16; i++) total[mt][nt][i] = 0.f;

    fetch(0);
    stage(0);
    __syncthreads();
    for (int kb = 0; kb < nk; kb++) {
        if (kb + 1 < nk) fetch(kb + 1);
        const uint8_t* base = smem + (size_t)(kb & 1) * stage_bytes(BM);
        const uint16_t* As = (const uint16_t*)base;
        const uint16_t* Bs = As + BM * kLd;
        const float* dsc = (const float*)(Bs + kBN * kLd);
        const float* cs = dsc + 2 * kBN;
#pragma unroll
        for (int blk = 0; blk < 2; blk++) {
            f32x16 ci[MT];
            bf16x8 a[MT][2], b[2][2];
            float dn[2];
#pragma unroll
            for (int mt = 0; mt < MT; mt++) {
                const float* cr = cs + blk * BM + wm * (32 * MT) + mt * 32 + lh * 4;
#pragma unroll
                for (int i0 = 0; i0 < 4; i0++) {
                    f32x4 c4 = *(const f32x4*)(cr + i0 * 8);
                    ci[mt][4 * i0] = c4[0]; ci[mt][4 * i0 + 1] = c4[1]; ci[mt][4 * i0 + 2] = c4[2]; ci[mt][4 * i0 + 3] = c4[3];
                }
#pragma unroll
                for (int s = 0; s < 2; s++)
                    a[mt][s] = *(const bf16x8*)(As + (wm * (32 * MT) + mt * 32 + l32) * kLd + blk * 32 + s * 16 + lh * 8);
            }
#pragma unroll
            for (int nt = 0; nt < 2; nt++) {
#pragma unroll
                for (int s = 0; s < 2; s++) b[nt][s] = *(const bf16x8*)(Bs + (wn * 64 + nt * 32 + l32) * kLd + blk * 32 + s * 16 + lh * 8);
                dn[nt] = dsc[blk * kBN + wn * 64 + nt * 32 + l32];
            }
#pragma unroll
            for (int mt = 0; mt < MT; mt++)
#pragma unroll
                for (int nt = 0; nt < 2; nt++) {
                    f32x16 S = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[mt][0], b[nt][0], ci[mt], 0, 0, 0);
                    S = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[mt][1], b[nt][1], S, 0, 0, 0);
#pragma unroll
                    for (int i = 0; i < 16; i++) total[mt][nt][i] = fmaf(S[i], dn[nt], total[mt][nt][i]);
                }
        }
        if (kb + 1 < nk) stage((kb + 1) & 1);
        __syncthreads();
    }

    // one rounding to the output's dtype (f32ToBF16, backend/cpu/half.go:42-51)
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int nt = 0; nt < 2; nt++) {
            const int n = n0 + wn * 64 + nt * 32 + l32;
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int m = m0 + wm * (32 * MT) + mt * 32 + (i >> 2) * 8 + lh * 4 + (i & 3);
                if (m < M && n < N) {
                    if (OUT_F32) ((float*)Yv)[(int64_t)m * N + n] = total[mt][nt][i];
                    else ((uint16_t*)Yv)[(int64_t)m * N + n] = f32_to_bf16_bits(total[mt][nt][i]);
                }
            }
        }
}

__global__ __launch_bounds__(256) void bf16_rows_to_f32_kernel(const uint16_t* __restrict__ x, float* __restrict__ y, int64_t M, int64_t K,
                                                               int64_t x_row_stride) {
    for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < M * K; t += (int64_t)gridDim.x * 256)
        y[t] = bf16_bits_to_f32(x[(t / K) * x_row_stride + t % K]);
}

__global__ __launch_bounds__(256) void f32_to_bf16_kernel(const float* __restrict__ x, uint16_t* __restrict__ y, int64_t n) {
    for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < n; t += (int64_t)gridDim.x * 256) y[t] = f32_to_bf16_bits(x[t]);
}

}  // namespace

hipError_t bf16_rows_to_f32(const void* x, float* y, int64_t M, int64_t K, int64_t x_row_stride, hipStream_t st) {
    int64_t g = (M * K + 255) / 256;
    hipLaunchKernelGGL(bf16_rows_to_f32_kernel, dim3((unsigned)(g > 65536 ? 65536 : g)), dim3(256), 0, st, (const uint16_t*)x, y, M, K,
                       x_row_stride);
    return hipGetLastError();
}

hipError_t f32_to_bf16(const float* x, void* y, int64_t n, hipStream_t st) {
    int64_t g = (n + 255) / 256;
    hipLaunchKernelGGL(f32_to_bf16_kernel, dim3((unsigned)(g > 65536 ? 65536 : g)), dim3(256), 0, st, x, (uint16_t*)y, n);
    return hipGetLastError();
}

// Whether the matrix-core kernel takes this product: whole steps of two blocks,
// rows of X aligned for 16-byte loads, W at least 2-byte aligned.
bool qgemm_q4_0_ok(const void* W, const void* X, int64_t M, int64_t N, int64_t K, int64_t x_row_stride) {
    return M > 0 && N > 0 && K > 0 && K % kKS == 0 && ((uintptr_t)X & 15) == 0 && x_row_stride % 8 == 0 && ((uintptr_t)W & 1) == 0 &&
           M <= (1 << 24) && N <= (1 << 24) && K <= (1 << 24);
}

size_t qgemm_q4_0_workspace_bytes(int64_t M, int64_t K) { return (size_t)M * (K / 32) * sizeof(float); }

// X [M, K] bfloat16 (rows x_row_stride elements apart), W [N, K] Q4_0, Y [M, N]
// bfloat16, or float32 if out_f32. workspace: qgemm_q4_0_workspace_bytes(M, K).
hipError_t qgemm_q4_0_bf16(const void* W, const void* X, void* Y, int64_t M, int64_t N, int64_t K, int64_t x_row_stride, bool out_f32,
                           void* workspace, hipStream_t st) {
    const int nb = (int)(K / 32);
    const int64_t items = M * nb;
    hipLaunchKernelGGL(qgemm_xsum_kernel, dim3((unsigned)((items + 255) / 256)), dim3(256), 0, st, (const uint16_t*)X, (float*)workspace,
                       items, nb, x_row_stride);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    // 128-row tiles unless they would leave compute units idle
    const int64_t tiles_n = (N + kBN - 1) / kBN;
    const bool tall = ((M + 127) / 128) * tiles_n >= 384;
    const int BM = tall ? 128 : 64;
    const int tiles_m = (int)((M + BM - 1) / BM);
    const int ntiles = (int)(tiles_m * tiles_n);
    dim3 grid((unsigned)(((ntiles + 7) / 8) * 8));
    const size_t lds = 2 * stage_bytes(BM);
    if (tall) {  // more dynamic LDS than a kernel gets by default
        static bool raised = false;
        if (!raised) {
            e = hipFuncSetAttribute((const void*)qgemm_q4_0_kernel<2, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e == hipSuccess)
                e = hipFuncSetAttribute((const void*)qgemm_q4_0_kernel<2, false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return e;
            raised = true;
        }
    }
#define QGEMM_LAUNCH(MT, F32)                                                                                                      \
    hipLaunchKernelGGL((qgemm_q4_0_kernel<MT, F32>), grid, dim3(256), lds, st, (const uint16_t*)X, (const uint8_t*)W,              \
                       (const float*)workspace, Y, (int)M, (int)N, (int)K, x_row_stride, tiles_m, ntiles)
    if (tall) {
        if (out_f32) QGEMM_LAUNCH(2, true); else QGEMM_LAUNCH(2, false);
    } else {
        if (out_f32) QGEMM_LAUNCH(1, true); else QGEMM_LAUNCH(1, false);
    }
#undef QGEMM_LAUNCH
    return hipGetLastError();
}

}  // namespace mimir
