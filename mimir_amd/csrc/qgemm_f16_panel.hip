// Q4_0 weights by many rows of X on the binary16 matrix cores, for products large enough to pay for a pass over W
// first: the approximate form of the prompt-sized product (weights rounded once to binary16, as qgemm_q4_0.hip's
// template argument HALF does inside its tiles), split into two launches.
//
//   1. q4_0_f16_panel_kernel writes W once as a plain binary16 panel P [N, K]: weight (n - 8) d rounded to nearest,
//      the same instruction sequence as the tile kernel's, so the same bits. A weight is converted once here instead
//      of once per 256 rows of X there.
//   2. hgemm_f16_nt_kernel multiplies X16 [M, K] (binary16, rows scaled by a power of two beforehand,
//      bf16_rows_to_f16_scaled in qgemm_q4_0.hip) by P: 256 x 256 tiles of Y, eight wavefronts of 128 x 64 each,
//      steps of 64 along K through two stages of LDS. Both operands go from global memory straight into LDS
//      (global_load_lds_dwordx4: no registers, no vector arithmetic in the wavefronts that share a SIMD with the MFMAs);
//      a row of a stage is 128 bytes and its eight 16-byte pieces are placed at piece ^ (row / 2 mod 8), which the
//      loading lane undoes in the address it reads from, so that the fragment reads of v_mfma_f32_32x32x16_f16
//      (32 rows, the same piece) spread over all banks. The loads of the next step are issued in four parts between
//      the four groups of MFMAs of a step, and the fragments of the next group are read while the current group
//      multiplies.
//
// Workgroups go round-robin over the eight dies; a die takes a contiguous range of tiles with the tile's row of X
// varying fastest, so the 32 workgroups a die runs together share 4 column panels of P and the 8 row panels of X
// through the die's L2.
//
// Reference semantics: Tensor.MatMulT for a half-precision x and block-quantized w, tensor/quant.go:45-48.
#include "device_util.h"
#include "kernels.h"

namespace mimir {

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kTile = 256;                        // rows of X and rows of W a workgroup multiplies
constexpr int kStep = 64;                         // of K a step
constexpr int kRowBytes = kStep * 2;              // a row of a stage in LDS
constexpr int kStageBytes = 2 * kTile * kRowBytes;  // X's 256 rows, then P's 256 rows
constexpr int kLoads = 8;                         // 1 KB loads a wavefront issues per step: 64 of the stage's 512 rows, 8 rows a load
constexpr size_t kLdsBytes = 2 * (size_t)kStageBytes;

// Eight weights a thread: the low or high nibbles of eight bytes of a block, as the binary16 values (n - 8) d.
__global__ __launch_bounds__(256) void q4_0_f16_panel_kernel(const uint8_t* __restrict__ W, uint16_t* __restrict__ P, int64_t pieces) {
    for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < pieces; t += (int64_t)gridDim.x * 256) {
        const int q = (int)(t & 3);
        const uint8_t* blk = W + (t >> 2) * 18;
        const uint16_t rd = *(const uint16_t*)blk;  // blocks are 2-byte aligned, no more
        const uint16_t* src = (const uint16_t*)(blk + 2 + 8 * (q & 1));
        const uint32_t raw[2] = {(uint32_t)src[0] | (uint32_t)src[1] << 16, (uint32_t)src[2] | (uint32_t)src[3] << 16};
        const _Float16 dh = __builtin_bit_cast(_Float16, rd);
        const f16x2 d2 = {dh, dh}, off = {(_Float16)1032.f, (_Float16)1032.f};
        u32x4 out;
#pragma unroll
        for (int i = 0; i < 2; i++) {
            // the nibble into the mantissa of binary16's 1024, minus 1032 is n - 8, times d rounds once
            const uint32_t nib = (raw[i] >> (4 * (q >> 1))) & 0x0f0f0f0fu;
            const uint32_t p0 = __builtin_amdgcn_perm(0x64646464u, nib, 0x04010400u);
            const uint32_t p1 = __builtin_amdgcn_perm(0x64646464u, nib, 0x04030402u);
            const f16x2 w0 = (__builtin_bit_cast(f16x2, p0) - off) * d2;
            const f16x2 w1 = (__builtin_bit_cast(f16x2, p1) - off) * d2;
            out[2 * i] = __builtin_bit_cast(uint32_t, w0);
            out[2 * i + 1] = __builtin_bit_cast(uint32_t, w1);
        }
        *(u32x4*)(P + 8 * t) = out;
    }
}

// 16 bytes a lane from global memory into LDS: lane l's piece lands at lds_base + 16 l. Written out because the
// compiler, given the builtin, waits for every load under way before any LDS access; these loads are counted by hand.
__device__ __forceinline__ void load_to_lds(const void* g, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_base), "v"(g) : "memory");
}
__device__ __forceinline__ void wait_loads() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// Y [M, N] = (X16 [M, K] . P [N, K]^T) row_scale[m], float32 sums, Y bfloat16 or float32. K a multiple of 64.
template <bool OUT_F32>
__global__ __launch_bounds__(512, 2) void hgemm_f16_nt_kernel(const uint16_t* __restrict__ X16, const uint16_t* __restrict__ P, void* __restrict__ Yv,
                                                              const float* __restrict__ row_scale, int M, int N, int K, int tiles_m, int ntiles) {
    extern __shared__ __align__(1024) char lds_gemm[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 2, wn = wave & 3;
    const int per_die = (ntiles + 7) >> 3;
    const int t = ((int)blockIdx.x & 7) * per_die + ((int)blockIdx.x >> 3);
    if (t >= ntiles) return;  // the whole workgroup
    const int m0 = (t % tiles_m) * kTile, n0 = (t / tiles_m) * kTile;

    // This wavefront's loads: rows [64 wave, 64 wave + 64) of the stage, X's for wavefronts 0-3 and P's for 4-7.
    // Rows past the matrix re-read its last row (their results are not stored).
    const char* from[kLoads];
    uint32_t into[kLoads];
#pragma unroll
    for (int j = 0; j < kLoads; j++) {
        const int row = 64 * wave + 8 * j + (lane >> 3);
        const int piece = (lane & 7) ^ ((row >> 1) & 7);
        const uint16_t* base;
        if (wave < 4) {
            const int m = m0 + row < M ? m0 + row : M - 1;
            base = X16 + (size_t)m * K;
        } else {
            const int n = n0 + row - kTile < N ? n0 + row - kTile : N - 1;
            base = P + (size_t)n * K;
        }
        from[j] = (const char*)(base + 8 * piece);
        into[j] = (uint32_t)((64 * wave + 8 * j) * kRowBytes);
    }
    const uint32_t lds0 = (uint32_t)(uintptr_t)lds_gemm;

    const int r32 = lane & 31, hi = lane >> 5;
    const int swz = (r32 >> 1) & 7;
    int piece_off[4];
#pragma unroll
    for (int kk = 0; kk < 4; kk++) piece_off[kk] = ((2 * kk + hi) ^ swz) * 16;
    const int a_row = (wm * 128 + r32) * kRowBytes, b_row = (kTile + wn * 64 + r32) * kRowBytes;

    f32x16 acc[4][2];
#pragma unroll
    for (int mt = 0; mt < 4; mt++)
#pragma unroll
        for (int nt = 0; nt < 2; nt++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[mt][nt][i] = 0.f;

    const int nk = K / kStep;
#pragma unroll
    for (int j = 0; j < kLoads; j++) {
        load_to_lds(from[j], __builtin_amdgcn_readfirstlane(lds0 + into[j]));
        from[j] += kRowBytes;
    }
    for (int i = 0; i < nk; i++) {
        wait_loads();   // this wavefront's part of step i has landed
        lds_barrier();  // everyone's has, and everyone has read the other stage for the last time
        const bool more = i + 1 < nk;
        const uint32_t next = lds0 + ((i + 1) & 1) * kStageBytes;
        const char* st = lds_gemm + (i & 1) * kStageBytes;
        f16x8 a[2][4], b[2][2];
#pragma unroll
        for (int mt = 0; mt < 4; mt++) a[0][mt] = *(const f16x8*)(st + a_row + mt * 32 * kRowBytes + piece_off[0]);
#pragma unroll
        for (int nt = 0; nt < 2; nt++) b[0][nt] = *(const f16x8*)(st + b_row + nt * 32 * kRowBytes + piece_off[0]);
#pragma unroll
        for (int kk = 0; kk < 4; kk++) {
            const int c = kk & 1, n = c ^ 1;
            if (more) {  // a quarter of the next step's loads
#pragma unroll
                for (int j = 2 * kk; j < 2 * kk + 2; j++) {
                    load_to_lds(from[j], __builtin_amdgcn_readfirstlane(next + into[j]));
                    from[j] += kRowBytes;
                }
            }
            if (kk + 1 < 4) {
#pragma unroll
                for (int mt = 0; mt < 4; mt++) a[n][mt] = *(const f16x8*)(st + a_row + mt * 32 * kRowBytes + piece_off[kk + 1]);
#pragma unroll
                for (int nt = 0; nt < 2; nt++) b[n][nt] = *(const f16x8*)(st + b_row + nt * 32 * kRowBytes + piece_off[kk + 1]);
            }
#pragma unroll
            for (int mt = 0; mt < 4; mt++)
#pragma unroll
                for (int nt = 0; nt < 2; nt++) acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[c][mt], b[c][nt], acc[mt][nt], 0, 0, 0);
            if (kk + 1 < 4) {  // one fragment read between two MFMAs
#pragma unroll
                for (int q = 0; q < 6; q++) {
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                }
                __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
            }
        }
    }

    // the row's scale undone (a power of two: exact), then one rounding to the output's dtype (f32ToBF16, backend/cpu/half.go:42-51)
#pragma unroll
    for (int mt = 0; mt < 4; mt++)
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int m = m0 + wm * 128 + mt * 32 + (i >> 2) * 8 + hi * 4 + (i & 3);
            if (m >= M) continue;
            const float back = row_scale[m];
#pragma unroll
            for (int nt = 0; nt < 2; nt++) {
                const int n = n0 + wn * 64 + nt * 32 + r32;
                if (n >= N) continue;
                const float v = acc[mt][nt][i] * back;
                if (OUT_F32) ((float*)Yv)[(int64_t)m * N + n] = v;
                else ((uint16_t*)Yv)[(int64_t)m * N + n] = f32_to_bf16_bits(v);
            }
        }
}

}  // namespace

size_t qgemm_f16_panel_bytes(int64_t N, int64_t K) { return ((size_t)N * K * 2 + 255) & ~(size_t)255; }

// Whether the two launches beat the one whose tiles convert W for themselves: the panel costs a pass over W
// (N K (0.5625 + 2) bytes), which 256 rows of X a tile and at least 1024 rows in all repay, and the 256 x 256 tiles
// must keep three quarters of the compute units busy.
bool qgemm_f16_panel_pays(int64_t M, int64_t N, int64_t K) {
    const int64_t tiles = ((M + kTile - 1) / kTile) * ((N + kTile - 1) / kTile);
    return M >= 1024 && K % kStep == 0 && K >= kStep && tiles >= 192 && M < (1 << 24) && N < (1 << 24) && K < (1 << 24);
}

hipError_t qgemm_f16_panel(const void* W, const void* X16, const float* row_scale, void* Y, int64_t M, int64_t N, int64_t K, bool out_f32,
                           void* panel, hipStream_t st) {
    {
        static std::atomic<bool> raised{false};  // threads may race here: both then set the same attribute
        if (!raised) {
            hipError_t e = hipFuncSetAttribute((const void*)hgemm_f16_nt_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsBytes);
            if (e == hipSuccess) e = hipFuncSetAttribute((const void*)hgemm_f16_nt_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsBytes);
            if (e != hipSuccess) return e;
            raised = true;
        }
    }
    const int64_t pieces = N * K / 8;
    const int64_t want = (pieces + 255) / 256;
    hipLaunchKernelGGL(q4_0_f16_panel_kernel, dim3((unsigned)(want > 8192 ? 8192 : want)), dim3(256), 0, st, (const uint8_t*)W, (uint16_t*)panel, pieces);
    const int tiles_m = (int)((M + kTile - 1) / kTile);
    const int ntiles = tiles_m * (int)((N + kTile - 1) / kTile);
    const dim3 grid((unsigned)(((ntiles + 7) / 8) * 8));
    if (out_f32)
        hipLaunchKernelGGL(hgemm_f16_nt_kernel<true>, grid, dim3(512), kLdsBytes, st, (const uint16_t*)X16, (const uint16_t*)panel, Y, row_scale, (int)M,
                           (int)N, (int)K, tiles_m, ntiles);
    else
        hipLaunchKernelGGL(hgemm_f16_nt_kernel<false>, grid, dim3(512), kLdsBytes, st, (const uint16_t*)X16, (const uint16_t*)panel, Y, row_scale, (int)M,
                           (int)N, (int)K, tiles_m, ntiles);
    return hipGetLastError();
}

}  // namespace mimir
