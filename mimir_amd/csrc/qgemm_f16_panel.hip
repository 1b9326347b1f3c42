// Q4_0 weights by many rows of X on the binary16 matrix cores, for products large enough to pay for a pass over W
// first: the approximate form of the prompt-sized product (weights rounded once to binary16, as qgemm_q4_0.hip's
// template argument HALF does inside its tiles), split into two launches.
//
//   1. panel_prepare_kernel writes W once as a plain binary16 panel P [N, K]: weight (n - 8) d rounded to nearest,
//      the same instruction sequence as the tile kernel's, so the same bits. A weight is converted once here instead
//      of once per 256 rows of X there. The same launch brings X to binary16 (X16, rows scaled by a power of two each,
//      half_rows.h), in workgroups of its own that run beside the panel's.
//   2. hgemm_f16_nt_kernel multiplies X16 [M, K] by P: 256 x 256 tiles of Y, eight wavefronts of 128 x 64 each,
//      steps of 64 along K through two stages of LDS. Both operands go from global memory straight into LDS
//      (global_load_lds_dwordx4: no registers, no vector arithmetic in the wavefronts that share a SIMD with the MFMAs);
//      a row of a stage is 128 bytes and its eight 16-byte pieces are placed at piece ^ (row / 2 mod 8), which the
//      loading lane undoes in the address it reads from, so that the fragment reads of v_mfma_f32_32x32x16_f16
//      (32 rows, the same piece) spread over all banks. The loads of the next step are issued in two parts with
//      the first two of a step's four groups of MFMAs (issued later they had not landed by the step's end, issued all
//      at once they hold the wavefront up), and the fragments of the next group are read while the current group
//      multiplies.
//
// A compute unit holds one workgroup (128 KB of LDS), so a product takes as long as the unit with the most tiles. Where
// 256 x 256 tiles would leave the last round partly empty (2048 x 14336: 448 tiles on 256 units), the right-hand
// columns of Y are cut into tiles of 256 x 192 instead, handed out after the wide ones (32 + 32 column tiles there: one
// wide and one narrow tile a unit); products with too few wide tiles for the device take 128 x 256 tiles. The cut is
// chosen on the host by the time the last tile ends (plan_panel).
//
// Workgroups go round-robin over the eight dies; a die takes a contiguous range of tiles with the tile's row of X
// varying fastest, so the 32 workgroups a die runs together share 4 column panels of P and the 8 row panels of X
// through the die's L2.
//
// Reference semantics: Tensor.MatMulT for a half-precision x and block-quantized w, tensor/quant.go:45-48.
#include "device_util.h"
#include "half_rows.h"
#include "kernels.h"
#include "tile_plan.h"

namespace mimir {

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kStep = 64;              // of K a step
constexpr int kRowBytes = kStep * 2;   // a row of a stage in LDS

// A workgroup's tile of Y: WM x (8 / WM) wavefronts of (32 MT) x (32 NT) each.
template <int WM, int MT, int NT>
struct Tile {
    static constexpr int WN = 8 / WM, kMT = MT, kNT = NT;
    static constexpr int BM = WM * 32 * MT, BN = WN * 32 * NT;
    static constexpr int kRows = BM + BN;                // rows of a stage: X's, then P's
    static constexpr int kLoads = kRows / 64;            // 1 KB loads (8 rows) a wavefront issues per step
    static constexpr int kStageBytes = kRows * kRowBytes;
    static_assert(kRows % 64 == 0 && BM % 8 == 0, "whole loads, none across the two operands");
};
using Wide = Tile<2, 4, 2>;    // 256 x 256: the most MFMAs per byte read from LDS (0.75 fragment reads an MFMA)
using Narrow = Tile<4, 2, 3>;  // 256 x 192: three quarters of a Wide tile, to fill a last round that Wide tiles would leave a quarter empty
using Low = Tile<2, 2, 2>;     // 128 x 256: for products with too few Wide tiles for the device
constexpr size_t kLdsBytes = 2 * (size_t)Wide::kStageBytes;

// The pass before the product, one launch: workgroups [0, M) bring a row of X each to binary16 (half_rows.h), the
// others write the panel. Sixteen weights a thread there: the low and the high nibbles of eight bytes of a block, as
// the binary16 values (n - 8) d.
__global__ __launch_bounds__(256) void panel_prepare_kernel(const uint16_t* __restrict__ X, uint16_t* __restrict__ X16, float* __restrict__ scale_back,
                                                            int M, int64_t K, int64_t x_row_stride, const uint8_t* __restrict__ W,
                                                            uint16_t* __restrict__ P, int64_t halves) {
    if ((int)blockIdx.x < M) {
        bf16_row_to_f16_scaled(X, X16, scale_back, K, x_row_stride, blockIdx.x);
        return;
    }
    const int64_t first = (int64_t)((int)blockIdx.x - M) * 256 + threadIdx.x, stride = (int64_t)((int)gridDim.x - M) * 256;
    for (int64_t t = first; t < halves; t += stride) {
        const int q = (int)(t & 1);
        const uint8_t* blk = W + (t >> 1) * 18;
        const uint16_t rd = *(const uint16_t*)blk;  // blocks are 2-byte aligned, no more
        const uint16_t* src = (const uint16_t*)(blk + 2 + 8 * q);
        const uint32_t raw[2] = {(uint32_t)src[0] | (uint32_t)src[1] << 16, (uint32_t)src[2] | (uint32_t)src[3] << 16};
        const _Float16 dh = __builtin_bit_cast(_Float16, rd);
        const f16x2 d2 = {dh, dh}, off = {(_Float16)1032.f, (_Float16)1032.f};
        uint16_t* out = P + (t >> 1) * 32 + 8 * q;  // elements 8 q .. 8 q + 7 (low nibbles) and 16 more on (high nibbles)
#pragma unroll
        for (int half = 0; half < 2; half++) {
            u32x4 v;
#pragma unroll
            for (int i = 0; i < 2; i++) {
                // the nibble into the mantissa of binary16's 1024, minus 1032 is n - 8, times d rounds once
                const uint32_t nib = (raw[i] >> (4 * half)) & 0x0f0f0f0fu;
                const uint32_t p0 = __builtin_amdgcn_perm(0x64646464u, nib, 0x04010400u);
                const uint32_t p1 = __builtin_amdgcn_perm(0x64646464u, nib, 0x04030402u);
                const f16x2 w0 = (__builtin_bit_cast(f16x2, p0) - off) * d2;
                const f16x2 w1 = (__builtin_bit_cast(f16x2, p1) - off) * d2;
                v[2 * i] = __builtin_bit_cast(uint32_t, w0);
                v[2 * i + 1] = __builtin_bit_cast(uint32_t, w1);
            }
            *(u32x4*)(out + 16 * half) = v;
        }
    }
}

// 16 bytes a lane from global memory into LDS: lane l's piece lands at lds_base + 16 l. Written out because the
// compiler, given the builtin, waits for every load under way before any LDS access; these loads are counted by hand.
// The instruction takes its LDS base from M0, which the compiler does not let an asm statement name as clobbered: nothing
// else in this kernel uses M0 (no dynamically indexed registers, no LDS-direct reads), and it is set anew before every load.
__device__ __forceinline__ void load_to_lds(const void* g, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_base), "v"(g) : "memory");
}
__device__ __forceinline__ void wait_loads() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// One tile: Y [m0 .. m0 + BM) x [n0 .. n0 + BN) = (X16 . P^T) row_scale[m], float32 sums, Y bfloat16 or float32.
template <class T, bool OUT_F32>
__device__ __forceinline__ void tile_body(const uint16_t* __restrict__ X16, const uint16_t* __restrict__ P, void* __restrict__ Yv,
                                          const float* __restrict__ row_scale, int M, int N, int K, int m0, int n0, char* lds) {
    constexpr int MT = T::kMT, NT = T::kNT;
    constexpr int kLoads = T::kLoads;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / T::WN, wn = wave % T::WN;

    // This wavefront's loads: load g = kLoads wave + j brings rows [8 g, 8 g + 8) of the stage, X's below BM and P's
    // from there. Rows past the matrix re-read its last row (their results are not stored).
    const char* from[kLoads];
    uint32_t into[kLoads];
#pragma unroll
    for (int j = 0; j < kLoads; j++) {
        const int first = 8 * (kLoads * wave + j);
        const int row = first + (lane >> 3);
        const int piece = (lane & 7) ^ ((row >> 1) & 7);
        const uint16_t* base;
        if (first < T::BM) {
            const int m = m0 + row < M ? m0 + row : M - 1;
            base = X16 + (size_t)m * K;
        } else {
            const int n = n0 + row - T::BM < N ? n0 + row - T::BM : N - 1;
            base = P + (size_t)n * K;
        }
        from[j] = (const char*)(base + 8 * piece);
        into[j] = (uint32_t)(first * kRowBytes);
    }
    const uint32_t lds0 = (uint32_t)(uintptr_t)lds;

    const int r32 = lane & 31, hi = lane >> 5;
    const int swz = (r32 >> 1) & 7;
    int piece_off[4];
#pragma unroll
    for (int kk = 0; kk < 4; kk++) piece_off[kk] = ((2 * kk + hi) ^ swz) * 16;
    const int a_row = (wm * 32 * MT + r32) * kRowBytes, b_row = (T::BM + wn * 32 * NT + r32) * kRowBytes;

    f32x16 acc[MT][NT];
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int nt = 0; nt < NT; nt++)
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
        const uint32_t next = lds0 + ((i + 1) & 1) * T::kStageBytes;
        const char* st = lds + (i & 1) * T::kStageBytes;
        f16x8 a[2][MT], b[2][NT];
#pragma unroll
        for (int mt = 0; mt < MT; mt++) a[0][mt] = *(const f16x8*)(st + a_row + mt * 32 * kRowBytes + piece_off[0]);
#pragma unroll
        for (int nt = 0; nt < NT; nt++) b[0][nt] = *(const f16x8*)(st + b_row + nt * 32 * kRowBytes + piece_off[0]);
#pragma unroll
        for (int kk = 0; kk < 4; kk++) {
            const int c = kk & 1, n = c ^ 1;
            if (more && kk < 2) {  // half of the next step's loads: all of them early in the step, so that they have landed by its end
#pragma unroll
                for (int j = kk * kLoads / 2; j < (kk + 1) * kLoads / 2; j++) {
                    load_to_lds(from[j], __builtin_amdgcn_readfirstlane(next + into[j]));
                    from[j] += kRowBytes;
                }
            }
            if (kk + 1 < 4) {
#pragma unroll
                for (int mt = 0; mt < MT; mt++) a[n][mt] = *(const f16x8*)(st + a_row + mt * 32 * kRowBytes + piece_off[kk + 1]);
#pragma unroll
                for (int nt = 0; nt < NT; nt++) b[n][nt] = *(const f16x8*)(st + b_row + nt * 32 * kRowBytes + piece_off[kk + 1]);
            }
#pragma unroll
            for (int mt = 0; mt < MT; mt++)
#pragma unroll
                for (int nt = 0; nt < NT; nt++) acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[c][mt], b[c][nt], acc[mt][nt], 0, 0, 0);
            if (kk + 1 < 4) {  // one fragment read between two MFMAs
#pragma unroll
                for (int q = 0; q < MT + NT; q++) {
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                }
                if (MT * NT > MT + NT) __builtin_amdgcn_sched_group_barrier(0x008, MT * NT - MT - NT, 0);
            }
        }
    }

    // The row's scale undone (a power of two: exact), then one rounding to the output's dtype (f32ToBF16,
    // backend/cpu/half.go:42-51). An MFMA leaves a lane one column of Y and four consecutive rows per group of four
    // registers; a 4 x 4 transposition within each quad of lanes turns that into one row and four consecutive columns a
    // lane, so that a group is stored with one 8-byte (bfloat16) or 16-byte (float32) store a lane instead of four
    // narrow ones (the stores of the untransposed form took 5 % of the launch).
    const bool wide_ok = (N & 3) == 0 && ((uintptr_t)Yv & 15) == 0;
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const int m = m0 + wm * 32 * MT + mt * 32 + q * 8 + hi * 4 + (lane & 3);
            const float back = m < M ? row_scale[m] : 0.f;
#pragma unroll
            for (int nt = 0; nt < NT; nt++) {
                float v[4] = {acc[mt][nt][4 * q], acc[mt][nt][4 * q + 1], acc[mt][nt][4 * q + 2], acc[mt][nt][4 * q + 3]};
                quad_transpose(v, lane);
                const int n = n0 + wn * 32 * NT + nt * 32 + (r32 & ~3);
                if (m >= M || n >= N) continue;
#pragma unroll
                for (int k = 0; k < 4; k++) v[k] = v[k] * back;
                if (wide_ok && n + 3 < N) {
                    if (OUT_F32) {
                        const f32x4 o = {v[0], v[1], v[2], v[3]};
                        *(f32x4*)((float*)Yv + (int64_t)m * N + n) = o;
                    } else {
                        const u32x2 o = {(uint32_t)f32_to_bf16_bits(v[0]) | (uint32_t)f32_to_bf16_bits(v[1]) << 16,
                                         (uint32_t)f32_to_bf16_bits(v[2]) | (uint32_t)f32_to_bf16_bits(v[3]) << 16};
                        *(u32x2*)((uint16_t*)Yv + (int64_t)m * N + n) = o;
                    }
                } else {
#pragma unroll
                    for (int k = 0; k < 4; k++) {
                        if (n + k >= N) continue;
                        if (OUT_F32) ((float*)Yv)[(int64_t)m * N + n + k] = v[k];
                        else ((uint16_t*)Yv)[(int64_t)m * N + n + k] = f32_to_bf16_bits(v[k]);
                    }
                }
            }
        }
}

// A die's workgroups (every eighth, round-robin) take a contiguous range of the tiles, the tile's row of X varying
// fastest: the 32 that run together share 4 column panels of P and the 8 row panels of X through the die's L2.
__device__ __forceinline__ int tile_of(int b, int ntiles) {
    const int per_die = (ntiles + 7) >> 3;
    return (b & 7) * per_die + (b >> 3);
}

template <bool OUT_F32>
__global__ __launch_bounds__(512, 2) void hgemm_f16_nt_kernel(const uint16_t* __restrict__ X16, const uint16_t* __restrict__ P, void* __restrict__ Yv,
                                                              const float* __restrict__ row_scale, int M, int N, int K, PanelPlan plan) {
    extern __shared__ __align__(1024) char lds_gemm[];
    int b = (int)blockIdx.x;
    if (plan.low) {
        const int ntiles = plan.tiles_m * plan.wide_cols;
        const int t = tile_of(b, ntiles);
        if (t >= ntiles) return;  // the whole workgroup
        tile_body<Low, OUT_F32>(X16, P, Yv, row_scale, M, N, K, (t % plan.tiles_m) * Low::BM, (t / plan.tiles_m) * Low::BN, lds_gemm);
        return;
    }
    const int nwide = plan.tiles_m * plan.wide_cols;
    const int wide_wgs = ((nwide + 7) >> 3) << 3;
    if (b < wide_wgs) {
        const int t = tile_of(b, nwide);
        if (t >= nwide) return;
        tile_body<Wide, OUT_F32>(X16, P, Yv, row_scale, M, N, K, (t % plan.tiles_m) * Wide::BM, (t / plan.tiles_m) * Wide::BN, lds_gemm);
        return;
    }
    b -= wide_wgs;
    const int nnarrow = plan.tiles_m * plan.narrow_cols;
    const int t = tile_of(b, nnarrow);
    if (t >= nnarrow) return;
    tile_body<Narrow, OUT_F32>(X16, P, Yv, row_scale, M, N, K, (t % plan.tiles_m) * Narrow::BM, plan.wide_cols * Wide::BN + (t / plan.tiles_m) * Narrow::BN,
                               lds_gemm);
}

// Costs in Wide tiles' time: a Narrow tile has three quarters of the MFMAs and reads a little more from LDS for each,
// a Low tile half of them and a third more.
constexpr double kNarrowCost = 0.78, kLowCost = 0.56;

}  // namespace

size_t qgemm_f16_panel_bytes(int64_t N, int64_t K) { return ((size_t)N * K * 2 + 255) & ~(size_t)255; }

// Whether the two launches beat the one whose tiles convert W for themselves: the panel costs a pass over W
// (N K (0.5625 + 2) bytes), which at least 1024 rows of X repay when the tiles keep 70 % of the device busy
// until the last one ends (at 512 x 14336 x 4096 the two routes measured the same, 544 and 551 TFLOP/s).
bool qgemm_f16_panel_pays(int64_t M, int64_t N, int64_t K) {
    if (!(M >= 1024 && K % kStep == 0 && K >= kStep && M < (1 << 24) && N < (1 << 24) && K < (1 << 24) && N > 0)) return false;
    PanelPlan plan;
    const double end = plan_panel(M, N, kNarrowCost, kLowCost, &plan);
    const double work = (double)M * (double)N / (256.0 * 256.0);
    return work >= 0.70 * kUnits * end;
}

hipError_t qgemm_f16_panel(const void* W, const void* X, int64_t x_row_stride, void* X16, float* row_scale, void* Y, int64_t M, int64_t N, int64_t K,
                           bool out_f32, void* panel, hipStream_t st) {
    {
        static std::atomic<bool> raised{false};  // threads may race here: both then set the same attribute
        if (!raised) {
            hipError_t e = hipFuncSetAttribute((const void*)hgemm_f16_nt_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsBytes);
            if (e == hipSuccess) e = hipFuncSetAttribute((const void*)hgemm_f16_nt_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsBytes);
            if (e != hipSuccess) return e;
            raised = true;
        }
    }
    const int64_t halves = N * K / 16;
    const int64_t want = (halves + 255) / 256;
    hipLaunchKernelGGL(panel_prepare_kernel, dim3((unsigned)(M + (want > 8192 ? 8192 : want))), dim3(256), 0, st, (const uint16_t*)X, (uint16_t*)X16, row_scale,
                       (int)M, K, x_row_stride, (const uint8_t*)W, (uint16_t*)panel, halves);
    PanelPlan plan;
    plan_panel(M, N, kNarrowCost, kLowCost, &plan);
    const int first = plan.tiles_m * plan.wide_cols, then = plan.tiles_m * plan.narrow_cols;
    note_kernel("hgemm_f16_nt_kernel: %d x %d tiles of %s, %d x %d tiles of 256 x 192", plan.tiles_m, plan.wide_cols, plan.low ? "128 x 256" : "256 x 256",
                plan.tiles_m, plan.narrow_cols);
    const dim3 grid((unsigned)(((first + 7) / 8) * 8 + ((then + 7) / 8) * 8));
    if (out_f32)
        hipLaunchKernelGGL(hgemm_f16_nt_kernel<true>, grid, dim3(512), kLdsBytes, st, (const uint16_t*)X16, (const uint16_t*)panel, Y, row_scale, (int)M,
                           (int)N, (int)K, plan);
    else
        hipLaunchKernelGGL(hgemm_f16_nt_kernel<false>, grid, dim3(512), kLdsBytes, st, (const uint16_t*)X16, (const uint16_t*)panel, Y, row_scale, (int)M,
                           (int)N, (int)K, plan);
    return hipGetLastError();
}

}  // namespace mimir
