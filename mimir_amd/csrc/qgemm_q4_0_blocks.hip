// The exact form of the prompt-sized Q4_0 product with bfloat16 activations (qgemm_q4_0.hip: no operand is rounded,
// float32 sums), for products large enough to pay for a pass over W first, with one MFMA a weight instead of two.
//
// The tile kernel multiplies x by the weights (n - 8) d, which have up to 15 significant bits and so enter the
// bfloat16 matrix cores as two halves. Here the scale stays out of the matrix cores: the weights enter as their
// integers n - 8, exact in bfloat16, so that a block's products x (n - 8) are exact (8 by 4 significant bits) and
// v_mfma_f32_32x32x16_bf16 leaves the block's sum in float32; one FMA per output and block then adds d times that sum
// (d, the block's binary16 scale, is exact in float32, and W's row is a lane's column of the MFMA's result, so the scale
// is one register a lane). Nothing is rounded but float32 sums, as in the tile kernel; which sums are formed differs, so
// the results differ in the last bits like two orders of addition do (the tests' bound is the same for both).
//
// Two launches. blocks_panel_kernel writes W's integers once as a bfloat16 panel P [N, K]. qgemm_q4_0_blocks_kernel
// multiplies X, read where the caller has it, by P: a workgroup of eight wavefronts owns a tile of Y of 256 x 256 (a
// wavefront 128 x 64), 256 x 192 (64 x 96) or 128 x 256 (64 x 64), cut as tile_plan.h says so that the last round of
// tiles leaves few compute units idle; a stage is a pair of
// blocks (64 of K); both operands go from global memory straight into LDS (global_load_lds_dwordx4), rows of 128 bytes
// with their 16-byte pieces at piece ^ (row / 2 mod 8), so that the 32 rows of a fragment read fall on all banks; the
// scales pass through registers, read from the blocks themselves. The two MFMAs of a 32 x 32 sub-tile and block are
// issued with the FMAs of the sub-tile before it.
//
// Reference semantics: Tensor.MatMulT for a half-precision x and block-quantized w, tensor/quant.go:45-48.
#include "device_util.h"
#include "kernels.h"
#include "tile_plan.h"

namespace mimir {

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kRowBytes = 128;  // a row of a stage: 64 bfloat16
constexpr int kScaleRows = 256; // rows of W whose scales a stage holds (every thread stores one: 512 = 2 blocks x 256)

// A workgroup's tile of Y: WM x (8 / WM) wavefronts of (32 MT) x (32 NT) each.
template <int WM, int MT_, int NT_>
struct Shape {
    static constexpr int WN = 8 / WM, MT = MT_, NT = NT_;
    static constexpr int BM = WM * 32 * MT, BN = WN * 32 * NT;
    static constexpr int kLoads = (BM + BN) / 64;        // 1 KB loads (8 rows) a wavefront issues per stage
    static constexpr int b = BM * kRowBytes;             // the stage in LDS: X's rows, P's rows,
    static constexpr int sw = b + BN * kRowBytes;        // float [2][kScaleRows]: W's scales of the stage's two blocks
    static constexpr int bytes = sw + 2 * kScaleRows * 4;
    static_assert(bytes % 1024 == 0 && (BM + BN) % 64 == 0 && BM % 8 == 0 && BN <= kScaleRows, "whole loads, none across the operands");
};
using Wide = Shape<2, 4, 2>;    // 256 x 256
using Narrow = Shape<4, 2, 3>;  // 256 x 192: to fill a last round that wide tiles would leave partly empty
using Low = Shape<2, 2, 2>;     // 128 x 256: for products with too few wide tiles for the device
constexpr size_t kLdsBytes = 2 * (size_t)Wide::bytes;

// Sixteen weights a thread: the low and the high nibbles of eight bytes of a block, as the bfloat16 integers n - 8.
__global__ __launch_bounds__(256) void blocks_panel_kernel(const uint8_t* __restrict__ W, uint16_t* __restrict__ P, int64_t halves) {
    const int64_t first = (int64_t)blockIdx.x * 256 + threadIdx.x, stride = (int64_t)gridDim.x * 256;
    for (int64_t t = first; t < halves; t += stride) {
        const int q = (int)(t & 1);
        const uint16_t* src = (const uint16_t*)(W + (t >> 1) * 18 + 2 + 8 * q);  // blocks are 2-byte aligned, no more
        const uint32_t raw[2] = {(uint32_t)src[0] | (uint32_t)src[1] << 16, (uint32_t)src[2] | (uint32_t)src[3] << 16};
        uint16_t* out = P + (t >> 1) * 32 + 8 * q;  // elements 8 q .. 8 q + 7 (low nibbles) and 16 more on (high nibbles)
#pragma unroll
        for (int half = 0; half < 2; half++) {
            u32x4 v;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                // a small integer's float32 has nothing below its upper 16 bits: those are its bfloat16
                const uint32_t two = raw[i >> 1] >> (16 * (i & 1) + 4 * half);
                const float lo = (float)((int)(two & 15) - 8), hi = (float)((int)((two >> 8) & 15) - 8);
                v[i] = (__builtin_bit_cast(uint32_t, lo) >> 16) | (__builtin_bit_cast(uint32_t, hi) & 0xffff0000u);
            }
            *(u32x4*)(out + 16 * half) = v;
        }
    }
}

// 16 bytes a lane from global memory into LDS: lane l's piece lands at lds_base + 16 l. Written out because the
// compiler, given the builtin, waits for every load under way before any LDS access; these loads are counted by hand
// (the compiler does not see them, so its own waits for the register loads of the scales can only be longer than
// needed, never shorter: loads return in order). The instruction takes its LDS base from M0, which an asm statement
// cannot name as clobbered: nothing else in this kernel uses M0, and it is set anew before every load.
__device__ __forceinline__ void load_to_lds(const void* g, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_base), "v"(g) : "memory");
}
__device__ __forceinline__ void wait_loads() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// A die's workgroups (every eighth, round-robin) take a contiguous range of the tiles, the tile's rows of X varying
// fastest: those that run together share few column panels of P through the die's L2.
__device__ __forceinline__ int tile_of(int b, int ntiles) {
    const int per_die = (ntiles + 7) >> 3;
    return (b & 7) * per_die + (b >> 3);
}

// One tile: Y [m0 .. m0 + BM) x [n0 .. n0 + BN).
template <class S, bool OUT_F32>
__device__ __forceinline__ void tile_body(const uint8_t* __restrict__ W, const uint16_t* __restrict__ P, const uint16_t* __restrict__ X,
                                          int64_t x_row_stride, void* __restrict__ Yv, int M, int N, int K, int m0, int n0, char* lds) {
    constexpr int MT = S::MT, NT = S::NT;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / S::WN, wn = wave % S::WN;
    const int nb = K >> 5;

    // This wavefront's loads: load g = kLoads wave + j brings rows [8 g, 8 g + 8) of the stage, X's below BM and P's
    // from there. Rows past the matrix re-read its last row (their results are not stored).
    const char* from[S::kLoads];
    uint32_t into[S::kLoads];
#pragma unroll
    for (int j = 0; j < S::kLoads; j++) {
        const int first = 8 * (S::kLoads * wave + j);
        const int row = first + (lane >> 3);
        const int piece = (lane & 7) ^ ((row >> 1) & 7);
        const uint16_t* base;
        if (first < S::BM) {
            const int m = m0 + row < M ? m0 + row : M - 1;
            base = X + (size_t)m * x_row_stride;
        } else {
            const int n = n0 + row - S::BM < N ? n0 + row - S::BM : N - 1;
            base = P + (size_t)n * K;
        }
        from[j] = (const char*)(base + 8 * piece);
        into[j] = (uint32_t)(first * kRowBytes);
    }
    // the scales: thread t takes block t % 2 of the stage for row t / 2 of W
    const int srow = tid >> 1, sodd = tid & 1;
    const uint8_t* wscale = W + ((size_t)(n0 + srow < N ? n0 + srow : N - 1) * nb + sodd) * 18;
    const uint32_t lds0 = (uint32_t)(uintptr_t)lds;

    const int r32 = lane & 31, hi = lane >> 5;
    const int swz = (r32 >> 1) & 7;
    int piece_off[4];  // of a row's pieces 2 p + hi: half p % 2 of the stage's block p / 2
#pragma unroll
    for (int p = 0; p < 4; p++) piece_off[p] = ((2 * p + hi) ^ swz) * 16;
    const int a_row = (wm * 32 * MT + r32) * kRowBytes, b_row = S::b + (wn * 32 * NT + r32) * kRowBytes;

    f32x16 acc[MT][NT];
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int nt = 0; nt < NT; nt++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[mt][nt][i] = 0.f;

    const int nstages = K / 64;
    {
        const float dw = f16_bits_to_f32(load_u16(wscale));
#pragma unroll
        for (int j = 0; j < S::kLoads; j++) load_to_lds(from[j], __builtin_amdgcn_readfirstlane(lds0 + into[j]));
        ((float*)(lds + S::sw))[sodd * kScaleRows + srow] = dw;
    }
    // No branches around the loads and stores: past the end the last stage is requested and stored again, into the
    // buffer that is not being read.
    for (int i = 0; i < nstages; i++) {
        wait_loads();   // this wavefront's part of stage i has landed
        lds_barrier();  // everyone's has, with the scales, and everyone has read the other stage for the last time
        const int step = i + 1 < nstages ? 1 : 0;
        const uint32_t next = lds0 + ((i + 1) & 1) * S::bytes;
        char* next_p = lds + ((i + 1) & 1) * S::bytes;
        const char* st = lds + (i & 1) * S::bytes;
        wscale += 36 * step;
        const float next_dw = f16_bits_to_f32(load_u16(wscale));
#pragma unroll
        for (int odd = 0; odd < 2; odd++) {
            // half of the next stage's loads with each block
#pragma unroll
            for (int j = odd * S::kLoads / 2; j < (odd + 1) * S::kLoads / 2; j++) {
                from[j] += kRowBytes * step;
                load_to_lds(from[j], __builtin_amdgcn_readfirstlane(next + into[j]));
            }
            bf16x8 a[MT][2], b[NT][2];  // [sub-tile][half of the block]
#pragma unroll
            for (int mt = 0; mt < MT; mt++)
#pragma unroll
                for (int h = 0; h < 2; h++) a[mt][h] = *(const bf16x8*)(st + a_row + mt * 32 * kRowBytes + piece_off[2 * odd + h]);
#pragma unroll
            for (int nt = 0; nt < NT; nt++)
#pragma unroll
                for (int h = 0; h < 2; h++) b[nt][h] = *(const bf16x8*)(st + b_row + nt * 32 * kRowBytes + piece_off[2 * odd + h]);
            float dw[NT];
#pragma unroll
            for (int nt = 0; nt < NT; nt++) dw[nt] = ((const float*)(st + S::sw))[odd * kScaleRows + wn * 32 * NT + nt * 32 + r32];
            // Sub-tile s = NT mt + nt: its two MFMAs are issued with the FMAs of the sub-tile before it, so that the
            // vector unit works while the matrix cores do.
            f32x16 c[2];
            auto multiply = [&](int sub) {
                const int mt = sub / NT, nt = sub % NT;
                f32x16 zero;
#pragma unroll
                for (int e = 0; e < 16; e++) zero[e] = 0.f;
                c[sub & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[mt][0], b[nt][0], zero, 0, 0, 0);
                c[sub & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[mt][1], b[nt][1], c[sub & 1], 0, 0, 0);
            };
            auto finish = [&](int sub) {
                const int mt = sub / NT, nt = sub % NT;
#pragma unroll
                for (int e = 0; e < 16; e++) acc[mt][nt][e] = fmaf(dw[nt], c[sub & 1][e], acc[mt][nt][e]);
            };
            multiply(0);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int sub = 1; sub < MT * NT; sub++) {
                multiply(sub);
                finish(sub - 1);
                __builtin_amdgcn_sched_barrier(0);
            }
            finish(MT * NT - 1);
        }
        // the next stage's scales, at the end: by now their load has landed with everything requested before it
        __builtin_amdgcn_sched_barrier(0);
        ((float*)(next_p + S::sw))[sodd * kScaleRows + srow] = next_dw;
    }

    // One rounding to the output's dtype (f32ToBF16, backend/cpu/half.go:42-51). An MFMA leaves a lane one column of Y
    // and four consecutive rows per group of four registers; a 4 x 4 transposition within each quad of lanes turns that
    // into one row and four consecutive columns a lane, stored with one 8-byte (bfloat16) or 16-byte (float32) store.
    const bool wide_ok = (N & 3) == 0 && ((uintptr_t)Yv & 15) == 0;
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const int m = m0 + wm * 32 * MT + mt * 32 + q * 8 + hi * 4 + (lane & 3);
#pragma unroll
            for (int nt = 0; nt < NT; nt++) {
                float v[4] = {acc[mt][nt][4 * q], acc[mt][nt][4 * q + 1], acc[mt][nt][4 * q + 2], acc[mt][nt][4 * q + 3]};
                quad_transpose(v, lane);
                const int n = n0 + wn * 32 * NT + nt * 32 + (r32 & ~3);
                if (m >= M || n >= N) continue;
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

template <bool OUT_F32>
__global__ __launch_bounds__(512) void qgemm_q4_0_blocks_kernel(const uint8_t* __restrict__ W, const uint16_t* __restrict__ P,
                                                                const uint16_t* __restrict__ X, int64_t x_row_stride, void* __restrict__ Yv,
                                                                int M, int N, int K, PanelPlan plan) {
    extern __shared__ __align__(1024) char lds[];
    int b = (int)blockIdx.x;
    if (plan.low) {
        const int ntiles = plan.tiles_m * plan.wide_cols;
        const int t = tile_of(b, ntiles);
        if (t >= ntiles) return;  // the whole workgroup
        tile_body<Low, OUT_F32>(W, P, X, x_row_stride, Yv, M, N, K, (t % plan.tiles_m) * Low::BM, (t / plan.tiles_m) * Low::BN, lds);
        return;
    }
    const int nwide = plan.tiles_m * plan.wide_cols;
    const int wide_wgs = ((nwide + 7) >> 3) << 3;
    if (b < wide_wgs) {
        const int t = tile_of(b, nwide);
        if (t >= nwide) return;
        tile_body<Wide, OUT_F32>(W, P, X, x_row_stride, Yv, M, N, K, (t % plan.tiles_m) * Wide::BM, (t / plan.tiles_m) * Wide::BN, lds);
        return;
    }
    b -= wide_wgs;
    const int nnarrow = plan.tiles_m * plan.narrow_cols;
    const int t = tile_of(b, nnarrow);
    if (t >= nnarrow) return;
    tile_body<Narrow, OUT_F32>(W, P, X, x_row_stride, Yv, M, N, K, (t % plan.tiles_m) * Narrow::BM,
                               plan.wide_cols * Wide::BN + (t / plan.tiles_m) * Narrow::BN, lds);
}

// Costs in wide tiles' time, measured: a tile of 256 x 192 has three quarters of the work, one of 128 x 256 half.
constexpr double kNarrowCost = 0.78, kLowCost = 0.56;

std::atomic<int> g_blocks{1};  // measurement aid: 0 keeps every product on the tile kernel, 2 takes this one whatever the shape

}  // namespace

void set_q4_0_blocks(int v) { g_blocks = v; }

// The panel: N K bfloat16.
size_t qgemm_q4_0_blocks_ws_bytes(int64_t N, int64_t K) { return (size_t)N * (size_t)K * 2; }

// Whether the product is the faster here than in the tile kernel, the pass over W included: from about 200 tiles of
// 128 x 256 on (measured at K = 4096: 512 x 14336 484 against 404 TFLOP/s, 2048 x 4096 569 against 438, 2048 x 14336 757
// against 435; 1024 x 4096, 128 tiles, 327 against 362).
bool qgemm_q4_0_blocks_pays(int64_t M, int64_t N, int64_t K) {
    if (g_blocks == 0 || M <= 0 || N <= 0 || K <= 0 || K % 64 != 0) return false;
    if (g_blocks == 2) return true;
    return M >= 256 && ((M + 127) / 128) * ((N + 255) / 256) >= 192;
}

// X [M, K] bfloat16 (16-byte aligned, rows x_row_stride elements apart, a multiple of 8), W [N, K] Q4_0, Y [M, N] bfloat16
// or float32; ws: qgemm_q4_0_blocks_ws_bytes(N, K) bytes, 16-byte aligned.
hipError_t qgemm_q4_0_blocks(const void* W, const void* X, int64_t x_row_stride, void* Y, int64_t M, int64_t N, int64_t K, bool out_f32, void* ws,
                             hipStream_t st) {
    if (!ws || ((uintptr_t)ws & 15) != 0 || ((uintptr_t)X & 15) != 0 || x_row_stride % 8 != 0 || x_row_stride < K || ((uintptr_t)W & 1) != 0 ||
        M <= 0 || N <= 0 || K <= 0 || K % 64 != 0 || M >= (1 << 24) || N >= (1 << 24) || K > (1 << 24))
        return hipErrorInvalidValue;
    static std::atomic<bool> raised{false};  // threads may race here: both then set the same attributes
    if (!raised) {
        hipError_t e = hipFuncSetAttribute((const void*)qgemm_q4_0_blocks_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsBytes);
        if (e == hipSuccess) e = hipFuncSetAttribute((const void*)qgemm_q4_0_blocks_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsBytes);
        if (e != hipSuccess) return e;
        raised = true;
    }
    uint16_t* P = (uint16_t*)ws;
    const int64_t halves = N * (K / 32) * 2;
    const int64_t want = (halves + 255) / 256;
    hipLaunchKernelGGL(blocks_panel_kernel, dim3((unsigned)(want < 8192 ? want : 8192)), dim3(256), 0, st, (const uint8_t*)W, P, halves);
    PanelPlan plan;
    plan_panel(M, N, kNarrowCost, kLowCost, &plan);
    const int first = plan.tiles_m * plan.wide_cols, then = plan.tiles_m * plan.narrow_cols;
    const dim3 grid((unsigned)(((first + 7) / 8) * 8 + ((then + 7) / 8) * 8));
    if (out_f32)
        hipLaunchKernelGGL(qgemm_q4_0_blocks_kernel<true>, grid, dim3(512), kLdsBytes, st, (const uint8_t*)W, P, (const uint16_t*)X, x_row_stride, Y, (int)M,
                           (int)N, (int)K, plan);
    else
        hipLaunchKernelGGL(qgemm_q4_0_blocks_kernel<false>, grid, dim3(512), kLdsBytes, st, (const uint8_t*)W, P, (const uint16_t*)X, x_row_stride, Y, (int)M,
                           (int)N, (int)K, plan);
    note_kernel("qgemm_q4_0_blocks_kernel: %d x %d tiles of %s, %d x %d tiles of 256 x 192", plan.tiles_m, plan.wide_cols, plan.low ? "128 x 256" : "256 x 256",
                plan.tiles_m, plan.narrow_cols);
    return hipGetLastError();
}

}  // namespace mimir
