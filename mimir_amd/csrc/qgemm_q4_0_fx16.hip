// The fixed-point Q4_0 product of many rows of float32 x (qgemm_q4_0_fx.hip: x as a 24-bit integer per element and
// a float32 scale per block of 32, the exact integer sum per block, one FMA per block with the product of the two
// scales), from some hundreds of rows on, through the binary16 matrix cores, with the same bits.
//
// What bounds the int8 form is the vector unit: three digit sums per output and block have to be joined, converted
// and scaled, five instructions against three MFMAs per 1024 outputs. Here the 24-bit integer a of an element is cut
// into two balanced 12-bit digits, a = d0 + 4096 d1 with d0 in [-2048, 2047] and d1 in [-2048, 2048], and each digit is
// a binary16 number (binary16 holds integers up to 2048 exactly). The weights enter as the binary16 integers n - 8. A
// v_mfma_f32_32x32x16_f16 then sums products that are integers below 2^15 into float32 sums that stay below 2^20:
// every partial sum is an integer float32 holds exactly, in whatever order the instruction adds. Per block and
// output, c0 = sum d0 (n - 8) and c1 = sum d1 (n - 8) are exact, fma(c1, 4096, c0) is the exact integer sum rounded
// once to float32, which is what the int8 form's conversion of its 32-bit sum gives, and the block's term follows as
// there: acc = fma(dw dx, that, acc), blocks in their order. Three vector instructions per output and block instead
// of five, and no offset term (n - 8 is signed here).
//
// Two launches. fx16_panel_kernel writes W's integers once as a binary16 panel P [N, K] (the pass the approximate
// form's panel takes too, qgemm_f16_panel.hip, without the scales). qgemm_q4_0_fx16_kernel multiplies: a workgroup
// of eight wavefronts owns 128 rows of x by 256 rows of W, a wavefront 64 by 64; a stage is a pair of blocks (64 of K):
// the rows of x (128 bytes a row and block: 32 digits d0, then 32 digits d1), the rows of P (128 bytes a row: the two
// blocks) and the scales. Operands go from global memory straight into LDS (global_load_lds_dwordx4) with the 16-byte
// pieces of a row placed at piece ^ (row / 2 mod 8), so that the 32 rows of a fragment read fall on all banks; the
// scales pass through registers (W's are read from the blocks themselves). Two stages, one barrier a stage.
//
// The products of the two scales come from the matrix cores as well: dw dx over a sub-tile is an outer product, an
// MFMA with K = 1 on float32 operands (one exact product per output, nothing added: the rounding of a multiplication).
// That leaves the vector unit two instructions per output and block.
//
// What was measured on the way (2048 and 4096 rows by 14336 x 4096): tiles of 128 x 128 in workgroups of four
// wavefronts, two a compute unit, with everything loaded straight into LDS and three stages, 335 to 340 TFLOP/s against
// 350 to 360 here (half as many bytes again from L2 per product); the barrier moved to the middle of a block with the
// next block's fragments read under the last vector work, and the order of MFMAs and vector instructions inside a
// group imposed: no change. Under this kernel the device clock settles near 1.6 GHz, lower the fewer cycles a variant
// needs: the time did not follow the cycle counts.
//
// x converted by fx16_convert_kernel: X16 [M, K / 32, 64] binary16 digits, then XS [M, K / 32] float32 scales; the
// integers and scales are those of fx_convert_kernel and q4_convert_item.
//
// Reference semantics: the float32 product with the dequantized weights (io/mim/dtype.go:118-123,
// backend/cpu/gemv.go:73-104), to which the result agrees within 1e-3.
#include "device_util.h"
#include "kernels.h"
#include "q4_act.h"

namespace mimir {

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x32 __attribute__((ext_vector_type(32)));

constexpr int kBM = 128;        // rows of x a workgroup
constexpr int kBN = 256;        // rows of W a workgroup
constexpr int kRowBytes = 128;  // a row of a stage: 64 binary16
constexpr int kLoads = 8;       // 1 KB loads (8 rows) a wavefront issues per stage: 512 rows
constexpr int kMinRows = 256;   // fewer rows stay with the int8 form

// A stage in LDS: the rows of x for the even block, for the odd block, the rows of P, then the scales.
struct Stage {
    static constexpr int a = 0;                          // [2][kBM] rows
    static constexpr int b = 2 * kBM * kRowBytes;        // [kBN] rows
    static constexpr int sx = b + kBN * kRowBytes;       // float [2][kBN]: x's in the first kBM of each, the rest so that every thread stores
    static constexpr int sw = sx + 2 * kBN * 4;          // float [2][kBN]
    static constexpr int bytes = sw + 2 * kBN * 4;
};
static_assert(Stage::bytes % 1024 == 0, "stages start on the boundary the loads assume");
constexpr size_t kLdsBytes = 2 * (size_t)Stage::bytes;

// Thread t takes elements 4t..4t+3 of row blockIdx.y; a block's eight threads are consecutive lanes.
__global__ __launch_bounds__(256) void fx16_convert_kernel(const float* __restrict__ x, int64_t x_row_stride, int K, uint16_t* __restrict__ X16,
                                                           float* __restrict__ XS) {
    const int nb = K >> 5;
    const float* xr = x + (int64_t)blockIdx.y * x_row_stride;
    uint16_t* row = X16 + (int64_t)blockIdx.y * nb * 64;
    float* xscale = XS + (int64_t)blockIdx.y * nb;
    const int nq = K >> 2;
    for (int t = blockIdx.x * blockDim.x + threadIdx.x; t < nq; t += gridDim.x * blockDim.x) {
        f32x4 v;
        __builtin_memcpy(&v, xr + 4 * (int64_t)t, 16);
        float amax = 0.f;
        bool finite = true;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            float a = __builtin_fabsf(v[k]);
            finite = finite && a < __builtin_inff();  // false for NaN too
            amax = fmaxf(amax, a);
        }
        amax = group8_max(amax);
        float bad = group8_max(finite ? 0.f : 1.f);
        float scale, inv;
        if (bad != 0.f) {  // a NaN or an infinity in the block: its products are NaN
            scale = __builtin_nanf("");
            inv = 0.f;
            v = f32x4{0.f, 0.f, 0.f, 0.f};
        } else if (amax < 0x1p-100f) {
            scale = 0.f;
            inv = 0.f;
        } else {
            scale = amax / (float)kFixMax;
            inv = (float)kFixMax / amax;
        }
        _Float16 lo[4], hi[4];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            int a = (int)__builtin_rintf(v[k] * inv);
            a = a > kFixMax ? kFixMax : a < -kFixMax ? -kFixMax : a;
            const int d0 = ((a + 2048) & 4095) - 2048;  // balanced: -2048..2047
            const int d1 = (a - d0) >> 12;              // -2048..2048
            lo[k] = (_Float16)(float)d0;
            hi[k] = (_Float16)(float)d1;
        }
        uint16_t* at = row + (t >> 3) * 64 + 4 * (t & 7);
        __builtin_memcpy(at, lo, 8);
        __builtin_memcpy(at + 32, hi, 8);
        if ((t & 7) == 0) xscale[t >> 3] = scale;
    }
}

// Sixteen weights a thread: the low and the high nibbles of eight bytes of a block, as the binary16 integers n - 8.
__global__ __launch_bounds__(256) void fx16_panel_kernel(const uint8_t* __restrict__ W, uint16_t* __restrict__ P, int64_t halves) {
    const int64_t first = (int64_t)blockIdx.x * 256 + threadIdx.x, stride = (int64_t)gridDim.x * 256;
    for (int64_t t = first; t < halves; t += stride) {
        const int q = (int)(t & 1);
        const uint16_t* src = (const uint16_t*)(W + (t >> 1) * 18 + 2 + 8 * q);  // blocks are 2-byte aligned, no more
        const uint32_t raw[2] = {(uint32_t)src[0] | (uint32_t)src[1] << 16, (uint32_t)src[2] | (uint32_t)src[3] << 16};
        const f16x2 off = {(_Float16)1032.f, (_Float16)1032.f};
        uint16_t* out = P + (t >> 1) * 32 + 8 * q;  // elements 8 q .. 8 q + 7 (low nibbles) and 16 more on (high nibbles)
#pragma unroll
        for (int half = 0; half < 2; half++) {
            u32x4 v;
#pragma unroll
            for (int i = 0; i < 2; i++) {
                // the nibble into the mantissa of binary16's 1024; minus 1032 is n - 8
                const uint32_t nib = (raw[i] >> (4 * half)) & 0x0f0f0f0fu;
                const uint32_t p0 = __builtin_amdgcn_perm(0x64646464u, nib, 0x04010400u);
                const uint32_t p1 = __builtin_amdgcn_perm(0x64646464u, nib, 0x04030402u);
                v[2 * i] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(f16x2, p0) - off);
                v[2 * i + 1] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(f16x2, p1) - off);
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

// A die's workgroups (every eighth, round-robin) take a contiguous range of the tiles, the tile's rows of x varying
// fastest: those that run together share few column panels of P through the die's L2.
__device__ __forceinline__ int tile_of(int b, int ntiles) {
    const int per_die = (ntiles + 7) >> 3;
    return (b & 7) * per_die + (b >> 3);
}

__global__ __launch_bounds__(512) void qgemm_q4_0_fx16_kernel(const uint8_t* __restrict__ W, const uint16_t* __restrict__ P,
                                                              const uint16_t* __restrict__ X16, const float* __restrict__ XS, float* y,
                                                              const float* resid,  // may be y
                                                              int M, int N, int K, int tiles_m, int ntiles) {
    extern __shared__ __align__(1024) char lds[];
    const int t = tile_of((int)blockIdx.x, ntiles);
    if (t >= ntiles) return;  // the whole workgroup
    const int m0 = (t % tiles_m) * kBM, n0 = (t / tiles_m) * kBN;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 2, wn = wave & 3;
    const int nb = K >> 5;

    // This wavefront's loads: load g = kLoads wave + j brings rows [8 g, 8 g + 8) of the stage: x's rows for the even
    // block, for the odd block, then P's. Rows past the matrix re-read its last row (their results are not stored).
    const char* from[kLoads];
    uint32_t into[kLoads];
    int advance[kLoads];
#pragma unroll
    for (int j = 0; j < kLoads; j++) {
        const int first = 8 * (kLoads * wave + j);
        const int row = first + (lane >> 3);
        const int piece = (lane & 7) ^ ((row >> 1) & 7);
        const uint16_t* base;
        if (first < 2 * kBM) {
            const int r = row & (kBM - 1), odd = row >> 7;
            const int m = m0 + r < M ? m0 + r : M - 1;
            base = X16 + ((size_t)m * nb + odd) * 64;
            advance[j] = 2 * kRowBytes;
        } else {
            const int r = row - 2 * kBM;
            const int n = n0 + r < N ? n0 + r : N - 1;
            base = P + (size_t)n * K;
            advance[j] = kRowBytes;
        }
        from[j] = (const char*)(base + 8 * piece);
        into[j] = (uint32_t)(first * kRowBytes);
    }
    // the scales: thread t takes block t % 2 of the stage for row t / 2 of W and of x (x's rows beyond kBM: loaded and
    // stored like the others, so that no branch is needed, and never read)
    const int srow = tid >> 1, sodd = tid & 1;
    const uint8_t* wscale = W + ((size_t)(n0 + srow < N ? n0 + srow : N - 1) * nb + sodd) * 18;
    const float* xscale = XS + (size_t)(m0 + srow < M ? m0 + srow : M - 1) * nb + sodd;
    const uint32_t lds0 = (uint32_t)(uintptr_t)lds;

    const int r32 = lane & 31, hi = lane >> 5;
    const int swz = (r32 >> 1) & 7;
    int piece_off[4];  // of a row's pieces 2 p + hi: of x, half p % 2 of digit p / 2; of P, half p % 2 of the stage's block p / 2
#pragma unroll
    for (int p = 0; p < 4; p++) piece_off[p] = ((2 * p + hi) ^ swz) * 16;
    const int a_row = (wm * 64 + r32) * kRowBytes, b_row = Stage::b + (wn * 64 + r32) * kRowBytes;

    f32x16 acc[2][2];
#pragma unroll
    for (int mt = 0; mt < 2; mt++)
#pragma unroll
        for (int nt = 0; nt < 2; nt++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[mt][nt][i] = 0.f;

    const int nstages = K / 64;
    {
        const float dw = f16_bits_to_f32(load_u16(wscale));
        const float dx = *xscale;
#pragma unroll
        for (int j = 0; j < kLoads; j++) load_to_lds(from[j], __builtin_amdgcn_readfirstlane(lds0 + into[j]));
        ((float*)(lds + Stage::sw))[sodd * kBN + srow] = dw;
        ((float*)(lds + Stage::sx))[sodd * kBN + srow] = dx;
    }
    // No branches around the loads and stores: past the end the last stage is requested and stored again, into the
    // buffer that is not being read.
    for (int i = 0; i < nstages; i++) {
        wait_loads();   // this wavefront's part of stage i has landed
        lds_barrier();  // everyone's has, with the scales, and everyone has read the other stage for the last time
        const int step = i + 1 < nstages ? 1 : 0;
        const uint32_t next = lds0 + ((i + 1) & 1) * Stage::bytes;
        char* next_p = lds + ((i + 1) & 1) * Stage::bytes;
        const char* st = lds + (i & 1) * Stage::bytes;
        wscale += 36 * step;
        xscale += 2 * step;
        const float next_dw = f16_bits_to_f32(load_u16(wscale));
        const float next_dx = *xscale;
#pragma unroll
        for (int odd = 0; odd < 2; odd++) {
            // half of the next stage's loads with each block
#pragma unroll
            for (int j = odd * kLoads / 2; j < (odd + 1) * kLoads / 2; j++) {
                from[j] += advance[j] * step;
                load_to_lds(from[j], __builtin_amdgcn_readfirstlane(next + into[j]));
            }
            f16x8 a[2][2][2], b[2][2];  // a[mt][digit][half], b[nt][half]
#pragma unroll
            for (int mt = 0; mt < 2; mt++)
#pragma unroll
                for (int p = 0; p < 4; p++)
                    a[mt][p >> 1][p & 1] = *(const f16x8*)(st + Stage::a + odd * kBM * kRowBytes + a_row + mt * 32 * kRowBytes + piece_off[p]);
#pragma unroll
            for (int nt = 0; nt < 2; nt++)
#pragma unroll
                for (int h = 0; h < 2; h++) b[nt][h] = *(const f16x8*)(st + b_row + nt * 32 * kRowBytes + piece_off[2 * odd + h]);
            // The operands of the outer products that give dw dx: v_mfma_f32_32x32x1_2b_f32 makes two, its first 32
            // lanes giving x's rows and W's rows of the first, the other 32 of the second; here the 32 rows of x of
            // sub-tiles (mt, 0) and (mt, 1), and the 64 rows of W of both (a lane each).
            const float dwv = ((const float*)(st + Stage::sw))[odd * kBN + wn * 64 + lane];
            float dxv[2];
#pragma unroll
            for (int mt = 0; mt < 2; mt++) dxv[mt] = ((const float*)(st + Stage::sx))[odd * kBN + wm * 64 + mt * 32 + r32];
            auto scales = [&](int mt, f32x32& w) {
                f32x32 zero;
#pragma unroll
                for (int e = 0; e < 32; e++) zero[e] = 0.f;
                w = __builtin_amdgcn_mfma_f32_32x32x1f32(dxv[mt], dwv, zero, 0, 0, 0);
            };
            // Sub-tile s = 2 mt + nt: its four MFMAs are issued with the finish of the sub-tile before it, so that the
            // vector unit works while the matrix cores do (two pairs of sums live at a time; more, and registers spill).
            auto multiply = [&](int sub, f32x16& c0, f32x16& c1) {
                const int mt = sub >> 1, nt = sub & 1;
                f32x16 zero;
#pragma unroll
                for (int e = 0; e < 16; e++) zero[e] = 0.f;
                c0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[mt][0][0], b[nt][0], zero, 0, 0, 0);
                c1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[mt][1][0], b[nt][0], zero, 0, 0, 0);
                c0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[mt][0][1], b[nt][1], c0, 0, 0, 0);
                c1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[mt][1][1], b[nt][1], c1, 0, 0, 0);
            };
            auto finish = [&](int sub, const f32x16& c0, const f32x16& c1, const f32x32& w) {
                const int mt = sub >> 1, nt = sub & 1;
#pragma unroll
                for (int e = 0; e < 16; e++) {
                    const float isum = fmaf(c1[e], 4096.f, c0[e]);  // the exact integer, rounded once
                    acc[mt][nt][e] = fmaf(w[16 * nt + e], isum, acc[mt][nt][e]);
                }
            };
            f32x16 p0, p1, q0, q1;
            f32x32 w;
            multiply(0, p0, p1);
            scales(0, w);
            __builtin_amdgcn_sched_barrier(0);
            multiply(1, q0, q1);
            finish(0, p0, p1, w);
            __builtin_amdgcn_sched_barrier(0);
            multiply(2, p0, p1);
            finish(1, q0, q1, w);
            __builtin_amdgcn_sched_barrier(0);
            scales(1, w);
            multiply(3, q0, q1);
            finish(2, p0, p1, w);
            __builtin_amdgcn_sched_barrier(0);
            finish(3, q0, q1, w);
        }
        // the next stage's scales, at the end: by now their loads have landed with everything requested before them
        __builtin_amdgcn_sched_barrier(0);
        ((float*)(next_p + Stage::sw))[sodd * kBN + srow] = next_dw;
        ((float*)(next_p + Stage::sx))[sodd * kBN + srow] = next_dx;
    }

    // An MFMA leaves a lane one column of y and four consecutive rows per group of four registers; a 4 x 4
    // transposition within each quad of lanes turns that into one row and four consecutive columns a lane.
    const bool wide_ok = (N & 3) == 0 && ((uintptr_t)y & 15) == 0 && (!resid || ((uintptr_t)resid & 15) == 0);
#pragma unroll
    for (int mt = 0; mt < 2; mt++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const int m = m0 + wm * 64 + mt * 32 + q * 8 + hi * 4 + (lane & 3);
#pragma unroll
            for (int nt = 0; nt < 2; nt++) {
                float v[4] = {acc[mt][nt][4 * q], acc[mt][nt][4 * q + 1], acc[mt][nt][4 * q + 2], acc[mt][nt][4 * q + 3]};
                quad_transpose(v, lane);
                const int n = n0 + wn * 64 + nt * 32 + (r32 & ~3);
                if (m >= M || n >= N) continue;
                if (wide_ok && n + 3 < N) {
                    f32x4 o = {v[0], v[1], v[2], v[3]};
                    if (resid) {
                        const f32x4 r = *(const f32x4*)(resid + (int64_t)m * N + n);
#pragma unroll
                        for (int k = 0; k < 4; k++) o[k] = o[k] + r[k];
                    }
                    *(f32x4*)(y + (int64_t)m * N + n) = o;
                } else {
#pragma unroll
                    for (int k = 0; k < 4; k++) {
                        if (n + k >= N) continue;
                        float o = v[k];
                        if (resid) o = o + resid[(int64_t)m * N + n + k];
                        y[(int64_t)m * N + n + k] = o;
                    }
                }
            }
        }
}

std::atomic<int> g_fx16{1};  // measurement aid: 0 keeps every product on the int8 form, 2 takes this one whatever the shape

}  // namespace

void set_q4_0_fx16(int v) { g_fx16 = v; }

// Whether the product is the faster here than in the int8 form (qgemm_q4_0_fx_cost_us), the pass over W included:
// that pass reads the blocks and writes the panel at about 4.4 TB/s; a workgroup takes about 2.85 us a stage of 64 of K,
// one a compute unit at a time (measured at 4096 x 4096, 14336 x 4096 and 4096 x 14336 weights, 512 to 4096 rows:
// 512 x 4096 x 4096 stays with the int8 form, 512 x 14336 x 4096 comes here).
bool qgemm_q4_0_fx16_pays(int64_t M, int64_t N, int64_t K) {
    if (g_fx16 == 0 || M <= 0 || N <= 0 || K <= 0 || K % 64 != 0) return false;
    if (g_fx16 == 2) return true;
    if (M < kMinRows) return false;
    const int64_t tiles = ((M + kBM - 1) / kBM) * ((N + kBN - 1) / kBN);
    const double product_us = (double)((tiles + 255) / 256) * (double)(K / 64) * 2.85;
    const double panel_us = (double)N * (double)K * (18.0 / 32.0 + 2.0) / 4.4e6;
    return panel_us + product_us < qgemm_q4_0_fx_cost_us(M, N, K);
}

// X16 [M, K / 32, 64] binary16, then XS [M, K / 32] float32: 4 K + K / 8 bytes a row.
size_t q4_0_fx16_act_bytes(int64_t K) { return (size_t)((4 * K + K / 8 + 15) / 16 * 16); }

hipError_t q4_0_fx16_convert_act(const float* x, int64_t M, int64_t K, int64_t x_row_stride, void* act, hipStream_t st) {
    const int gx = (int)((K / 4 + 255) / 256);
    uint16_t* X16 = (uint16_t*)act;
    float* XS = (float*)(X16 + (size_t)M * K * 2);
    hipLaunchKernelGGL(fx16_convert_kernel, dim3((unsigned)gx, (unsigned)M), dim3(256), 0, st, x, x_row_stride, (int)K, X16, XS);
    return hipGetLastError();
}

// The panel: N K binary16.
size_t qgemm_q4_0_fx16_ws_bytes(int64_t N, int64_t K) { return (size_t)N * (size_t)K * 2; }

// act: q4_0_fx16_convert_act's for these M rows; ws: qgemm_q4_0_fx16_ws_bytes(N, K) bytes, 16-byte aligned.
// y = x . W^T (+ resid, which may be y itself).
hipError_t qgemm_q4_0_fx16(const void* W, const void* act, float* y, const float* resid, int64_t M, int64_t N, int64_t K, void* ws, hipStream_t st) {
    if (!ws || ((uintptr_t)ws & 15) != 0 || ((uintptr_t)act & 15) != 0 || ((uintptr_t)W & 1) != 0 || M <= 0 || N <= 0 || K <= 0 || K % 64 != 0 ||
        M >= (1 << 30) || N >= (1 << 30) || K > (1 << 20))
        return hipErrorInvalidValue;
    static std::atomic<bool> raised{false};  // threads may race here: both then set the same attribute
    if (!raised) {
        hipError_t e = hipFuncSetAttribute((const void*)qgemm_q4_0_fx16_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsBytes);
        if (e != hipSuccess) return e;
        raised = true;
    }
    const int64_t tiles_m = (M + kBM - 1) / kBM, ntiles = tiles_m * ((N + kBN - 1) / kBN);
    if (ntiles >= ((int64_t)1 << 28)) return hipErrorInvalidValue;
    uint16_t* P = (uint16_t*)ws;
    const int64_t halves = N * (K / 32) * 2;
    const int64_t want = (halves + 255) / 256;
    hipLaunchKernelGGL(fx16_panel_kernel, dim3((unsigned)(want < 8192 ? want : 8192)), dim3(256), 0, st, (const uint8_t*)W, P, halves);
    const uint16_t* X16 = (const uint16_t*)act;
    const float* XS = (const float*)(X16 + (size_t)M * K * 2);
    const int wgs = (int)(((ntiles + 7) / 8) * 8);
    hipLaunchKernelGGL(qgemm_q4_0_fx16_kernel, dim3((unsigned)wgs), dim3(512), kLdsBytes, st, (const uint8_t*)W, P, X16, XS, y, resid, (int)M, (int)N,
                       (int)K, (int)tiles_m, (int)ntiles);
    note_kernel("qgemm_q4_0_fx16_kernel: %lld x %lld tiles of 128 x 256", (long long)tiles_m, (long long)(ntiles / tiles_m));
    return hipGetLastError();
}

}  // namespace mimir
