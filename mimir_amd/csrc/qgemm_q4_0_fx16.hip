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
// of four wavefronts owns 128 rows of x by 128 rows of W, a wavefront 64 by 64, and a compute unit runs two such
// workgroups, so that one computes while the other waits at its barrier or for its operands. A stage is one block (32
// of K): the rows of x (128 bytes a row: 32 digits d0, then 32 digits d1), the rows of P (64 bytes) and the scales of
// both (W's binary16 bits as they lie in the blocks). Everything goes from global memory straight into LDS
// (global_load_lds_*), operands with the 16-byte pieces of a row placed so that the 16 rows a quarter wavefront reads
// fall on all banks (piece ^ (row / 2 mod 8) in the 128-byte rows, piece ^ (row / 4 mod 4) in the 64-byte ones, which
// the loading lane undoes in the address it reads from). Three stages in a ring, requested two blocks ahead, one
// barrier a block.
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
constexpr int kBN = 128;        // rows of W a workgroup
constexpr int kMinRows = 256;   // fewer rows stay with the int8 form
constexpr int kStages = 3;

// A stage in LDS: the rows of x for the block, the rows of P, then the scales of both.
struct Stage {
    static constexpr int a = 0;                      // [kBM] rows of 128 bytes
    static constexpr int b = kBM * 128;              // [kBN] rows of 64 bytes
    static constexpr int sx = b + kBN * 64;          // float [kBM]
    static constexpr int sw = sx + kBM * 4;          // uint32 [kBN]: binary16 bits
    static constexpr int bytes = sw + kBN * 4;
};
static_assert(Stage::bytes % 1024 == 0, "stages start on a boundary the loads' layout can assume");
constexpr size_t kLdsBytes = kStages * (size_t)Stage::bytes;  // 75 KB: two workgroups a compute unit

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
// 4 bytes a lane (lane l's lands at lds_base + 4 l), and 2 bytes a lane, which LDS receives as a zero-extended dword.
__device__ __forceinline__ void load_dword_to_lds(const void* g, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dword %1, off" ::"s"(lds_base), "v"(g) : "memory");
}
__device__ __forceinline__ void load_ushort_to_lds(const void* g, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_ushort %1, off" ::"s"(lds_base), "v"(g) : "memory");
}
constexpr int kLoads = 7;  // a wavefront's loads per stage: four of x's rows, two of P's, one of scales
__device__ __forceinline__ void wait_all_but_last_stage() { asm volatile("s_waitcnt vmcnt(7)" ::: "memory"); }
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// A die's workgroups (every eighth, round-robin) take a contiguous range of the tiles, the tile's rows of x varying
// fastest: those that run together share few column panels of P through the die's L2.
__device__ __forceinline__ int tile_of(int b, int ntiles) {
    const int per_die = (ntiles + 7) >> 3;
    return (b & 7) * per_die + (b >> 3);
}

__global__ __launch_bounds__(256, 2) void qgemm_q4_0_fx16_kernel(const uint8_t* __restrict__ W, const uint16_t* __restrict__ P,
                                                                 const uint16_t* __restrict__ X16, const float* __restrict__ XS, float* y,
                                                                 const float* resid,  // may be y
                                                                 int M, int N, int K, int tiles_m, int ntiles) {
    extern __shared__ __align__(1024) char lds[];
    const int t = tile_of((int)blockIdx.x, ntiles);
    if (t >= ntiles) return;  // the whole workgroup
    const int m0 = (t % tiles_m) * kBM, n0 = (t / tiles_m) * kBN;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int nb = K >> 5;

    // This wavefront's loads of a stage. Rows past the matrix re-read its last row (their results are not stored).
    //   j = 0..3: rows [8 (4 wave + j), + 8) of x: a lane one 16-byte piece of a 128-byte row
    //   j = 4, 5: rows [16 (2 wave + j - 4), + 16) of P: a lane one piece of a 64-byte row
    //   j = 6:    wavefronts 0 and 1 the scales of x's rows [64 wave, + 64), 2 and 3 those of W's rows [64 (wave - 2), + 64)
    const char* from[kLoads];
    uint32_t into[kLoads];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int first = 8 * (4 * wave + j), row = first + (lane >> 3);
        const int piece = (lane & 7) ^ ((row >> 1) & 7);
        const int m = m0 + row < M ? m0 + row : M - 1;
        from[j] = (const char*)(X16 + (size_t)m * nb * 64 + 8 * piece);
        into[j] = (uint32_t)(Stage::a + first * 128);
    }
#pragma unroll
    for (int j = 4; j < 6; j++) {
        const int first = 16 * (2 * wave + j - 4), row = first + (lane >> 2);
        const int piece = (lane & 3) ^ ((row >> 2) & 3);
        const int n = n0 + row < N ? n0 + row : N - 1;
        from[j] = (const char*)(P + (size_t)n * K + 8 * piece);
        into[j] = (uint32_t)(Stage::b + first * 64);
    }
    const bool x_scales = wave < 2;  // uniform
    if (x_scales) {
        const int row = 64 * wave + lane;
        from[6] = (const char*)(XS + (size_t)(m0 + row < M ? m0 + row : M - 1) * nb);
        into[6] = (uint32_t)(Stage::sx + 4 * 64 * wave);
    } else {
        const int row = 64 * (wave - 2) + lane;
        from[6] = (const char*)(W + (size_t)(n0 + row < N ? n0 + row : N - 1) * nb * 18);
        into[6] = (uint32_t)(Stage::sw + 4 * 64 * (wave - 2));
    }
    const int scale_step = x_scales ? 4 : 18;
    const uint32_t lds0 = (uint32_t)(uintptr_t)lds;
    // Every load into the stage at stage_base, `ahead` (0 or 1) blocks on from the last request.
    auto request = [&](uint32_t stage_base, int ahead) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            from[j] += 128 * ahead;
            load_to_lds(from[j], __builtin_amdgcn_readfirstlane(stage_base + into[j]));
        }
#pragma unroll
        for (int j = 4; j < 6; j++) {
            from[j] += 64 * ahead;
            load_to_lds(from[j], __builtin_amdgcn_readfirstlane(stage_base + into[j]));
        }
        from[6] += scale_step * ahead;
        if (x_scales) load_dword_to_lds(from[6], __builtin_amdgcn_readfirstlane(stage_base + into[6]));
        else load_ushort_to_lds(from[6], __builtin_amdgcn_readfirstlane(stage_base + into[6]));
    };

    const int r32 = lane & 31, hi = lane >> 5;
    int a_off[4], b_off[2];  // x: piece 2 p + hi is half p % 2 of digit p / 2; P: piece 2 h + hi is half h
#pragma unroll
    for (int p = 0; p < 4; p++) a_off[p] = ((2 * p + hi) ^ ((r32 >> 1) & 7)) * 16;
#pragma unroll
    for (int h = 0; h < 2; h++) b_off[h] = ((2 * h + hi) ^ ((r32 >> 2) & 3)) * 16;
    const int a_row = Stage::a + (wm * 64 + r32) * 128, b_row = Stage::b + (wn * 64 + r32) * 64;

    f32x16 acc[2][2];
#pragma unroll
    for (int mt = 0; mt < 2; mt++)
#pragma unroll
        for (int nt = 0; nt < 2; nt++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[mt][nt][i] = 0.f;

    // Blocks 0 and 1 are requested before the loop, block i + 2 during block i. No branches around the loads, and
    // always seven a stage, so that the count the wait leaves under way is right: past the end the last block is
    // requested again, into a stage that is not read any more.
    request(lds0, 0);
    request(lds0 + Stage::bytes, 1);  // K has at least two blocks
    int cur = 0;  // the stage of block i
    for (int i = 0; i < nb; i++) {
        wait_all_but_last_stage();  // this wavefront's part of block i has landed (the seven loads after it may be under way)
        lds_barrier();              // everyone's has, and everyone has read block i - 1's stage for the last time
        const int nxt2 = cur == 0 ? 2 : cur - 1;  // (cur + 2) % 3: block i - 1's stage
        const char* st = lds + cur * Stage::bytes;
        request(lds0 + nxt2 * Stage::bytes, i + 2 < nb ? 1 : 0);
        cur = cur == 2 ? 0 : cur + 1;

        f16x8 a[2][2][2], b[2][2];  // a[mt][digit][half], b[nt][half]
        auto read_a = [&](int mt) {
#pragma unroll
            for (int p = 0; p < 4; p++) a[mt][p >> 1][p & 1] = *(const f16x8*)(st + a_row + mt * 32 * 128 + a_off[p]);
        };
#pragma unroll
        for (int nt = 0; nt < 2; nt++)
#pragma unroll
            for (int h = 0; h < 2; h++) b[nt][h] = *(const f16x8*)(st + b_row + nt * 32 * 64 + b_off[h]);
        read_a(0);
        // The products of the two scales, dw dx rounded to float32, come from the matrix cores as well: an outer
        // product is an MFMA with K = 1 (float32 operands, one exact product per output and nothing added to it, so
        // the same rounding as a multiplication). v_mfma_f32_32x32x1_2b_f32 makes two of them: its first 32 lanes give
        // x's rows and W's rows for the first, the other 32 for the second; here the 32 rows of x of sub-tiles
        // (mt, 0) and (mt, 1) and the 64 rows of W of both.
        const float dwv = f16_bits_to_f32((uint16_t)((const uint32_t*)(st + Stage::sw))[wn * 64 + lane]);
        float dxv[2];
#pragma unroll
        for (int mt = 0; mt < 2; mt++) dxv[mt] = ((const float*)(st + Stage::sx))[wm * 64 + mt * 32 + r32];
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
        read_a(1);
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
// that pass reads the blocks and writes the panel at about 4.4 TB/s; a workgroup takes 0.82 us a block when it has its
// compute unit to itself, and two that share one 0.74 us a block each (measured at 4096 x 4096, 14336 x 4096 and
// 4096 x 14336 weights, 512 to 4096 rows: 512 x 4096 x 4096 stays with the int8 form, 512 x 14336 x 4096 comes here).
bool qgemm_q4_0_fx16_pays(int64_t M, int64_t N, int64_t K) {
    if (g_fx16 == 0 || M <= 0 || N <= 0 || K <= 0 || K % 64 != 0) return false;
    if (g_fx16 == 2) return true;
    if (M < kMinRows) return false;
    const double tiles = (double)((M + kBM - 1) / kBM) * (double)((N + kBN - 1) / kBN);
    const double per_unit = tiles / 256.0, blocks = (double)(K / 32);
    const double rounds = (double)(int64_t)(per_unit + 0.999999);
    const double product_us = per_unit <= 1.0 ? 0.82 * blocks : 0.74 * blocks * rounds;
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
    hipLaunchKernelGGL(qgemm_q4_0_fx16_kernel, dim3((unsigned)wgs), dim3(256), kLdsBytes, st, (const uint8_t*)W, P, X16, XS, y, resid, (int)M, (int)N,
                       (int)K, (int)tiles_m, (int)ntiles);
    note_kernel("qgemm_q4_0_fx16_kernel: %lld x %lld tiles of 128 x 128", (long long)tiles_m, (long long)(ntiles / tiles_m));
    return hipGetLastError();
}

}  // namespace mimir
