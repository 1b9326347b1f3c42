// Products of many rows of float32 x with Q4_0 weights on the int8 matrix
// cores of gfx950: y[M, N] = x[M, K] . W[N, K]^T (+ a residual), the prompt-sized
// counterpart of the fixed-point decode kernel (qgemv_q4_0.hip), with that
// kernel's arithmetic. What the reference's CPU computes here is the float32
// product with the dequantized weights (io/mim/dtype.go:118-123,
// backend/cpu/gemv.go:73-104), to which a product has to agree within 1e-3.
//
// x is held as in the decode kernel, a 24-bit fixed-point number per element
// and one float32 scale per block of 32 (the same integers and scales:
// q4_convert_item and fx_convert below round alike), here cut into three
// balanced base-256 digits, int8 each, instead of six base-16 ones. A Q4_0
// block is 32 weights (n - 8) d with 4-bit n: exactly the K of one
// v_mfma_i32_32x32x32_i8. Per block and tile of 32 rows of x by 32 rows of W:
// three MFMAs (one per digit plane, weights n - 8 as int8), the exact integer
// sum T0 + 256 T1 + 65536 T2, converted once and multiplied by the product of
// the block's two scales into the float32 sum (one FMA, as the decode kernel
// does it). Only the order of those float32 additions differs from the decode
// kernel's, so the two agree to a few units in the last place.
//
// The vector unit bounds it: five instructions per output and block against
// three MFMAs of 32 cycles per 1024 outputs. A workgroup of eight wavefronts
// owns 128 rows of x by 64 rows of W, a wavefront 32 by 32; steps of four
// blocks (128 of K); W requested two steps ahead, x one; two LDS step buffers,
// rows padded to 144 bytes (conflict-free 128-bit fragment reads).
#include "device_util.h"
#include "kernels.h"
#include "q4_act.h"

namespace mimir {

namespace {

typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kTM = 128;          // rows of x per workgroup
constexpr int kTN = 64;           // rows of W per workgroup
constexpr int kStepK = 128;       // K per step: four blocks
constexpr int kRow = kStepK + 16; // bytes per LDS row of int8

// LDS: two step buffers (three planes of x, the weights) and, per step buffer, the scales of its
// four blocks: x's as [block][row], W's as [block][row].
struct Layout {
    static constexpr int x = 0;                       // int8[3][kTM][kRow]
    static constexpr int w = 3 * kTM * kRow;          // int8[kTN][kRow]
    static constexpr int sx = w + kTN * kRow;         // float[4][kTM]
    static constexpr int sw = sx + 4 * kTM * 4;       // float[4][kTN]
    static constexpr int step = sw + 4 * kTN * 4;
    static constexpr int total = 2 * step;
};

__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

__device__ __forceinline__ u32x2 load_u32x2_unaligned(const uint8_t* p) {
    u32x2 v;
    __builtin_memcpy(&v, p, 8);
    return v;
}

// Four nibbles in the bytes of v (each below 16) to four int8 n - 8.
__device__ __forceinline__ uint32_t nibbles_to_i8(uint32_t v) { return ((v | 0x80808080u) - 0x08080808u) ^ 0x80808080u; }

}  // namespace

// One row of x with nb blocks, converted for this kernel (K = 32 nb):
//   int8 plane[3][K]   digit j of element e at plane[j][e]; x[e] ~ scale * (d0 + 256 d1 + 65536 d2)
//   float scale[nb]
size_t q4_0_fx_act_bytes(int64_t K) { return (size_t)((3 * K + K / 8 + 15) / 16 * 16); }

// Thread t takes elements 4t..4t+3; a block's eight threads are consecutive lanes. The integers and
// scales are those of q4_convert_item: the block's largest magnitude maps to kFixMax.
__global__ __launch_bounds__(256) void fx_convert_kernel(const float* __restrict__ x, int64_t x_row_stride, int K,
                                                         uint8_t* __restrict__ act, int64_t act_row_bytes) {
    const float* xr = x + (int64_t)blockIdx.y * x_row_stride;
    uint8_t* row = act + (int64_t)blockIdx.y * act_row_bytes;
    float* xscale = (float*)(row + 3 * (int64_t)K);
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
        uint32_t d[3] = {0, 0, 0};
#pragma unroll
        for (int k = 0; k < 4; k++) {
            int a = (int)__builtin_rintf(v[k] * inv);
            a = a > kFixMax ? kFixMax : a < -kFixMax ? -kFixMax : a;
            const int d0 = (int)(int8_t)a;  // balanced digits: each in -128..127
            const int a1 = (a - d0) >> 8;
            const int d1 = (int)(int8_t)a1;
            const int d2 = (a1 - d1) >> 8;
            d[0] |= (uint32_t)(d0 & 0xff) << (8 * k);
            d[1] |= (uint32_t)(d1 & 0xff) << (8 * k);
            d[2] |= (uint32_t)(d2 & 0xff) << (8 * k);
        }
#pragma unroll
        for (int j = 0; j < 3; j++) ((uint32_t*)(row + (int64_t)j * K))[t] = d[j];
        if ((t & 7) == 0) xscale[t >> 3] = scale;
    }
}

hipError_t q4_0_fx_convert_act(const float* x, int64_t M, int64_t K, int64_t x_row_stride, void* act, bool pairs, hipStream_t st) {
    if (pairs) return q4_0_fx16_convert_act(x, M, K, x_row_stride, act, st);
    int gx = (int)((K / 4 + 255) / 256);
    hipLaunchKernelGGL(fx_convert_kernel, dim3((unsigned)gx, (unsigned)M), dim3(256), 0, st, x, x_row_stride, (int)K, (uint8_t*)act,
                       (int64_t)q4_0_fx_act_bytes(K));
    return hipGetLastError();
}

namespace {

// What a thread holds between the loads of a step and its LDS stores.
struct FetchedW {
    u32x2 q;      // 8 bytes of nibbles: half a block
    uint32_t d;   // the block's scale (binary16 bits)
};
struct FetchedX {
    u32x4 x[6];   // 16-byte pieces of the three planes
    float s;      // one scale of x: row tid / 4, block tid % 4 of the step
};

__global__ __launch_bounds__(512) void qgemm_q4_0_fx_kernel(const uint8_t* __restrict__ W, const uint8_t* __restrict__ act,
                                                             float* y, const float* resid, int M, int N, int K,  // resid may be y
                                                             int64_t act_row_bytes, int tiles_m, int ntiles) {
    typedef Layout L;
    extern __shared__ __align__(16) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave & 3, wn = wave >> 2, l32 = lane & 31, lh = lane >> 5;
    const int nb = K >> 5;

    // Tiles that share rows of W run next to each other on one XCD (workgroup i goes to XCD i % 8).
    const int id = blockIdx.x, xcd = id & 7, slot = id >> 3;
    const int per_xcd = (ntiles + 7) >> 3;
    const int t = slot / tiles_m + xcd * per_xcd;
    const int tm = slot % tiles_m;
    if (slot >= per_xcd * tiles_m || t >= ntiles) return;
    const int m0 = tm * kTM, n0 = t * kTN;

    // This thread's part of the W tile: half c8 % 2 of block c8 / 2 of the step, of row wrow_i.
    const int wrow_i = tid >> 3, c8 = tid & 7;
    const int last_n = N - 1 - n0, last_m = M - 1 - m0;
    const uint8_t* w_t = W + (int64_t)n0 * nb * 18;
    const uint32_t woff = (uint32_t)(wrow_i < last_n ? wrow_i : last_n) * (uint32_t)(nb * 18) + 18 * (c8 >> 1);
    const uint8_t* act_t = act + (int64_t)m0 * act_row_bytes;
    // pieces of x: piece p = tid + 512 i is plane p / 1024, row (p % 1024) / 8, bytes 16 (p % 8)..
    uint32_t xoff[6];
#pragma unroll
    for (int i = 0; i < 6; i++) {
        const int p = tid + 512 * i, r = (p & 1023) >> 3;
        xoff[i] = (uint32_t)(r < last_m ? r : last_m) * (uint32_t)act_row_bytes + (uint32_t)(p >> 10) * (uint32_t)K + 16 * (p & 7);
    }
    const int srow = tid >> 2, sblk = tid & 3;
    const uint32_t soff = (uint32_t)(srow < last_m ? srow : last_m) * (uint32_t)act_row_bytes + 4 * sblk;
    const uint8_t* xs_t = act_t + 3 * (int64_t)K;

    FetchedW fw0, fw1;
    FetchedX fx;
    auto fetch_w = [&](FetchedW& f, int step) {
        const uint8_t* wb = w_t + (int64_t)step * 72 + woff;  // four blocks a step
        f.q = load_u32x2_unaligned(wb + 2 + 8 * (c8 & 1));
        f.d = load_u16(wb);
    };
    auto fetch_x = [&](int step) {
#pragma unroll
        for (int i = 0; i < 6; i++) fx.x[i] = *(const u32x4*)(act_t + (int64_t)step * kStepK + xoff[i]);
        fx.s = *(const float*)(xs_t + (int64_t)step * 16 + soff);
    };
    auto stage = [&](const FetchedW& f, int parity) {
        uint8_t* buf = smem + parity * L::step;
#pragma unroll
        for (int i = 0; i < 6; i++) {
            const int p = tid + 512 * i;
            *(u32x4*)(buf + L::x + ((p >> 10) * kTM + ((p & 1023) >> 3)) * kRow + 16 * (p & 7)) = fx.x[i];
        }
        ((float*)(buf + L::sx))[sblk * kTM + srow] = fx.s;
        // bytes j..j+7 of the block's nibbles: low nibbles are elements j.., high nibbles elements 16 + j..
        u32x2 lo, hi;
#pragma unroll
        for (int d = 0; d < 2; d++) {
            lo[d] = nibbles_to_i8(f.q[d] & 0x0F0F0F0Fu);
            hi[d] = nibbles_to_i8((f.q[d] >> 4) & 0x0F0F0F0Fu);
        }
        uint8_t* wrow = buf + L::w + wrow_i * kRow + 32 * (c8 >> 1) + 8 * (c8 & 1);
        *(u32x2*)wrow = lo;
        *(u32x2*)(wrow + 16) = hi;
        ((float*)(buf + L::sw))[(c8 >> 1) * kTN + wrow_i] = f16_bits_to_f32((uint16_t)f.d);  // both halves' threads store it
    };

    f32x16 acc;
#pragma unroll
    for (int i = 0; i < 16; i++) acc[i] = 0.f;

    auto compute = [&](int step) {
        const uint8_t* buf = smem + (step & 1) * L::step;
        const uint8_t* xa = buf + L::x + (wm * 32 + l32) * kRow + 16 * lh;
        const uint8_t* wa = buf + L::w + (wn * 32 + l32) * kRow + 16 * lh;
        const float* sx = (const float*)(buf + L::sx) + wm * 32 + 4 * lh;
        const float* sw = (const float*)(buf + L::sw) + wn * 32 + l32;
#pragma unroll
        for (int b = 0; b < 4; b++) {
            i32x16 zero;
#pragma unroll
            for (int i = 0; i < 16; i++) zero[i] = 0;
            const i32x4 wv = *(const i32x4*)(wa + 32 * b);
            const i32x4 x0 = *(const i32x4*)(xa + 32 * b);
            const i32x4 x1 = *(const i32x4*)(xa + kTM * kRow + 32 * b);
            const i32x4 x2 = *(const i32x4*)(xa + 2 * kTM * kRow + 32 * b);
            const i32x16 t0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(x0, wv, zero, 0, 0, 0);
            const i32x16 t1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(x1, wv, zero, 0, 0, 0);
            const i32x16 t2 = __builtin_amdgcn_mfma_i32_32x32x32_i8(x2, wv, zero, 0, 0, 0);
            const float dw = sw[b * kTN];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const f32x4 dx = *(const f32x4*)(sx + b * kTM + 8 * j);
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const int i = 4 * j + k;
                    const int isum = t0[i] + (t1[i] << 8) + (t2[i] << 16);  // below 2^31: 32 * 8 * kFixMax
                    const float wsc = dw * dx[k];
                    acc[i] = fmaf(wsc, (float)isum, acc[i]);
                }
            }
        }
    };

    const int steps = K / kStepK;
    fetch_w(fw0, 0);
    fetch_x(0);
    fetch_w(fw1, steps > 1 ? 1 : 0);
    stage(fw0, 0);
    lds_barrier();
    // Even steps live in buffer 0, odd ones in buffer 1. No branches around the loads and stores: past the
    // end the last step is requested and staged again, into the buffer that is not being read.
    for (int step = 0; step < steps; step += 2) {
        const int s1 = step + 1 < steps ? step + 1 : steps - 1, s2 = step + 2 < steps ? step + 2 : steps - 1,
                  s3 = step + 3 < steps ? step + 3 : steps - 1;
        fetch_w(fw0, s2);
        fetch_x(s1);
        compute(step);
        stage(fw1, 1);
        lds_barrier();
        if (step + 1 < steps) {
            fetch_w(fw1, s3);
            fetch_x(s2);
            compute(step + 1);
            stage(fw0, 0);
            lds_barrier();
        }
    }

    const int n = n0 + wn * 32 + l32;
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const int m = m0 + wm * 32 + 8 * (i >> 2) + 4 * lh + (i & 3);
        if (m < M && n < N) {
            float v = acc[i];
            if (resid) v = v + resid[(int64_t)m * N + n];
            y[(int64_t)m * N + n] = v;
        }
    }
}

}  // namespace

bool qgemm_q4_0_fx_ok(const void* W, int64_t M, int64_t N, int64_t K) {
    return K > 0 && K % kStepK == 0 && K <= (1 << 20) && ((uintptr_t)W & 1) == 0 && M > 0 && N > 0 &&
           ((M + kTM - 1) / kTM) * ((N + kTN - 1) / kTN) < ((int64_t)1 << 28);
}

// Whether this kernel beats the row kernels: those take about 1 us per row of x and 8.7 MB of W; a
// workgroup here about 2.8 us per step of 128 of K, 256 workgroups at a time (measured at 4096 x 4096
// to 14336 x 4096, 32 to 2048 rows).
double qgemm_q4_0_fx_cost_us(int64_t M, int64_t N, int64_t K) {
    const int64_t tiles = ((M + kTM - 1) / kTM) * ((N + kTN - 1) / kTN);
    return (double)((tiles + 255) / 256) * (double)(K / kStepK) * 2.8;
}

bool qgemm_q4_0_fx_pays(const void* W, int64_t M, int64_t N, int64_t K) {
    if (M < 16 || !qgemm_q4_0_fx_ok(W, M, N, K)) return false;
    const double rows_us = (double)M * ((double)N * (double)(K / 32) * 18.0) / 8.7e6;
    return qgemm_q4_0_fx_cost_us(M, N, K) < rows_us;
}

// act: q4_0_fx_convert_act's rows, as pairs if ws is given. y = x . W^T (+ resid, which may be y itself).
hipError_t qgemm_q4_0_fx(const void* W, const void* act, float* y, const float* resid, int64_t M, int64_t N, int64_t K, void* ws, hipStream_t st) {
    if (ws) return qgemm_q4_0_fx16(W, act, y, resid, M, N, K, ws, st);
    static std::atomic<bool> raised{false};  // threads may race here: both then set the same attribute
    if (!raised) {
        hipError_t e = hipFuncSetAttribute((const void*)qgemm_q4_0_fx_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, Layout::total);
        if (e != hipSuccess) return e;
        raised = true;
    }
    const int tiles_m = (int)((M + kTM - 1) / kTM), ntiles = (int)((N + kTN - 1) / kTN);
    const int per_xcd = (ntiles + 7) / 8;
    hipLaunchKernelGGL(qgemm_q4_0_fx_kernel, dim3((unsigned)(8 * per_xcd * tiles_m)), dim3(512), Layout::total, st, (const uint8_t*)W,
                       (const uint8_t*)act, y, resid, (int)M, (int)N, (int)K, (int64_t)q4_0_fx_act_bytes(K), tiles_m, ntiles);
    note_kernel("qgemm_q4_0_fx_kernel");
    return hipGetLastError();
}

}  // namespace mimir
