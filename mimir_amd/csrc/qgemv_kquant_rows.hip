// Products of a few rows of x with Q4_K or Q6_K weights on the int8 matrix cores
// of gfx950, W read once per eight rows of x: the decoding step of a batch of
// sequences for models with K-quant linears. The arithmetic is qdotQ4KGo's and
// qdotQ6KGo's (backend/cpu/qmatmul.go:148-172, 180-200), operation for operation,
// so the results are the CPU's bits like those of the other K-quant kernels
// (qgemv_kquant.hip, qgemm_kquant.hip). Q4_K: per super-block of 256 the integer sums
//   sumi = sum_j sc_j (sub-block j's quants . x),  summ = sum_j m_j (sum of x over sub-block j)
// with the 6-bit scales and mins of scale_min_k4, then in float32
//   dd = d_w d_x, dm = dmin_w d_x, acc += dd float(sumi), accm += dm float(summ)
// over the super-blocks in order, and acc - accm at the end.
//
// x comes rounded to int8 per super-block (kq_convert_act: quants, sums of 16,
// scale). A sub-block is 32 weights: the K of one v_mfma_i32_32x32x32_i8, whose
// first operand holds the eight rows of x (8 of its 32 rows) and whose second
// 32 rows of W as their nibbles 0..15. A lane ends up with its row of W's
// sub-block sums for four rows of x; the scales are per lane, so sc_j times the
// sum is one multiply-add, and m_j times the two sums of 16 one v_dot2.
//
// A workgroup of eight wavefronts (four for Q6_K) owns 32 rows of W; a wavefront
// takes every eighth super-block and leaves its float32 terms per output (two
// for Q4_K, one for Q6_K) in LDS; when all are there the first wavefront adds
// them in the super-blocks' order, which is the CPU's. x of a super-block (2.3 KB
// for eight rows) is staged per wavefront in LDS; a lane loads its row's header
// and its half of each group of nibbles where they lie (five aligned 16-byte
// loads a super-block; for Q6_K see WBlock<kQ6_K>).
#include "device_util.h"
#include "kernels.h"

namespace mimir {

#pragma clang fp contract(off)

namespace {

typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef short s16x2 __attribute__((ext_vector_type(2)));

constexpr int kRows = 8;                        // rows of x a group holds
constexpr int kXq = 0, kXs = 2048, kXd = 2304;  // a super-block of x for eight rows in LDS: quants [8][256], sums [8][16] int16, scales [8]
constexpr int kXBytes = 2336;

// scale_min_k4 (backend/cpu/quant.go:129-134) on the twelve scale bytes held as three dwords.
__device__ __forceinline__ int q4k_sc(uint32_t s0, uint32_t s2, int j) {
    const int sh = 8 * (j & 3);
    return j < 4 ? (int)((s0 >> sh) & 63) : (int)(((s2 >> sh) & 0xf) | (((s0 >> (sh + 6)) & 3) << 4));
}
__device__ __forceinline__ int q4k_mn(uint32_t s1, uint32_t s2, int j) {
    const int sh = 8 * (j & 3);
    return j < 4 ? (int)((s1 >> sh) & 63) : (int)(((s2 >> (sh + 4)) & 0xf) | (((s1 >> (sh + 6)) & 3) << 4));
}

// What a lane holds of its row's super-block between the loads and the arithmetic, how it loads it, and the float32 terms it
// makes of it for its four rows of x (x of the super-block lies in the wavefront's LDS at xl).
template <int DT> struct WBlock;

template <> struct WBlock<kQ4_K> {
    static constexpr int kBytes = 144, kTerms = 2;
    u32x4 hdr, q[4];  // d, dmin, scales; the lane's 16 bytes of nibbles of each of the four groups of 64
    __device__ __forceinline__ void load(const uint8_t* wb, int lh) {
        hdr = *(const u32x4*)wb;
#pragma unroll
        for (int g = 0; g < 4; g++) q[g] = *(const u32x4*)(wb + 16 + 32 * g + 16 * lh);
    }
    // t[0] = d_w d_x float(sumi), t[1] = dmin_w d_x float(summ)
    __device__ __forceinline__ void terms(const uint8_t* xl, int l32, int lh, f32x4* t) const {
        const uint8_t* xrow = xl + kXq + (l32 & 7) * 256 + 16 * lh;  // this lane's operand row of x (rows 8.. of the operand repeat rows 0..7)
        const uint32_t s0 = hdr[1], s1 = hdr[2], s2 = hdr[3];
        int sumi[4] = {0, 0, 0, 0}, summ[4] = {0, 0, 0, 0};
        // the sums of 16 of this lane's four rows of x: dword c holds chunks 2c and 2c + 1
        u32x4 sv[4][2];
#pragma unroll
        for (int jj = 0; jj < 4; jj++) {
            sv[jj][0] = *(const u32x4*)(xl + kXs + (4 * lh + jj) * 32);
            sv[jj][1] = *(const u32x4*)(xl + kXs + (4 * lh + jj) * 32 + 16);
        }
        const f32x4 xd = *(const f32x4*)(xl + kXd + 16 * lh);
#pragma unroll
        for (int g = 0; g < 4; g++) {
            i32x4 wlo, whi;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                wlo[i] = (int)(q[g][i] & 0x0F0F0F0Fu);
                whi[i] = (int)((q[g][i] >> 4) & 0x0F0F0F0Fu);
            }
            const i32x4 xa = *(const i32x4*)(xrow + 64 * g), xb = *(const i32x4*)(xrow + 64 * g + 32);
            i32x16 zero;
#pragma unroll
            for (int i = 0; i < 16; i++) zero[i] = 0;
            const i32x16 ca = __builtin_amdgcn_mfma_i32_32x32x32_i8(xa, wlo, zero, 0, 0, 0);
            const i32x16 cb = __builtin_amdgcn_mfma_i32_32x32x32_i8(xb, whi, zero, 0, 0, 0);
            const int sca = q4k_sc(s0, s2, 2 * g), scb = q4k_sc(s0, s2, 2 * g + 1);
            const int ma = q4k_mn(s1, s2, 2 * g), mb = q4k_mn(s1, s2, 2 * g + 1);
            const uint32_t ma2 = (uint32_t)ma * 0x00010001u, mb2 = (uint32_t)mb * 0x00010001u;
#pragma unroll
            for (int jj = 0; jj < 4; jj++) {
                sumi[jj] += sca * ca[jj] + scb * cb[jj];
                // sub-block 2g is chunks 4g, 4g + 1 (dword 2g of the sums), sub-block 2g + 1 chunks 4g + 2, 4g + 3
                const uint32_t pa = sv[jj][g >> 1][2 * (g & 1)], pb = sv[jj][g >> 1][2 * (g & 1) + 1];
                summ[jj] = __builtin_amdgcn_sdot2(__builtin_bit_cast(s16x2, pa), __builtin_bit_cast(s16x2, ma2), summ[jj], false);
                summ[jj] = __builtin_amdgcn_sdot2(__builtin_bit_cast(s16x2, pb), __builtin_bit_cast(s16x2, mb2), summ[jj], false);
            }
        }
        const float dw = f16_bits_to_f32((uint16_t)hdr[0]), dmin = f16_bits_to_f32((uint16_t)(hdr[0] >> 16));
#pragma unroll
        for (int jj = 0; jj < 4; jj++) {
            const float dd = dw * xd[jj], dm = dmin * xd[jj];
            t[0][jj] = dd * (float)sumi[jj];
            t[1][jj] = dm * (float)summ[jj];
        }
    }
};

// Q6_K (qdotQ6KGo, backend/cpu/qmatmul.go:180-200): 210-byte blocks, so a row's blocks start on even addresses only and the
// 16-byte loads below are unaligned ones. Half h2 of a super-block (128 weights) is 64 bytes of ql and 32 of qh: slab s = 0..3 of the
// half (32 weights) has its low four bits in the low (s < 2) or high nibbles of ql[64 h2 + 32 (s & 1) ..] and its upper two at bit 2 s
// of qh[32 h2 ..]; a scale per chunk of 16, a zero point of 32. The matrix-core product must keep the two chunks of a slab apart: the
// operand's row 8 c + m holds row m of x with everything but chunk c of the slab zeroed, so the result's rows 0..7 are chunk 0's sums
// and rows 8..15 chunk 1's (rows 16..31 are unused).
template <> struct WBlock<kQ6_K> {
    static constexpr int kBytes = 210, kTerms = 1;
    u32x4 ql[2][2], qh[2], sc;
    uint32_t d;
    __device__ __forceinline__ static u32x4 load16(const uint8_t* p) {
        u32x4 v;
        __builtin_memcpy(&v, __builtin_assume_aligned(p, 2), 16);
        return v;
    }
    __device__ __forceinline__ void load(const uint8_t* wb, int lh) {
#pragma unroll
        for (int h2 = 0; h2 < 2; h2++) {
            ql[h2][0] = load16(wb + 64 * h2 + 16 * lh);
            ql[h2][1] = load16(wb + 64 * h2 + 32 + 16 * lh);
            qh[h2] = load16(wb + 128 + 32 * h2 + 16 * lh);
        }
        sc = load16(wb + 192);
        d = *(const uint16_t*)(wb + 208);
    }
    // t[0] = d_w d_x float(sum over the chunks of sc (q . x - 32 sum of x))
    __device__ __forceinline__ void terms(const uint8_t* xl, int l32, int lh, f32x4* t) const {
        const bool keep = (l32 >> 3) == lh;  // operand rows 0..7 keep the first 16 of a slab (held by lanes of half 0), rows 8..15 the second
        const uint8_t* xrow = xl + kXq + (l32 & 7) * 256 + 16 * lh;
        int sumi[4] = {0, 0, 0, 0}, summ[4] = {0, 0, 0, 0};
        u32x4 sv[4][2];
#pragma unroll
        for (int jj = 0; jj < 4; jj++) {
            sv[jj][0] = *(const u32x4*)(xl + kXs + (4 * lh + jj) * 32);
            sv[jj][1] = *(const u32x4*)(xl + kXs + (4 * lh + jj) * 32 + 16);
        }
        const f32x4 xd = *(const f32x4*)(xl + kXd + 16 * lh);
#pragma unroll
        for (int h2 = 0; h2 < 2; h2++)
#pragma unroll
            for (int s = 0; s < 4; s++) {
                i32x4 w, xa = *(const i32x4*)(xrow + 128 * h2 + 32 * s);
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const uint32_t lo = (ql[h2][s & 1][i] >> (s & 2 ? 4 : 0)) & 0x0F0F0F0Fu, hi = (qh[h2][i] >> (2 * s)) & 0x03030303u;
                    w[i] = (int)(lo | (hi << 4));  // 0..63
                    xa[i] = keep ? xa[i] : 0;
                }
                i32x16 zero;
#pragma unroll
                for (int i = 0; i < 16; i++) zero[i] = 0;
                const i32x16 c = __builtin_amdgcn_mfma_i32_32x32x32_i8(xa, w, zero, 0, 0, 0);
                // the scales of chunks 8 h2 + 2 s and + 1: bytes 2 (s & 1), 2 (s & 1) + 1 of dword 2 h2 + s / 2
                const uint32_t sd = sc[2 * h2 + (s >> 1)];
                const int sca = (int)(int8_t)(sd >> (16 * (s & 1))), scb = (int)(int8_t)(sd >> (16 * (s & 1) + 8));
                const uint32_t pair = ((uint32_t)sca & 0xffffu) | ((uint32_t)scb << 16);
#pragma unroll
                for (int jj = 0; jj < 4; jj++) {
                    sumi[jj] += sca * c[jj] + scb * c[4 + jj];
                    const uint32_t ps = sv[jj][h2][s];  // a copy: __builtin_bit_cast of a vector's element takes element 0 with this compiler
                    summ[jj] = __builtin_amdgcn_sdot2(__builtin_bit_cast(s16x2, ps), __builtin_bit_cast(s16x2, pair), summ[jj], false);
                }
            }
        const float dw = f16_bits_to_f32((uint16_t)d);
#pragma unroll
        for (int jj = 0; jj < 4; jj++) {
            const float dd = dw * xd[jj];
            t[0][jj] = dd * (float)(sumi[jj] - 32 * summ[jj]);
        }
    }
};

// The pieces of x of a super-block a lane fetches for the wavefront's LDS.
struct XPieces {
    u32x4 xq[2];  // two 16-byte pieces of the eight rows' quants
    u32x4 xs;     // lanes 0..15: a piece of their sums
    float xd;     // lanes 0..7: a row's scale
};

template <int DT, int kWaves>
__global__ __launch_bounds__(64 * kWaves) void qgemv_kq_rows_kernel(const uint8_t* __restrict__ W, const uint8_t* act, float* y, const float* resid,
                                                                     int M_all, int N, int nsb, int64_t act_row_bytes) {
    typedef WBlock<DT> WB;
    constexpr int kT = WB::kTerms;
    extern __shared__ __align__(16) uint8_t smem[];  // terms [nsb][kT][64] of four floats, then a super-block of x per wavefront
    const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, lh = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // blockIdx.z: the group of eight rows of x
    const int64_t row0 = (int64_t)kRows * blockIdx.z;
    act += row0 * act_row_bytes;
    const int M = M_all - (int)row0 < kRows ? M_all - (int)row0 : kRows;
    const int n = blockIdx.x * 32 + l32;
    const uint8_t* wrow = W + (int64_t)(n < N ? n : N - 1) * nsb * WB::kBytes;
    f32x4* terms = (f32x4*)smem;
    uint8_t* xl = smem + (size_t)nsb * kT * 1024 + wave * kXBytes;

    // pieces of x a lane fetches: quants p = lane, 64 + lane (row p / 16, bytes 16 (p % 16)..); sums (lanes below 16:
    // row lane / 2, half lane % 2); scale (lanes below 8: row lane). Rows from M on repeat the last one.
    const uint8_t* xsrc[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int p = 64 * i + lane, r = p >> 4;
        xsrc[i] = act + (int64_t)(r < M ? r : M - 1) * act_row_bytes + 16 * (p & 15);
    }
    const int rs = (lane >> 1) < M ? (lane >> 1) : M - 1, rd = lane < M ? lane : M - 1;  // used by lanes below 16 and 8
    const uint8_t* ssrc = act + (int64_t)(rs & 7) * act_row_bytes + (int64_t)nsb * 256 + 16 * (lane & 1);
    const uint8_t* dsrc = act + (int64_t)(rd & 7) * act_row_bytes + (int64_t)nsb * 288;

    auto fetch = [&](WB& w, XPieces& f, int sb) {
        w.load(wrow + (int64_t)sb * WB::kBytes, lh);
#pragma unroll
        for (int i = 0; i < 2; i++) f.xq[i] = *(const u32x4*)(xsrc[i] + (int64_t)sb * 256);
        if (lane < 16) f.xs = *(const u32x4*)(ssrc + (int64_t)sb * 32);
        if (lane < 8) f.xd = ((const float*)dsrc)[sb];
    };

    WB wcur, wnxt;
    XPieces xcur, xnxt;
    if (wave < nsb) fetch(wcur, xcur, wave);
    for (int sb = wave; sb < nsb; sb += kWaves) {
        fetch(wnxt, xnxt, sb + kWaves < nsb ? sb + kWaves : sb);
        // x of the super-block into this wavefront's LDS (its own: a wavefront's LDS operations complete in order)
#pragma unroll
        for (int i = 0; i < 2; i++) *(u32x4*)(xl + kXq + 16 * (64 * i + lane)) = xcur.xq[i];
        if (lane < 16) *(u32x4*)(xl + kXs + 16 * lane) = xcur.xs;
        if (lane < 8) *(float*)(xl + kXd + 4 * lane) = xcur.xd;
        f32x4 t[kT];
        wcur.terms(xl, l32, lh, t);
#pragma unroll
        for (int i = 0; i < kT; i++) terms[(sb * kT + i) * 64 + lane] = t[i];
        wcur = wnxt;
        xcur = xnxt;
    }
    __syncthreads();
    if (wave != 0) return;
    f32x4 acc[kT];
#pragma unroll
    for (int i = 0; i < kT; i++) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int sb = 0; sb < nsb; sb++) {  // the CPU's order
#pragma unroll
        for (int i = 0; i < kT; i++) {
            const f32x4 t = terms[(sb * kT + i) * 64 + lane];
#pragma unroll
            for (int jj = 0; jj < 4; jj++) acc[i][jj] = acc[i][jj] + t[jj];
        }
    }
    if (n < N) {
#pragma unroll
        for (int jj = 0; jj < 4; jj++) {
            const int m = 4 * lh + jj;
            if (m < M) {
                const int64_t at = (row0 + m) * N + n;
                const float v = kT == 2 ? acc[0][jj] - acc[kT - 1][jj] : acc[0][jj];
                y[at] = resid ? v + resid[at] : v;
            }
        }
    }
}

}  // namespace

static int g_kq_rows = 0;  // measurement aid: 1 = never, 2 = for any number of rows the kernel takes
void set_kquant_rows(int v) { g_kq_rows = v; }

static int g_kq_rows_waves = 0;  // measurement aid: 4 or 8 wavefronts to a workgroup whatever the type
void set_kquant_rows_waves(int v) { g_kq_rows_waves = v; }
// Q6_K's kernel holds more of W in registers (three wavefronts to a SIMD): four wavefronts to a workgroup let three workgroups share a
// compute unit where eight would leave it to one.
static int rows_waves(int dt) { return g_kq_rows_waves == 4 || g_kq_rows_waves == 8 ? g_kq_rows_waves : dt == kQ4_K ? 8 : 4; }
static size_t rows_lds(int dt, int64_t nsb) { return (size_t)nsb * (dt == kQ4_K ? 2 : 1) * 1024 + 8 * kXBytes; }

// Two rows of x or more, converted (kq_convert_act); the terms of 32 rows of W in LDS; Q4_K's W 16-byte aligned, Q6_K's on an even address.
bool qgemv_kquant_rows_ok(int dt, const QGemvArgs& a) {
    const int64_t nsb = a.K / 256;
    return (dt == kQ4_K || dt == kQ6_K) && g_kq_rows != 1 && a.M >= 2 && a.M <= 8 * 65535 && a.act && a.K % 256 == 0 && nsb > 0 &&
           ((uintptr_t)a.W & (dt == kQ4_K ? 15 : 1)) == 0 && ((uintptr_t)a.act & 15) == 0 && a.N > 0 && a.N <= (1ll << 30) &&
           rows_lds(dt, nsb) <= 160 * 1024;
}

// Where it is the faster choice. A pass over W for eight rows of x runs at about 3.3 TB/s (Q4_K; 14336 x 4096 in 11 us, 28672 x 4096
// in 20 us, after 4 us for converting x) or 2.6 TB/s (Q6_K; 19 and 37 us); the tiled kernel of qgemm_kquant.hip spends about 2.1 us per
// super-block of K and round of 256 tiles of 128 x 128 (at 32 rows of x and 14336 x 4096: 36 us here, 34 us there; at 4096 x 14336: 36
// and 100 us).
bool qgemv_kquant_rows_pays(int dt, const QGemvArgs& a) {
    if (!qgemv_kquant_rows_ok(dt, a)) return false;
    if (g_kq_rows == 2 || a.M <= 8) return true;
    if (a.M > 64) return false;
    const double nsb = (double)(a.K / 256), groups = (double)((a.M + kRows - 1) / kRows);
    const double rows_us = groups * (double)a.N * nsb * (dt == kQ4_K ? 144 / 3.3e6 : 210 / 2.6e6);
    const int64_t tiles = ((a.M + 127) / 128) * ((a.N + 127) / 128);
    return rows_us < (double)((tiles + 255) / 256) * nsb * 2.1;
}

template <int DT, int WAVES>
static hipError_t launch_kq_rows(const QGemvArgs& a, hipStream_t st) {
    const int nsb = (int)(a.K / 256);
    static bool raised = false;
    if (!raised) {
        hipError_t e = hipFuncSetAttribute((const void*)qgemv_kq_rows_kernel<DT, WAVES>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return e;
        raised = true;
    }
    const size_t lds = (size_t)nsb * WBlock<DT>::kTerms * 1024 + WAVES * kXBytes;
    hipLaunchKernelGGL((qgemv_kq_rows_kernel<DT, WAVES>), dim3((unsigned)((a.N + 31) / 32), 1, (unsigned)((a.M + kRows - 1) / kRows)), dim3(64 * WAVES),
                       lds, st, (const uint8_t*)a.W, (const uint8_t*)a.act, a.y, a.resid, (int)a.M, (int)a.N, nsb, (int64_t)kq_act_bytes(a.K));
    return hipGetLastError();
}

hipError_t qgemv_kquant_rows(int dt, const QGemvArgs& a, hipStream_t st) {
    const bool eight = rows_waves(dt) == 8;
    if (dt == kQ4_K) return eight ? launch_kq_rows<kQ4_K, 8>(a, st) : launch_kq_rows<kQ4_K, 4>(a, st);
    return eight ? launch_kq_rows<kQ6_K, 8>(a, st) : launch_kq_rows<kQ6_K, 4>(a, st);
}

}  // namespace mimir
