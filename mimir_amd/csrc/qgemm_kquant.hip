// Products of many rows of x with Q4_K and Q6_K weights on the matrix cores of
// gfx950: y[M, N] = x[M, K] . W[N, K]^T with x already rounded to int8 per
// super-block of 256 (kq_convert_act), computing what the reference's CPU tiles
// compute (backend/cpu/qtile.go:124-271), which is what its dot products
// compute (qdotQ4KGo and qdotQ6KGo, backend/cpu/qmatmul.go:148-200): per
// super-block an integer sum, one float32 product of the two scales, one
// multiply and one add, the super-blocks of a row taken in order. Every output
// here goes through the same float32 operations in the same order, so the
// results are the CPU's bit for bit.
//
// The integer sum of a super-block is sum_i s(i) q_i x_i with a 6-bit scale and
// a 4-bit quant (Q4_K) or an int8 scale and a 6-bit quant less 32 (Q6_K). The
// scaled weight s q has 10 or 14 bits, too many for the int8 matrix
// instruction, so it is split: s q = 64 a + b (Q4_K) or 128 a + b (Q6_K) with
// both digits in int8 range, and the sum is 64 A + B from two planes of
// v_mfma_i32_32x32x32_i8 against the same fragment of x. Integer sums are
// exact, so the split changes nothing. Q4_K's second sum, the mins against the
// sums of x, is sum over the sixteen 16-element groups of m(g / 2) S(g): one
// v_mfma_f32_32x32x16_f16 per tile and super-block, exact because S (at most
// 16 * 127) and m (at most 63) are integers binary16 holds and the products
// and their sum stay below 2^24.
//
// A workgroup of eight wavefronts owns a tile of 128 or 256 rows of x by 64 rows
// of W; a wavefront owns 32 or 64 by 32 of it. The loop runs over halves of a
// super-block (128 of K): the int8 rows of x and the two planes of W for the
// next half are loaded from global memory before the current half is
// multiplied, and split and stored into the other of two LDS buffers
// afterwards; rows are padded to 144 bytes, which makes the 128-bit fragment
// reads conflict-free. After the second half the wavefront turns its integer
// sums into float32 as above. Both matrix instructions take, per lane, the
// bytes or halves k = 16 or 8 (lane / 32).. of row (lane % 32); the result holds
// column (lane % 32) and rows 8 (i / 4) + 4 (lane / 32) + i % 4 in register i.
#include "device_util.h"
#include "kernels.h"

namespace mimir {

#pragma clang fp contract(off)

namespace {

typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef short s16x2 __attribute__((ext_vector_type(2)));
typedef short s16x8 __attribute__((ext_vector_type(8)));

constexpr int kTN = 64;          // rows of W per workgroup
constexpr int kHalf = 128;       // K per step
constexpr int kRow = kHalf + 16; // bytes per LDS row of int8
constexpr int kSumRow = 48;      // bytes per LDS row of sixteen binary16 (32 used)

// LDS: two step buffers (x rows, plane A, plane B) and what the end of a
// super-block needs (scales of x, sums of x, scales and mins of W), stored with
// the second half's step: the barrier that ends the super-block's last step
// also separates its readers from the next writers.
template <int TM>
struct Layout {
    static constexpr int x = 0;
    static constexpr int wa = TM * kRow;
    static constexpr int wb = wa + kTN * kRow;
    static constexpr int step = wb + kTN * kRow;
    static constexpr int side0 = 2 * step;
    static constexpr int dx = 0;                       // float[TM]
    static constexpr int xsum = TM * 4;                // binary16[TM][16], rows of kSumRow bytes
    static constexpr int dw = xsum + TM * kSumRow;     // float[kTN][2]: d, dmin
    static constexpr int mins = dw + kTN * 8;          // binary16[kTN][16], rows of kSumRow bytes
    static constexpr int side = mins + kTN * kSumRow;
    static constexpr int total = side0 + side;
};

__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

__device__ __forceinline__ u32x2 load_u32x2_unaligned(const uint8_t* p) {
    u32x2 v;
    __builtin_memcpy(&v, p, 8);
    return v;
}

// Bytes 0 and 2 of lo, then bytes 0 and 2 of hi.
__device__ __forceinline__ uint32_t even_bytes(uint32_t lo, uint32_t hi) { return __builtin_amdgcn_perm(hi, lo, 0x06040200u); }
// Bytes 0 and 1 (or 2 and 3) of v, each widened to 16 bits.
__device__ __forceinline__ uint32_t widen01(uint32_t v) { return __builtin_amdgcn_perm(0u, v, 0x0c010c00u); }
__device__ __forceinline__ uint32_t widen23(uint32_t v) { return __builtin_amdgcn_perm(0u, v, 0x0c030c02u); }

// Four quants in the bytes of q (each below 16) times the 6-bit scale s, split
// into the digits of 64 a + b.
__device__ __forceinline__ void split_q4k(uint32_t q, uint32_t s, uint32_t& a, uint32_t& b) {
    uint32_t p01 = __umul24(widen01(q), s), p23 = __umul24(widen23(q), s);  // two products below 1024 each
    a = even_bytes(p01 >> 6, p23 >> 6);
    b = even_bytes(p01 & 0x003F003Fu, p23 & 0x003F003Fu);
}

// Four quants in the bytes of q (each below 64) less 32, times the int8 scale
// s, split into the digits of 128 a + b with b in 0..127.
__device__ __forceinline__ void split_q6k(uint32_t q, int s, uint32_t& a, uint32_t& b) {
    const s16x2 bias = {32, 32}, sc = {(short)s, (short)s};
    s16x2 p01 = (__builtin_bit_cast(s16x2, widen01(q)) - bias) * sc;
    s16x2 p23 = (__builtin_bit_cast(s16x2, widen23(q)) - bias) * sc;
    a = even_bytes(__builtin_bit_cast(uint32_t, p01 >> 7), __builtin_bit_cast(uint32_t, p23 >> 7));
    b = even_bytes(__builtin_bit_cast(uint32_t, p01) & 0x007F007Fu, __builtin_bit_cast(uint32_t, p23) & 0x007F007Fu);
}

// scale_min_k4 (backend/cpu/quant.go:129-134) on the twelve scale bytes held as three dwords.
__device__ __forceinline__ uint32_t q4k_scale(uint32_t s0, uint32_t s2, int j) {
    const int sh = 8 * (j & 3);
    return j < 4 ? (s0 >> sh) & 63 : ((s2 >> sh) & 0xf) | (((s0 >> (sh + 6)) & 3) << 4);
}
__device__ __forceinline__ uint32_t q4k_min(uint32_t s1, uint32_t s2, int j) {
    const int sh = 8 * (j & 3);
    return j < 4 ? (s1 >> sh) & 63 : ((s2 >> (sh + 4)) & 0xf) | (((s1 >> (sh + 6)) & 3) << 4);
}

// What a thread holds between the loads of a step and its LDS stores: its
// piece of W, requested two steps ahead (it comes from HBM), and its pieces of
// the x tile, requested one step ahead (they come from the L2, every tile of
// the same rows reads them).
struct FetchedW {
    u32x4 hdr;      // Q4_K: d, dmin and the scales. Q6_K: x, y = the 8 scales of the half, z = d
    u32x2 q;        // 8 bytes of nibbles
    u32x2 qh;       // Q6_K: the 8 bytes of upper bits that go with them
};
template <int XV>
struct FetchedX {
    u32x4 x[XV];    // 16-byte pieces of the x tile
    u32x4 sums;     // second half only: eight int16 sums of x
    float dx;       // second half only: the scale of one row of x
};

template <int H>
struct Half {
    static constexpr int value = H;
};

// MT 32-row tiles per wavefront: the workgroup's tile is (128 MT) x 64. DEPTH says how far ahead of
// its LDS stores a step's global loads are requested: 0 one step for W and x, 1 two steps for W, 2 two
// steps for both; each step further costs the registers of one more set of loads.
template <int DT, int MT, int DEPTH, bool OUT_BF16>
__global__ __launch_bounds__(512) void qgemm_kquant_kernel(const uint8_t* __restrict__ W, const uint8_t* __restrict__ act,
                                                            void* __restrict__ yv, int M, int N, int nsb,
                                                            int64_t act_row_bytes, int tiles_m, int ntiles) {
    constexpr int TM = 128 * MT;
    constexpr int XV = TM * 8 / 512;  // 16-byte pieces of x per thread and step: piece p is row p / 8, bytes 16 (p % 8)..
    constexpr int BB = DT == kQ4_K ? 144 : 210;
    typedef Layout<TM> L;
    extern __shared__ __align__(16) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave & 3, wn = wave >> 2, l32 = lane & 31, lh = lane >> 5;

    // Tiles that share rows of W run next to each other on one XCD (workgroup i
    // goes to XCD i % 8), so the second and later tiles find W in that L2.
    const int id = blockIdx.x, xcd = id & 7, slot = id >> 3;
    const int per_xcd = (ntiles + 7) >> 3;
    const int t = slot / tiles_m + xcd * per_xcd;
    const int tm = slot % tiles_m;
    if (slot >= per_xcd * tiles_m || t >= ntiles) return;
    const int m0 = tm * TM, n0 = t * kTN;

    // This thread's part of the W tile: 8 bytes of nibbles of row wrow_i, piece c8 of the half. Its
    // addresses, and those of its pieces of x, are a base the workgroup shares plus 32 bits of its own.
    const int wrow_i = tid >> 3, c8 = tid & 7;
    const int last_n = N - 1 - n0, last_m = M - 1 - m0;
    const uint8_t* w_t = W + (int64_t)n0 * nsb * BB;
    const uint32_t woff = (uint32_t)(wrow_i < last_n ? wrow_i : last_n) * (uint32_t)(nsb * BB);
    const uint8_t* act_t = act + (int64_t)m0 * act_row_bytes;
    uint32_t xoff[XV];
#pragma unroll
    for (int i = 0; i < XV; i++) {
        const int r = (tid + 512 * i) >> 3;
        xoff[i] = (uint32_t)(r < last_m ? r : last_m) * (uint32_t)act_row_bytes + 16 * (tid & 7);
    }
    // sums: two threads a row; scales: a thread a row
    // (with 128-row tiles two threads do the same row's part: branch-free, and the same bytes to the same place)
    const int srow = (tid >> 1) & (TM - 1), drow = tid & (TM - 1);
    const uint32_t soff = (uint32_t)(srow < last_m ? srow : last_m) * (uint32_t)act_row_bytes + 16 * (tid & 1);
    const uint32_t doff = (uint32_t)(drow < last_m ? drow : last_m) * (uint32_t)act_row_bytes;
    const uint8_t* sums_t = act_t + (int64_t)nsb * 256;
    const uint8_t* dx_t = act_t + (int64_t)nsb * 288;

    FetchedW fw0, fw1;
    FetchedX<XV> fx0, fx1;
    auto fetch_w = [&](FetchedW& f, int sb, auto half) {
        constexpr int h = decltype(half)::value;
        const uint8_t* wb = w_t + (int64_t)sb * BB + woff;
        if (DT == kQ4_K) {
            f.hdr = *(const u32x4*)wb;
            f.q = *(const u32x2*)(wb + 16 + 64 * h + 8 * c8);
        } else {
            f.q = load_u32x2_unaligned(wb + 64 * h + 8 * c8);
            f.qh = load_u32x2_unaligned(wb + 128 + 32 * h + 8 * (c8 & 3));
            u32x2 sc = load_u32x2_unaligned(wb + 192 + 8 * h);
            f.hdr[0] = sc[0];
            f.hdr[1] = sc[1];
            f.hdr[2] = load_u16(wb + 208);
        }
    };
    auto fetch_x = [&](FetchedX<XV>& fx, int sb, auto half) {
        constexpr int h = decltype(half)::value;
#pragma unroll
        for (int i = 0; i < XV; i++) fx.x[i] = *(const u32x4*)(act_t + ((int64_t)sb * 256 + kHalf * h) + xoff[i]);
        if (h == 1) {
            if (DT == kQ4_K) fx.sums = *(const u32x4*)(sums_t + (int64_t)sb * 32 + soff);
            fx.dx = *(const float*)(dx_t + (int64_t)sb * 4 + doff);
        }
    };
    auto stage = [&](const FetchedW& f, const FetchedX<XV>& fx, int sb, auto half) {
        constexpr int h = decltype(half)::value;
        uint8_t* buf = smem + h * L::step;
        uint8_t* side = smem + L::side0;
#pragma unroll
        for (int i = 0; i < XV; i++) {
            const int p = tid + 512 * i;
            *(u32x4*)(buf + L::x + (p >> 3) * kRow + 16 * (p & 7)) = fx.x[i];
        }
        u32x2 alo, blo, ahi, bhi;
        int klo, khi;
        if (DT == kQ4_K) {
            const int j = 4 * h + 2 * (c8 >> 2);  // sub-blocks j (low nibbles) and j + 1 (high) of this thread's bytes
            const uint32_t sl = q4k_scale(f.hdr[1], f.hdr[3], j), sh = q4k_scale(f.hdr[1], f.hdr[3], j + 1);
#pragma unroll
            for (int d = 0; d < 2; d++) {
                const uint32_t w = f.q[d];
                uint32_t a0, b0, a1, b1;
                split_q4k(w & 0x0F0F0F0Fu, sl, a0, b0);
                split_q4k((w >> 4) & 0x0F0F0F0Fu, sh, a1, b1);
                alo[d] = a0, blo[d] = b0, ahi[d] = a1, bhi[d] = b1;
            }
            klo = 64 * (c8 >> 2) + 8 * (c8 & 3);
            khi = klo + 32;
            if (h == 1) {
                float* dw = (float*)(side + L::dw) + 2 * wrow_i;  // the row's eight threads store the same two values
                dw[0] = f16_bits_to_f32((uint16_t)f.hdr[0]);
                dw[1] = f16_bits_to_f32((uint16_t)(f.hdr[0] >> 16));
                // sub-block c8's min, once for each of its two groups of 16
                const _Float16 mn = (_Float16)(float)q4k_min(f.hdr[2], f.hdr[3], c8);
                const uint32_t pair = (uint32_t)__builtin_bit_cast(uint16_t, mn) * 0x00010001u;
                *(uint32_t*)(side + L::mins + wrow_i * kSumRow + 4 * c8) = pair;
            }
        } else {
            const int shl = c8 >= 4 ? 2 : 0;
            const int si = c8 >> 1;  // scale of the low nibbles' group; the high nibbles' is four further
            const int sl = (int)(int8_t)(f.hdr[0] >> (8 * si)), sh = (int)(int8_t)(f.hdr[1] >> (8 * si));
#pragma unroll
            for (int d = 0; d < 2; d++) {
                const uint32_t a = f.q[d], b = f.qh[d] >> shl;
                uint32_t a0, b0, a1, b1;
                split_q6k((a & 0x0F0F0F0Fu) | ((b & 0x03030303u) << 4), sl, a0, b0);
                split_q6k(((a >> 4) & 0x0F0F0F0Fu) | (((b >> 4) & 0x03030303u) << 4), sh, a1, b1);
                alo[d] = a0, blo[d] = b0, ahi[d] = a1, bhi[d] = b1;
            }
            klo = 8 * c8;
            khi = klo + 64;
            if (h == 1) {
                float* dw = (float*)(side + L::dw) + 2 * wrow_i;
                dw[0] = f16_bits_to_f32((uint16_t)f.hdr[2]);
            }
        }
        uint8_t* wa = buf + L::wa + wrow_i * kRow;
        uint8_t* wbp = buf + L::wb + wrow_i * kRow;
        *(u32x2*)(wa + klo) = alo;
        *(u32x2*)(wa + khi) = ahi;
        *(u32x2*)(wbp + klo) = blo;
        *(u32x2*)(wbp + khi) = bhi;
        if (h == 1) {
            if (DT == kQ4_K) {
                const s16x8 s = __builtin_bit_cast(s16x8, fx.sums);
                const f16x8 hsum = __builtin_convertvector(s, f16x8);
                *(f16x8*)(side + L::xsum + srow * kSumRow + 16 * (tid & 1)) = hsum;
            }
            ((float*)(side + L::dx))[drow] = fx.dx;
        }
    };

    i32x16 acc_a[MT], acc_b[MT];
    f32x16 acc[MT], accm[MT];
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[mt][i] = accm[mt][i] = 0.f;

    auto compute = [&](int sb, auto half) {
        constexpr int h = decltype(half)::value;
        const uint8_t* buf = smem + h * L::step;
        const uint8_t* xa = buf + L::x + (wm * 32 * MT + l32) * kRow + 16 * lh;
        const uint8_t* pa = buf + L::wa + (wn * 32 + l32) * kRow + 16 * lh;
        const uint8_t* pb = buf + L::wb + (wn * 32 + l32) * kRow + 16 * lh;
#pragma unroll
        for (int s = 0; s < 4; s++) {
            const i32x4 wa = *(const i32x4*)(pa + 32 * s), wb = *(const i32x4*)(pb + 32 * s);
#pragma unroll
            for (int mt = 0; mt < MT; mt++) {
                const i32x4 x = *(const i32x4*)(xa + mt * 32 * kRow + 32 * s);
                if (h == 0 && s == 0) {  // a super-block's first products start its sums from the constant zero
                    i32x16 zero;
#pragma unroll
                    for (int i = 0; i < 16; i++) zero[i] = 0;
                    acc_a[mt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(x, wa, zero, 0, 0, 0);
                    acc_b[mt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(x, wb, zero, 0, 0, 0);
                } else {
                    acc_a[mt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(x, wa, acc_a[mt], 0, 0, 0);
                    acc_b[mt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(x, wb, acc_b[mt], 0, 0, 0);
                }
            }
        }
    };
    // The end of a super-block: its integer sums into the float32 sums, as the CPU does it.
    auto finish = [&]() {
        {
            const uint8_t* side = smem + L::side0;
            const float* dwp = (const float*)(side + L::dw) + 2 * (wn * 32 + l32);
            const float dw = dwp[0], dmin = DT == kQ4_K ? dwp[1] : 0.f;
#pragma unroll
            for (int mt = 0; mt < MT; mt++) {
                const int r0 = wm * 32 * MT + 32 * mt;
                f32x16 summ;
                if (DT == kQ4_K) {
                    const f16x8 xs = *(const f16x8*)(side + L::xsum + (r0 + l32) * kSumRow + 16 * lh);
                    const f16x8 mn = *(const f16x8*)(side + L::mins + (wn * 32 + l32) * kSumRow + 16 * lh);
                    f32x16 zero;
#pragma unroll
                    for (int i = 0; i < 16; i++) zero[i] = 0.f;
                    summ = __builtin_amdgcn_mfma_f32_32x32x16_f16(xs, mn, zero, 0, 0, 0);
                }
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const f32x4 dx = *(const f32x4*)(side + L::dx + 4 * (r0 + 8 * j + 4 * lh));
#pragma unroll
                    for (int k = 0; k < 4; k++) {
                        const int i = 4 * j + k;
                        const int sumi = (acc_a[mt][i] << (DT == kQ4_K ? 6 : 7)) + acc_b[mt][i];
                        const float dd = dw * dx[k];
                        const float tt = dd * (float)sumi;
                        acc[mt][i] = acc[mt][i] + tt;
                        if (DT == kQ4_K) {
                            const float dm = dmin * dx[k];
                            const float u = dm * summ[i];
                            accm[mt][i] = accm[mt][i] + u;
                        }
                    }
                }
                __builtin_amdgcn_sched_barrier(0);  // one tile at a time: interleaving them costs registers the kernel lacks
            }
        }
    };

    const Half<0> h0;
    const Half<1> h1;
    // Sets of loads: with two steps of lead, the steps of a first half use fw0 / fx0 and those of a
    // second half fw1 / fx1; with one step of lead there is one set.
    FetchedW& fwb = DEPTH >= 1 ? fw1 : fw0;
    FetchedX<XV>& fxb = DEPTH >= 2 ? fx1 : fx0;
    fetch_w(fw0, 0, h0);
    fetch_x(fx0, 0, h0);
    if (DEPTH >= 1) fetch_w(fw1, 0, h1);
    if (DEPTH >= 2) fetch_x(fx1, 0, h1);
    stage(fw0, fx0, 0, h0);
    lds_barrier();
    // No branches inside: the last super-block requests and stages itself again, into buffers nobody reads.
    for (int sb = 0; sb < nsb; sb++) {
        const int nx = sb + 1 < nsb ? sb + 1 : sb;
        if (DEPTH >= 1) fetch_w(fw0, nx, h0); else fetch_w(fw0, sb, h1);
        if (DEPTH >= 2) fetch_x(fx0, nx, h0); else fetch_x(fx0, sb, h1);
        compute(sb, h0);
        stage(fwb, fxb, sb, h1);
        lds_barrier();
        if (DEPTH >= 1) fetch_w(fw1, nx, h1); else fetch_w(fw0, nx, h0);
        if (DEPTH >= 2) fetch_x(fx1, nx, h1); else fetch_x(fx0, nx, h0);
        compute(sb, h1);
        __builtin_amdgcn_sched_barrier(0);
        finish();
        stage(fw0, fx0, nx, h0);
        lds_barrier();
    }

    const int n = n0 + wn * 32 + l32;
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int m = m0 + wm * 32 * MT + 32 * mt + 8 * (i >> 2) + 4 * lh + (i & 3);
            if (m < M && n < N) {
                const float v = DT == kQ4_K ? acc[mt][i] - accm[mt][i] : acc[mt][i];
                if (OUT_BF16) ((uint16_t*)yv)[(int64_t)m * N + n] = f32_to_bf16_bits(v);
                else ((float*)yv)[(int64_t)m * N + n] = v;
            }
        }
}

template <int DT, int MT, bool OUT_BF16>
hipError_t launch(const QGemvArgs& a, int nsb, hipStream_t st) {
    // What the registers allow: 256 a lane at two wavefronts a SIMD.
    constexpr int DEPTH = MT == 1 ? 2 : 1;
    typedef Layout<128 * MT> L;
    static std::atomic<bool> raised{false};  // threads may race here: both then set the same attribute
    if (!raised) {
        hipError_t e = hipFuncSetAttribute((const void*)qgemm_kquant_kernel<DT, MT, DEPTH, OUT_BF16>, hipFuncAttributeMaxDynamicSharedMemorySize, L::total);
        if (e != hipSuccess) return e;
        raised = true;
    }
    const int tiles_m = (int)((a.M + 128 * MT - 1) / (128 * MT)), ntiles = (int)((a.N + kTN - 1) / kTN);
    const int per_xcd = (ntiles + 7) / 8;
    hipLaunchKernelGGL((qgemm_kquant_kernel<DT, MT, DEPTH, OUT_BF16>), dim3((unsigned)(8 * per_xcd * tiles_m)), dim3(512), L::total, st,
                       (const uint8_t*)a.W, (const uint8_t*)a.act, (void*)a.y, (int)a.M, (int)a.N, nsb, (int64_t)kq_act_bytes(a.K),
                       tiles_m, ntiles);
    return hipGetLastError();
}

}  // namespace

bool qgemm_kquant_ok(int dt, const QGemvArgs& a) {
    // Q4_K's blocks are read with aligned loads (144 bytes keep a 16-byte aligned W aligned); Q6_K's 2-byte aligned.
    return (dt == kQ4_K || dt == kQ6_K) && a.K % 256 == 0 && a.K > 0 && ((uintptr_t)a.W & (dt == kQ4_K ? 15 : 1)) == 0 &&
           ((uintptr_t)a.act & 15) == 0 && a.M * ((a.N + kTN - 1) / kTN) < ((int64_t)1 << 30) && a.K <= (1 << 20);
}

static bool tall_tiles(const QGemvArgs& a) {
    // 256-row tiles halve the work of splitting W; 128-row tiles where those would leave compute units idle.
    return a.M > 128 && ((a.M + 255) / 256) * ((a.N + kTN - 1) / kTN) >= 256;
}

// The row-by-row kernels read W once per row of x, at about 5.8 TB/s (Q4_K) or 5.1 TB/s (Q6_K) while it sits in
// the caches; a workgroup here spends about 2.1 us (5.5 with 256-row tiles) per super-block of K, 256 workgroups
// at a time. Measured on 4096 x 4096, 4096 x 14336 and 14336 x 4096 weights, 2 to 64 rows (at 14336 x 4096 and
// eight rows: 49 and 79 us by rows, 35 and 37 us here).
bool qgemm_kquant_pays(int dt, const QGemvArgs& a) {
    if (a.M < 4) return false;
    const double nsb = (double)(a.K / 256);
    const double rows_us = (double)a.M * (double)a.N * nsb * (dt == kQ4_K ? 144 : 210) / (dt == kQ4_K ? 5.8e6 : 5.1e6);
    const bool tall = tall_tiles(a);
    const int64_t tiles = ((a.M + (tall ? 255 : 127)) / (tall ? 256 : 128)) * ((a.N + kTN - 1) / kTN);
    return (double)((tiles + 255) / 256) * nsb * (tall ? 5.5 : 2.1) < rows_us;
}

template <bool OUT_BF16>
static hipError_t pick(int dt, const QGemvArgs& a, hipStream_t st) {
    const int nsb = (int)(a.K / 256);
    const bool tall = tall_tiles(a);
    if (dt == kQ4_K) return tall ? launch<kQ4_K, 2, OUT_BF16>(a, nsb, st) : launch<kQ4_K, 1, OUT_BF16>(a, nsb, st);
    return tall ? launch<kQ6_K, 2, OUT_BF16>(a, nsb, st) : launch<kQ6_K, 1, OUT_BF16>(a, nsb, st);
}

hipError_t qgemm_kquant(int dt, const QGemvArgs& a, hipStream_t st, bool out_bf16) {
    return out_bf16 ? pick<true>(dt, a, st) : pick<false>(dt, a, st);
}

}  // namespace mimir
