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
// A workgroup of four or eight wavefronts owns 32 rows of W; its wavefronts take
// the super-blocks round robin and leave their float32 terms per output (two
// for Q4_K, one for Q6_K) in LDS; when all are there the first wavefront adds
// them in the super-blocks' order, which is the CPU's. (Long rows: contiguous
// runs of super-blocks, terms in registers, the sums handed from wavefront to
// wavefront in that order; see the kernel.) x of a super-block (2.6 KB for eight
// rows) and W of it (32 rows, loaded as whole cache lines) pass through LDS that
// is the wavefront's own, so no barrier but those around the sums.
#include "device_util.h"
#include "kernels.h"
#include "rope_tail.h"

namespace mimir {

#pragma clang fp contract(off)

namespace {

typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef short s16x2 __attribute__((ext_vector_type(2)));

constexpr int kRows = 8;                        // rows of x a group holds
// A super-block of x for eight rows in LDS: quants [8][256] with rows 288 bytes apart (72 dwords: the sixteen 16-byte pieces the
// lanes of a matrix-core operand read, eight rows by two halves, fall on all 64 banks; 256 apart they would share four), sums [8][16]
// int16, scales [8].
constexpr int kXRow = 288;
constexpr int kXq = 0, kXs = 8 * kXRow, kXd = kXs + 256;
constexpr int kXBytes = kXd + 32;

// scale_min_k4 (backend/cpu/quant.go:129-134) on the twelve scale bytes held as three dwords.
__device__ __forceinline__ int q4k_sc(uint32_t s0, uint32_t s2, int j) {
    const int sh = 8 * (j & 3);
    return j < 4 ? (int)((s0 >> sh) & 63) : (int)(((s2 >> sh) & 0xf) | (((s0 >> (sh + 6)) & 3) << 4));
}
__device__ __forceinline__ int q4k_mn(uint32_t s1, uint32_t s2, int j) {
    const int sh = 8 * (j & 3);
    return j < 4 ? (int)((s1 >> sh) & 63) : (int)(((s2 >> (sh + 4)) & 0xf) | (((s1 >> (sh + 6)) & 3) << 4));
}

// W comes through LDS: a wavefront loads a super-block of its 32 rows as 16-byte pieces in row order (consecutive lanes, consecutive
// pieces of a row: whole cache lines per request, where a load of a lane's own row would touch 64 lines for 16 bytes each and wait for
// the cache's tag lookups), stores them into a slab of its own and reads its row's pieces back. WBlock<DT> says how a row's
// super-block is cut into pieces and makes the float32 terms of a lane's four rows of x from its row in the slab (wl) and the
// super-block of x in LDS (xl).
template <int DT> struct WBlock;

template <> struct WBlock<kQ4_K> {
    static constexpr int kBytes = 144, kTerms = 2;
    static constexpr int kPieces = 9, kStride = 144;  // rows 36 dwords apart: the 16 lanes of a 128-bit read's phase fall on all 64 banks
    __device__ __forceinline__ static int piece_offset(int c) { return 16 * c; }
    // t[0] = d_w d_x float(sumi), t[1] = dmin_w d_x float(summ)
    __device__ __forceinline__ static void terms(const uint8_t* wl, const uint8_t* xl, int l32, int lh, f32x4* t) {
        const u32x4 hdr = *(const u32x4*)wl;  // d, dmin, scales
        const uint8_t* xrow = xl + kXq + (l32 & 7) * kXRow + 16 * lh;  // this lane's operand row of x (rows 8.. of the operand repeat rows 0..7)
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
            const u32x4 q = *(const u32x4*)(wl + 16 + 32 * g + 16 * lh);  // the lane's 16 bytes of nibbles of group g
            i32x4 wlo, whi;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                wlo[i] = (int)(q[i] & 0x0F0F0F0Fu);
                whi[i] = (int)((q[i] >> 4) & 0x0F0F0F0Fu);
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
                // 24-bit multiplies (full rate; a 32-bit one takes four times as long): |sum| <= 32 * 15 * 127, scales below 64
                sumi[jj] += __mul24(sca, ca[jj]) + __mul24(scb, cb[jj]);
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
// 16-byte loads are unaligned ones: thirteen pieces from the block's start and a fourteenth over its last 16 bytes (194..209), which
// lands behind them in the slab (bytes 208..223 of the row there: the scale d at 222). Half h2 of a super-block (128 weights) is 64
// bytes of ql and 32 of qh: slab s = 0..3 of the half (32 weights) has its low four bits in the low (s < 2) or high nibbles of
// ql[64 h2 + 32 (s & 1) ..] and its upper two at bit 2 s of qh[32 h2 ..]; a scale per chunk of 16, a zero point of 32. The matrix-core
// product must keep the two chunks of a slab apart: the operand's row 8 c + m holds row m of x with everything but chunk c of the slab
// zeroed, so the result's rows 0..7 are chunk 0's sums and rows 8..15 chunk 1's (rows 16..31 are unused).
template <> struct WBlock<kQ6_K> {
    static constexpr int kBytes = 210, kTerms = 1;
    static constexpr int kPieces = 14, kStride = 240;  // 60 dwords: as above
    __device__ __forceinline__ static int piece_offset(int c) { return c < 13 ? 16 * c : 194; }
    // t[0] = d_w d_x float(sum over the chunks of sc (q . x - 32 sum of x))
    __device__ __forceinline__ static void terms(const uint8_t* wl, const uint8_t* xl, int l32, int lh, f32x4* t) {
        const bool keep = (l32 >> 3) == lh;  // operand rows 0..7 keep the first 16 of a slab (held by lanes of half 0), rows 8..15 the second
        const uint8_t* xrow = xl + kXq + (l32 & 7) * kXRow + 16 * lh;
        int sumi[4] = {0, 0, 0, 0}, summ[4] = {0, 0, 0, 0};
        u32x4 sv[4][2];
#pragma unroll
        for (int jj = 0; jj < 4; jj++) {
            sv[jj][0] = *(const u32x4*)(xl + kXs + (4 * lh + jj) * 32);
            sv[jj][1] = *(const u32x4*)(xl + kXs + (4 * lh + jj) * 32 + 16);
        }
        const f32x4 xd = *(const f32x4*)(xl + kXd + 16 * lh);
        const u32x4 sc = *(const u32x4*)(wl + 192);
#pragma unroll
        for (int h2 = 0; h2 < 2; h2++) {
            const u32x4 ql[2] = {*(const u32x4*)(wl + 64 * h2 + 16 * lh), *(const u32x4*)(wl + 64 * h2 + 32 + 16 * lh)};
            const u32x4 qh = *(const u32x4*)(wl + 128 + 32 * h2 + 16 * lh);
#pragma unroll
            for (int s = 0; s < 4; s++) {
                i32x4 w, xa = *(const i32x4*)(xrow + 128 * h2 + 32 * s);
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const uint32_t lo = (ql[s & 1][i] >> (s & 2 ? 4 : 0)) & 0x0F0F0F0Fu, hi = (qh[i] >> (2 * s)) & 0x03030303u;
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
                    sumi[jj] += __mul24(sca, c[jj]) + __mul24(scb, c[4 + jj]);  // |sum| <= 16 * 63 * 127, int8 scales
                    const uint32_t ps = sv[jj][h2][s];  // a copy: __builtin_bit_cast of a vector's element takes element 0 with this compiler
                    summ[jj] = __builtin_amdgcn_sdot2(__builtin_bit_cast(s16x2, ps), __builtin_bit_cast(s16x2, pair), summ[jj], false);
                }
            }
        }
        const float dw = f16_bits_to_f32(*(const uint16_t*)(wl + 222));
#pragma unroll
        for (int jj = 0; jj < 4; jj++) {
            const float dd = dw * xd[jj];
            t[0][jj] = dd * (float)(sumi[jj] - 32 * summ[jj]);
        }
    }
};

// What a lane fetches of a super-block: its pieces of W, and of x for the wavefront's LDS.
template <int LOADS> struct Stage {
    u32x4 w[LOADS];
    u32x4 xq[2];  // two 16-byte pieces of the eight rows' quants
    u32x4 xs;     // a piece of their sums (lanes 0..15 store theirs)
    float xd;     // a row's scale (lanes 0..7 store theirs)
};

// CHAIN > 0: a wavefront takes a contiguous run of at most CHAIN super-blocks and keeps its terms in registers; the sums then pass
// from wavefront to wavefront through LDS in the super-blocks' order (a barrier a wavefront). LDS holds no terms then, so more
// workgroups share a compute unit and long rows leave room for eight wavefronts. CHAIN = 0: super-blocks round robin, terms
// [nsb][kT][64] in LDS, summed by the first wavefront (any K that fits).
// ROPE: W is q | k | v of a decoding step; the rotation and the cache writes ride on the results (rope_kv's arithmetic, interleaved
// pairs), y gets the rotated queries only.
template <int DT, int kWaves, int CHAIN, bool ROPE = false>
__global__ __launch_bounds__(64 * kWaves) void qgemv_kq_rows_kernel(const uint8_t* __restrict__ W, const uint8_t* act, float* y, const float* resid,
                                                                     int M_all, int N, int nsb, int64_t act_row_bytes, const Q4RopeTail rope) {
    typedef WBlock<DT> WB;
    constexpr int kT = WB::kTerms, kAll = 32 * WB::kPieces, kLoads = (kAll + 63) / 64, kSlab = 32 * WB::kStride;
    typedef Stage<kLoads> St;
    extern __shared__ __align__(16) uint8_t smem[];  // terms (or the sums handed on), then per wavefront a super-block of x and the slab of W
    const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, lh = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // blockIdx.z: the group of eight rows of x
    const int64_t row0 = (int64_t)kRows * blockIdx.z;
    act += row0 * act_row_bytes;
    const int M = M_all - (int)row0 < kRows ? M_all - (int)row0 : kRows;
    const int n0 = blockIdx.x * 32, n = n0 + l32;
    f32x4* terms = (f32x4*)smem;
    uint8_t* xl = smem + (size_t)(CHAIN ? 1 : nsb) * kT * 1024 + wave * (kXBytes + kSlab);
    uint8_t* slab = xl + kXBytes;

    // piece p = 64 i + lane of a super-block of the 32 rows: row p / kPieces, piece p % kPieces of it
    const uint8_t* wbase = W + (int64_t)n0 * nsb * WB::kBytes;
    uint32_t goff[kLoads], loff[kLoads];
#pragma unroll
    for (int i = 0; i < kLoads; i++) {
        int p = 64 * i + lane;
        p = p < kAll ? p : kAll - 1;  // a last load that is not full repeats the last piece in its upper lanes
        const int r = p / WB::kPieces, c = p - WB::kPieces * r;
        const int row = n0 + r < N ? n0 + r : N - 1;
        goff[i] = (uint32_t)(row - n0) * (uint32_t)(nsb * WB::kBytes) + WB::piece_offset(c);  // 32 rows of W within 4 GB (checked by the host)
        loff[i] = r * WB::kStride + 16 * c;
    }
    // pieces of x a lane fetches: quants p = lane, 64 + lane (row p / 16, bytes 16 (p % 16)..); sums (lanes below 16:
    // row lane / 2, half lane % 2); scale (lanes below 8: row lane). Rows from M on repeat the last one.
    const uint8_t* xsrc[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int p = 64 * i + lane, r = p >> 4;
        xsrc[i] = act + (int64_t)(r < M ? r : M - 1) * act_row_bytes + 16 * (p & 15);
    }
    // (every lane loads, the upper ones what lower ones load too: with a load under a branch the compiler waits for all loads under
    // way, the next super-block's with them, before it touches this one's)
    const int rs = ((lane >> 1) & 7) < M ? ((lane >> 1) & 7) : M - 1, rd = (lane & 7) < M ? (lane & 7) : M - 1;
    const uint8_t* ssrc = act + (int64_t)rs * act_row_bytes + (int64_t)nsb * 256 + 16 * (lane & 1);
    const uint8_t* dsrc = act + (int64_t)rd * act_row_bytes + (int64_t)nsb * 288;

    auto fetch = [&](St& f, int sb) {
        const uint8_t* wb = wbase + (int64_t)sb * WB::kBytes;
#pragma unroll
        for (int i = 0; i < kLoads; i++) {
            if (DT == kQ4_K) f.w[i] = *(const u32x4*)(wb + goff[i]);
            else __builtin_memcpy(&f.w[i], __builtin_assume_aligned(wb + goff[i], 2), 16);
        }
#pragma unroll
        for (int i = 0; i < 2; i++) f.xq[i] = *(const u32x4*)(xsrc[i] + (int64_t)sb * 256);
        f.xs = *(const u32x4*)(ssrc + (int64_t)sb * 32);
        f.xd = ((const float*)dsrc)[sb];
    };
    auto work = [&](const St& f, f32x4* t) {
        // W and x of the super-block into this wavefront's LDS (its own: a wavefront's LDS operations complete in order)
#pragma unroll
        for (int i = 0; i < kLoads; i++)
            if (64 * (i + 1) <= kAll || lane < kAll - 64 * i) *(u32x4*)(slab + loff[i]) = f.w[i];
#pragma unroll
        for (int i = 0; i < 2; i++) *(u32x4*)(xl + kXq + ((64 * i + lane) >> 4) * kXRow + 16 * (lane & 15)) = f.xq[i];
        if (lane < 16) *(u32x4*)(xl + kXs + 16 * lane) = f.xs;
        if (lane < 8) *(float*)(xl + kXd + 4 * lane) = f.xd;
        WB::terms(slab + l32 * WB::kStride, xl, l32, lh, t);
    };
    f32x4 acc[kT];
#pragma unroll
    for (int i = 0; i < kT; i++) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    if constexpr (CHAIN > 0) {
        const int sb_lo = wave * nsb / kWaves, count = (wave + 1) * nsb / kWaves - sb_lo;  // at most CHAIN (the host's choice of CHAIN)
        St f[2];
        f32x4 tt[CHAIN][kT];
        if (count > 0) fetch(f[0], sb_lo);
#pragma unroll
        for (int j = 0; j < CHAIN; j++) {
            if (j < count) {  // the same for the whole wavefront
                if (j + 1 < count) fetch(f[(j + 1) & 1], sb_lo + j + 1);
                work(f[j & 1], tt[j]);
            }
            __builtin_amdgcn_sched_barrier(0);  // one super-block's work at a time: interleaved they would not fit the registers
        }
        // wavefront w adds its terms, the CPU's next ones, to the sums of those before it and hands them on
        for (int w = 0; w < kWaves; w++) {
            if (w == wave) {
                if (w > 0) {
#pragma unroll
                    for (int i = 0; i < kT; i++) acc[i] = terms[i * 64 + lane];
                }
#pragma unroll
                for (int j = 0; j < CHAIN; j++) {
                    if (j < count) {
#pragma unroll
                        for (int i = 0; i < kT; i++)
#pragma unroll
                            for (int jj = 0; jj < 4; jj++) acc[i][jj] = acc[i][jj] + tt[j][i][jj];
                    }
                }
                if (w + 1 < kWaves) {
#pragma unroll
                    for (int i = 0; i < kT; i++) terms[i * 64 + lane] = acc[i];
                }
            }
            if (w + 1 < kWaves) __syncthreads();
        }
        if (wave != kWaves - 1) return;
    } else {
        St cur, nxt;  // one in work, the next requested
        if (wave < nsb) fetch(cur, wave);
        for (int sb = wave; sb < nsb; sb += kWaves) {
            fetch(nxt, sb + kWaves < nsb ? sb + kWaves : sb);
            f32x4 t[kT];
            work(cur, t);
#pragma unroll
            for (int i = 0; i < kT; i++) terms[(sb * kT + i) * 64 + lane] = t[i];
            cur = nxt;
        }
        __syncthreads();
        if (wave != 0) return;
        // the CPU's order; eight super-blocks' terms are requested together so that the chain of additions does not wait for LDS each time
        for (int sb0 = 0; sb0 < nsb; sb0 += 8) {
            f32x4 t[8][kT];
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const int sb = sb0 + j < nsb ? sb0 + j : nsb - 1;
#pragma unroll
                for (int i = 0; i < kT; i++) t[j][i] = terms[(sb * kT + i) * 64 + lane];
            }
#pragma unroll
            for (int j = 0; j < 8; j++) {
                if (sb0 + j >= nsb) break;
#pragma unroll
                for (int i = 0; i < kT; i++)
#pragma unroll
                    for (int jj = 0; jj < 4; jj++) acc[i][jj] = acc[i][jj] + t[j][i][jj];
            }
        }
    }
    if constexpr (ROPE) {
        // rows (n, n + 1), n even, are a pair of features: the even lane takes its neighbour's result and stores both
        const int pos = *rope.pos;
#pragma unroll
        for (int jj = 0; jj < 4; jj++) {
            const float v = kT == 2 ? acc[0][jj] - acc[kT - 1][jj] : acc[0][jj];
            const float other = dpp_f32<0xb1>(v);  // quad_perm [1,0,3,2]
            const int m = 4 * lh + jj, seq = (int)row0 + m;
            if ((lane & 1) == 0 && n < N && m < M) q4_rope_store(rope, pos, seq, n, v, other, y + (int64_t)seq * N);
        }
        return;
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

static std::atomic<int> g_kq_rows{0};  // measurement aid: 1 = never, 2 = for any number of rows the kernel takes
void set_kquant_rows(int v) { g_kq_rows = v; }

static std::atomic<int> g_kq_rows_waves{0};  // measurement aid: 4 or 8 wavefronts to a workgroup whatever the shape
static std::atomic<int> g_kq_rows_chain{0};  // measurement aid: 1 = terms in LDS whatever the shape
void set_kquant_rows_waves(int v) {
    if (v == 0) g_kq_rows_chain = g_kq_rows_waves = 0;
    else if (v == 1) g_kq_rows_chain = 1;
    else g_kq_rows_waves = v;
}

// LDS of a workgroup: the terms (or the sums handed on), and per wavefront a super-block of x and the slab of W.
static size_t rows_lds(int dt, int64_t nsb, int waves, bool chain) {
    return (size_t)(chain ? 1 : nsb) * (dt == kQ4_K ? 2 : 1) * 1024 +
           (size_t)waves * (kXBytes + 32 * (dt == kQ4_K ? WBlock<kQ4_K>::kStride : WBlock<kQ6_K>::kStride));
}

// Two rows of x or more, converted (kq_convert_act); the terms of 32 rows of W in LDS; Q4_K's W 16-byte aligned, Q6_K's on an even address.
bool qgemv_kquant_rows_ok(int dt, const QGemvArgs& a) {
    const int64_t nsb = a.K / 256;
    return (dt == kQ4_K || dt == kQ6_K) && g_kq_rows != 1 && a.M >= 2 && a.M <= 8 * 65535 && a.act && a.K % 256 == 0 && nsb > 0 &&
           ((uintptr_t)a.W & (dt == kQ4_K ? 15 : 1)) == 0 && ((uintptr_t)a.act & 15) == 0 && a.N > 0 && a.N <= (1ll << 30) &&
           (nsb <= 64 || rows_lds(dt, nsb, 4, false) <= 160 * 1024) && 32 * nsb * 210 < ((int64_t)1 << 32);
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
    // (its 2.1 us hold up to some 128 tiles at a time: 112 tiles take 35 us at K = 4096, 224 take 63)
    const double tiles = (double)(((a.M + 127) / 128) * ((a.N + 127) / 128));
    return rows_us < (tiles > 128 ? tiles / 128 : 1.0) * nsb * 2.1;
}

template <int DT, int WAVES, int CHAIN, bool ROPE = false>
static hipError_t launch_kq_rows(const QGemvArgs& a, hipStream_t st, const Q4RopeTail* rope = nullptr) {
    const int nsb = (int)(a.K / 256);
    static std::atomic<bool> raised{false};  // threads may race here: both then set the same attribute
    if (!raised) {
        hipError_t e = hipFuncSetAttribute((const void*)qgemv_kq_rows_kernel<DT, WAVES, CHAIN, ROPE>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return e;
        raised = true;
    }
    hipLaunchKernelGGL((qgemv_kq_rows_kernel<DT, WAVES, CHAIN, ROPE>), dim3((unsigned)((a.N + 31) / 32), 1, (unsigned)((a.M + kRows - 1) / kRows)),
                       dim3(64 * WAVES), rows_lds(DT, nsb, WAVES, CHAIN > 0), st, (const uint8_t*)a.W, (const uint8_t*)a.act, a.y, a.resid, (int)a.M,
                       (int)a.N, nsb, (int64_t)kq_act_bytes(a.K), rope ? *rope : Q4RopeTail{});
    return hipGetLastError();
}

// Eight wavefronts where the workgroups are at most one to a compute unit or the rows are long, four where they are many (measured at
// eight rows of x already converted, us a call, Q4_K | Q6_K, four and eight wavefronts: 14336 x 4096 11.1 14.2 | 16.0 19.2; 4096 x 4096
// 7.6 7.1 | 10.1 9.3; 28672 x 4096 20.5 27.3 | 33.5 41.8). Rows of more than four super-blocks a wavefront (K above 8192 with eight) keep
// the terms in registers, in runs of up to eight super-blocks (4096 x 14336: 16.3 | 21.3 us, 19.9 | 21.9 with the terms in LDS, which leave
// room for four wavefronts only); shorter ones gain nothing from it (the registers cost what the LDS gives), longer ones have no choice.
static void rows_shape(int dt, const QGemvArgs& a, int* waves_out, bool* chain_out) {
    const int64_t nsb = a.K / 256, wgs = (a.N + 31) / 32 * ((a.M + kRows - 1) / kRows);
    int waves = wgs <= 256 || nsb > 32 ? 8 : 4;
    if (g_kq_rows_waves == 4 || g_kq_rows_waves == 8) waves = g_kq_rows_waves;
    bool chain = g_kq_rows_chain != 1 && nsb > 4 * waves && nsb <= 64;
    if (chain) waves = 8;
    else if (rows_lds(dt, nsb, waves, false) > 160 * 1024) waves = 4;
    *waves_out = waves;
    *chain_out = chain;
}

// The q | k | v product of a decoding step with the rotation and the cache writes as its tail (see Q4RopeTail; interleaved pairs,
// even widths): where the rows kernel takes the shape with its terms in LDS (K up to 8192).
bool qgemv_kquant_rows_rope_ok(int dt, const QGemvArgs& a) {
    if (!qgemv_kquant_rows_ok(dt, a) || a.resid || a.N % 2) return false;
    int waves;
    bool chain;
    rows_shape(dt, a, &waves, &chain);
    return !chain;
}

hipError_t qgemv_kquant_rows_rope(int dt, const QGemvArgs& a, const Q4RopeTail& rope, hipStream_t st) {
    int waves;
    bool chain;
    rows_shape(dt, a, &waves, &chain);
    if (chain) return hipErrorInvalidValue;
    if (dt == kQ4_K) return waves == 8 ? launch_kq_rows<kQ4_K, 8, 0, true>(a, st, &rope) : launch_kq_rows<kQ4_K, 4, 0, true>(a, st, &rope);
    return waves == 8 ? launch_kq_rows<kQ6_K, 8, 0, true>(a, st, &rope) : launch_kq_rows<kQ6_K, 4, 0, true>(a, st, &rope);
}

hipError_t qgemv_kquant_rows(int dt, const QGemvArgs& a, hipStream_t st) {
    int waves;
    bool chain;
    rows_shape(dt, a, &waves, &chain);
    if (dt == kQ4_K) return chain ? launch_kq_rows<kQ4_K, 8, 8>(a, st) : waves == 8 ? launch_kq_rows<kQ4_K, 8, 0>(a, st) : launch_kq_rows<kQ4_K, 4, 0>(a, st);
    return chain ? launch_kq_rows<kQ6_K, 8, 8>(a, st) : waves == 8 ? launch_kq_rows<kQ6_K, 8, 0>(a, st) : launch_kq_rows<kQ6_K, 4, 0>(a, st);
}

}  // namespace mimir
