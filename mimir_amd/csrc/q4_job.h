// What the fixed-point Q4_0 kernels share: how a lane fetches its pair of blocks, the integer dot
// products of a pair against the digit planes of x, and the description of a launch (which matrices,
// which tail, where x comes from).
#pragma once

#include "device_util.h"
#include "kernels.h"
#include "q4_act.h"

namespace mimir {

// A 128-bit load that is only dword aligned (gfx950 serves it at full rate).
typedef u32x4 u32x4_a4 __attribute__((aligned(4)));

template <int RR, int PC>
struct Q4PairTile {
    u32x4 a[RR][PC], b[RR][PC];
    uint32_t c[RR][PC];
};

// Lane `lane` owns blocks 2p, 2p+1 with p = lane + 64 * pc of each row: nine
// aligned dwords. Plain (cached) loads: the three touch the same cache lines,
// which must stay cached between them.
template <int RR, int PC>
__device__ __forceinline__ void q4_load_pairs(Q4PairTile<RR, PC>& t, const uint8_t* const rowp[RR], int npairs, int pc0, int lane) {
#pragma unroll
    for (int pc = 0; pc < PC; pc++) {
        int p = lane + 64 * (pc0 + pc);
        p = p < npairs ? p : npairs - 1;
#pragma unroll
        for (int r = 0; r < RR; r++) {
            const uint32_t* src = (const uint32_t*)rowp[r] + p * 9;
            t.a[r][pc] = *(const u32x4_a4*)src;
            t.b[r][pc] = *(const u32x4_a4*)(src + 4);
            t.c[r][pc] = src[8];
        }
    }
}

// For the two blocks of a pair: sum over the block of (n - 8) * X, X the
// fixed-point activations. Digit planes run from the most significant down,
// each four v_dot8 accumulating on sixteen times the sum so far; the two
// blocks' chains are independent and interleaved so that neither waits on
// its own previous result.
__device__ __forceinline__ void q4_pair_dot(const uint32_t q0[4], const uint32_t q1[4], const u32x4 d0[kDigits],
                                            const u32x4 d1[kDigits], int& out0, int& out1) {
    int w0[4], w1[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        w0[i] = (int)(q0[i] ^ 0x88888888u);
        w1[i] = (int)(q1[i] ^ 0x88888888u);
    }
    int t0 = 0, t1 = 0;
#pragma unroll
    for (int j = kDigits - 1; j >= 0; j--) {
        t0 *= 16;
        t1 *= 16;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            t0 = __builtin_amdgcn_sdot8(w0[i], (int)d0[j][i], t0, false);
            t1 = __builtin_amdgcn_sdot8(w1[i], (int)d1[j][i], t1, false);
        }
    }
    out0 = t0;  // |t| <= 32 * 8 * 7829367 < 2^31
    out1 = t1;
}

// What one launch of the fixed-point kernel computes, for each row m of x:
//   kPlain    y[m, :] = x[m, :] . W0^T (+ resid[m, :])
//   kMulti    y[m, :] = x[m, :] . [W0; W1; W2]^T: up to three matrices that share
//             K, their rows concatenated (queries, keys and values of a block)
//   kSwiGLU   y[m, r] = SiLU(x[m, :] . W0[r]) * (x[m, :] . W1[r]): gate and up
//             of a SwiGLU feed-forward (llm/model.go:446-448), the activation
//             applied as tensor/elementwise.go:520-525,583-585 computes it
//   kRope     kMulti for the q, k, v projections of a decoding step, then what
//             rope_kv does with the result: pairs of features (2i, 2i+1) of the
//             query and key heads rotated by the angle of the position read on
//             the device (nn/transformer.go:146-257, interleaved layout), queries
//             left in y, keys and values cast into their caches at that position
//             (KVCache.Write, nn/transformer.go:464). Rows per wavefront even.
enum Q4Mode { kPlain = 0, kMulti = 1, kSwiGLU = 2, kRope = 3 };

struct Q4Job {
    const uint8_t* W[3];
    int n[3];
    int total;           // rows of y
    const float* resid;  // [M, total] or null
    Q4RopeTail rope;     // kRope only
    // kSwiGLU only: if set, the results go to act_out in the fixed-point form the next product
    // reads (row m at act_out + m * act_out_row_bytes) instead of y. A workgroup then owns exactly
    // the 32 results of one block, so rows_per_wg is 32 and total a multiple of 32.
    uint8_t* act_out;
    int64_t act_out_row_bytes;
    // HEAD 1: the product's x is RMSNorm(norm_x[m, :]) * norm_w, normalized and converted by
    // every workgroup for itself as its first phase instead of read from act. HEAD 2: x is
    // norm_x[m, :] itself (rows x_row_stride floats apart), converted likewise.
    const float* norm_x;
    const float* norm_w;
    float norm_inv_d, norm_eps;
    int64_t x_row_stride;
};

constexpr int kHeadAct = 0, kHeadNorm = 1, kHeadConvert = 2;

// ---- one pair of blocks a lane, the digits of x in registers (qgemv_q4_0_stream.hip) ----
struct PairRegs {
    u32x4 a, b;
    uint32_t c;
};

// The nine dwords of the lane's pair of blocks of one row.
__device__ __forceinline__ void load_pair(PairRegs& t, const uint8_t* rowp, int p) {
    const uint32_t* src = (const uint32_t*)rowp + p * 9;
    t.a = *(const u32x4_a4*)src;
    t.b = *(const u32x4_a4*)(src + 4);
    t.c = src[8];
}

// The lane's share of one row's sum: its pair of blocks against its digits of x.
__device__ __forceinline__ float pair_term(const PairRegs& t, const u32x4 d0[kDigits], const u32x4 d1[kDigits], float s0, float s1, bool live) {
    // block 0: scale in the low half of a[0], nibbles at bytes 2..17; block 1: scale in the high half of b[0], nibbles at bytes 20..35
    const uint32_t q0[4] = {__builtin_amdgcn_alignbyte(t.a[1], t.a[0], 2), __builtin_amdgcn_alignbyte(t.a[2], t.a[1], 2),
                            __builtin_amdgcn_alignbyte(t.a[3], t.a[2], 2), __builtin_amdgcn_alignbyte(t.b[0], t.a[3], 2)};
    const uint32_t q1[4] = {t.b[1], t.b[2], t.b[3], t.c};
    int i0, i1;
    q4_pair_dot(q0, q1, d0, d1, i0, i1);
    const float f0 = (float)i0, f1 = (float)i1;
    // a lane without a pair of its own re-reads a neighbour's: it must add exactly zero
    const float w0 = live ? f16_bits_to_f32((uint16_t)(t.a[0] & 0xffffu)) * s0 : 0.f;
    const float w1 = live ? f16_bits_to_f32((uint16_t)(t.b[0] >> 16)) * s1 : 0.f;
    float acc = 0.f;
    acc = fmaf(w0, f0, acc);
    acc = fmaf(w1, f1, acc);
    return acc;
}


}  // namespace mimir
