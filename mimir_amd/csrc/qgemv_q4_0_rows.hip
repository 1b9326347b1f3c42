// Products of two to eight rows of float32 x with Q4_0 weights on the int8
// matrix cores of gfx950: y[M, N] = x[M, K] . W[N, K]^T (+ a residual), the
// decoding step of a batch of sequences. W is read once for all the rows, and
// the arithmetic is that of the other two fixed-point kernels (qgemv_q4_0.hip
// for one row, qgemm_q4_0_fx.hip for many): x as a 24-bit fixed-point number
// per element and a float32 scale per block of 32, the exact integer sum per
// block, one FMA per block with the product of the two scales. What the
// reference's CPU computes here is the float32 product with the dequantized
// weights (io/mim/dtype.go:118-123, backend/cpu/gemv.go:73-104), to which a
// product has to agree within 1e-3.
//
// One v_mfma_i32_32x32x32_i8 per block of 32 weights and 32 rows of W: its
// other operand holds the three base-256 digits of the eight rows of x as 24
// of its 32 rows (row 8 d + m: digit d of row m of x), so digit sums of all
// eight rows come out of one instruction, each lane holding those of its row of
// W for four rows of x. The weights enter as their nibbles n (0..15); the
// offset of -8 is taken out per block as 8 times the sum of the block's x,
// which the conversion of x leaves beside the scales.
//
// A lane takes one block of 18 bytes per step, the lower half of the wavefront
// an even block and the upper half the odd one after it; v_permlane32_swap
// trades the halves' high and low nibbles so that each of the two blocks gets a
// whole operand. A workgroup of eight wavefronts owns 32 rows of W, a wavefront
// every eighth run of eight blocks; their sums meet in LDS in a fixed order.
// The operand wants a lane per row of W, memory wants neighbouring lanes on
// neighbouring bytes (a load of 64 different rows costs the L1 cache 64 lookups,
// and that bounded the first version): so a wavefront loads a run of eight
// blocks of its 32 rows as 288 aligned 16-byte pieces in row order, passes them
// through LDS, and each lane reads its block back as dwords. Shapes that do not
// allow this (K not a multiple of 256, W not 16-byte aligned) take a kernel that
// loads each lane's block where it lies.
#include <type_traits>

#include "device_util.h"
#include "kernels.h"
#include "q4_rows_act.h"
#include "rope_tail.h"

namespace mimir {

namespace {

typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));

constexpr int kRows = 8;     // rows of x a launch takes
constexpr int kWaves = 8;    // wavefronts of a workgroup: shares of K
constexpr int kDepth = 4;    // steps (pairs of blocks) requested ahead
constexpr int kFragBytes = kRowsFragBytes;  // one block of the eight rows as an MFMA operand: 64 lanes x 16 bytes
constexpr int kTailBytes = kRowsTailBytes;  // per block: float scale[8], int32 eight_sums[8]

__device__ __forceinline__ int group8_sum_i32(int v) {
    v += __builtin_amdgcn_update_dpp(0, v, 0xb1, 0xf, 0xf, true);   // quad_perm [1,0,3,2]
    v += __builtin_amdgcn_update_dpp(0, v, 0x4e, 0xf, 0xf, true);   // quad_perm [2,3,0,1]
    v += __builtin_amdgcn_update_dpp(0, v, 0x141, 0xf, 0xf, true);  // row_half_mirror
    return v;
}

}  // namespace

// The converted form of up to eight rows of x: see q4_rows_act.h.
size_t q4_0_rows_act_bytes(int64_t K) { return q4_0_rows_act_size(K); }

// Thread t of row blockIdx.y takes elements 4t..4t+3; a block's eight threads are consecutive lanes.
// The integers and scales are those of q4_convert_item and of fx_convert_kernel. Rows from M on are
// written as zeros, so that a launch always defines the whole buffer.
__global__ __launch_bounds__(256) void q4_0_rows_convert_kernel(const float* __restrict__ x, int64_t x_row_stride, int M, int K,
                                                                uint8_t* act) {
    const int nb = K >> 5;
    const int m = blockIdx.y + kRows * blockIdx.z;  // row of x; blockIdx.z: its group of eight, converted into a buffer of its own
    act += (int64_t)blockIdx.z * nb * (kFragBytes + kTailBytes);
    const float* xr = x + (int64_t)(m < M ? m : 0) * x_row_stride;
    uint8_t* tail = act + (int64_t)nb * kFragBytes;
    const int nq = K >> 2;
    for (int t = blockIdx.x * blockDim.x + threadIdx.x; t < nq; t += gridDim.x * blockDim.x) {
        f32x4 v;
        __builtin_memcpy(&v, xr + 4 * (int64_t)t, 16);
        if (m >= M) v = f32x4{0.f, 0.f, 0.f, 0.f};
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
        int sum = 0;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            int a = (int)__builtin_rintf(v[k] * inv);
            a = a > kFixMax ? kFixMax : a < -kFixMax ? -kFixMax : a;
            sum += a;
            const int d0 = (int)(int8_t)a;  // balanced digits: each in -128..127
            const int a1 = (a - d0) >> 8;
            const int d1 = (int)(int8_t)a1;
            const int d2 = (a1 - d1) >> 8;
            d[0] |= (uint32_t)(d0 & 0xff) << (8 * k);
            d[1] |= (uint32_t)(d1 & 0xff) << (8 * k);
            d[2] |= (uint32_t)(d2 & 0xff) << (8 * k);
        }
        sum = group8_sum_i32(sum);  // below 2^28
        const int b = t >> 3, q = t & 7;
        uint32_t* frag = (uint32_t*)(act + (int64_t)b * kFragBytes) + (q & 3);
        const int lane0 = 32 * (q >> 2) + (int)blockIdx.y;
#pragma unroll
        for (int j = 0; j < 3; j++) frag[4 * (lane0 + 8 * j)] = d[j];
        frag[4 * (lane0 + 24)] = 0;
        if (q == 0) {
            ((float*)(tail + (int64_t)b * kTailBytes))[blockIdx.y] = scale;
            ((int32_t*)(tail + (int64_t)b * kTailBytes))[8 + blockIdx.y] = 8 * sum;
        }
    }
}

hipError_t q4_0_rows_convert_act(const float* x, int64_t M, int64_t K, int64_t x_row_stride, void* act, hipStream_t st) {
    int gx = (int)((K / 4 + 255) / 256);
    // more than eight rows: a buffer of q4_0_rows_act_bytes(K) per group of eight, one after the other
    hipLaunchKernelGGL(q4_0_rows_convert_kernel, dim3((unsigned)gx, kRows, (unsigned)((M + kRows - 1) / kRows)), dim3(256), 0, st, x, x_row_stride,
                       (int)M, (int)K, (uint8_t*)act);
    return hipGetLastError();
}

namespace {

// What a lane holds of a step between its loads and its arithmetic.
struct Step {
    u32x4 q;       // the 16 bytes of nibbles of the lane's block
    uint32_t d;    // its scale (binary16 bits)
    i32x4 xa, xb;  // the operands of x for the step's two blocks
};

__global__ __launch_bounds__(64 * kWaves) void qgemv_q4_0_rows_direct_kernel(const uint8_t* __restrict__ W, const uint8_t* __restrict__ act,
                                                                       float* y, const float* resid,  // resid may be y
                                                                       int M, int N, int nb) {
    extern __shared__ __align__(16) uint8_t smem[];  // the tail of act, then the wavefronts' sums
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, lh = lane >> 5;
    const int n = blockIdx.x * 32 + l32;
    const uint8_t* wrow = W + (int64_t)(n < N ? n : N - 1) * nb * 18 + 18 * lh;
    const uint8_t* xfrag = act + 16 * lane;
    const int nsteps = nb >> 1;
    const int per = (nsteps + kWaves - 1) / kWaves;
    const int s_begin = wave * per, s_end = s_begin + per < nsteps ? s_begin + per : nsteps;

    // the scales and sums of x: every wavefront reads its blocks' from LDS
    {
        const u32x4* tail = (const u32x4*)(act + (int64_t)nb * kFragBytes);
        for (int i = tid; i < nb * (kTailBytes / 16); i += 64 * kWaves) ((u32x4*)smem)[i] = tail[i];
    }
    auto fetch = [&](Step& f, int s) {
        s = s < nsteps - 1 ? s : nsteps - 1;
        const uint8_t* p = wrow + 36 * (int64_t)s;
        f.q = load_u32x4_unaligned(p + 2);
        f.d = load_u16(p);
        f.xa = *(const i32x4*)(xfrag + (int64_t)(2 * s) * kFragBytes);
        f.xb = *(const i32x4*)(xfrag + (int64_t)(2 * s + 1) * kFragBytes);
    };
    Step st[kDepth];
#pragma unroll
    for (int u = 0; u < kDepth; u++) fetch(st[u], s_begin + u);
    __syncthreads();

    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    // one block: c = digit sums against the nibbles; lane: row l32 of W, rows 4 lh + j of x
    auto block = [&](const i32x4 xop, const i32x4 wop, float dw, int b) {
        i32x16 zero;
#pragma unroll
        for (int i = 0; i < 16; i++) zero[i] = 0;
        const i32x16 c = __builtin_amdgcn_mfma_i32_32x32x32_i8(xop, wop, zero, 0, 0, 0);
        const f32x4 dx = *(const f32x4*)(smem + b * kTailBytes + 16 * lh);
        const i32x4 off = *(const i32x4*)(smem + b * kTailBytes + 32 + 16 * lh);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            // sum of x (n - 8), below 2^31 in magnitude (32 * 8 * kFixMax); the partial terms may wrap
            const int isum = (int)((uint32_t)c[j] + ((uint32_t)c[4 + j] << 8) + ((uint32_t)c[8 + j] << 16) - (uint32_t)off[j]);
            const float wsc = dw * dx[j];
            acc[j] = fmaf(wsc, (float)isum, acc[j]);
        }
    };
    for (int s0 = s_begin; s0 < s_end; s0 += kDepth) {
#pragma unroll
        for (int u = 0; u < kDepth; u++) {
            const int s = s0 + u;
            const Step cur = st[u];
            fetch(st[u], s + kDepth);
            if (s < s_end) {
                i32x4 wa, wb;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const uint32_t lo = cur.q[i] & 0x0F0F0F0Fu, hi = (cur.q[i] >> 4) & 0x0F0F0F0Fu;
                    // lower lanes keep their low nibbles and take the upper lanes' in exchange for their high ones
                    const auto r = __builtin_amdgcn_permlane32_swap(lo, hi, false, false);
                    wa[i] = (int)r[0];
                    wb[i] = (int)r[1];
                }
                const auto dd = __builtin_amdgcn_permlane32_swap(cur.d, cur.d, false, false);
                block(cur.xa, wa, f16_bits_to_f32((uint16_t)dd[0]), 2 * s);
                block(cur.xb, wb, f16_bits_to_f32((uint16_t)dd[1]), 2 * s + 1);
            }
        }
    }

    // the eight shares of K, added in their order
    f32x4* red = (f32x4*)(smem + (size_t)nb * kTailBytes);
    red[wave * 64 + lane] = f32x4{acc[0], acc[1], acc[2], acc[3]};
    __syncthreads();
    if (wave != 0) return;
    f32x4 sum = red[lane];
#pragma unroll
    for (int w = 1; w < kWaves; w++) {
        const f32x4 t = red[w * 64 + lane];
#pragma unroll
        for (int j = 0; j < 4; j++) sum[j] = sum[j] + t[j];
    }
    if (n < N) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int m = 4 * lh + j;
            if (m < M) {
                float v = sum[j];
                if (resid) v = v + resid[(int64_t)m * N + n];
                y[(int64_t)m * N + n] = v;
            }
        }
    }
}

// Up to three matrices with the same K, multiplied in one launch (q, k and v; gate and up): n[i] rows
// each (all but the last a multiple of 32), groups[i] workgroups.
struct RowsJob {
    const uint8_t* W[3];
    int n[3], groups[3];
};

constexpr int kRunBlocks = 8;                   // blocks a wavefront takes at a time: 144 bytes a row, nine pieces
constexpr int kRunBytes = 18 * kRunBlocks;
constexpr int kSlabStride = kRunBytes + 32;     // bytes between rows of a wavefront's slab in LDS
constexpr int kSlabBytes = 32 * kSlabStride;
constexpr int kWaveLds = kSlabBytes + kRunBlocks * kTailBytes;  // the slab, then the run's scales and sums of x

enum RowsTail { kRowsPlain = 0, kRowsRope = 1, kRowsSwiGLU = 2 };

// What the tails need beside the job.
struct RowsTailArgs {
    Q4RopeTail rope;              // kRowsRope: the three matrices are q, k, v; y gets the rotated queries, the caches k and v
    uint8_t* act_out = nullptr;   // kRowsSwiGLU: the two matrices are gate and up; SiLU(gate) * up converted for the next product
    int nb_out = 0;               //   whose rows have nb_out blocks
};

// gridDim.y shares of K: with more than one, share s writes its sums to y + s * M * N and nothing is added
// (a later kernel adds the shares in their order); resid only with one share.
// TAIL: kRowsRope, the rotation of a decoding step and its cache writes on the results (rope_kv's arithmetic,
// interleaved pairs); kRowsSwiGLU, a workgroup multiplies its 32 rows of gate and of up and leaves SiLU(gate) * up
// (swiglu_kernel's arithmetic) converted as block blockIdx.x of the next product's x. One share for both.
template <int WAVES, int TAIL>  // WAVES: wavefronts of a workgroup, among which the runs of its share of K go round
__global__ __launch_bounds__(64 * WAVES) __attribute__((amdgpu_waves_per_eu(3))) void qgemv_q4_0_rows_kernel(const RowsJob job, const uint8_t* __restrict__ act_all,
                                                                       float* y, const float* resid,  // resid may be y
                                                                       int M_all, int nb, const RowsTailArgs tail_args) {
    extern __shared__ __align__(16) uint8_t smem[];  // per wavefront: slab and tail of its run; later the wavefronts' sums
    // blockIdx.z: the group of eight rows of x, each converted into a buffer of its own
    const uint8_t* __restrict__ act = act_all + (int64_t)blockIdx.z * nb * (kFragBytes + kTailBytes);
    const int M = M_all - kRows * (int)blockIdx.z < kRows ? M_all - kRows * (int)blockIdx.z : kRows;
    const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, lh = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // in a scalar register: what depends on it alone is scalar arithmetic
    // up to three matrices, their rows one after the other in y: this workgroup's, and its first row there
    int g = blockIdx.x, which = 0;
    if (TAIL != kRowsSwiGLU) {
        if (g >= job.groups[0]) { g -= job.groups[0]; which = 1; }
        if (which == 1 && g >= job.groups[1]) { g -= job.groups[1]; which = 2; }
    }
    const uint8_t* __restrict__ W = which == 0 ? job.W[0] : which == 1 ? job.W[1] : job.W[2];
    const int N = which == 0 ? job.n[0] : which == 1 ? job.n[1] : job.n[2];
    const int ybase = which == 0 ? 0 : which == 1 ? job.n[0] : job.n[0] + job.n[1];
    const int ny = job.n[0] + job.n[1] + job.n[2];
    const int n0 = g * 32, n = n0 + l32;
    const int nruns = nb / kRunBlocks;
    const int per_share = (nruns + (int)gridDim.y - 1) / (int)gridDim.y;
    const int run0 = (int)blockIdx.y * per_share + wave;
    const int run_end = ((int)blockIdx.y + 1) * per_share < nruns ? ((int)blockIdx.y + 1) * per_share : nruns;
    uint8_t* slab = smem + wave * kWaveLds;
    const uint32_t xlane = 16 * lane;

    // piece p = 64 i + lane of a run: row p / 9 of the 32, bytes 16 (p % 9).. of its 144. The fifth load's
    // upper lanes fetch the run's 32 pieces of scales and sums of x instead (512 bytes after the operands).
    uint32_t goff[4], loff[5];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int p = 64 * i + lane, r = p / 9, c = p - 9 * r;
        const int row = n0 + r < N ? n0 + r : N - 1;
        goff[i] = (uint32_t)(row - n0) * (uint32_t)(nb * 18) + 16 * c;  // rows of W below 2^32 bytes apart from the first (checked by the host)
        loff[i] = r * kSlabStride + 16 * c;
    }
    const int64_t group_bytes = (int64_t)n0 * nb * 18;
    int64_t off4, stride4;  // the fifth load: relative to the matrix for the lower lanes, to act for the upper
    if (lane < 32) {
        const int p = 256 + lane, r = p / 9, c = p - 9 * r;
        const int row = n0 + r < N ? n0 + r : N - 1;
        off4 = group_bytes + (int64_t)(row - n0) * nb * 18 + 16 * c;
        stride4 = kRunBytes;
        loff[4] = r * kSlabStride + 16 * c;
    } else {
        off4 = (int64_t)nb * kFragBytes + 16 * (lane - 32);
        stride4 = kRunBlocks * kTailBytes;
        loff[4] = kSlabBytes + 16 * (lane - 32);
    }

    struct Run { u32x4 w[5]; };
    auto fetch_w = [&](Run& f, const uint8_t* wm, int run) {
        const uint8_t* p = wm + group_bytes + (int64_t)run * kRunBytes;
#pragma unroll
        for (int i = 0; i < 4; i++) f.w[i] = *(const u32x4*)(p + goff[i]);
        f.w[4] = *(const u32x4*)((lane < 32 ? wm : act) + off4 + run * stride4);
    };
    struct XPair { i32x4 a, b; };
    auto fetch_x = [&](XPair& f, int step) {  // blocks 2 step and 2 step + 1
        const uint8_t* p = act + (int64_t)step * (2 * kFragBytes);
        f.a = *(const i32x4*)(p + xlane);
        f.b = *(const i32x4*)(p + kFragBytes + xlane);
    };

    const uint8_t* tail = slab + kSlabBytes + 16 * lh;
    // c: a block's digit sums against the nibbles; lane: row l32 of W, rows 4 lh + j of x. dx, off: the block's scales and 8 * sums of x.
    auto finish = [&](float (&acc)[4], const i32x16& c, float dw, const f32x4 dx, const i32x4 off) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            // sum of x (n - 8), below 2^31 in magnitude (32 * 8 * kFixMax); the partial terms may wrap
            uint32_t t = ((uint32_t)c[8 + j] << 8) + (uint32_t)c[4 + j];
            asm volatile("" : "+v"(t));  // keeps the two shift-and-add steps (otherwise: two shifts and a three-way add)
            const int isum = (int)((t << 8) + ((uint32_t)c[j] - (uint32_t)off[j]));
            const float wsc = dw * dx[j];
            acc[j] = fmaf(wsc, (float)isum, acc[j]);
        }
    };

    Run cur, nxt;
    XPair xs[4];
    if (run0 < run_end) {
        fetch_w(cur, W, run0);
#pragma unroll
        for (int u = 0; u < 4; u++) fetch_x(xs[u], 4 * run0 + u);
    }
    // this lane's block of step j of a run: bytes 36 j + 18 lh.. of row l32; read as dwords from 36 j + 20 lh (the
    // upper half's nibbles start on a dword, the lower half's two bytes into one), the scale from 36 j + 16 lh
    const uint8_t* mine = slab + l32 * kSlabStride + 20 * lh;
    const uint8_t* mine_d = slab + l32 * kSlabStride + 16 * lh;
    const uint32_t shift = lh ? 0u : 16u;
    // One run of `cur` into acc, with the run (wn, nrun) requested for afterwards; x_too: also the operands of x
    // for run nrun (not when the run after has the same, as up's after gate's).
    auto one_run = [&](auto x_too, float (&acc)[4], const uint8_t* wn, int nrun) {
        fetch_w(nxt, wn, nrun);
        // slab and tail are this wavefront's alone: every lane's reads of the last run were waited for before
        // its last MFMAs and FMAs, and a wavefront's LDS operations complete in order
#pragma unroll
        for (int i = 0; i < 5; i++) *(u32x4*)(slab + loff[i]) = cur.w[i];
        // The LDS reads of a step are issued a step ahead of their use, the scales and sums of x before the
        // MFMAs whose results they meet: a wavefront has few neighbours on its SIMD to fill its waits with.
        uint32_t r[5], dword;
        auto read_block = [&](int j) {
#pragma unroll
            for (int i = 0; i < 5; i++) r[i] = *(const uint32_t*)(mine + 36 * j + 4 * i);
            dword = *(const uint32_t*)(mine_d + 36 * j);
        };
        read_block(0);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const XPair xp = xs[j];
            if constexpr (decltype(x_too)::value) fetch_x(xs[j], 4 * nrun + j);
            i32x4 wa, wb;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t q = __builtin_amdgcn_alignbit(r[i + 1], r[i], shift);
                const uint32_t lo = q & 0x0F0F0F0Fu, hi = (q >> 4) & 0x0F0F0F0Fu;
                const auto t = __builtin_amdgcn_permlane32_swap(lo, hi, false, false);
                wa[i] = (int)t[0];
                wb[i] = (int)t[1];
            }
            // every lane gets both blocks' scales (kept as integers across the swap: with its results cast to
            // float in place, this compiler read the first of the two for both)
            const uint32_t dbits = (dword >> (16 - shift)) & 0xffffu;
            const auto dd = __builtin_amdgcn_permlane32_swap(dbits, dbits, false, false);
            if (j < 3) read_block(j + 1);
            const f32x4 dxa = *(const f32x4*)(tail + (2 * j) * kTailBytes), dxb = *(const f32x4*)(tail + (2 * j + 1) * kTailBytes);
            const i32x4 offa = *(const i32x4*)(tail + (2 * j) * kTailBytes + 32), offb = *(const i32x4*)(tail + (2 * j + 1) * kTailBytes + 32);
            i32x16 zero;
#pragma unroll
            for (int i = 0; i < 16; i++) zero[i] = 0;
            // both products are issued before the first one's sums are touched
            const i32x16 ca = __builtin_amdgcn_mfma_i32_32x32x32_i8(xp.a, wa, zero, 0, 0, 0);
            const i32x16 cb = __builtin_amdgcn_mfma_i32_32x32x32_i8(xp.b, wb, zero, 0, 0, 0);
            finish(acc, ca, f16_bits_to_f32((uint16_t)dd[0]), dxa, offa);
            finish(acc, cb, f16_bits_to_f32((uint16_t)dd[1]), dxb, offb);
        }
        cur = nxt;
    };

    // this wavefront's runs one after the other; with the SwiGLU tail, each run of gate is followed by the same
    // run of up, which meets the same operands of x
    float acc[4] = {0.f, 0.f, 0.f, 0.f}, gate_acc[4] = {0.f, 0.f, 0.f, 0.f};
    const int mine_runs = run0 < run_end ? (run_end - run0 + WAVES - 1) / WAVES : 0;
    for (int it = 0; it < mine_runs; it++) {
        const int nx = it + 1 < mine_runs ? it + 1 : it;  // the run requested ahead
        if (TAIL == kRowsSwiGLU) {
            one_run(std::false_type{}, gate_acc, job.W[1], run0 + it * WAVES);
            one_run(std::true_type{}, acc, W, run0 + nx * WAVES);
        } else {
            one_run(std::true_type{}, acc, W, run0 + nx * WAVES);
        }
    }

    __syncthreads();  // every wavefront is done with its slab
    f32x4* red = (f32x4*)smem;
    if (TAIL == kRowsSwiGLU) {
        red[wave * 64 + lane] = f32x4{gate_acc[0], gate_acc[1], gate_acc[2], gate_acc[3]};
        red[(WAVES + wave) * 64 + lane] = f32x4{acc[0], acc[1], acc[2], acc[3]};
    } else {
        red[wave * 64 + lane] = f32x4{acc[0], acc[1], acc[2], acc[3]};
    }
    __syncthreads();
    if (wave != 0) return;
    f32x4 sum = red[lane];
#pragma unroll
    for (int w = 1; w < WAVES; w++) {
        const f32x4 t = red[w * 64 + lane];
#pragma unroll
        for (int j = 0; j < 4; j++) sum[j] = sum[j] + t[j];
    }
    if (TAIL == kRowsPlain) {
        if (n < N) {
            const int64_t row0 = (int64_t)kRows * blockIdx.z;
            float* yo = y + ((int64_t)blockIdx.y * M_all + row0) * ny + ybase;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int m = 4 * lh + j;
                if (m < M) {
                    float v = sum[j];
                    if (resid) v = v + resid[(row0 + m) * ny + ybase + n];
                    yo[(int64_t)m * ny + n] = v;
                }
            }
        }
    } else if (TAIL == kRowsRope) {
        // rows (n, n + 1), n even, are a pair of features: the even lane takes its neighbour's sums and stores both
        const int pos = *tail_args.rope.pos;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const float other = dpp_f32<0xb1>(sum[j]);  // quad_perm [1,0,3,2]
            const int m = 4 * lh + j, seq = kRows * (int)blockIdx.z + m;
            if ((lane & 1) == 0 && n < N && m < M) q4_rope_store(tail_args.rope, pos, seq, ybase + n, sum[j], other, y + (int64_t)seq * ny);
        }
    } else {
        f32x4 up = red[WAVES * 64 + lane];
#pragma unroll
        for (int w = 1; w < WAVES; w++) {
            const f32x4 t = red[(WAVES + w) * 64 + lane];
#pragma unroll
            for (int j = 0; j < 4; j++) up[j] = up[j] + t[j];
        }
        // this workgroup's 32 results of row m are block blockIdx.x of the next product's row m: the lanes of a half
        // hold its elements. Largest magnitude and sum over the half's 32 lanes, digits through LDS into the operand's
        // 16-byte pieces (lane 32 h + 8 d + m of the block: digit d of elements 16 h.. of row m).
        uint8_t* stage = smem + 2 * WAVES * 64 * 16;  // 64 pieces
        const float nl2e = (float)(-1.4426950408889634);
        float scale_j[4];
        int sum_j[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            float v = 0.f;
            if (n < N) {
                const float e = __builtin_exp2f(sum[j] * nl2e);
                const float sg = 1.0f / (1.0f + e);
                const float a = sum[j] * sg;
                v = a * up[j];
            }
            // magnitudes as integers order like the floats, with infinities and NaNs above every finite value
            uint32_t mag = __builtin_bit_cast(uint32_t, v) & 0x7fffffffu;
            mag = max(mag, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)mag, 0xb1, 0xf, 0xf, true));
            mag = max(mag, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)mag, 0x4e, 0xf, 0xf, true));
            mag = max(mag, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)mag, 0x141, 0xf, 0xf, true));
            mag = max(mag, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)mag, 0x140, 0xf, 0xf, true));
            mag = max(mag, (uint32_t)__builtin_amdgcn_ds_swizzle((int)mag, 0x401F));  // lane ^ 16
            const float amax = __builtin_bit_cast(float, mag);
            float scale, inv;
            if (mag >= 0x7f800000u) {  // a NaN or an infinity in the block: its products are NaN
                scale = __builtin_nanf("");
                inv = 0.f;
                v = 0.f;
            } else if (amax < 0x1p-100f) {
                scale = 0.f;
                inv = 0.f;
            } else {
                scale = amax / (float)kFixMax;
                inv = (float)kFixMax / amax;
            }
            int a = (int)__builtin_rintf(v * inv);
            a = a > kFixMax ? kFixMax : a < -kFixMax ? -kFixMax : a;
            int t = a;
            t += __builtin_amdgcn_update_dpp(0, t, 0xb1, 0xf, 0xf, true);
            t += __builtin_amdgcn_update_dpp(0, t, 0x4e, 0xf, 0xf, true);
            t += __builtin_amdgcn_update_dpp(0, t, 0x141, 0xf, 0xf, true);
            t += __builtin_amdgcn_update_dpp(0, t, 0x140, 0xf, 0xf, true);
            t += __builtin_amdgcn_ds_swizzle(t, 0x401F);
            scale_j[j] = scale;
            sum_j[j] = t;
            const int d0 = (int)(int8_t)a;
            const int a1 = (a - d0) >> 8;
            const int d1 = (int)(int8_t)a1;
            const int d2 = (a1 - d1) >> 8;
            const int m = 4 * lh + j;
            uint8_t* at = stage + (32 * (l32 >> 4) + m) * 16 + (l32 & 15);
            at[0] = (uint8_t)d0;
            at[8 * 16] = (uint8_t)d1;
            at[16 * 16] = (uint8_t)d2;
        }
        uint8_t* group_out = tail_args.act_out + (int64_t)blockIdx.z * tail_args.nb_out * (kFragBytes + kTailBytes);
        uint8_t* out = group_out + (int64_t)blockIdx.x * kFragBytes;
        if ((lane & 31) < 24) *(u32x4*)(out + 16 * lane) = *(const u32x4*)(stage + 16 * lane);
        if (l32 == 0) {
            uint8_t* to = group_out + (int64_t)tail_args.nb_out * kFragBytes + (int64_t)blockIdx.x * kTailBytes;
            *(f32x4*)(to + 16 * lh) = f32x4{scale_j[0], scale_j[1], scale_j[2], scale_j[3]};
            *(i32x4*)(to + 32 + 16 * lh) = i32x4{8 * sum_j[0], 8 * sum_j[1], 8 * sum_j[2], 8 * sum_j[3]};
        }
    }
}

// ---- the kernels around the product in a decoding step of a few sequences ------------------------

// RMSNorm of rows of x (RMSNorm.Forward, nn/transformer.go:50-61) into the converted form, with the
// arithmetic of rmsnorm_q4act_kernel (norm_load's sums in its order). With shares, x[m] first
// becomes x[m] + parts[0][m] + parts[1][m] + ... (the shares of K of the product before, added in
// their order) and is written back: the residual connection.
__global__ __launch_bounds__(256) void rows_norm_act_kernel(float* __restrict__ x, const float* __restrict__ parts, int shares,
                                                            int64_t share_stride, const float* __restrict__ w, uint8_t* act, int d,
                                                            float inv_d, float eps) {
    __shared__ float part[4];
    const int m = blockIdx.x, t0 = threadIdx.x, nq = d >> 3, nb = d >> 5;
    float* xr = x + (int64_t)m * d;
    act += (int64_t)(m / kRows) * nb * (kFragBytes + kTailBytes);  // the row's group of eight has a buffer of its own
    NormRow r;
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < kNormItems; i++) {
        const int t = t0 + i * 256;
        if (t < nq) {
            const int o = 32 * (t >> 2) + 4 * (t & 3);
            __builtin_memcpy(&r.lo[i], xr + o, 16);
            __builtin_memcpy(&r.hi[i], xr + o + 16, 16);
            __builtin_memcpy(&r.wl[i], w + o, 16);
            __builtin_memcpy(&r.wh[i], w + o + 16, 16);
        }
    }
    if (shares > 0) {
#pragma unroll
        for (int i = 0; i < kNormItems; i++) {
            const int t = t0 + i * 256;
            if (t < nq) {
                const int o = 32 * (t >> 2) + 4 * (t & 3);
                for (int s = 0; s < shares; s++) {
                    f32x4 pl, ph;
                    const float* pr = parts + s * share_stride + (int64_t)m * d + o;
                    __builtin_memcpy(&pl, pr, 16);
                    __builtin_memcpy(&ph, pr + 16, 16);
#pragma unroll
                    for (int k = 0; k < 4; k++) {
                        r.lo[i][k] = r.lo[i][k] + pl[k];
                        r.hi[i][k] = r.hi[i][k] + ph[k];
                    }
                }
                __builtin_memcpy(xr + o, &r.lo[i], 16);
                __builtin_memcpy(xr + o + 16, &r.hi[i], 16);
            }
        }
    }
#pragma unroll
    for (int i = 0; i < kNormItems; i++) {
        if (t0 + i * 256 < nq) {
#pragma unroll
            for (int k = 0; k < 4; k++) {
                float a = r.lo[i][k] * r.lo[i][k], c = r.hi[i][k] * r.hi[i][k];
                ss = ss + a;
                ss = ss + c;
            }
        }
    }
    ss = wave_sum(ss);
    if ((t0 & 63) == 0) part[t0 >> 6] = ss;
    __syncthreads();
    const float total = (part[0] + part[1]) + (part[2] + part[3]);
    const float ms = total * inv_d;
    const float scale = 1.0f / __builtin_sqrtf(ms + eps);
#pragma unroll
    for (int i = 0; i < kNormItems; i++) {
        const int t = t0 + i * 256;
        if (t < nq) {
            float l4[4], h4[4];
#pragma unroll
            for (int k = 0; k < 4; k++) {
                float a = r.lo[i][k] * scale, c = r.hi[i][k] * scale;
                l4[k] = a * r.wl[i][k];
                h4[k] = c * r.wh[i][k];
            }
            rows_convert_item(l4, h4, act, nb, m % kRows, t >> 2, t & 3);
        }
    }
}

// SiLU(g) * u (llm/model.go:446-448, the arithmetic of swiglu_kernel) into the converted form: g and u
// rows `stride` floats apart, n a multiple of 32.
__global__ __launch_bounds__(256) void rows_swiglu_act_kernel(const float* __restrict__ g, const float* __restrict__ u, int64_t stride,
                                                              uint8_t* act, int n) {
    const float nl2e = (float)(-1.4426950408889634);
    const int m = blockIdx.y, nq = n >> 3, nb = n >> 5;
    const int t = blockIdx.x * 256 + threadIdx.x;
    if (t >= nq) return;  // whole quads: nq is a multiple of 4
    act += (int64_t)(m / kRows) * nb * (kFragBytes + kTailBytes);
    const int o = 32 * (t >> 2) + 4 * (t & 3);
    f32x4 gl, gh, ul, uh;
    __builtin_memcpy(&gl, g + m * stride + o, 16);
    __builtin_memcpy(&gh, g + m * stride + o + 16, 16);
    __builtin_memcpy(&ul, u + m * stride + o, 16);
    __builtin_memcpy(&uh, u + m * stride + o + 16, 16);
    float l4[4], h4[4];
#pragma unroll
    for (int k = 0; k < 4; k++) {
        float e = __builtin_exp2f(gl[k] * nl2e);
        float sg = 1.0f / (1.0f + e);
        float a = gl[k] * sg;
        l4[k] = a * ul[k];
        e = __builtin_exp2f(gh[k] * nl2e);
        sg = 1.0f / (1.0f + e);
        a = gh[k] * sg;
        h4[k] = a * uh[k];
    }
    rows_convert_item(l4, h4, act, nb, m % kRows, t >> 2, t & 3);
}

// x += parts[0] + parts[1] + ..., added in that order, n floats.
__global__ __launch_bounds__(256) void rows_add_parts_kernel(float* __restrict__ x, const float* __restrict__ parts, int shares,
                                                             int64_t share_stride, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    float v = x[i];
    for (int s = 0; s < shares; s++) v = v + parts[s * share_stride + i];
    x[i] = v;
}

}  // namespace

hipError_t rows_norm_act(float* x, const float* parts, int shares, const float* w, void* act, int64_t rows, int64_t d, double eps,
                         hipStream_t st) {
    if (rows <= 0) return hipSuccess;
    if (rows > kRows * 65535 || d % 32 != 0 || d > 8 * 256 * kNormItems) return hipErrorInvalidValue;
    hipLaunchKernelGGL(rows_norm_act_kernel, dim3((unsigned)rows), dim3(256), 0, st, x, parts, parts ? shares : 0, rows * d, w, (uint8_t*)act,
                       (int)d, (float)(1.0 / (double)d), (float)eps);
    return hipGetLastError();
}

hipError_t rows_swiglu_act(const float* g, const float* u, void* act, int64_t rows, int64_t n, int64_t stride, hipStream_t st) {
    if (rows <= 0) return hipSuccess;
    if (rows > 65535 || n % 32 != 0) return hipErrorInvalidValue;
    hipLaunchKernelGGL(rows_swiglu_act_kernel, dim3((unsigned)((n / 8 + 255) / 256), (unsigned)rows), dim3(256), 0, st, g, u, stride,
                       (uint8_t*)act, (int)n);
    return hipGetLastError();
}

hipError_t rows_add_parts(float* x, const float* parts, int shares, int64_t n, hipStream_t st) {
    if (n <= 0 || shares <= 0) return hipSuccess;
    hipLaunchKernelGGL(rows_add_parts_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, x, parts, shares, n, n);
    return hipGetLastError();
}

static std::atomic<int> g_rows_direct{0};  // measurement aid: 1 = always the kernel without the LDS pass
static std::atomic<int> g_rows_waves{0};   // measurement aid: 4 or 8 = that many wavefronts a workgroup, whatever the shape
void set_q4_rows_direct(int v) { g_rows_direct = v; }
void set_q4_rows_waves(int v) { g_rows_waves = v; }

// W 2-byte aligned (ggml blocks), pairs of blocks, at most eight rows of x.
static bool rows_base_ok(const void* W, int64_t M, int64_t N, int64_t K) {
    return K > 0 && K % 64 == 0 && K <= (1 << 20) && ((uintptr_t)W & 1) == 0 && M > 0 && M <= kRows * 65535 && N > 0 && N <= (1ll << 30);
}

// Whether the product can be cut into `shares` shares of K whose sums a later kernel adds: the kernel that
// passes rows of W through LDS (runs of eight blocks, W 16-byte aligned), at least a run per share.
bool qgemv_q4_0_rows_shares_ok(const void* W, int64_t M, int64_t N, int64_t K, int shares) {
    return rows_base_ok(W, M, N, K) && shares >= 1 && shares <= 8 && K % 256 == 0 && K / 256 >= shares && ((uintptr_t)W & 15) == 0 &&
           32 * (K / 32) * 18 < ((int64_t)1 << 32) && g_rows_direct == 0;
}

bool qgemv_q4_0_rows_ok(const void* W, int64_t M, int64_t N, int64_t K) {
    return rows_base_ok(W, M, N, K) &&
           (qgemv_q4_0_rows_shares_ok(W, M, N, K, 1) || (size_t)(K / 32) * kTailBytes + kWaves * 64 * 16 <= 64 * 1024);
}

static int64_t grid_z(int64_t M) { return (M + kRows - 1) / kRows; }

// Many workgroups: four wavefronts each, so that all are resident at once and each wavefront has runs to request
// ahead of; few: eight, for the parallelism.
static hipError_t launch_rows(const RowsJob& job, unsigned groups, int shares, int tail, const RowsTailArgs& t, const void* act, float* y,
                              const float* resid, int64_t M, int64_t K, hipStream_t st) {
    const bool four = tail != kRowsSwiGLU && (g_rows_waves == 4 || (g_rows_waves == 0 && (int64_t)groups * shares * grid_z(M) >= 384));
    const dim3 grid(groups, (unsigned)shares, (unsigned)((M + kRows - 1) / kRows));
#define ROWS_LAUNCH(WV, TL)                                                                                                       \
    hipLaunchKernelGGL((qgemv_q4_0_rows_kernel<WV, TL>), grid, dim3(64 * WV), (size_t)WV * kWaveLds, st, job, (const uint8_t*)act, y, \
                       resid, (int)M, (int)(K / 32), t)
    if (tail == kRowsSwiGLU) ROWS_LAUNCH(4, kRowsSwiGLU);
    else if (tail == kRowsRope) { if (four) ROWS_LAUNCH(4, kRowsRope); else ROWS_LAUNCH(8, kRowsRope); }
    else { if (four) ROWS_LAUNCH(4, kRowsPlain); else ROWS_LAUNCH(8, kRowsPlain); }
#undef ROWS_LAUNCH
    return hipGetLastError();
}

// act: q4_0_rows_convert_act's buffer. y[M, N] = x . W^T (+ resid, which may be y itself). With shares > 1
// (qgemv_q4_0_rows_shares_ok, no resid): y[shares, M, N], share s of K summed into y[s].
hipError_t qgemv_q4_0_rows(const void* W, const void* act, float* y, const float* resid, int64_t M, int64_t N, int64_t K, int shares,
                           hipStream_t st) {
    const int nb = (int)(K / 32);
    const dim3 wg(64 * kWaves);
    if (qgemv_q4_0_rows_shares_ok(W, M, N, K, shares)) {
        const void* w1[3] = {W, nullptr, nullptr};
        const int64_t n1[3] = {N, 0, 0};
        return qgemv_q4_0_rows_multi(w1, n1, act, y, resid, M, K, shares, st);
    }
    if (shares != 1 || M > kRows) return hipErrorInvalidValue;  // this kernel: a group of eight rows a launch
    const size_t lds = (size_t)nb * kTailBytes + kWaves * 64 * 16;
    if (lds > 64 * 1024) return hipErrorInvalidValue;
    hipLaunchKernelGGL(qgemv_q4_0_rows_direct_kernel, dim3((unsigned)((N + 31) / 32)), wg, lds, st, (const uint8_t*)W, (const uint8_t*)act, y,
                       resid, (int)M, (int)N, nb);
    return hipGetLastError();
}

// About what a product of M rows takes, conversion included: 5 us and a pass over W per eight rows at 4.2 TB/s
// (measured at 4096 x 4096, 4096 x 14336 and 14336 x 4096, 8 to 128 rows: 131, 125 and 41 us at 128 rows).
double qgemv_q4_0_rows_cost_us(int64_t M, int64_t N, int64_t K) {
    return (double)((M + kRows - 1) / kRows) * ((double)N * (double)(K / 32) * 18.0 / 4.2e6) + 5.0;
}

// Up to three matrices (n[i] = 0: none) that share act and K, their rows one after the other in
// y[shares, M, n[0] + n[1] + n[2]]; every matrix must satisfy qgemv_q4_0_rows_shares_ok and all but the last have
// a multiple of 32 rows.
hipError_t qgemv_q4_0_rows_multi(const void* const W[3], const int64_t n[3], const void* act, float* y, const float* resid, int64_t M,
                                 int64_t K, int shares, hipStream_t st) {
    RowsJob job;
    int last = -1;
    for (int i = 0; i < 3; i++)
        if (n[i] > 0) last = i;
    unsigned groups = 0;
    for (int i = 0; i < 3; i++) {
        job.W[i] = (const uint8_t*)W[i];
        job.n[i] = (int)n[i];
        job.groups[i] = (int)((n[i] + 31) / 32);
        groups += (unsigned)job.groups[i];
        if (n[i] > 0 && (!qgemv_q4_0_rows_shares_ok(W[i], M, n[i], K, shares) || (i != last && n[i] % 32 != 0))) return hipErrorInvalidValue;
        if (n[i] == 0 && i < last) return hipErrorInvalidValue;
    }
    if (last < 0 || (shares > 1 && resid)) return hipErrorInvalidValue;
    return launch_rows(job, groups, shares, kRowsPlain, RowsTailArgs{}, act, y, resid, M, K, st);
}

// q, k and v in one launch with the rotation and the cache writes of a decoding step as its tail: y [M, n[0] + n[1] + n[2]]
// receives the rotated queries only (interleaved pairs, even row counts).
hipError_t qgemv_q4_0_rows_qkv_rope(const void* const W[3], const int64_t n[3], const void* act, float* y, int64_t M, int64_t K,
                                    const Q4RopeTail& rope, hipStream_t st) {
    RowsJob job;
    unsigned groups = 0;
    for (int i = 0; i < 3; i++) {
        if (n[i] <= 0 || n[i] % 32 != 0 || !qgemv_q4_0_rows_shares_ok(W[i], M, n[i], K, 1)) return hipErrorInvalidValue;
        job.W[i] = (const uint8_t*)W[i];
        job.n[i] = (int)n[i];
        job.groups[i] = (int)(n[i] / 32);
        groups += (unsigned)job.groups[i];
    }
    RowsTailArgs t;
    t.rope = rope;
    return launch_rows(job, groups, 1, kRowsRope, t, act, y, nullptr, M, K, st);
}

// SiLU(x . gate^T) * (x . up^T), gate and up [N, K], converted into act_out as the x of a product over N (N a multiple of 32).
hipError_t qgemv_q4_0_rows_swiglu_act(const void* gate, const void* up, const void* act, void* act_out, int64_t M, int64_t N, int64_t K,
                                      hipStream_t st) {
    if (N % 32 != 0 || !qgemv_q4_0_rows_shares_ok(gate, M, N, K, 1) || !qgemv_q4_0_rows_shares_ok(up, M, N, K, 1)) return hipErrorInvalidValue;
    RowsJob job;
    job.W[0] = (const uint8_t*)gate; job.W[1] = (const uint8_t*)up; job.W[2] = nullptr;
    job.n[0] = (int)N; job.n[1] = 0; job.n[2] = 0;
    job.groups[0] = (int)(N / 32); job.groups[1] = job.groups[2] = 0;
    RowsTailArgs t;
    t.act_out = (uint8_t*)act_out;
    t.nb_out = (int)(N / 32);
    return launch_rows(job, (unsigned)(N / 32), 1, kRowsSwiGLU, t, act, nullptr, nullptr, M, K, st);
}

}  // namespace mimir
