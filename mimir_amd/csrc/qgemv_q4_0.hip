// Decode products by Q4_0 weights, y = x . W^T with few rows of x, for gfx950.
// They replace the reference's generated qmatmul kernel
// (backend/internal/gen/quant.go:152-209). What the reference's CPU computes
// for a Q4_0 linear is the float32 product with the dequantized weights: it
// decodes Q4_0 to float32 at load (io/mim/dtype.go:118-123) and multiplies in
// float32 (backend/cpu/gemv.go:73-104).
//
// W stays in ggml's layout (18-byte blocks: binary16 scale, 16 bytes of
// nibbles), read in place. A wavefront owns R rows of W at a time and splits K
// across its 64 lanes; every load of a tile is issued before the first is
// used; the activations are staged once per workgroup in LDS, laid out so that
// the lanes' 128-bit LDS reads are conflict-free; row sums are reduced over
// the wavefront with DPP.
//
// Two kernels:
//
//  qgemv_q4_0_i4_kernel   the fast path. The kernel is bound by vector-ALU
//    issue as much as by HBM (a 16-lane SIMD needs four cycles per wavefront
//    instruction), so it multiplies eight weights per instruction with
//    v_dot8_i32_i4: XOR 0x88888888 turns a dword of offset-binary nibbles n
//    into two's-complement (n - 8), and each block of 32 activations is held
//    as a 24-bit fixed-point number per element, split into six planes of
//    signed 4-bit digits, with one float32 scale per block. The integer sums
//    are exact; the only error is the fixed-point rounding of x, at most
//    2^-23 of the block's largest magnitude per element: float32's own
//    precision for the block's large values, and below 1e-7 of the result. Lanes own pairs of blocks (36 bytes, dword aligned)
//    and fetch them with aligned 128-bit loads. Needs K a multiple of 64 and W
//    dword aligned.
//
//  qgemv_q4_0_kernel      any shape and any 2-byte aligned W: float32
//    multiply-adds through v_fma_mix_f32 on nibbles masked in place as
//    binary16 subnormals.
#include <hip/hip_ext.h>
#include "device_util.h"
#include "kernels.h"
#include "q4_act.h"
#include "q4_job.h"
#include "rope_tail.h"

namespace mimir {

// LDS layout of the staged activations of one row of x with nb blocks:
//   float4 xs[8][nbp]   part j of block b at xs[j * nbp + b]; nbp = nb | 1
//   float  xsum[nb]     sum of the block's 32 values
__host__ __device__ inline int q4_nbp(int nb) { return nb | 1; }
__host__ __device__ inline size_t q4_lds_bytes(int nb) { return (size_t)q4_nbp(nb) * 8 * 16 + (size_t)nb * 4; }

// ---- Q4_0 -------------------------------------------------------------------
//
// The nibbles are multiplied without an integer-to-float conversion: masked
// in place, a nibble at bits 0-3 (or 4-7) of a 16-bit half is the binary16
// subnormal n * 2^-24 (or 16n * 2^-24), which v_fma_mix_f32 widens for free.
// Per dword of 8 nibbles that is 5 bit operations and 8 fused multiply-adds.
// The factors 2^-24 and 16 are powers of two and are taken out exactly when
// the block's scale is applied; the offset 8 is applied through the block sum
// of x: sum (n-8) x = sum n x - 8 sum x.
// x values a thread parks in registers between their global load and their
// LDS store, so that the weights' loads can be issued in between.
constexpr int kStage = 8;

__device__ __forceinline__ f32x4 load_f32x4(const float* p) {
    f32x4 v;
    __builtin_memcpy(&v, p, 16);
    return v;
}

template <int R, int C>
struct Q4Tile {
    u32x4 q[R][C];
    uint16_t d[R][C];
};

template <int R, int C>
__device__ __forceinline__ void q4_load_tile(Q4Tile<R, C>& t, const uint8_t* __restrict__ W, int64_t row_bytes, int N, int nb,
                                             int row0, int c0, int lane) {
#pragma unroll
    for (int c = 0; c < C; c++) {
        int b = lane + 64 * (c0 + c);
        int bc = b < nb ? b : nb - 1;
#pragma unroll
        for (int r = 0; r < R; r++) {
            int row = row0 + r;
            row = row < N ? row : N - 1;
            const uint8_t* p = W + (int64_t)row * row_bytes + (int64_t)bc * 18;
            t.d[r][c] = load_u16(p);
            t.q[r][c] = load_u32x4_unaligned(p + 2);
        }
    }
}

template <int R, int C, bool XLDS>
__global__ __launch_bounds__(512) void qgemv_q4_0_kernel(const uint8_t* __restrict__ W, const float* __restrict__ x,
                                                         float* __restrict__ y, int N, int nb, int64_t x_row_stride,
                                                         int rows_per_wg) {
    extern __shared__ f32x4 lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, waves = blockDim.x >> 6;
    const int m = blockIdx.y;
    const float* xr = x + (int64_t)m * x_row_stride;
    float* yr = y + (int64_t)m * N;
    const int nbp = q4_nbp(nb);
    float* xsum = (float*)(lds + 8 * nbp);
    const int64_t row_bytes = (int64_t)nb * 18;
    const int wg_row0 = blockIdx.x * rows_per_wg;
    const int ncol = (nb + 63) >> 6;
    const int nf = nb * 8;  // float4s of x

    Q4Tile<R, C> tile;
    int r0 = wave * R;
    // The first tile's loads go out between the loads of x and its LDS stores.
    f32x4 park[kStage];
    if (XLDS) {
#pragma unroll
        for (int i = 0; i < kStage; i++) {
            int f = tid + i * (int)blockDim.x;
            if (f < nf) park[i] = load_f32x4(xr + 4 * (int64_t)f);
        }
    }
    const bool first_live = r0 < rows_per_wg && wg_row0 + r0 < N;
    if (first_live) q4_load_tile<R, C>(tile, W, row_bytes, N, nb, wg_row0 + r0, 0, lane);
    if (XLDS) {
#pragma unroll
        for (int i = 0; i < kStage; i++) {
            int f = tid + i * (int)blockDim.x;
            if (f < nf) {
                f32x4 v = park[i];
                int b = f >> 3, j = f & 7;
                lds[j * nbp + b] = v;
                // all 8 lanes of a block are live together: nf is a multiple of 8 and so is the stride
                float s = group8_sum((v[0] + v[1]) + (v[2] + v[3]));
                if (j == 7) xsum[b] = s;
            }
        }
        for (int f = tid + kStage * (int)blockDim.x; f < nf; f += (int)blockDim.x) {
            f32x4 v = load_f32x4(xr + 4 * (int64_t)f);
            int b = f >> 3, j = f & 7;
            lds[j * nbp + b] = v;
            float s = group8_sum((v[0] + v[1]) + (v[2] + v[3]));
            if (j == 7) xsum[b] = s;
        }
        __syncthreads();
    }

    bool loaded = first_live;
    for (; r0 < rows_per_wg; r0 += waves * R) {
        const int row0 = wg_row0 + r0;
        if (row0 >= N) break;
        float acc[R];
#pragma unroll
        for (int r = 0; r < R; r++) acc[r] = 0.f;

        for (int c0 = 0; c0 < ncol; c0 += C) {
            if (!loaded) q4_load_tile<R, C>(tile, W, row_bytes, N, nb, row0, c0, lane);
            loaded = false;
#pragma unroll
            for (int c = 0; c < C; c++) {
                int b = lane + 64 * (c0 + c);
                bool live = b < nb;
                int bc = live ? b : nb - 1;
                f32x4 xv[8];
                float xs;
                if (XLDS) {
#pragma unroll
                    for (int j = 0; j < 8; j++) xv[j] = lds[j * nbp + bc];
                    xs = xsum[bc];
                } else {
                    xs = 0.f;
#pragma unroll
                    for (int j = 0; j < 8; j++) {
                        xv[j] = load_f32x4(xr + 32 * (int64_t)bc + 4 * j);
                        xs += (xv[j][0] + xv[j][1]) + (xv[j][2] + xv[j][3]);
                    }
                }
                if (!live) {
#pragma unroll
                    for (int j = 0; j < 8; j++) xv[j] = f32x4{0.f, 0.f, 0.f, 0.f};
                    xs = 0.f;
                }
#pragma unroll
                for (int r = 0; r < R; r++) {
                    float lo = 0.f, hi = 0.f;
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        uint32_t w = tile.q[r][c][i], s = w >> 8;
                        f16x2 p0 = as_f16x2(w & 0x000F000Fu), p1 = as_f16x2(w & 0x00F000F0u);
                        f16x2 p2 = as_f16x2(s & 0x000F000Fu), p3 = as_f16x2(s & 0x00F000F0u);
                        // byte k of the dword holds elements 4i+k (low nibble) and 16+4i+k (high)
                        lo = fmaf((float)p0[0], xv[i][0], lo);
                        lo = fmaf((float)p2[0], xv[i][1], lo);
                        lo = fmaf((float)p0[1], xv[i][2], lo);
                        lo = fmaf((float)p2[1], xv[i][3], lo);
                        hi = fmaf((float)p1[0], xv[4 + i][0], hi);
                        hi = fmaf((float)p3[0], xv[4 + i][1], hi);
                        hi = fmaf((float)p1[1], xv[4 + i][2], hi);
                        hi = fmaf((float)p3[1], xv[4 + i][3], hi);
                    }
                    // lo = 2^-24 sum n x over the low nibbles, hi = 2^-20 sum n x over the high ones
                    float t = fmaf(hi, 0.0625f, lo);
                    t = fmaf(xs, -8.0f * 0x1p-24f, t);
                    float d = f16_bits_to_f32(tile.d[r][c]) * 0x1p24f;
                    acc[r] = fmaf(d, t, acc[r]);
                }
            }
        }
#pragma unroll
        for (int r = 0; r < R; r++) {
            float s = wave_sum(acc[r]);
            if (lane == 0 && row0 + r < N) yr[row0 + r] = s;
        }
    }
}

template <int R, int C>
static hipError_t launch_q4_0(const QGemvArgs& a, int waves, bool xlds, hipStream_t st) {
    int rows_per_wg = a.rows_per_wg > 0 ? a.rows_per_wg : R * waves;
    dim3 grid((unsigned)((a.N + rows_per_wg - 1) / rows_per_wg), (unsigned)a.M);
    size_t lds = xlds ? q4_lds_bytes((int)(a.K / 32)) : 0;
    if (xlds)
        hipLaunchKernelGGL((qgemv_q4_0_kernel<R, C, true>), grid, dim3(64 * waves), lds, st, (const uint8_t*)a.W, a.x, a.y,
                           (int)a.N, (int)(a.K / 32), a.x_row_stride, rows_per_wg);
    else
        hipLaunchKernelGGL((qgemv_q4_0_kernel<R, C, false>), grid, dim3(64 * waves), lds, st, (const uint8_t*)a.W, a.x, a.y,
                           (int)a.N, (int)(a.K / 32), a.x_row_stride, rows_per_wg);
    return hipGetLastError();
}

// ---- fixed-point activations, v_dot8_i32_i4 ---------------------------------
//
// One row of x with nb blocks, converted (nbp = nb | 1; q4_0_act_bytes(K) bytes):
//   u32x4 plane[6][nbp]  digit plane j of block b at plane[j * nbp + b]: dword i
//                        holds, nibble for nibble as dword i of the block's
//                        weights does (byte k: low nibble element 4i+k, high
//                        nibble element 16+4i+k), digit j of those elements
//   float scale[nb]      x[e] ~ scale * sum_j 16^j digit_j[e]
// The conversion runs once per x (q4_0_convert_act), not once per workgroup
// of the product: a decode step multiplies the same x by several matrices.
size_t q4_0_act_bytes(int64_t K) { return q4_0_act_row_bytes(K); }

// Thread t of a row takes item t: block t / 4, dword t % 4. The block's four
// items sit in consecutive lanes (the item count and the stride are multiples
// of 4), so its largest magnitude is a quad reduction.
__global__ __launch_bounds__(256) void q4_0_convert_act_kernel(const float* __restrict__ x, int64_t x_row_stride, int nb,
                                                               uint8_t* __restrict__ act, int64_t act_row_bytes) {
    const float* xr = x + (int64_t)blockIdx.y * x_row_stride;
    u32x4* plane = (u32x4*)(act + (int64_t)blockIdx.y * act_row_bytes);
    const int nbp = nb | 1;
    float* xscale = (float*)(plane + kDigits * nbp);
    const int nq = nb * 4;
    for (int t = blockIdx.x * blockDim.x + threadIdx.x; t < nq; t += gridDim.x * blockDim.x) {
        int b = t >> 2, d = t & 3;
        f32x4 vlo = load_f32x4(xr + 32 * (int64_t)b + 4 * d), vhi = load_f32x4(xr + 32 * (int64_t)b + 16 + 4 * d);
        float lo[4] = {vlo[0], vlo[1], vlo[2], vlo[3]}, hi[4] = {vhi[0], vhi[1], vhi[2], vhi[3]};
        q4_convert_item(lo, hi, plane, xscale, nbp, b, d);
    }
}

hipError_t q4_0_convert_act(const float* x, int64_t M, int64_t K, int64_t x_row_stride, void* act, hipStream_t st) {
    int nb = (int)(K / 32);
    int gx = (nb * 4 + 255) / 256;
    hipLaunchKernelGGL(q4_0_convert_act_kernel, dim3((unsigned)gx, (unsigned)M), dim3(256), 0, st, x, x_row_stride, nb,
                       (uint8_t*)act, (int64_t)q4_0_act_bytes(K));
    return hipGetLastError();
}

static std::atomic<int> g_q4_batch_off{0};  // measurement aid: 1 keeps products of several rows of x on the one-row kernel, 2 puts all on the batch kernel
void set_q4_batch_off(int v) { g_q4_batch_off = v; }

template <int R, int PC, int MODE, int HEAD = kHeadAct>
__global__ __launch_bounds__(512) void qgemv_q4_0_i4_kernel(Q4Job job, const uint8_t* __restrict__ act, float* __restrict__ y,
                                                             int nb, int64_t act_row_bytes, int rows_per_wg) {
    constexpr int RR = MODE == kSwiGLU ? 2 * R : R;  // rows of weights a tile reads
    extern __shared__ u32x4 lds_i4[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), waves = blockDim.x >> 6;
    const int m = blockIdx.y;
    const int N = job.total;
    float* yr = y + (int64_t)m * N;
    const int nbp = nb | 1;
    const float* xscale = (const float*)(lds_i4 + kDigits * nbp);
    const int64_t row_bytes = (int64_t)nb * 18;
    const int wg_row0 = blockIdx.x * rows_per_wg;
    const int npairs = nb >> 1;
    const int npc = (npairs + 63) >> 6;
    const int rope_pos = MODE == kRope ? *job.rope.pos : 0;

    // The address of the weights behind row t of the tile at row0; rows past
    // the end are clamped into the matrix (their sums are never stored).
    auto row_ptr = [&](int row0, int t) -> const uint8_t* {
        if (MODE == kSwiGLU) {
            int r = row0 + (t < R ? t : t - R);
            r = r < N ? r : N - 1;
            return job.W[t < R ? 0 : 1] + (int64_t)r * row_bytes;
        }
        int g = row0 + t;
        g = g < N ? g : N - 1;
        if (MODE == kMulti || MODE == kRope) {
            if (g >= job.n[0] + job.n[1]) return job.W[2] + (int64_t)(g - job.n[0] - job.n[1]) * row_bytes;
            if (g >= job.n[0]) return job.W[1] + (int64_t)(g - job.n[0]) * row_bytes;
        }
        return job.W[0] + (int64_t)g * row_bytes;
    };

    // Loads return in order, so the activations' loads go out first: they come
    // back from L2 well before the weights do from HBM, and the LDS stores and
    // the barrier are then over by the time the first weights arrive.
    constexpr int kPark = PC == 1 ? 2 : 6;
    const u32x4* act_row = (const u32x4*)(act + (int64_t)m * act_row_bytes);
    const int n16 = (int)(act_row_bytes >> 4);
    u32x4 park[kPark];
    __shared__ float norm_part[4];
    NormRow norm_row;
    float norm_ss = 0.f;
    constexpr int kCv = 2;  // items of x a thread requests ahead of the weights when it converts x itself
    f32x4 cv_lo[kCv], cv_hi[kCv];
    const int nq = nb * 4;
    if (HEAD == kHeadNorm) {  // eight wavefronts; the first four hold the row between its sum of squares and its conversion
        if (tid < 256) norm_ss = norm_load(norm_row, job.norm_x + (int64_t)m * nb * 32, job.norm_w, nq, tid);
    } else if (HEAD == kHeadConvert) {
        const float* xr = job.norm_x + (int64_t)m * job.x_row_stride;
#pragma unroll
        for (int i = 0; i < kCv; i++) {
            int t = tid + i * (int)blockDim.x;
            t = t < nq ? t : nq - 1;
            cv_lo[i] = load_f32x4(xr + 32 * (t >> 2) + 4 * (t & 3));
            cv_hi[i] = load_f32x4(xr + 32 * (t >> 2) + 16 + 4 * (t & 3));
        }
    } else {
#pragma unroll
        for (int i = 0; i < kPark; i++) {
            int idx = tid + i * (int)blockDim.x;
            if (idx < n16) park[i] = act_row[idx];
        }
    }
    Q4PairTile<RR, PC> tile;
    int r0 = wave * R;
    const uint8_t* rowp[RR];
#pragma unroll
    for (int t = 0; t < RR; t++) rowp[t] = row_ptr(wg_row0 + r0, t);
    // Unconditional (rows are clamped into W): a branch here would make the
    // wait before the LDS stores below cover the weights' loads as well.
    q4_load_pairs<RR, PC>(tile, rowp, npairs, 0, lane);
    if (HEAD != kHeadAct) __builtin_amdgcn_sched_barrier(0);  // the weights' loads stay ahead of the arithmetic on x below
    if (HEAD == kHeadNorm) {
        if (tid < 256) {
            norm_ss = wave_sum(norm_ss);
            if (lane == 0) norm_part[wave] = norm_ss;
        }
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");  // LDS only: the weights' loads stay in flight
        if (tid < 256)
            norm_convert(norm_row, norm_part, nullptr, (u32x4*)lds_i4, (float*)(lds_i4 + kDigits * nbp), nbp, nq, tid,
                         job.norm_inv_d, job.norm_eps);
    } else if (HEAD == kHeadConvert) {
        // items t = tid, tid + blockDim, ...: the four items of a block sit in four consecutive lanes
        const float* xr = job.norm_x + (int64_t)m * job.x_row_stride;
        u32x4* plane = (u32x4*)lds_i4;
        float* xs = (float*)(lds_i4 + kDigits * nbp);
#pragma unroll
        for (int i = 0; i < kCv; i++) {
            const int t = tid + i * (int)blockDim.x;
            if (t < nq) {
                float lo[4] = {cv_lo[i][0], cv_lo[i][1], cv_lo[i][2], cv_lo[i][3]}, hi[4] = {cv_hi[i][0], cv_hi[i][1], cv_hi[i][2], cv_hi[i][3]};
                q4_convert_item(lo, hi, plane, xs, nbp, t >> 2, t & 3);
            }
        }
        for (int t = tid + kCv * (int)blockDim.x; t < nq; t += (int)blockDim.x) {
            const f32x4 vlo = load_f32x4(xr + 32 * (t >> 2) + 4 * (t & 3)), vhi = load_f32x4(xr + 32 * (t >> 2) + 16 + 4 * (t & 3));
            float lo[4] = {vlo[0], vlo[1], vlo[2], vlo[3]}, hi[4] = {vhi[0], vhi[1], vhi[2], vhi[3]};
            q4_convert_item(lo, hi, plane, xs, nbp, t >> 2, t & 3);
        }
    } else {
#pragma unroll
        for (int i = 0; i < kPark; i++) {
            int idx = tid + i * (int)blockDim.x;
            if (idx < n16) lds_i4[idx] = park[i];
        }
        for (int idx = tid + kPark * (int)blockDim.x; idx < n16; idx += (int)blockDim.x) lds_i4[idx] = act_row[idx];
    }
    __syncthreads();

    bool loaded = true;
    for (; r0 < rows_per_wg; r0 += waves * R) {
        const int row0 = wg_row0 + r0;
        if (row0 >= N) break;
        if (!loaded) {
#pragma unroll
            for (int t = 0; t < RR; t++) rowp[t] = row_ptr(row0, t);
        }
        float acc[RR];
#pragma unroll
        for (int r = 0; r < RR; r++) acc[r] = 0.f;
        for (int pc0 = 0; pc0 < npc; pc0 += PC) {
            if (!loaded) q4_load_pairs<RR, PC>(tile, rowp, npairs, pc0, lane);
            loaded = false;
#pragma unroll
            for (int pc = 0; pc < PC; pc++) {
                int p = lane + 64 * (pc0 + pc);
                const bool live = p < npairs;
                p = live ? p : npairs - 1;
                u32x4 d0[kDigits], d1[kDigits];
#pragma unroll
                for (int j = 0; j < kDigits; j++) {
                    d0[j] = lds_i4[j * nbp + 2 * p];
                    d1[j] = lds_i4[j * nbp + 2 * p + 1];
                }
                const float s0 = live ? xscale[2 * p] : 0.f, s1 = live ? xscale[2 * p + 1] : 0.f;
#pragma unroll
                for (int r = 0; r < RR; r++) {
                    const u32x4 a = tile.a[r][pc], b = tile.b[r][pc];
                    const uint32_t c = tile.c[r][pc];
                    // block 0: scale in the low half of a[0], nibbles at bytes 2..17
                    const uint32_t q0[4] = {__builtin_amdgcn_alignbyte(a[1], a[0], 2), __builtin_amdgcn_alignbyte(a[2], a[1], 2),
                                            __builtin_amdgcn_alignbyte(a[3], a[2], 2), __builtin_amdgcn_alignbyte(b[0], a[3], 2)};
                    // block 1: scale in the high half of b[0], nibbles at bytes 20..35
                    const uint32_t q1[4] = {b[1], b[2], b[3], c};
                    int i0, i1;
                    q4_pair_dot(q0, q1, d0, d1, i0, i1);
                    const float f0 = (float)i0, f1 = (float)i1;
                    // a lane past the row's end re-reads the last pair: it must add exactly zero
                    const float w0 = live ? f16_bits_to_f32((uint16_t)(a[0] & 0xffffu)) * s0 : 0.f;
                    const float w1 = live ? f16_bits_to_f32((uint16_t)(b[0] >> 16)) * s1 : 0.f;
                    acc[r] = fmaf(w0, f0, acc[r]);
                    acc[r] = fmaf(w1, f1, acc[r]);
                }
            }
        }
        if (MODE == kRope) {
#pragma unroll
            for (int r = 0; r + 1 < R; r += 2) {
                const float a = wave_sum(acc[r]), b = wave_sum(acc[r + 1]);
                if (lane == 0 && row0 + r < N) q4_rope_store(job.rope, rope_pos, m, row0 + r, a, b, yr);
            }
            continue;
        }
#pragma unroll
        for (int r = 0; r < R; r++) {
            float s = wave_sum(acc[r]);
            if (MODE == kSwiGLU) {
                const float u = wave_sum(acc[R + r]);
                const float e = __builtin_exp2f(s * (float)(-1.4426950408889634));
                const float sg = 1.0f / (1.0f + e);
                const float a = s * sg;
                s = a * u;
            }
            if (MODE == kSwiGLU && job.act_out) {
                if (lane == 0) ((float*)(lds_i4 + n16))[r0 + r] = s;  // behind the staged activations
            } else if (lane == 0 && row0 + r < N) {
                if (MODE == kPlain && job.resid) s = s + job.resid[(int64_t)m * N + row0 + r];
                yr[row0 + r] = s;
            }
        }
    }
    if (MODE == kSwiGLU && job.act_out) {  // the workgroup's 32 results are block blockIdx.x of the next product's x
        __syncthreads();
        if (tid < 4) {
            const f32x4* v = (const f32x4*)(lds_i4 + n16);
            const f32x4 vlo = v[tid], vhi = v[4 + tid];
            float lo[4] = {vlo[0], vlo[1], vlo[2], vlo[3]}, hi[4] = {vhi[0], vhi[1], vhi[2], vhi[3]};
            u32x4* plane = (u32x4*)(job.act_out + (int64_t)m * job.act_out_row_bytes);
            const int nbp_out = (N >> 5) | 1;
            q4_convert_item(lo, hi, plane, (float*)(plane + kDigits * nbp_out), nbp_out, blockIdx.x, tid);
        }
    }
}

// The same product for several rows of x at once: a workgroup stages MB converted rows in LDS, a
// wavefront unpacks its rows of W once per step and multiplies them with one row of x after the
// other, so W is read from memory once for MB rows of x instead of once for each. Every row of x
// meets the same lanes, steps and reductions as in the kernel above, so its results are the same
// bits. Over converted activations only; tails as above (the block of SwiGLU results per row of x).
template <int R, int MODE, int MB>
__global__ __launch_bounds__(512) void qgemv_q4_0_i4_batch_kernel(Q4Job job, const uint8_t* __restrict__ act, float* __restrict__ y, int M,
                                                                   int nb, int64_t act_row_bytes, int rows_per_wg) {
    constexpr int RR = MODE == kSwiGLU ? 2 * R : R;
    extern __shared__ u32x4 lds_i4[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), waves = blockDim.x >> 6;
    const int m0 = blockIdx.y * MB;
    const int mc = M - m0 < MB ? M - m0 : MB;  // rows of x this workgroup has
    const int N = job.total;
    const int nbp = nb | 1;
    const int n16 = (int)(act_row_bytes >> 4);
    const int64_t row_bytes = (int64_t)nb * 18;
    const int wg_row0 = blockIdx.x * rows_per_wg;
    const int npairs = nb >> 1;
    const int npc = (npairs + 63) >> 6;
    const int rope_pos = MODE == kRope ? *job.rope.pos : 0;
    float* outv = (float*)(lds_i4 + MB * n16);  // kSwiGLU with act_out: 32 results per row of x

    auto row_ptr = [&](int row0, int t) -> const uint8_t* {
        if (MODE == kSwiGLU) {
            int r = row0 + (t < R ? t : t - R);
            r = r < N ? r : N - 1;
            return job.W[t < R ? 0 : 1] + (int64_t)r * row_bytes;
        }
        int g = row0 + t;
        g = g < N ? g : N - 1;
        if (MODE == kMulti || MODE == kRope) {
            if (g >= job.n[0] + job.n[1]) return job.W[2] + (int64_t)(g - job.n[0] - job.n[1]) * row_bytes;
            if (g >= job.n[0]) return job.W[1] + (int64_t)(g - job.n[0]) * row_bytes;
        }
        return job.W[0] + (int64_t)g * row_bytes;
    };

    Q4PairTile<RR, 1> tile;
    int r0 = wave * R;
    const uint8_t* rowp[RR];
#pragma unroll
    for (int t = 0; t < RR; t++) rowp[t] = row_ptr(wg_row0 + r0, t);
    q4_load_pairs<RR, 1>(tile, rowp, npairs, 0, lane);  // in flight while the rows of x are staged
    const u32x4* src = (const u32x4*)(act + (int64_t)m0 * act_row_bytes);
    for (int idx = tid; idx < mc * n16; idx += (int)blockDim.x) lds_i4[idx] = src[idx];
    __syncthreads();

    bool loaded = true;
    for (; r0 < rows_per_wg; r0 += waves * R) {
        const int row0 = wg_row0 + r0;
        if (row0 >= N) break;
        if (!loaded) {
#pragma unroll
            for (int t = 0; t < RR; t++) rowp[t] = row_ptr(row0, t);
        }
        float acc[MB][RR];
#pragma unroll
        for (int mi = 0; mi < MB; mi++)
#pragma unroll
            for (int r = 0; r < RR; r++) acc[mi][r] = 0.f;
        for (int pc = 0; pc < npc; pc++) {
            if (!loaded) q4_load_pairs<RR, 1>(tile, rowp, npairs, pc, lane);
            loaded = false;
            int p = lane + 64 * pc;
            const bool live = p < npairs;
            p = live ? p : npairs - 1;
            // the rows of W of this step, unpacked once for all rows of x
            uint32_t q0[RR][4], q1[RR][4];
            float dw0[RR], dw1[RR];
#pragma unroll
            for (int r = 0; r < RR; r++) {
                const u32x4 a = tile.a[r][0], b = tile.b[r][0];
                q0[r][0] = __builtin_amdgcn_alignbyte(a[1], a[0], 2);
                q0[r][1] = __builtin_amdgcn_alignbyte(a[2], a[1], 2);
                q0[r][2] = __builtin_amdgcn_alignbyte(a[3], a[2], 2);
                q0[r][3] = __builtin_amdgcn_alignbyte(b[0], a[3], 2);
                q1[r][0] = b[1], q1[r][1] = b[2], q1[r][2] = b[3], q1[r][3] = tile.c[r][0];
                dw0[r] = f16_bits_to_f32((uint16_t)(a[0] & 0xffffu));
                dw1[r] = f16_bits_to_f32((uint16_t)(b[0] >> 16));
            }
#pragma unroll
            for (int mi = 0; mi < MB; mi++) {
                if (mi < mc) {
                    const u32x4* xrow = lds_i4 + mi * n16;
                    const float* xscale = (const float*)(xrow + kDigits * nbp);
                    u32x4 d0[kDigits], d1[kDigits];
#pragma unroll
                    for (int j = 0; j < kDigits; j++) {
                        d0[j] = xrow[j * nbp + 2 * p];
                        d1[j] = xrow[j * nbp + 2 * p + 1];
                    }
                    const float s0 = live ? xscale[2 * p] : 0.f, s1 = live ? xscale[2 * p + 1] : 0.f;
#pragma unroll
                    for (int r = 0; r < RR; r++) {
                        int i0, i1;
                        q4_pair_dot(q0[r], q1[r], d0, d1, i0, i1);
                        const float f0 = (float)i0, f1 = (float)i1;
                        // a lane past the row's end re-reads the last pair: it must add exactly zero
                        const float w0 = live ? dw0[r] * s0 : 0.f;
                        const float w1 = live ? dw1[r] * s1 : 0.f;
                        acc[mi][r] = fmaf(w0, f0, acc[mi][r]);
                        acc[mi][r] = fmaf(w1, f1, acc[mi][r]);
                    }
                }
            }
        }
#pragma unroll
        for (int mi = 0; mi < MB; mi++) {
            if (mi >= mc) break;
            const int m = m0 + mi;
            float* yr = y + (int64_t)m * N;
            if (MODE == kRope) {
#pragma unroll
                for (int r = 0; r + 1 < R; r += 2) {
                    const float a = wave_sum(acc[mi][r]), b = wave_sum(acc[mi][r + 1]);
                    if (lane == 0 && row0 + r < N) q4_rope_store(job.rope, rope_pos, m, row0 + r, a, b, yr);
                }
                continue;
            }
#pragma unroll
            for (int r = 0; r < R; r++) {
                float s = wave_sum(acc[mi][r]);
                if (MODE == kSwiGLU) {
                    const float u = wave_sum(acc[mi][R + r]);
                    const float e = __builtin_exp2f(s * (float)(-1.4426950408889634));
                    const float sg = 1.0f / (1.0f + e);
                    const float a = s * sg;
                    s = a * u;
                }
                if (MODE == kSwiGLU && job.act_out) {
                    if (lane == 0) outv[32 * mi + r0 + r] = s;
                } else if (lane == 0 && row0 + r < N) {
                    if (MODE == kPlain && job.resid) s = s + job.resid[(int64_t)m * N + row0 + r];
                    yr[row0 + r] = s;
                }
            }
        }
    }
    if (MODE == kSwiGLU && job.act_out) {  // per row of x, the workgroup's 32 results are block blockIdx.x of the next product's x
        __syncthreads();
        if (tid < 4 * mc) {
            const int mi = tid >> 2, d = tid & 3;
            const f32x4* v = (const f32x4*)(outv + 32 * mi);
            const f32x4 vlo = v[d], vhi = v[4 + d];
            float lo[4] = {vlo[0], vlo[1], vlo[2], vlo[3]}, hi[4] = {vhi[0], vhi[1], vhi[2], vhi[3]};
            u32x4* plane = (u32x4*)(job.act_out + (int64_t)(m0 + mi) * job.act_out_row_bytes);
            const int nbp_out = (N >> 5) | 1;
            q4_convert_item(lo, hi, plane, (float*)(plane + kDigits * nbp_out), nbp_out, blockIdx.x, d);
        }
    }
}

// Rows of x a workgroup of the batch kernel can stage (8, 4, 2; 0: none fits).
static int q4_batch_rows(int64_t M, int64_t K) {
    const size_t row = q4_0_act_bytes(K);
    for (int mb = 8; mb >= 2; mb >>= 1)
        if (M >= mb && (size_t)mb * row + 1024 <= 144 * 1024) return mb;
    return M >= 2 && 2 * row + 1024 <= 144 * 1024 ? 2 : 0;
}

template <int R, int MODE, int MB>
static hipError_t launch_q4_0_i4_batch(const Q4Job& job, const void* act, float* y, int64_t M, int64_t K, hipStream_t st) {
    static std::atomic<bool> raised{false};  // threads may race here: both then set the same attribute
    const size_t act_bytes = q4_0_act_bytes(K), lds_bytes = MB * act_bytes + MB * 128;
    if (!raised) {
        hipError_t e = hipFuncSetAttribute((const void*)qgemv_q4_0_i4_batch_kernel<R, MODE, MB>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                           160 * 1024);
        if (e != hipSuccess) return e;
        raised = true;
    }
    const int rows_per_wg = MODE == kSwiGLU && job.act_out ? 32 : R * 8;
    dim3 grid((unsigned)((job.total + rows_per_wg - 1) / rows_per_wg), (unsigned)((M + MB - 1) / MB));
    hipLaunchKernelGGL((qgemv_q4_0_i4_batch_kernel<R, MODE, MB>), grid, dim3(512), lds_bytes, st, job, (const uint8_t*)act, y, (int)M,
                       (int)(K / 32), (int64_t)act_bytes, rows_per_wg);
    return hipGetLastError();
}

// From two rows of x on the batch kernel, where it is the faster: both kernels are bound by the
// vector arithmetic of the six digit planes, not by reading W, so sharing W gains only where staging
// x per workgroup is what costs (rows of x from 8192 on: 20 % faster at 4096 x 14336, 15 to 60 %
// slower at K = 4096; measured for 2 to 512 rows of x).
template <int MODE>
static bool dispatch_q4_0_i4_batch(const Q4Job& job, const void* act, float* y, int64_t M, int64_t K, hipStream_t st, hipError_t* err) {
    if (job.norm_x || g_q4_batch_off == 1 || (K < 8192 && g_q4_batch_off != 2)) return false;
    const int mb = q4_batch_rows(M, K);
    if (mb == 0) return false;
    constexpr int R = MODE == kSwiGLU ? 2 : 4;
    *err = mb == 8 ? launch_q4_0_i4_batch<R, MODE, 8>(job, act, y, M, K, st)
           : mb == 4 ? launch_q4_0_i4_batch<R, MODE, 4>(job, act, y, M, K, st)
                     : launch_q4_0_i4_batch<R, MODE, 2>(job, act, y, M, K, st);
    return true;
}

template <int R, int PC, int MODE, int HEAD = kHeadAct>
static hipError_t launch_q4_0_i4(const Q4Job& job, const void* act, float* y, int64_t M, int64_t K, int waves, hipStream_t st) {
    int rows_per_wg = R * waves;
    if (MODE == kSwiGLU && job.act_out) rows_per_wg = 32;  // a block of results a workgroup, in one or two turns of its wavefronts
    dim3 grid((unsigned)((job.total + rows_per_wg - 1) / rows_per_wg), (unsigned)M);
    size_t act_bytes = q4_0_act_bytes(K);
    const size_t lds_bytes = act_bytes + (MODE == kSwiGLU ? 128 : 0);  // kSwiGLU: room for a block of results
    note_kernel("qgemv_q4_0_i4_kernel<%d, %d, %d, %d>", R, PC, MODE, HEAD);
    hipEvent_t t0, t1;
    if (next_timing_events(&t0, &t1))  // a measurement is on: this launch's own begin and end
        hipExtLaunchKernelGGL((qgemv_q4_0_i4_kernel<R, PC, MODE, HEAD>), grid, dim3(64 * waves), lds_bytes, st, t0, t1, 0, job,
                              (const uint8_t*)act, y, (int)(K / 32), (int64_t)act_bytes, rows_per_wg);
    else
        hipLaunchKernelGGL((qgemv_q4_0_i4_kernel<R, PC, MODE, HEAD>), grid, dim3(64 * waves), lds_bytes, st, job, (const uint8_t*)act, y,
                           (int)(K / 32), (int64_t)act_bytes, rows_per_wg);
    return hipGetLastError();
}

// Shape of a launch: R rows per wavefront, C column steps in flight, waves
// per workgroup. A 16-lane SIMD issues a wavefront instruction over four
// cycles, so the tiles must cover all four SIMDs of each of the 256 CUs: the
// plan aims at 2048 tiles or more (8 wavefronts per CU), with up to 16
// 128-bit loads in flight per lane, in workgroups as large as leaves at
// least one per CU, which share one staging of x.
struct Q4Plan { int R, C, waves; };

static int floor_to_instantiated_rows(int64_t r, int c) {
    static const int rows1[] = {16, 8, 4, 2, 1}, rows2[] = {8, 7, 4, 2, 1}, rows4[] = {4, 2, 1}, rows7[] = {2, 1};
    const int* set = c == 1 ? rows1 : c == 2 ? rows2 : c == 4 ? rows4 : rows7;
    int n = c == 1 ? 5 : c == 2 ? 5 : c == 4 ? 3 : 2;
    for (int i = 0; i < n; i++)
        if (set[i] <= r) return set[i];
    return 1;
}

static Q4Plan plan_q4_0(int64_t N, int64_t K, const int* tune) {
    Q4Plan p;
    int ncol = (int)((K / 32 + 63) / 64);
    p.C = ncol <= 1 ? 1 : ncol <= 2 ? 2 : ncol <= 4 ? 4 : 7;
    if (tune[1] > 0) p.C = tune[1];
    p.R = floor_to_instantiated_rows(N / 2048 > 0 ? N / 2048 : 1, p.C);
    if (p.R == 8 && p.C == 2 && N % 7 == 0) p.R = 7;
    if (tune[0] > 0) p.R = tune[0];
    int64_t tiles = (N + p.R - 1) / p.R;
    p.waves = 8;
    while (p.waves > 1 && tiles / p.waves < 256) p.waves >>= 1;
    if (tune[2] > 0) p.waves = tune[2];
    return p;
}

bool q4_0_fixed_point_ok(const void* W, int64_t K) {
    int64_t nb = K / 32;
    return nb > 0 && nb % 2 == 0 && ((uintptr_t)W & 3) == 0 && q4_0_act_bytes(K) <= 64 * 1024;
}

// Launch shape of the fixed-point kernel. Many small tiles: measured on MI355X,
// two rows per wavefront in workgroups of eight wavefronts stream best at the
// decode shapes. tune: {rows, pair steps, waves}.
template <int MODE>
static hipError_t dispatch_q4_0_i4(const Q4Job& job, const void* act, float* y, int64_t M, int64_t K, const int* tune, hipStream_t st) {
    if constexpr (MODE != kMulti) {
        hipError_t e;
        if (M >= 2 && tune[0] == 0 && tune[1] == 0 && tune[2] == 0 && dispatch_q4_0_i4_batch<MODE>(job, act, y, M, K, st, &e)) return e;
    }
    if (tune[0] == 0 && tune[1] == 0 && tune[2] == 0) {  // no launch plan forced: the kernel shaped for the whole chip where it takes the shape
        hipError_t e;
        if (q4_0_dma_dispatch(MODE, job, act, y, M, K, st, &e)) return e;
        if (q4_0_stream_dispatch(MODE, job, act, y, M, K, st, &e)) return e;
    }
    int nb = (int)(K / 32);
    int npc = (nb / 2 + 63) / 64;  // steps of 64 pairs of blocks that cover a row
    int PC = npc <= 1 ? 1 : 2;
    if (tune[1] > 0) PC = tune[1];
    int R = MODE == kSwiGLU ? (job.total >= 8192 ? 2 : 1) : (job.total >= 4096 ? 2 : 1);
    if (MODE == kPlain && job.total >= 8192 && npc <= 1) R = 4;  // many short rows: fewer, longer-lived wavefronts stream a little better
    if (tune[0] > 0) R = tune[0];
    if (MODE == kRope) R = 2;  // a wavefront's two rows are the pair of features a rotation takes
    if (MODE == kSwiGLU && job.act_out) R = tune[0] == 4 ? 4 : 2, PC = 1;  // eight wavefronts, two turns of two rows (or one of four)
    int64_t tiles = (job.total + R - 1) / R;
    int waves = 8;
    while (waves > 1 && tiles / waves < 256) waves >>= 1;
    if (tune[2] > 0) waves = tune[2];
    if (waves > 8) waves = 8;
    if (MODE == kSwiGLU && job.act_out) waves = 8;
#define Q4ICASE(RR, PP) if (R == RR && PC == PP) return launch_q4_0_i4<RR, PP, MODE>(job, act, y, M, K, waves, st)
    if (job.norm_w) {  // kRope, and kSwiGLU with converted results: two rows, eight wavefronts, rows one step long
        if constexpr (MODE == kRope || MODE == kSwiGLU) return launch_q4_0_i4<2, 1, MODE, kHeadNorm>(job, act, y, M, K, 8, st);
        return hipErrorInvalidValue;
    }
    if constexpr (MODE == kRope) {
        Q4ICASE(2, 1);
        return launch_q4_0_i4<2, 2, MODE>(job, act, y, M, K, waves, st);
    } else {
        if constexpr (MODE == kPlain) {
            if (job.norm_x) {  // x itself, converted by every workgroup
#define Q4CCASE(RR, PP) if (R == RR && PC == PP) return launch_q4_0_i4<RR, PP, MODE, kHeadConvert>(job, act, y, M, K, waves, st)
                Q4CCASE(1, 1); Q4CCASE(2, 1); Q4CCASE(4, 1);
                Q4CCASE(1, 2); Q4CCASE(2, 2); Q4CCASE(4, 2);
#undef Q4CCASE
                return launch_q4_0_i4<1, 1, MODE, kHeadConvert>(job, act, y, M, K, waves, st);
            }
        }
        Q4ICASE(1, 1); Q4ICASE(2, 1); Q4ICASE(4, 1);
        Q4ICASE(1, 2); Q4ICASE(2, 2);
        if constexpr (MODE != kSwiGLU) { Q4ICASE(4, 2); }
        return launch_q4_0_i4<1, 1, MODE>(job, act, y, M, K, waves, st);
    }
#undef Q4ICASE
}

// The fixed-point product from converted activations (a.act), plus a.resid
// if set. Needs q4_0_fixed_point_ok.
hipError_t qgemv_q4_0_act(const QGemvArgs& a, const int* tune, hipStream_t st) {
    // without converted activations every workgroup converts its row of a.x for itself (few rows of x: a launch saved)
    Q4Job job{{(const uint8_t*)a.W, nullptr, nullptr}, {(int)a.N, 0, 0}, (int)a.N, a.resid, {}, nullptr, 0, a.act ? nullptr : a.x, nullptr, 0.f, 0.f,
              a.x_row_stride};
    return dispatch_q4_0_i4<kPlain>(job, a.act, a.y, a.M, a.K, tune, st);
}

// y[m, :] = x[m, :] . [W0; W1; W2]^T for up to three matrices [n_i, K] (n_i may
// be 0), each qualifying for the fixed-point kernel; y rows are n0 + n1 + n2 long.
hipError_t qgemv_q4_0_act_multi(const void* const W[3], const int64_t n[3], const void* act, float* y, int64_t M, int64_t K,
                                const int* tune, hipStream_t st) {
    Q4Job job{{(const uint8_t*)W[0], (const uint8_t*)W[1], (const uint8_t*)W[2]}, {(int)n[0], (int)n[1], (int)n[2]},
              (int)(n[0] + n[1] + n[2]), nullptr, {}, nullptr, 0, nullptr, nullptr, 0.f, 0.f, 0};
    return dispatch_q4_0_i4<kMulti>(job, act, y, M, K, tune, st);
}

// The q, k, v projections of a decoding step with the rotation and the cache
// writes behind them (see kRope): y [M, n0 + n1 + n2] receives the rotated
// queries only. Needs the interleaved layout, even head and rotation widths.
hipError_t qgemv_q4_0_act_qkv_rope(const void* const W[3], const int64_t n[3], const void* act, float* y, int64_t M, int64_t K,
                                   const Q4RopeTail& rope, const Q4NormHead& norm, const int* tune, hipStream_t st) {
    Q4Job job{{(const uint8_t*)W[0], (const uint8_t*)W[1], (const uint8_t*)W[2]}, {(int)n[0], (int)n[1], (int)n[2]},
              (int)(n[0] + n[1] + n[2]), nullptr, rope, nullptr, 0, norm.x, norm.w, (float)(1.0 / (double)K), (float)norm.eps, K};
    return dispatch_q4_0_i4<kRope>(job, act, y, M, K, tune, st);
}

// Whether a product can take the norm of its x as its first phase (Q4NormHead): x short enough for
// the norm's 256 threads and for one step of a wavefront.
bool q4_0_norm_head_ok(int64_t K) { return K % 64 == 0 && K / 8 <= 256 * kNormItems && K / 64 <= 64; }

// y[m, r] = SiLU(x[m, :] . gate[r]) * (x[m, :] . up[r]), gate and up [N, K].
hipError_t qgemv_q4_0_act_swiglu(const void* gate, const void* up, const void* act, float* y, int64_t M, int64_t N, int64_t K,
                                 const int* tune, hipStream_t st) {
    Q4Job job{{(const uint8_t*)gate, (const uint8_t*)up, nullptr}, {(int)N, (int)N, 0}, (int)N, nullptr, {}, nullptr, 0, nullptr, nullptr, 0.f, 0.f, 0};
    return dispatch_q4_0_i4<kSwiGLU>(job, act, y, M, K, tune, st);
}

// Whether qgemv_q4_0_act_swiglu_convert takes the shape: rows of x that one
// step of the wavefront covers, and whole blocks of results.
bool q4_0_swiglu_convert_ok(int64_t N, int64_t K) { return K / 64 <= 64 && N % 64 == 0; }

// The same, with the results left in the fixed-point form of activations in
// act_out (q4_0_act_bytes(N) bytes a row, not the buffer act points into)
// instead of float32: the conversion that would follow as a launch of its own.
hipError_t qgemv_q4_0_act_swiglu_convert(const void* gate, const void* up, const void* act, void* act_out, int64_t M, int64_t N,
                                         int64_t K, const Q4NormHead& norm, const int* tune, hipStream_t st) {
    Q4Job job{{(const uint8_t*)gate, (const uint8_t*)up, nullptr}, {(int)N, (int)N, 0}, (int)N, nullptr, {}, (uint8_t*)act_out,
              (int64_t)q4_0_act_bytes(N), norm.x, norm.w, (float)(1.0 / (double)K), (float)norm.eps, K};
    return dispatch_q4_0_i4<kSwiGLU>(job, act, nullptr, M, K, tune, st);
}

// The float32 product, any shape. tune: {rows, cols, waves, no_lds}.
hipError_t qgemv_q4_0(const QGemvArgs& a, const int* tune, hipStream_t st) {
    int nb = (int)(a.K / 32);
    Q4Plan p = plan_q4_0(a.N, a.K, tune);
    bool xlds = q4_lds_bytes(nb) <= 64 * 1024 && tune[3] == 0;
#define Q4CASE(RR, CC) if (p.R == RR && p.C == CC) return launch_q4_0<RR, CC>(a, p.waves, xlds, st)
    Q4CASE(1, 1); Q4CASE(2, 1); Q4CASE(4, 1); Q4CASE(8, 1); Q4CASE(16, 1);
    Q4CASE(1, 2); Q4CASE(2, 2); Q4CASE(4, 2); Q4CASE(7, 2); Q4CASE(8, 2);
    Q4CASE(1, 4); Q4CASE(2, 4); Q4CASE(4, 4);
    Q4CASE(1, 7); Q4CASE(2, 7);
#undef Q4CASE
    // any other shape: one row per wavefront, one step at a time
    return launch_q4_0<1, 1>(a, p.waves, xlds, st);
}

}  // namespace mimir
