// Decode products by block-quantized weights, y = x . W^T with few rows of x,
// for gfx950. They replace the reference's generated qmatmul kernel
// (backend/internal/gen/quant.go:152-209) and compute what its CPU backend
// computes (backend/cpu/qmatmul.go:310-405):
//
//   Q4_0          the float32 product with the dequantized weights (the
//                 reference decodes Q4_0 to float32 at load, io/mim/dtype.go:118-123,
//                 and multiplies in float32, backend/cpu/gemv.go:73-104)
//   Q8_0/Q4_K/Q6_K  activations rounded to int8 per block (quantizeRow,
//                 qmatmul.go:208-254), integer dot products, scales applied
//                 once per block (qdotQ8_0Go/qdotQ4KGo/qdotQ6KGo, :125-200)
//
// W stays in ggml's layout, read in place. A wavefront owns R rows of W at a
// time and splits K across its 64 lanes, one block of 32 weights per lane and
// step; each lane fetches its block with one (unaligned) 128-bit load, so a
// wavefront's load covers 64 consecutive blocks, and every load of a tile is
// issued before the first is used. The activations are staged once per
// workgroup in LDS, transposed so that the lanes' 128-bit LDS reads are
// conflict-free. Row sums are reduced over the wavefront with DPP.
#include "device_util.h"
#include "kernels.h"

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

hipError_t qgemv_q4_0(const QGemvArgs& a, const int* tune, hipStream_t st) {
    Q4Plan p = plan_q4_0(a.N, a.K, tune);
    int nb = (int)(a.K / 32);
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
