// Decode products by Q8_0 weights, y = x . W^T with few rows of x, for gfx950.
// They replace the reference's generated qmatmul kernel
// (backend/internal/gen/quant.go:152-209) and compute what its CPU backend
// computes (backend/cpu/qmatmul.go:310-405): each block of 32 activations is
// rounded to int8 with a float32 scale (quantizeRow, qmatmul.go:208-254), the
// products of a block are summed in four int32 lanes, value p into lane
// p/4 mod 4, each lane times the product of the two scales is added to a
// float32 lane of its own (a multiply, then an add: never fused), and the lanes
// are added (0+2)+(1+3) (qdotQ8_0Go, qmatmul.go:125-139). The integer sums are
// exact; the result differs from the CPU's only in the order in which the
// blocks of a row are added, a few units in the last place.
//
// W stays in ggml's layout (34-byte blocks: binary16 scale, 32 int8), read in
// place. A lane owns a pair of blocks, 68 bytes, dword aligned, fetched with
// four aligned 128-bit loads and one dword; the second block's quants are
// dword aligned, the first's are realigned with v_alignbyte. The activations
// are converted once per x by q8_convert_act and staged in LDS per workgroup.
#include "device_util.h"
#include "kernels.h"

namespace mimir {

#pragma clang fp contract(off)

// One row of x with nb blocks, converted (nbp = nb | 1):
//   u32x4 q[2][nbp]   quants 16h..16h+15 of block b at q[h * nbp + b]
//   float d[nb]       the block's scale
size_t q8_act_bytes(int64_t K) {
    int64_t nb = K / 32;
    return (size_t)(((nb | 1) * 2 * 16 + nb * 4 + 15) / 16 * 16);
}

// quantizeRow (backend/cpu/qmatmul.go:208-254) for blocks of 32. Thread t takes
// four values: block t / 8, dword t % 8; a block's eight threads are
// consecutive lanes.
// Item t of a row (block t / 8, dword t % 8; a block's eight items in eight consecutive lanes,
// all active) from its four values: the dword of quants into q, the block's scale from its first item.
__device__ __forceinline__ void q8_convert_item(const f32x4 v, uint32_t* q, float* dscale, int nbp, int t) {
    const int b = t >> 3, i = t & 7;
    float amax = 0.f;
    bool finite = true;
#pragma unroll
    for (int k = 0; k < 4; k++) {
        float a = __builtin_fabsf(v[k]);
        finite = finite && a < __builtin_inff();  // false for NaN too
        if (a > amax) amax = a;
    }
    amax = group8_max(amax);
    float bad = group8_max(finite ? 0.f : 1.f);
    float d = 0.f;
    uint32_t packed = 0;
    if (bad != 0.f) {
        d = __builtin_nanf("");
    } else if (amax != 0.f) {
        d = amax / 127.0f;
        float id = 127.0f / amax;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            int r = (int)__builtin_rintf(v[k] * id);  // nearest, ties to even
            r = r > 127 ? 127 : r < -127 ? -127 : r;
            packed |= (uint32_t)(r & 0xff) << (8 * k);
        }
    }
    q[((i >> 2) * nbp + b) * 4 + (i & 3)] = packed;
    if (i == 0) dscale[b] = d;
}

__global__ __launch_bounds__(256) void q8_convert_act_kernel(const float* __restrict__ x, int64_t x_row_stride, int nb,
                                                             uint8_t* __restrict__ act, int64_t act_row_bytes) {
    const float* xr = x + (int64_t)blockIdx.y * x_row_stride;
    uint32_t* q = (uint32_t*)(act + (int64_t)blockIdx.y * act_row_bytes);
    const int nbp = nb | 1;
    float* dscale = (float*)(q + 2 * nbp * 4);
    const int nq = nb * 8;
    for (int t = blockIdx.x * blockDim.x + threadIdx.x; t < nq; t += gridDim.x * blockDim.x) {
        f32x4 v;
        __builtin_memcpy(&v, xr + 4 * (int64_t)t, 16);
        q8_convert_item(v, q, dscale, nbp, t);
    }
}

hipError_t q8_convert_act(const float* x, int64_t M, int64_t K, int64_t x_row_stride, void* act, hipStream_t st) {
    int nb = (int)(K / 32);
    int gx = (nb * 8 + 255) / 256;
    hipLaunchKernelGGL(q8_convert_act_kernel, dim3((unsigned)gx, (unsigned)M), dim3(256), 0, st, x, x_row_stride, nb,
                       (uint8_t*)act, (int64_t)q8_act_bytes(K));
    return hipGetLastError();
}

typedef u32x4 u32x4_a4 __attribute__((aligned(4)));
typedef u32x4 u32x4_a2 __attribute__((aligned(2)));

// The 17 dwords of a pair of blocks, or, for an odd last block or a W that is
// only 2-byte aligned, one block at a time through unaligned loads.
struct Q8Pair {
    u32x4 v[4];
    uint32_t tail;
};

// acc[l] += (d_w * d_x) * float(s_l) for the four lane sums of one block,
// with the reference's roundings: the scales' product, its product with each
// sum, and the addition are each rounded to float32.
__device__ __forceinline__ void q8_block(const uint32_t w[8], const u32x4 xa, const u32x4 xb, float dw, float dx, float acc[4]) {
    const float dd = dw * dx;
#pragma unroll
    for (int l = 0; l < 4; l++) {
        int s = __builtin_amdgcn_sdot4((int)w[l], (int)xa[l], 0, false);
        s = __builtin_amdgcn_sdot4((int)w[l + 4], (int)xb[l], s, false);
        float t = dd * (float)s;
        acc[l] = acc[l] + t;
    }
}

// CONVERT: act is float32 x (rows act_row_bytes bytes apart) and every workgroup rounds its row to
// int8 for itself (few rows of x: a launch saved); otherwise act holds rows converted beforehand.
template <int R, bool ALIGNED, bool CONVERT>
__global__ __launch_bounds__(512) void qgemv_q8_0_kernel(const uint8_t* __restrict__ W, const uint8_t* __restrict__ act, float* y,
                                                         const float* resid, int N, int nb, int64_t act_row_bytes, int rows_per_wg) {
    extern __shared__ u32x4 lds_q8[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), waves = blockDim.x >> 6;
    const int m = blockIdx.y;
    float* yr = y + (int64_t)m * N;
    const int nbp = nb | 1;
    const float* xd = (const float*)(lds_q8 + 2 * nbp);
    const int64_t row_bytes = (int64_t)nb * 34;
    const int wg_row0 = blockIdx.x * rows_per_wg;
    // ALIGNED: lanes own pairs of blocks; otherwise single blocks.
    const int nunits = ALIGNED ? nb >> 1 : nb;
    const int nsteps = (nunits + 63) >> 6;

    // The blocks of W a lane multiplies at one step of its rows [row0, row0 + R).
    Q8Pair pr[R];
    uint32_t single[R][9];
    auto request = [&](int row0, int step) {
        int u = lane + 64 * step;
        u = u < nunits ? u : nunits - 1;
#pragma unroll
        for (int r = 0; r < R; r++) {
            int row = row0 + r;
            row = row < N ? row : N - 1;
            const uint8_t* rowp = W + (int64_t)row * row_bytes;
            if (ALIGNED) {
                const uint32_t* src = (const uint32_t*)rowp + u * 17;
#pragma unroll
                for (int k = 0; k < 4; k++) pr[r].v[k] = *(const u32x4_a4*)(src + 4 * k);
                pr[r].tail = src[16];
            } else {
                const uint8_t* src = rowp + (int64_t)u * 34;
                u32x4 a = *(const u32x4_a2*)(src + 2), b = *(const u32x4_a2*)(src + 18);
                single[r][0] = load_u16(src);
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    single[r][1 + k] = a[k];
                    single[r][5 + k] = b[k];
                }
            }
        }
    };
    // W does not depend on x: where the workgroup converts x itself (a product on its own, few workgroups), the wavefront's
    // first blocks are requested behind x's first loads (loads return in order) and are on their way while x is staged:
    // 6.6 -> 5.7 us at 4096 x 4096. With x converted beforehand (the decoder's head: thousands of workgroups that hide
    // one another's waits) the blocks are requested where they are used.
    const int first_r0 = wave * R;

    // Stage the converted activations (see qgemv_q4_0_i4_kernel for the order).
    constexpr int kPark = 2;
    if (CONVERT) {
        const float* xr = (const float*)(act + (int64_t)m * act_row_bytes);
        const int nq = nb * 8;
        f32x4 park[kPark];
#pragma unroll
        for (int i = 0; i < kPark; i++) {
            const int t = tid + i * (int)blockDim.x;
            if (t < nq) __builtin_memcpy(&park[i], xr + 4 * (int64_t)t, 16);
        }
        request(wg_row0 + first_r0, 0);  // rows past the end are clamped: no branch, so that the waits below are counted
#pragma unroll
        for (int i = 0; i < kPark; i++) {
            const int t = tid + i * (int)blockDim.x;
            if (t < nq) q8_convert_item(park[i], (uint32_t*)lds_q8, (float*)(lds_q8 + 2 * nbp), nbp, t);
        }
        for (int t = tid + kPark * (int)blockDim.x; t < nq; t += (int)blockDim.x) {
            f32x4 v;
            __builtin_memcpy(&v, xr + 4 * (int64_t)t, 16);
            q8_convert_item(v, (uint32_t*)lds_q8, (float*)(lds_q8 + 2 * nbp), nbp, t);
        }
    } else {
        const u32x4* act_row = (const u32x4*)(act + (int64_t)m * act_row_bytes);
        const int n16 = (int)(act_row_bytes >> 4);
        u32x4 park[kPark];
#pragma unroll
        for (int i = 0; i < kPark; i++) {
            int idx = tid + i * (int)blockDim.x;
            if (idx < n16) park[i] = act_row[idx];
        }
#pragma unroll
        for (int i = 0; i < kPark; i++) {
            int idx = tid + i * (int)blockDim.x;
            if (idx < n16) lds_q8[idx] = park[i];
        }
        for (int idx = tid + kPark * (int)blockDim.x; idx < n16; idx += (int)blockDim.x) lds_q8[idx] = act_row[idx];
    }
    __syncthreads();

    for (int r0 = wave * R; r0 < rows_per_wg; r0 += waves * R) {
        const int row0 = wg_row0 + r0;
        if (row0 >= N) break;
        float acc[R][4];
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int l = 0; l < 4; l++) acc[r][l] = 0.f;
        for (int step = 0; step < nsteps; step++) {
            int u = lane + 64 * step;
            const bool live = u < nunits;
            u = live ? u : nunits - 1;
            if (!CONVERT || r0 != first_r0 || step != 0) request(row0, step);
            if (ALIGNED) {
                const u32x4 xa0 = lds_q8[2 * u], xb0 = lds_q8[nbp + 2 * u];
                const u32x4 xa1 = lds_q8[2 * u + 1], xb1 = lds_q8[nbp + 2 * u + 1];
                const float dx0 = live ? xd[2 * u] : 0.f, dx1 = live ? xd[2 * u + 1] : 0.f;
#pragma unroll
                for (int r = 0; r < R; r++) {
                    uint32_t d[17];
#pragma unroll
                    for (int k = 0; k < 16; k++) d[k] = pr[r].v[k >> 2][k & 3];
                    d[16] = pr[r].tail;
                    // block 0: scale in the low half of d[0], quants at bytes 2..33
                    uint32_t w0[8], w1[8];
#pragma unroll
                    for (int k = 0; k < 8; k++) {
                        w0[k] = __builtin_amdgcn_alignbyte(d[k + 1], d[k], 2);
                        w1[k] = d[9 + k];  // block 1: scale in the high half of d[8], quants at bytes 36..67
                    }
                    // a lane past the row's end re-reads the last pair: it must add exactly zero
                    q8_block(w0, xa0, xb0, live ? f16_bits_to_f32((uint16_t)(d[0] & 0xffffu)) : 0.f, dx0, acc[r]);
                    q8_block(w1, xa1, xb1, live ? f16_bits_to_f32((uint16_t)(d[8] >> 16)) : 0.f, dx1, acc[r]);
                }
            } else {
                const u32x4 xa = lds_q8[u], xb = lds_q8[nbp + u];
                const float dx = live ? xd[u] : 0.f;
#pragma unroll
                for (int r = 0; r < R; r++)
                    q8_block(&single[r][1], xa, xb, live ? f16_bits_to_f32((uint16_t)single[r][0]) : 0.f, dx, acc[r]);
            }
        }
#pragma unroll
        for (int r = 0; r < R; r++) {
            float a0 = wave_sum(acc[r][0]), a1 = wave_sum(acc[r][1]), a2 = wave_sum(acc[r][2]), a3 = wave_sum(acc[r][3]);
            float s02 = a0 + a2, s13 = a1 + a3;
            if (lane == 0 && row0 + r < N) {
                const float v = s02 + s13;
                yr[row0 + r] = resid ? v + resid[(int64_t)m * N + row0 + r] : v;
            }
        }
    }
}

// Several rows of x against W read once: MB converted rows staged in LDS once per workgroup, whose wavefronts
// then walk rows_per_wave rows of W each (pairs of blocks, W 4-byte aligned; the next row's first blocks are
// requested before the current row is multiplied). Every (row of W, row of x) sum is formed exactly as the
// kernel above forms it.
template <int MB>
__global__ __launch_bounds__(512) void qgemv_q8_0_rows_kernel(const uint8_t* __restrict__ W, const uint8_t* __restrict__ act, float* y, int M,
                                                              int N, int nb, int64_t act_row_bytes, int rows_per_wave) {
    extern __shared__ u32x4 lds_q8[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), waves = blockDim.x >> 6;
    const int m0 = blockIdx.y * MB;
    const int nbp = nb | 1;
    const int n16 = (int)(act_row_bytes >> 4);
    const int64_t row_bytes = (int64_t)nb * 34;
    const int nunits = nb >> 1, nsteps = (nunits + 63) >> 6;
    const int wg_row0 = blockIdx.x * waves * rows_per_wave;
    auto fetch = [&](Q8Pair& f, int row, int step) {
        int u = lane + 64 * step;
        u = u < nunits ? u : nunits - 1;
        const uint32_t* src = (const uint32_t*)(W + (int64_t)(row < N ? row : N - 1) * row_bytes) + u * 17;
#pragma unroll
        for (int k = 0; k < 4; k++) f.v[k] = *(const u32x4_a4*)(src + 4 * k);
        f.tail = src[16];
    };
    Q8Pair next;  // the first row's first step is requested before x is staged
    fetch(next, wg_row0 + wave, 0);
    for (int mb = 0; mb < MB; mb++) {
        const int m = m0 + mb < M ? m0 + mb : M - 1;
        const u32x4* act_row = (const u32x4*)(act + (int64_t)m * act_row_bytes);
        for (int idx = tid; idx < n16; idx += (int)blockDim.x) lds_q8[mb * n16 + idx] = act_row[idx];
    }
    __syncthreads();
    for (int i = 0; i < rows_per_wave; i++) {
        const int row = wg_row0 + wave + waves * i;
        if (row >= N) break;
        float acc[MB][4];
#pragma unroll
        for (int mb = 0; mb < MB; mb++)
#pragma unroll
            for (int l = 0; l < 4; l++) acc[mb][l] = 0.f;
        for (int step = 0; step < nsteps; step++) {
            int u = lane + 64 * step;
            const bool live = u < nunits;
            u = live ? u : nunits - 1;
            const Q8Pair pr = next;
            if (step + 1 < nsteps) fetch(next, row, step + 1);
            else fetch(next, row + waves, 0);  // past the end of W: the last row again, not used
            uint32_t d[17];
#pragma unroll
            for (int k = 0; k < 16; k++) d[k] = pr.v[k >> 2][k & 3];
            d[16] = pr.tail;
            uint32_t w0[8], w1[8];
#pragma unroll
            for (int k = 0; k < 8; k++) {
                w0[k] = __builtin_amdgcn_alignbyte(d[k + 1], d[k], 2);
                w1[k] = d[9 + k];
            }
            const float dw0 = live ? f16_bits_to_f32((uint16_t)(d[0] & 0xffffu)) : 0.f;
            const float dw1 = live ? f16_bits_to_f32((uint16_t)(d[8] >> 16)) : 0.f;
#pragma unroll
            for (int mb = 0; mb < MB; mb++) {
                const u32x4* xr = lds_q8 + mb * n16;
                const float* xd = (const float*)(xr + 2 * nbp);
                const u32x4 xa0 = xr[2 * u], xb0 = xr[nbp + 2 * u];
                const u32x4 xa1 = xr[2 * u + 1], xb1 = xr[nbp + 2 * u + 1];
                const float dx0 = live ? xd[2 * u] : 0.f, dx1 = live ? xd[2 * u + 1] : 0.f;
                q8_block(w0, xa0, xb0, dw0, dx0, acc[mb]);
                q8_block(w1, xa1, xb1, dw1, dx1, acc[mb]);
                __builtin_amdgcn_sched_barrier(0);  // one row of x at a time: its operands need not all be held at once
            }
        }
#pragma unroll
        for (int mb = 0; mb < MB; mb++) {
            float a0 = wave_sum(acc[mb][0]), a1 = wave_sum(acc[mb][1]), a2 = wave_sum(acc[mb][2]), a3 = wave_sum(acc[mb][3]);
            float s02 = a0 + a2, s13 = a1 + a3;
            if (lane == 0 && m0 + mb < M) y[(int64_t)(m0 + mb) * N + row] = s02 + s13;
        }
    }
}

// Rows of x converted beforehand (q8_convert_act), W 4-byte aligned with an even number of blocks a row.
bool qgemv_q8_0_rows_ok(const QGemvArgs& a) {
    return a.M >= 2 && a.act && !a.resid && (a.K / 32) % 2 == 0 && ((uintptr_t)a.W & 3) == 0 && 8 * q8_act_bytes(a.K) <= 64 * 1024;
}

hipError_t qgemv_q8_0_rows(const QGemvArgs& a, hipStream_t st) {
    const int waves = 8;
    const size_t ab = q8_act_bytes(a.K);
    const int mb = a.M > 4 ? 8 : a.M > 2 ? 4 : 2;
    // rows of W per wavefront: as many as still leave every compute unit four workgroups
    int rpw = 16;
    while (rpw > 1 && (a.N + waves * rpw - 1) / (waves * rpw) < 1024) rpw >>= 1;
    dim3 grid((unsigned)((a.N + waves * rpw - 1) / (waves * rpw)), (unsigned)((a.M + mb - 1) / mb));
#define Q8ROWS(MB)                                                                                                                      \
    hipLaunchKernelGGL((qgemv_q8_0_rows_kernel<MB>), grid, dim3(64 * waves), MB * ab, st, (const uint8_t*)a.W, (const uint8_t*)a.act, a.y, \
                       (int)a.M, (int)a.N, (int)(a.K / 32), (int64_t)ab, rpw)
    if (mb == 8) Q8ROWS(8); else if (mb == 4) Q8ROWS(4); else Q8ROWS(2);
#undef Q8ROWS
    return hipGetLastError();
}

bool q8_act_fits(int64_t K) { return q8_act_bytes(K) <= 64 * 1024; }

template <int R, bool ALIGNED>
static hipError_t launch_q8(const QGemvArgs& a, int waves, hipStream_t st) {
    int rows_per_wg = R * waves;
    dim3 grid((unsigned)((a.N + rows_per_wg - 1) / rows_per_wg), (unsigned)a.M);
    size_t act_bytes = q8_act_bytes(a.K);
    if (a.act)
        hipLaunchKernelGGL((qgemv_q8_0_kernel<R, ALIGNED, false>), grid, dim3(64 * waves), act_bytes, st, (const uint8_t*)a.W,
                           (const uint8_t*)a.act, a.y, a.resid, (int)a.N, (int)(a.K / 32), (int64_t)act_bytes, rows_per_wg);
    else  // float32 x, converted by every workgroup
        hipLaunchKernelGGL((qgemv_q8_0_kernel<R, ALIGNED, true>), grid, dim3(64 * waves), act_bytes, st, (const uint8_t*)a.W,
                           (const uint8_t*)a.x, a.y, a.resid, (int)a.N, (int)(a.K / 32), a.x_row_stride * 4, rows_per_wg);
    return hipGetLastError();
}

// tune: {rows, -, waves}. Needs q8_act_fits(K).
hipError_t qgemv_q8_0_act(const QGemvArgs& a, const int* tune, hipStream_t st) {
    int nb = (int)(a.K / 32);
    const bool aligned = nb % 2 == 0 && ((uintptr_t)a.W & 3) == 0;
    int R = a.N >= 4096 ? 2 : 1;
    if (tune[0] > 0) R = tune[0];
    int64_t tiles = (a.N + R - 1) / R;
    int waves = 8;
    while (waves > 1 && tiles / waves < 256) waves >>= 1;
    if (tune[2] > 0) waves = tune[2];
#define Q8CASE(RR)                                                           \
    if (R == RR) return aligned ? launch_q8<RR, true>(a, waves, st) : launch_q8<RR, false>(a, waves, st)
    Q8CASE(1); Q8CASE(2); Q8CASE(4);
#undef Q8CASE
    return aligned ? launch_q8<1, true>(a, waves, st) : launch_q8<1, false>(a, waves, st);
}

}  // namespace mimir
