// Products of two to eight rows of x with Q8_0 weights on the int8 matrix cores
// of gfx950, W read once for all the rows: the output projection of a batch's
// decoding step. The arithmetic is qdotQ8_0Go's (backend/cpu/qmatmul.go:125-139,
// see qgemv_q8_0.hip): per block four int32 lane sums (value p into lane
// p/4 mod 4), each times the product of the two scales added to a float32 lane
// of its own (a multiply, then an add), the lanes added (0+2)+(1+3).
//
// The four lane sums of eight rows of x are the 32 rows of one
// v_mfma_i32_32x32x32_i8: its first operand's row 8 l + m holds row m's int8
// block with everything but the values of lane sum l zeroed (of the 16 values a
// lane holds, that is dword l), its other operand 32 rows of W. A lane ends up
// with the four lane sums of its row of W for four rows of x. The integer sums
// are the CPU's; the float32 sums run over the blocks of a row in another order
// than the CPU's or the one-row kernel's (a wavefront takes every fourth run of
// eight blocks, the wavefronts' sums are added in order), a few units in the
// last place.
//
// W stays in ggml's layout. As in qgemv_q4_0_rows.hip, a wavefront loads a run
// of eight blocks of its 32 rows as aligned 16-byte pieces in row order (272
// bytes a row), passes them through a private LDS slab and reads its 16 int8 of
// each block back as dwords. x comes converted by q8_convert_act (its one-row
// form): a lane loads the one dword of it that its operand row keeps.
#include "device_util.h"
#include "kernels.h"

namespace mimir {

#pragma clang fp contract(off)

namespace {

typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));

constexpr int kWaves = 4;                      // wavefronts of a workgroup, among which the runs of K go round
constexpr int kRunBlocks = 8;
constexpr int kRunBytes = 34 * kRunBlocks;     // 272: seventeen pieces a row
constexpr int kPieces = kRunBytes / 16;
constexpr int kSlabStride = kRunBytes + 32;    // 304 bytes = 76 dwords: rows fall on eight banks, four to each
constexpr int kSlabBytes = 32 * kSlabStride;
constexpr int kLoads = (32 * kPieces + 63) / 64;  // 9: the last one half full

__global__ __launch_bounds__(64 * kWaves) void qgemv_q8_0_mfma_kernel(const uint8_t* __restrict__ W, const uint8_t* act, float* y, int M, int N,
                                                                       int nb, int64_t act_row_bytes) {
    extern __shared__ __align__(16) uint8_t smem[];  // a slab per wavefront; later the wavefronts' sums
    const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, lh = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // The grid runs over the groups of eight rows of x first: the workgroups that read the same 32 rows of W are handed
    // out together, so the rows come from HBM once and from the memory-side cache for the other groups.
    const int ngroups = (M + 7) >> 3, group = (int)(blockIdx.x % (unsigned)ngroups);
    const int n0 = (int)(blockIdx.x / (unsigned)ngroups) * 32, n = n0 + l32;
    const int nruns = nb / kRunBlocks, nbp = nb | 1;
    uint8_t* slab = smem + wave * kSlabBytes;
    act += (int64_t)8 * group * act_row_bytes;
    y += (int64_t)8 * group * N;
    M = M - 8 * group < 8 ? M - 8 * group : 8;

    // piece p = 64 i + lane of a run: row p / 17 of the 32, bytes 16 (p % 17).. of its 272
    uint32_t goff[kLoads], loff[kLoads];
#pragma unroll
    for (int i = 0; i < kLoads; i++) {
        int p = 64 * i + lane;
        p = p < 32 * kPieces ? p : 32 * kPieces - 1;  // the last load's upper lanes repeat the last piece
        const int r = p / kPieces, c = p - kPieces * r;
        const int row = n0 + r < N ? n0 + r : N - 1;
        goff[i] = (uint32_t)(row - n0) * (uint32_t)(nb * 34) + 16 * c;  // 32 rows of W within 4 GB (checked by the host)
        loff[i] = r * kSlabStride + 16 * c;
    }
    const uint8_t* wbase = W + (int64_t)n0 * nb * 34;
    // this lane's operand row of x: lane sum xl of row xm; it keeps dword xl of the 16 bytes a lane holds
    const int xl = (l32 >> 3), xm = l32 & 7;
    const uint8_t* xrow = act + (int64_t)(xm < M ? xm : M - 1) * act_row_bytes;
    const uint32_t* xq = (const uint32_t*)xrow + (int64_t)lh * nbp * 4 + xl;  // + 4 b: dword xl of half lh of block b
    const bool x_live = xm < M;

    struct Run {
        u32x4 w[kLoads];
        uint32_t x[kRunBlocks];  // the lane's dword of x per block
        float dx;                // one scale of x, see below
    };
    // The scales of x a lane needs are those of rows 4 lh .. 4 lh + 3 for every block of the run: 32 floats.
    // They are loaded once a run by the lanes (block l32 >> 2 of the run, row 4 lh + (l32 & 3)) and handed
    // round through LDS behind the slab.
    float* dxs = (float*)(smem + kWaves * kSlabBytes) + wave * 64;  // [half][block of the run][4 rows]
    auto fetch = [&](Run& f, int run) {
        const uint8_t* p = wbase + (int64_t)run * kRunBytes;
#pragma unroll
        for (int i = 0; i < kLoads; i++) f.w[i] = *(const u32x4*)(p + goff[i]);
#pragma unroll
        for (int b = 0; b < kRunBlocks; b++) f.x[b] = xq[(int64_t)(run * kRunBlocks + b) * 4];
        const int drow = 4 * lh + (l32 & 3);
        f.dx = ((const float*)(act + (int64_t)(drow < M ? drow : M - 1) * act_row_bytes + (int64_t)nbp * 32))[run * kRunBlocks + (l32 >> 2)];
    };

    float acc[4][4];  // [lane sum][row of x 4 lh + j]
#pragma unroll
    for (int l = 0; l < 4; l++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[l][j] = 0.f;

    Run cur, nxt;
    if (wave < nruns) fetch(cur, wave);
    const uint8_t* mine = slab + l32 * kSlabStride + 16 * lh;  // the lane's 16 int8 of block b: bytes 34 b + 2 + 16 lh
    const uint32_t keep0 = xl == 0 && x_live ? ~0u : 0u, keep1 = xl == 1 && x_live ? ~0u : 0u, keep2 = xl == 2 && x_live ? ~0u : 0u,
                   keep3 = xl == 3 && x_live ? ~0u : 0u;
    for (int run = wave; run < nruns; run += kWaves) {
        const int nrun = run + kWaves < nruns ? run + kWaves : run;
        fetch(nxt, nrun);
        // slab and scales are this wavefront's alone, and a wavefront's LDS operations complete in order
#pragma unroll
        for (int i = 0; i < kLoads - 1; i++) *(u32x4*)(slab + loff[i]) = cur.w[i];
        if (lane < 32 * kPieces - 64 * (kLoads - 1)) *(u32x4*)(slab + loff[kLoads - 1]) = cur.w[kLoads - 1];
        dxs[32 * lh + l32] = cur.dx;  // [half][block l32 >> 2][row l32 & 3]
#pragma unroll
        for (int b = 0; b < kRunBlocks; b++) {
            // bytes 34 b + 2 ..: on a dword for odd b, two bytes into one for even b
            i32x4 wop;
            float dw;
            if (b & 1) {
                const uint8_t* p = mine + 34 * b + 2;
#pragma unroll
                for (int i = 0; i < 4; i++) wop[i] = (int)*(const uint32_t*)(p + 4 * i);
                dw = f16_bits_to_f32((uint16_t)(*(const uint32_t*)(slab + l32 * kSlabStride + 34 * b - 2) >> 16));
            } else {
                const uint8_t* p = mine + 34 * b;
                uint32_t r[5];
#pragma unroll
                for (int i = 0; i < 5; i++) r[i] = *(const uint32_t*)(p + 4 * i);
#pragma unroll
                for (int i = 0; i < 4; i++) wop[i] = (int)__builtin_amdgcn_alignbit(r[i + 1], r[i], 16);
                dw = f16_bits_to_f32((uint16_t)(*(const uint32_t*)(slab + l32 * kSlabStride + 34 * b) & 0xffffu));
            }
            const uint32_t xv = cur.x[b];
            const i32x4 xop = {(int)(xv & keep0), (int)(xv & keep1), (int)(xv & keep2), (int)(xv & keep3)};
            i32x16 zero;
#pragma unroll
            for (int i = 0; i < 16; i++) zero[i] = 0;
            const i32x16 c = __builtin_amdgcn_mfma_i32_32x32x32_i8(xop, wop, zero, 0, 0, 0);
            const f32x4 dx = *(const f32x4*)(dxs + 32 * lh + 4 * b);
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const float dd = dw * dx[j];
#pragma unroll
                for (int l = 0; l < 4; l++) {
                    const float t = dd * (float)c[4 * l + j];
                    acc[l][j] = acc[l][j] + t;
                }
            }
        }
        cur = nxt;
    }

    __syncthreads();  // every wavefront is done with its slab
    f32x4* red = (f32x4*)smem;  // [wave][lane sum][lane]
#pragma unroll
    for (int l = 0; l < 4; l++) red[(wave * 4 + l) * 64 + lane] = f32x4{acc[l][0], acc[l][1], acc[l][2], acc[l][3]};
    __syncthreads();
    if (wave != 0) return;
    f32x4 a[4];
#pragma unroll
    for (int l = 0; l < 4; l++) {
        a[l] = red[l * 64 + lane];
#pragma unroll
        for (int w = 1; w < kWaves; w++) {
            const f32x4 t = red[(w * 4 + l) * 64 + lane];
#pragma unroll
            for (int j = 0; j < 4; j++) a[l][j] = a[l][j] + t[j];
        }
    }
    if (n < N) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int m = 4 * lh + j;
            if (m < M) {
                const float s02 = a[0][j] + a[2][j], s13 = a[1][j] + a[3][j];
                y[(int64_t)m * N + n] = s02 + s13;
            }
        }
    }
}

}  // namespace

// Rows of x converted beforehand (q8_convert_act), taken eight at a time; whole runs of eight blocks; W 16-byte aligned.
bool qgemv_q8_0_mfma_ok(const QGemvArgs& a) {
    const int64_t nb = a.K / 32;
    return a.M >= 2 && a.M <= 8 * 65535 && a.act && !a.resid && a.K % 256 == 0 && nb > 0 && ((uintptr_t)a.W & 15) == 0 && 32 * nb * 34 < ((int64_t)1 << 32) &&
           a.N > 0 && a.N <= (1ll << 30);
}

static std::atomic<int> g_q8_mfma{0};  // measurement aid: 1 = wherever the kernel takes the shape, 2 = never
void set_q8_mfma(int v) { g_q8_mfma = v; }

bool qgemv_q8_0_mfma_pays(const QGemvArgs& a) {
    if (g_q8_mfma == 2 || !qgemv_q8_0_mfma_ok(a)) return false;
    return g_q8_mfma == 1 || a.N * a.K >= ((int64_t)64 << 20);
}

hipError_t qgemv_q8_0_mfma(const QGemvArgs& a, hipStream_t st) {
    const size_t lds = (size_t)kWaves * kSlabBytes + kWaves * 64 * 4;
    const int64_t wgs = ((a.N + 31) / 32) * ((a.M + 7) / 8);
    if (wgs > 0x7fffffff) return hipErrorInvalidValue;
    hipLaunchKernelGGL(qgemv_q8_0_mfma_kernel, dim3((unsigned)wgs), dim3(64 * kWaves), lds, st, (const uint8_t*)a.W,
                       (const uint8_t*)a.act, a.y, (int)a.M, (int)a.N, (int)(a.K / 32), (int64_t)q8_act_bytes(a.K));
    return hipGetLastError();
}

}  // namespace mimir
