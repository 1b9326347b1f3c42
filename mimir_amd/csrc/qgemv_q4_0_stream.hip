// The fixed-point Q4_0 product of one row of x (or a few, each on its own) shaped for the
// whole chip: one workgroup per compute unit, up to four rows of the matrix in flight per
// wavefront from the moment x is staged, and the arithmetic done row by row as the rows arrive.
//
// The arithmetic is that of qgemv_q4_0_i4_kernel (qgemv_q4_0.hip; what the reference's CPU
// computes for a Q4_0 linear is the float32 product with the dequantized weights,
// io/mim/dtype.go:118-123 and backend/cpu/gemv.go:73-104): x as 24-bit fixed point per block of
// 32 in six planes of signed 4-bit digits, v_dot8_i32_i4 against the weights' nibbles, one
// float32 multiply-add per block and row. What differs is the shape of a launch:
//
//  - A lane keeps the digit planes and scales of its own pair of blocks in registers for the
//    whole launch (48 + 2 registers), read from LDS once, instead of re-reading them from LDS
//    for every row: the loop over rows touches no LDS.
//  - Rows longer than 64 pairs of blocks are cut into `nchunks` equal chunks of at most 64
//    pairs; wavefront w of a workgroup serves chunk w % nchunks of rows w / nchunks,
//    w / nchunks + waves / nchunks, ...; the chunks' sums of a row meet in LDS and are added
//    in the chunks' order.
//  - A workgroup owns `items_per_wg` consecutive items (an item is a row of W; for the rotation
//    tail two consecutive rows, a pair of features), and every wavefront takes exactly NIT of them (a wavefront whose last items fall
//    beyond the workgroup's range repeats its previous item and drops the result), so that
//    the whole schedule of a wavefront is straight-line code: DEPTH items requested before
//    anything else happens, the next requested as soon as a slot has been multiplied, and
//    every wait counts exactly the loads that may still be under way.
//  - The grid is one workgroup per compute unit where the rows divide that way.
#include <hip/hip_ext.h>

#include <mutex>

#include "device_util.h"
#include "kernels.h"
#include "q4_act.h"
#include "q4_job.h"
#include "rope_tail.h"

namespace mimir {

namespace {

constexpr size_t kStreamLdsMost = 64 * 1024;  // dynamic LDS of a launch

struct StreamShape {
    int items_per_wg;  // items a workgroup owns
    int nchunks;       // chunks a row is cut into (wavefronts per row)
    int ppc;           // pairs of blocks per chunk, at most 64
    int nrl;           // rows under way side by side in a workgroup: wavefronts / nchunks
};

// MODE and HEAD as in qgemv_q4_0_i4_kernel. NIT: items a wavefront takes; DEPTH: how many of them are
// requested ahead: up to four rows of W (sixteen wavefronts of 128 registers a lane). Measured and dropped:
// workgroups of eight wavefronts with 256 registers and a wavefront's whole share under way from its first
// instructions (x then arrives later, behind the other workgroups' weights); stores that bypass the cache.
// Where the instantiation that takes clock readings leaves them (null: nowhere).
__device__ long long* g_stream_stamps_dev = nullptr;

// STAMPS: the build that reads the clock at five points per workgroup (a measurement aid, launched only on request).
template <int MODE, int HEAD, int NIT, bool STAMPS = false>
__global__ __launch_bounds__(1024) void qgemv_q4_0_stream_kernel(Q4Job job, const uint8_t* __restrict__ act, float* __restrict__ y, int nb,
                                                                       int64_t act_row_bytes, StreamShape sh) {
    long long* const stamps = STAMPS ? g_stream_stamps_dev : nullptr;
    static_assert(MODE == kPlain || MODE == kRope, "the modes this launch shape is faster on");
    constexpr int RR = MODE == kRope ? 2 : 1;  // rows of W an item reads
    constexpr int kMaxRows = 4;
    constexpr int DEPTH = NIT < kMaxRows / RR ? NIT : kMaxRows / RR;
    extern __shared__ u32x4 lds_i4[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int m = blockIdx.y;
    const int N = job.total;
    const int nitems = MODE == kRope ? N >> 1 : N;
    float* yr = y + (int64_t)m * N;
    const int nbp = nb | 1;
    const int64_t row_bytes = (int64_t)nb * 18;
    const int npairs = nb >> 1;
    const int n16 = (int)(act_row_bytes >> 4);
    const int chunk = wave % sh.nchunks, rl = wave / sh.nchunks;
    const int item0 = blockIdx.x * sh.items_per_wg;
    const int item_end = item0 + sh.items_per_wg < nitems ? item0 + sh.items_per_wg : nitems;
    const int rope_pos = MODE == kRope ? *job.rope.pos : 0;
    long long t_entry = 0;
    if (STAMPS && tid == 0) t_entry = wall_clock64();

    // the lane's pair of blocks; lanes beyond the chunk (or the row) re-read its first pair and add nothing
    const int p_own = chunk * sh.ppc + lane;
    const bool live = lane < sh.ppc && p_own < npairs;
    const int p = live ? p_own : chunk * sh.ppc < npairs ? chunk * sh.ppc : 0;

    // The address of the weights behind row t of an item; items past the workgroup's range are clamped by the caller.
    auto row_ptr = [&](int item, int t) -> const uint8_t* {
        const int g = MODE == kRope ? 2 * item + t : item;
        if (MODE == kRope) {
            if (g >= job.n[0] + job.n[1]) return job.W[2] + (int64_t)(g - job.n[0] - job.n[1]) * row_bytes;
            if (g >= job.n[0]) return job.W[1] + (int64_t)(g - job.n[0]) * row_bytes;
        }
        return job.W[0] + (int64_t)g * row_bytes;
    };
    // Item i of this wavefront; one that falls beyond the range repeats the one before it (whose lines the caches hold).
    auto item_at = [&](int i) -> int {
        int it = item0 + rl + i * sh.nrl;
        while (it >= item_end && it - sh.nrl >= item0 + rl) it -= sh.nrl;
        return it < item_end ? it : item_end - 1;  // a wavefront with no item of its own at all: the workgroup's last
    };

    // ---- requests, in the order they are wanted back (loads return in order): what the head needs of x, the few
    // values the tails add (residuals, the rotation's cosines and sines), then the first DEPTH items of W ----
    __shared__ float norm_part[4];
    constexpr int kPark = 6;  // 16-byte pieces of converted x a thread carries from global memory to LDS
    const int nq = nb * 4;
    NormRow norm_row;
    float norm_ss = 0.f;
    f32x4 cv_lo = {0.f, 0.f, 0.f, 0.f}, cv_hi = {0.f, 0.f, 0.f, 0.f};
    u32x4 park[kPark];
    const u32x4* act_row = (const u32x4*)(act + (int64_t)m * act_row_bytes);
    if (HEAD == kHeadNorm) {  // the first four wavefronts hold the row between its sum of squares and its conversion
        if (tid < 256) norm_ss = norm_load(norm_row, job.norm_x + (int64_t)m * nb * 32, job.norm_w, nq, tid);
    } else if (HEAD == kHeadConvert) {
        // items t = tid, tid + blockDim, ...: the four items of a block sit in four consecutive lanes
        const float* xr = job.norm_x + (int64_t)m * job.x_row_stride;
        const int t = tid < nq ? tid : nq - 1;
        __builtin_memcpy(&cv_lo, xr + 32 * (t >> 2) + 4 * (t & 3), 16);
        __builtin_memcpy(&cv_hi, xr + 32 * (t >> 2) + 16 + 4 * (t & 3), 16);
    } else {
#pragma unroll
        for (int i = 0; i < kPark; i++) {
            const int idx = tid + i * (int)blockDim.x;
            if (idx < n16) park[i] = act_row[idx];
        }
    }
    float resid_v[NIT], rope_c[NIT], rope_s[NIT];
    bool rope_turns[NIT];
#pragma unroll
    for (int i = 0; i < NIT; i++) {
        resid_v[i] = 0.f;
        rope_c[i] = 1.f;
        rope_s[i] = 0.f;
        rope_turns[i] = false;
        if (MODE == kPlain && job.resid && sh.nchunks == 1) resid_v[i] = job.resid[(int64_t)m * N + item_at(i)];
        if (MODE == kRope && sh.nchunks == 1) rope_turns[i] = q4_rope_coeffs(job.rope, rope_pos, 2 * item_at(i), &rope_c[i], &rope_s[i]);
    }
    asm volatile("s_barrier" ::: "memory");
    // Only the first item of W is requested before x is staged: what the whole chip has under way then (some 4 MB) keeps
    // the memory busy without standing in the way of the x of workgroups that start a little later; the rest of the
    // first DEPTH follow once x is in LDS.
    constexpr int EARLY = 1;
    PairRegs tile[DEPTH][RR];
#pragma unroll
    for (int u = 0; u < EARLY; u++) {
        const int it = item_at(u);
#pragma unroll
        for (int t = 0; t < RR; t++) load_pair(tile[u][t], row_ptr(it, t), p);
    }
    __builtin_amdgcn_sched_barrier(0);  // the requests above stay ahead of the arithmetic on x below

    // ---- x into LDS in its fixed-point form ----
    if (HEAD == kHeadNorm) {
        if (tid < 256) {
            norm_ss = wave_sum(norm_ss);
            if (lane == 0) norm_part[wave] = norm_ss;
        }
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");  // LDS only: the weights' loads stay in flight
        if (tid < 256)
            norm_convert(norm_row, norm_part, nullptr, (u32x4*)lds_i4, (float*)(lds_i4 + kDigits * nbp), nbp, nq, tid, job.norm_inv_d, job.norm_eps);
    } else if (HEAD == kHeadConvert) {
        const float* xr = job.norm_x + (int64_t)m * job.x_row_stride;
        u32x4* plane = (u32x4*)lds_i4;
        float* xs = (float*)(lds_i4 + kDigits * nbp);
        if (tid < nq) {
            float lo[4] = {cv_lo[0], cv_lo[1], cv_lo[2], cv_lo[3]}, hi[4] = {cv_hi[0], cv_hi[1], cv_hi[2], cv_hi[3]};
            q4_convert_item(lo, hi, plane, xs, nbp, tid >> 2, tid & 3);
        }
        for (int t = tid + (int)blockDim.x; t < nq; t += (int)blockDim.x) {  // rows of x longer than the workgroup
            f32x4 vlo, vhi;
            __builtin_memcpy(&vlo, xr + 32 * (t >> 2) + 4 * (t & 3), 16);
            __builtin_memcpy(&vhi, xr + 32 * (t >> 2) + 16 + 4 * (t & 3), 16);
            float lo[4] = {vlo[0], vlo[1], vlo[2], vlo[3]}, hi[4] = {vhi[0], vhi[1], vhi[2], vhi[3]};
            q4_convert_item(lo, hi, plane, xs, nbp, t >> 2, t & 3);
        }
    } else {
#pragma unroll
        for (int i = 0; i < kPark; i++) {
            const int idx = tid + i * (int)blockDim.x;
            if (idx < n16) lds_i4[idx] = park[i];
        }
        for (int idx = tid + kPark * (int)blockDim.x; idx < n16; idx += (int)blockDim.x) lds_i4[idx] = act_row[idx];
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
#pragma unroll
    for (int u = EARLY; u < DEPTH; u++) {
        const int it = item_at(u);
#pragma unroll
        for (int t = 0; t < RR; t++) load_pair(tile[u][t], row_ptr(it, t), p);
    }
    long long t_staged = 0;
    if (STAMPS && tid == 0) t_staged = wall_clock64();
    __builtin_amdgcn_sched_barrier(0);  // the schedule below is written in program order: nothing moves across these points

    // the lane's digits and scales, for every row of the launch
    u32x4 d0[kDigits], d1[kDigits];
#pragma unroll
    for (int j = 0; j < kDigits; j++) {
        d0[j] = lds_i4[j * nbp + 2 * p];
        d1[j] = lds_i4[j * nbp + 2 * p + 1];
    }
    const float* xscale = (const float*)(lds_i4 + kDigits * nbp);
    const float s0 = xscale[2 * p], s1 = xscale[2 * p + 1];

    // ---- the rows: multiply a slot, request the item DEPTH ahead into it, reduce; nothing is stored to memory
    // before the last row's weights have been used (a store under way would stand in the way of counting loads) ----
    float* part = (float*)(lds_i4 + n16);  // [items_per_wg][RR][nchunks] sums of chunks
    float res[NIT][RR];
    long long t_first = 0;
#pragma unroll
    for (int i = 0; i < NIT; i++) {
        const int u = i % DEPTH;
#pragma unroll
        for (int t = 0; t < RR; t++) res[i][t] = pair_term(tile[u][t], d0, d1, s0, s1, live);
        if (i + DEPTH < NIT) {
            const int nx = item_at(i + DEPTH);
#pragma unroll
            for (int t = 0; t < RR; t++) load_pair(tile[u][t], row_ptr(nx, t), p);
        }
#pragma unroll
        for (int t = 0; t < RR; t++) res[i][t] = wave_sum(res[i][t]);
        if (STAMPS && tid == 0 && i == 0) t_first = wall_clock64();
        __builtin_amdgcn_sched_barrier(0);  // a row's multiply, refill and reduction stay together
    }
    long long t_last = 0;
    if (STAMPS && tid == 0) t_last = wall_clock64();

    // ---- the tails ----
#pragma unroll
    for (int i = 0; i < NIT; i++) {
        const int it = item_at(i);
        const bool mine = item0 + rl + i * sh.nrl < item_end;  // else a repeated item: nothing is stored
        if (!mine) continue;
        if (sh.nchunks > 1) {
            if (lane == 0) {
#pragma unroll
                for (int t = 0; t < RR; t++) part[((it - item0) * RR + t) * sh.nchunks + chunk] = res[i][t];
            }
            continue;
        }
        if (MODE == kRope) {
            if (lane == 0) q4_rope_store_with(job.rope, rope_pos, m, 2 * it, res[i][0], res[i][RR - 1], rope_turns[i], rope_c[i], rope_s[i], yr);
            continue;
        }
        if (lane == 0) {
            float s = res[i][0];
            if (job.resid) s = s + resid_v[i];
            yr[it] = s;
        }
    }

    if (sh.nchunks > 1) {  // the chunks' sums of each row, added in the chunks' order
        __syncthreads();
        for (int r = tid; r < item_end - item0; r += (int)blockDim.x) {
            float sum[RR];
#pragma unroll
            for (int t = 0; t < RR; t++) {
                float s = 0.f;
                for (int c = 0; c < sh.nchunks; c++) s = s + part[(r * RR + t) * sh.nchunks + c];
                sum[t] = s;
            }
            const int it = item0 + r;
            if (MODE == kRope) {
                q4_rope_store(job.rope, rope_pos, m, 2 * it, sum[0], sum[RR - 1], yr);
                continue;
            }
            float s = sum[0];
            if (job.resid) s = s + job.resid[(int64_t)m * N + it];
            yr[it] = s;
        }
    }
    if (STAMPS && stamps && tid == 0) {
        long long* s = stamps + 5 * ((int64_t)blockIdx.y * gridDim.x + blockIdx.x);
        s[0] = t_entry; s[1] = t_staged; s[2] = t_first; s[3] = t_last; s[4] = wall_clock64();
    }
}

int compute_units() {
    static std::once_flag once;
    static int n = 256;
    std::call_once(once, [] {
        int dev = 0, v = 0;
        if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) n = v;
    });
    return n;
}

std::atomic<int> g_stream_off{0};         // "q4_0.stream": 1 keeps every product off this kernel
std::atomic<int> g_stream_waves{0};       // "q4_0.stream_waves": wavefronts a workgroup, where the shape allows (0: by the cost below)
std::atomic<long long*> g_stamps{nullptr};  // where the next launches leave their workgroups' timestamps, if anywhere

struct StreamPlan {
    bool ok = false;
    int grid = 0, waves = 0, nit = 0;
    StreamShape sh{};
};

// How a product of `nitems` items over rows of `npairs` pairs of blocks is laid over the chip. min_waves: what the
// head needs.
StreamPlan plan_stream(int nitems, int npairs, int min_waves) {
    StreamPlan pl;
    if (nitems <= 0 || npairs <= 0) return pl;
    const int cus = compute_units();
    int nchunks = (npairs + 63) / 64;
    if (nchunks > 16) return pl;
    // equal chunks: K = 14336 is four chunks of 56 pairs rather than three of 64 and one of 32
    int ppc = (npairs + nchunks - 1) / nchunks;
    int ipw = (nitems + cus - 1) / cus;
    int grid = (nitems + ipw - 1) / ipw;
    // two workgroups to a compute unit at most (eight wavefronts each then: 128 registers a lane)
    const int max_waves = grid > cus ? 8 : 16;
    if (grid > 2 * cus) return pl;
    int best_cost = 1 << 30, best_waves = 0, best_nit = 0;
    const int forced = g_stream_waves.load(std::memory_order_relaxed);
    for (int w = nchunks; w <= max_waves; w += nchunks) {
        if (w < min_waves) continue;
        const int nrl = w / nchunks, nit = (ipw + nrl - 1) / nrl;
        if (nit > 8) continue;
        if (forced > 0 && w != forced) continue;
        const int cost = nit * ((w + 3) / 4);  // rows the busiest SIMD multiplies
        if (cost < best_cost || (cost == best_cost && w > best_waves)) best_cost = cost, best_waves = w, best_nit = nit;
    }
    if (best_waves == 0) return pl;
    pl.ok = true;
    pl.grid = grid;
    pl.waves = best_waves;
    pl.nit = best_nit;
    pl.sh = StreamShape{ipw, nchunks, ppc, best_waves / nchunks};
    return pl;
}

template <int MODE, int HEAD, int NIT>
hipError_t launch_stream(const Q4Job& job, const void* act, float* y, int64_t M, int64_t K, const StreamPlan& pl, hipStream_t st) {
    constexpr int RR = MODE == kRope ? 2 : 1;
    const size_t act_bytes = q4_0_act_bytes(K);
    const size_t part_bytes = pl.sh.nchunks > 1 ? (size_t)pl.sh.items_per_wg * RR * pl.sh.nchunks * 4 : 0;
    const size_t lds_bytes = act_bytes + part_bytes;
    if (lds_bytes > kStreamLdsMost) return hipErrorInvalidValue;  // the dispatch keeps such products off this kernel
    dim3 grid((unsigned)pl.grid, (unsigned)M);
    note_kernel("qgemv_q4_0_stream_kernel<%d, %d, %d>", MODE, HEAD, NIT);
    if constexpr (MODE == kPlain && HEAD == kHeadConvert) {
        if (g_stamps.load(std::memory_order_relaxed)) {  // clock readings asked for: the build that takes them
            hipLaunchKernelGGL((qgemv_q4_0_stream_kernel<MODE, HEAD, NIT, true>), grid, dim3(64 * pl.waves), lds_bytes, st, job, (const uint8_t*)act, y,
                               (int)(K / 32), (int64_t)act_bytes, pl.sh);
            return hipGetLastError();
        }
    }
    hipEvent_t t0, t1;
    if (next_timing_events(&t0, &t1))  // a measurement is on: this launch's own begin and end
        hipExtLaunchKernelGGL((qgemv_q4_0_stream_kernel<MODE, HEAD, NIT>), grid, dim3(64 * pl.waves), lds_bytes, st, t0, t1, 0, job, (const uint8_t*)act, y,
                              (int)(K / 32), (int64_t)act_bytes, pl.sh);
    else
        hipLaunchKernelGGL((qgemv_q4_0_stream_kernel<MODE, HEAD, NIT>), grid, dim3(64 * pl.waves), lds_bytes, st, job, (const uint8_t*)act, y, (int)(K / 32),
                           (int64_t)act_bytes, pl.sh);
    return hipGetLastError();
}

template <int MODE, int HEAD>
hipError_t launch_stream_nit(const Q4Job& job, const void* act, float* y, int64_t M, int64_t K, const StreamPlan& pl, hipStream_t st) {
    switch (pl.nit) {
    case 1: return launch_stream<MODE, HEAD, 1>(job, act, y, M, K, pl, st);
    case 2: return launch_stream<MODE, HEAD, 2>(job, act, y, M, K, pl, st);
    case 3: return launch_stream<MODE, HEAD, 3>(job, act, y, M, K, pl, st);
    case 4: return launch_stream<MODE, HEAD, 4>(job, act, y, M, K, pl, st);
    case 5: return launch_stream<MODE, HEAD, 5>(job, act, y, M, K, pl, st);
    case 6: return launch_stream<MODE, HEAD, 6>(job, act, y, M, K, pl, st);
    case 7: return launch_stream<MODE, HEAD, 7>(job, act, y, M, K, pl, st);
    case 8: return launch_stream<MODE, HEAD, 8>(job, act, y, M, K, pl, st);
    }
    return hipErrorInvalidValue;
}

}  // namespace

void set_q4_stream_off(int v) { g_stream_off = v; }
void set_q4_stream_waves(int v) { g_stream_waves = v; }
hipError_t set_q4_stream_stamps(long long* p) {  // synchronous
    g_stamps = p;
    return hipMemcpyToSymbol(HIP_SYMBOL(g_stream_stamps_dev), &p, sizeof(p));
}

// Whether this kernel takes the product (then *err is the launch's status). mode: a Q4Mode; head: kHeadAct, kHeadNorm or
// kHeadConvert, as the job's fields say. Few rows of x only: each is a pass over W of its own.
bool q4_0_stream_dispatch(int mode, const Q4Job& job, const void* act, float* y, int64_t M, int64_t K, hipStream_t st, hipError_t* err) {
    if (g_stream_off.load(std::memory_order_relaxed) == 1 || M < 1 || M > 4 || K % 64 != 0) return false;
    const int npairs = (int)(K / 64);
    const int head = job.norm_w ? kHeadNorm : job.norm_x ? kHeadConvert : kHeadAct;
    const int nitems = mode == kRope ? job.total / 2 : job.total;
    if (mode == kRope && (job.total % 2 != 0 || job.n[0] % 2 != 0 || job.n[1] % 2 != 0)) return false;
    if (mode != kPlain && mode != kRope) return false;
    if (head == kHeadNorm && !q4_0_norm_head_ok(K)) return false;
    const StreamPlan pl = plan_stream(nitems, npairs, head == kHeadNorm ? 4 : 1);
    if (!pl.ok) return false;
    // x and the chunks' sums within what a launch gets of LDS without asking for more (rows of x up to some 20 000
    // elements): longer rows and very tall matrices stay on the finer-grained launch
    const size_t rr = mode == kRope ? 2 : 1;
    if (q4_0_act_bytes(K) + (pl.sh.nchunks > 1 ? (size_t)pl.sh.items_per_wg * rr * pl.sh.nchunks * 4 : 0) > kStreamLdsMost) return false;
#define STREAM_CASE(MM, HH) \
    if (mode == MM && head == HH) { *err = launch_stream_nit<MM, HH>(job, act, y, M, K, pl, st); return true; }
    // The products this shape was measured faster on than the finer-grained launch: x in float32 converted here, and the
    // q|k|v product with its rotation. The others (SwiGLU, the residual's products on prepared activations, several
    // matrices in one launch) measured a few per cent slower and stay where they were.
    STREAM_CASE(kPlain, kHeadConvert)
    STREAM_CASE(kRope, kHeadAct) STREAM_CASE(kRope, kHeadNorm)
#undef STREAM_CASE
    return false;
}

}  // namespace mimir
