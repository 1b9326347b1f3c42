// The fixed-point Q4_0 product of one row of x with the weights brought into LDS by wavefronts that do
// nothing else: one workgroup per compute unit, whose first wavefronts convert x and multiply, while its
// last ones ("feeders") request the unit's whole share of W with loads that write LDS directly
// (global_load_lds_dwordx4) and say, through a counter in LDS, how many rows have arrived.
//
// Why the roles are split: a wavefront that requests more than the unit's memory pipeline holds is
// stalled at the request itself until earlier data has come back, not at the wait for its data. With
// every wavefront requesting its own rows (measured: the first wavefront of a workgroup needs 3.5 us to
// get 21 requests accepted while x, requested before them, has long arrived) nobody converts x or
// multiplies in the meantime. A feeder stalls there for the whole launch and that costs nothing.
//
// The arithmetic is that of qgemv_q4_0_i4_kernel and qgemv_q4_0_stream_kernel (what the reference's CPU
// computes for a Q4_0 linear is the float32 product with the dequantized weights, io/mim/dtype.go:118-123
// and backend/cpu/gemv.go:73-104): x as 24-bit fixed point per block of 32 in six planes of signed 4-bit
// digits, v_dot8_i32_i4 against the weights' nibbles, one float32 multiply-add per block and row, the
// same sums in the same order, so the three kernels give the same bits.
//
// How a launch is laid out:
//  - A workgroup owns `items_per_wg` consecutive items (an item is a row of W; with the rotation tail two
//    consecutive rows, a pair of features). Rows longer than 64 pairs of blocks are cut into `nchunks`
//    equal chunks; multiplying wavefront w serves chunk w % nchunks of items w / nchunks,
//    w / nchunks + nrl, ..., exactly NIT of them (one that falls beyond the range repeats an earlier one
//    and drops the result), each in a slot of LDS of its own.
//  - The slots are filled in the order q = i * NC + w (item i of wavefront w): feeder l of NL takes
//    q = l, l + NL, ..., P loads of 1 KB a row (64 lanes x 16 bytes; the last one with the lanes beyond
//    the chunk's end switched off), keeps at most `window` of its rows under way, and after each
//    request waits for the row `window` back and publishes the count of its rows that are complete.
//    Only a feeder's own count of loads under way says that a row is in LDS, hence the hand-written
//    loads and waits: the compiler would wait for every load before any read of LDS.
//  - The multiplying wavefronts request x (and the residuals) before the feeders start, one barrier of
//    the whole workgroup apart, so that x is ahead of all the weights in the unit's queue; from there
//    on they meet among themselves through counters in LDS and never wait for a feeder at a barrier.
#include <hip/hip_ext.h>

#include <mutex>

#include "device_util.h"
#include "kernels.h"
#include "q4_act.h"
#include "q4_job.h"
#include "rope_tail.h"

namespace mimir {

namespace {

constexpr size_t kDmaLdsMost = 160 * 1024 - 512;  // dynamic LDS of a launch: a compute unit's 160 KB less what the kernel declares itself
constexpr int kCtrlBytes = 64;                    // the counters at the front of the dynamic LDS

struct DmaShape {
    int items_per_wg;  // items a workgroup owns
    int nchunks;       // chunks a row is cut into (wavefronts per row)
    int ppc;           // pairs of blocks per chunk, at most 64, a multiple of 4
    int nrl;           // items under way side by side in a workgroup: multiplying wavefronts / nchunks
    int slots_off;     // where the slots start in LDS, in bytes (after the counters, x and the chunks' sums)
    int nc, nl;        // multiplying wavefronts, feeders
    int window;        // rows a feeder keeps under way
};

// Where the per-workgroup clock readings of the instantiation that takes them go (null: nowhere).
__device__ long long* g_dma_stamps_dev = nullptr;

// ---- loads and waits written out: the compiler neither sees nor counts them ----
// 16 bytes a lane from global memory into LDS: lane l's piece lands at lds_base + OFF + 16 l, read from g + OFF.
template <int OFF>
__device__ __forceinline__ void dma16(const void* g, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off offset:%2" ::"s"(lds_base), "v"(g), "n"(OFF) : "memory");
}
__device__ __forceinline__ void gload16(u32x4& v, const void* g) { asm volatile("global_load_dwordx4 %0, %1, off" : "=&v"(v) : "v"(g) : "memory"); }
__device__ __forceinline__ void gload4(float& v, const void* g) { asm volatile("global_load_dword %0, %1, off" : "=&v"(v) : "v"(g) : "memory"); }
// At most N of the wavefront's loads are still under way (they complete in the order they were issued).
template <int N>
__device__ __forceinline__ void vm_wait() {
    static_assert(N >= 0 && N < 64, "the counter has six bits");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
__device__ __forceinline__ void vm_wait_n(int n) {  // n uniform over the wavefront
    switch (n) {
#define VMW(i) case i: vm_wait<i>(); break;
#define VMW8(b) VMW(b) VMW(b + 1) VMW(b + 2) VMW(b + 3) VMW(b + 4) VMW(b + 5) VMW(b + 6) VMW(b + 7)
    VMW8(0) VMW8(8) VMW8(16) VMW8(24) VMW8(32) VMW8(40) VMW8(48) VMW8(56)
#undef VMW8
#undef VMW
    default: vm_wait<0>(); break;
    }
}
// A register that a hand-written load fills may be read only behind the wait for it: this pins every use below it.
__device__ __forceinline__ void settled(u32x4& v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ void settled(float& v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
__device__ __forceinline__ f32x4 as_f32x4(u32x4 v) { return __builtin_bit_cast(f32x4, v); }

// Counters in LDS. A feeder's count of complete rows, read by the wavefront that multiplies them; and the meeting
// points of the multiplying wavefronts (a barrier instruction would wait for the feeders too). The LDS serves a
// wavefront's instructions in order, so a counter written after data (or read before it) needs no fence, only the
// compiler kept from reordering; a release or acquire here would have the compiler wait for every load under way.
__device__ __forceinline__ void publish(uint32_t* c, uint32_t v) {
    asm volatile("" ::: "memory");
    __hip_atomic_store(c, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}
__device__ __forceinline__ void await_above(const uint32_t* c, uint32_t v) {  // until *c > v
    while (__hip_atomic_load(c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) <= v) __builtin_amdgcn_s_sleep(1);
    asm volatile("" ::: "memory");
}
// Every one of the nc multiplying wavefronts calls this once per counter; returns when all have.
__device__ __forceinline__ void meet(uint32_t* c, int nc, int lane) {
    asm volatile("" ::: "memory");
    if (lane == 0) __hip_atomic_fetch_add(c, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    await_above(c, (uint32_t)nc - 1);
}

// MODE: kPlain or kRope (q4_job.h). HEAD: where x comes from (kHeadAct converted beforehand, kHeadNorm RMSNorm of
// job.norm_x as the first phase, kHeadConvert job.norm_x itself). NIT: items a multiplying wavefront takes. P: loads of
// 1 KB that cover a row's chunk. STAMPS: the instantiation that leaves clock readings (a measurement aid).
template <int MODE, int HEAD, int NIT, int P, bool STAMPS>
__global__ __launch_bounds__(1024) void qgemv_q4_0_dma_kernel(Q4Job job, const uint8_t* __restrict__ act, float* __restrict__ y, int nb,
                                                                    int64_t act_row_bytes, DmaShape sh) {
    static_assert(MODE == kPlain || MODE == kRope, "the modes this launch shape serves");
    constexpr int RR = MODE == kRope ? 2 : 1;  // rows of W an item reads
    constexpr int NTAIL = MODE == kRope ? 2 * NIT : NIT + 1;  // values the tail adds, a load each
    constexpr int kPark = 4;   // kHeadAct: 16-byte pieces of converted x a thread carries from global memory to LDS
    extern __shared__ u32x4 lds_all[];
    __shared__ float norm_part[4];
    uint32_t* ctrl = (uint32_t*)lds_all;           // [0..3] feeders' counts, [8], [9], [10] meeting points
    u32x4* lds_i4 = lds_all + kCtrlBytes / 16;     // x in its fixed-point form, then the chunks' sums, then the slots
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int N = job.total;
    const int nitems = MODE == kRope ? N >> 1 : N;
    const int nbp = nb | 1;
    const int64_t row_bytes = (int64_t)nb * 18;
    const int n16 = (int)(act_row_bytes >> 4);
    const int nq = nb * 4;
    const int NC = sh.nc, NL = sh.nl;
    const int item0 = blockIdx.x * sh.items_per_wg;
    const int item_end = item0 + sh.items_per_wg < nitems ? item0 + sh.items_per_wg : nitems;
    const int chunk_bytes = sh.ppc * 36;
    const uint32_t slots_lds = (uint32_t)(uintptr_t)lds_all + (uint32_t)sh.slots_off;

    auto row_ptr = [&](int item, int t) -> const uint8_t* {
        const int g = MODE == kRope ? 2 * item + t : item;
        if (MODE == kRope) {
            if (g >= job.n[0] + job.n[1]) return job.W[2] + (int64_t)(g - job.n[0] - job.n[1]) * row_bytes;
            if (g >= job.n[0]) return job.W[1] + (int64_t)(g - job.n[0]) * row_bytes;
        }
        return job.W[0] + (int64_t)g * row_bytes;
    };
    // Item i of the multiplying wavefront whose items start at item0 + rl; one that falls beyond the range repeats the one before it.
    auto item_of = [&](int rl, int i) -> int {
        int it = item0 + rl + i * sh.nrl;
        while (it >= item_end && it - sh.nrl >= item0 + rl) it -= sh.nrl;
        return it < item_end ? it : item_end - 1;
    };

    if (tid < kCtrlBytes / 4) ctrl[tid] = 0;

    if (wave >= NC) {
        // ================= a feeder =================
        lds_barrier();  // the counters are zero and x is requested
        const int l = wave - NC;
        const int total = NIT * NC;                 // slots of the workgroup
        const int mine = (total - l + NL - 1) / NL;  // of which this feeder fills
        const int window = sh.window < mine ? sh.window : mine;
        const bool in_last = 1024 * (P - 1) + 16 * lane < chunk_bytes;  // the last piece: lanes within the chunk
        for (int s = 0; s < mine; s++) {
            const int q = l + s * NL, w = q % NC, i = q / NC;
            const int it = item_of(w / sh.nchunks, i);
            const int64_t lane_off = (int64_t)(w % sh.nchunks) * chunk_bytes + 16 * lane;
#pragma unroll
            for (int t = 0; t < RR; t++) {
                const uint8_t* src = row_ptr(it, t) + lane_off;
                const uint32_t dst = slots_lds + (uint32_t)(((w * NIT + i) * RR + t) * chunk_bytes);
                if (P > 1) dma16<0>(src, dst);
                if (P > 2) dma16<1024>(src, dst);
                if (in_last) dma16<1024 * (P - 1)>(src, dst);
            }
            if (s + 1 >= window) {  // slot s + 1 - window is complete once at most window - 1 younger ones are under way
                vm_wait_n((window - 1) * RR * P);
                if (lane == 0) publish(&ctrl[l], (uint32_t)(s + 2 - window));
            }
        }
        for (int s = mine - window + 1; s < mine; s++) {  // the rest, as they arrive
            vm_wait_n((mine - 1 - s) * RR * P);
            if (lane == 0) publish(&ctrl[l], (uint32_t)(s + 1));
        }
        return;
    }

    // ================= a multiplying wavefront =================
    const int chunk = wave % sh.nchunks, rl = wave / sh.nchunks;
    const int rope_pos = MODE == kRope ? *job.rope.pos : 0;
    long long t_entry = 0, t_staged = 0, t_first = 0, t_last = 0;
    if (STAMPS && tid == 0) t_entry = wall_clock64();

    // ---- 1. what the head needs of x, and the residuals: every index clamped, every load unconditional ----
    NormRow norm_row;
    u32x4 cv_lo, cv_hi, park[kPark];
    float tail_v[NTAIL];
    if (HEAD == kHeadNorm) {
        if (wave < 4) {  // the first four wavefronts hold the row between its sum of squares and its conversion
#pragma unroll
            for (int i = 0; i < kNormItems; i++) {
                int t = tid + i * 256;
                t = t < nq ? t : nq - 1;
                const int b = t >> 2, q = t & 3;
                u32x4 a, c, d, e;
                gload16(a, job.norm_x + 32 * b + 4 * q);
                gload16(c, job.norm_x + 32 * b + 16 + 4 * q);
                gload16(d, job.norm_w + 32 * b + 4 * q);
                gload16(e, job.norm_w + 32 * b + 16 + 4 * q);
                norm_row.lo[i] = as_f32x4(a); norm_row.hi[i] = as_f32x4(c); norm_row.wl[i] = as_f32x4(d); norm_row.wh[i] = as_f32x4(e);
            }
        }
    } else if (HEAD == kHeadConvert) {
        const int t = tid < nq ? tid : nq - 1;  // item t: block t / 4, dword t % 4; nq <= 64 NC (the host checks)
        gload16(cv_lo, job.norm_x + 32 * (t >> 2) + 4 * (t & 3));
        gload16(cv_hi, job.norm_x + 32 * (t >> 2) + 16 + 4 * (t & 3));
    } else {
        const u32x4* act_row = (const u32x4*)act;
#pragma unroll
        for (int i = 0; i < kPark; i++) {
            int idx = tid + i * 64 * NC;
            idx = idx < n16 ? idx : n16 - 1;
            gload16(park[i], act_row + idx);
        }
    }
    if (MODE == kPlain) {
        // a product without a residual reads its own weights' first bytes instead and ignores them
        const float* rs = job.resid ? job.resid : (const float*)job.W[0];
#pragma unroll
        for (int i = 0; i < NIT; i++) gload4(tail_v[i], rs + (job.resid ? item_of(rl, i) : 0));
        const int r = item0 + tid < item_end ? item0 + tid : item_end - 1;  // the row whose chunks this thread adds at the end
        gload4(tail_v[NIT], rs + (job.resid ? r : 0));
    }
    __builtin_amdgcn_sched_barrier(0);
    lds_barrier();  // every request for x is out before the first for W, and the counters are zero
    if (MODE == kRope) {
        // the rotation's cosine and sine wait for the position; they queue behind the weights and are there at the end
        const int half = job.rope.rope_dim >> 1;
#pragma unroll
        for (int i = 0; i < NIT; i++) {
            const int row = 2 * item_of(rl, i), head = row / job.rope.dim, f = row - head * job.rope.dim;
            const bool turns = head < job.rope.H + job.rope.HK && f < job.rope.rope_dim;
            const int64_t at = turns ? (int64_t)rope_pos * half + (f >> 1) : 0;
            gload4(tail_v[2 * i], job.rope.cosv + at);
            gload4(tail_v[2 * i + 1], job.rope.sinv + at);
        }
    }
    __builtin_amdgcn_sched_barrier(0);

    // ---- 2. x into LDS in its fixed-point form, while the weights travel ----
    vm_wait<MODE == kRope ? NTAIL : 0>();
    u32x4* plane = lds_i4;
    float* xs = (float*)(lds_i4 + kDigits * nbp);
    if (HEAD == kHeadNorm) {
        if (wave < 4) {
            float ss = 0.f;
#pragma unroll
            for (int i = 0; i < kNormItems; i++) {
                u32x4 a = __builtin_bit_cast(u32x4, norm_row.lo[i]), c = __builtin_bit_cast(u32x4, norm_row.hi[i]);
                u32x4 d = __builtin_bit_cast(u32x4, norm_row.wl[i]), e = __builtin_bit_cast(u32x4, norm_row.wh[i]);
                settled(a); settled(c); settled(d); settled(e);
                norm_row.lo[i] = as_f32x4(a); norm_row.hi[i] = as_f32x4(c); norm_row.wl[i] = as_f32x4(d); norm_row.wh[i] = as_f32x4(e);
                if (tid + i * 256 < nq) {  // norm_load's sum, term for term
#pragma unroll
                    for (int k = 0; k < 4; k++) {
                        float sa = norm_row.lo[i][k] * norm_row.lo[i][k], sc = norm_row.hi[i][k] * norm_row.hi[i][k];
                        ss = ss + sa;
                        ss = ss + sc;
                    }
                }
            }
            ss = wave_sum(ss);
            if (lane == 0) norm_part[wave] = ss;
        }
        meet(&ctrl[8], NC, lane);
        if (wave < 4) norm_convert(norm_row, norm_part, nullptr, plane, xs, nbp, nq, tid, job.norm_inv_d, job.norm_eps);
    } else if (HEAD == kHeadConvert) {
        settled(cv_lo); settled(cv_hi);
        if (tid < nq) {
            const f32x4 lo4 = as_f32x4(cv_lo), hi4 = as_f32x4(cv_hi);
            float lo[4] = {lo4[0], lo4[1], lo4[2], lo4[3]}, hi[4] = {hi4[0], hi4[1], hi4[2], hi4[3]};
            q4_convert_item(lo, hi, plane, xs, nbp, tid >> 2, tid & 3);
        }
    } else {
#pragma unroll
        for (int i = 0; i < kPark; i++) {
            settled(park[i]);
            const int idx = tid + i * 64 * NC;
            if (idx < n16) lds_i4[idx] = park[i];
        }
    }
    meet(&ctrl[9], NC, lane);
    if (STAMPS && tid == 0) t_staged = wall_clock64();

    // the lane's pair of blocks: its digits and scales, for every row of the launch
    const bool live = lane < sh.ppc;
    const int p = chunk * sh.ppc + (live ? lane : 0);
    u32x4 d0[kDigits], d1[kDigits];
#pragma unroll
    for (int j = 0; j < kDigits; j++) {
        d0[j] = lds_i4[j * nbp + 2 * p];
        d1[j] = lds_i4[j * nbp + 2 * p + 1];
    }
    const float s0 = xs[2 * p], s1 = xs[2 * p + 1];

    // ---- 3. the rows, as their feeder reports them ----
    const uint8_t* my_slots = (const uint8_t*)lds_all + sh.slots_off + (size_t)wave * (NIT * RR) * chunk_bytes + 36 * (live ? lane : 0);
    float res[NIT][RR];
#pragma unroll
    for (int i = 0; i < NIT; i++) {
        const int q = i * NC + wave;
        await_above(&ctrl[q % NL], (uint32_t)(q / NL));
#pragma unroll
        for (int t = 0; t < RR; t++) {
            const uint32_t* s = (const uint32_t*)(my_slots + (i * RR + t) * chunk_bytes);
            PairRegs tile;
            tile.a = u32x4{s[0], s[1], s[2], s[3]};
            tile.b = u32x4{s[4], s[5], s[6], s[7]};
            tile.c = s[8];
            res[i][t] = pair_term(tile, d0, d1, s0, s1, live);
        }
#pragma unroll
        for (int t = 0; t < RR; t++) res[i][t] = wave_sum(res[i][t]);
        if (STAMPS && tid == 0 && i == 0) t_first = wall_clock64();
    }
    if (STAMPS && tid == 0) t_last = wall_clock64();
    vm_wait<0>();
#pragma unroll
    for (int i = 0; i < NTAIL; i++) settled(tail_v[i]);

    // ---- 4. the tails ----
    float* part = (float*)(lds_i4 + n16);  // [items_per_wg][RR][nchunks] sums of chunks
#pragma unroll
    for (int i = 0; i < NIT; i++) {
        const int it = item_of(rl, i);
        const bool own = item0 + rl + i * sh.nrl < item_end;  // else a repeated item: nothing is stored
        if (!own) continue;
        if (sh.nchunks > 1) {
            if (lane == 0) {
#pragma unroll
                for (int t = 0; t < RR; t++) part[((it - item0) * RR + t) * sh.nchunks + chunk] = res[i][t];
            }
            continue;
        }
        if (MODE == kRope) {
            if (lane == 0) {
                const int row = 2 * it, head = row / job.rope.dim, f = row - head * job.rope.dim;
                const bool turns = head < job.rope.H + job.rope.HK && f < job.rope.rope_dim;
                q4_rope_store_with(job.rope, rope_pos, 0, row, res[i][0], res[i][RR - 1], turns, tail_v[(2 * i) % NTAIL], tail_v[(2 * i + 1) % NTAIL], y);
            }
            continue;
        }
        if (lane == 0) {
            float s = res[i][0];
            if (job.resid) s = s + tail_v[i];
            y[it] = s;
        }
    }
    if (sh.nchunks > 1) {  // the chunks' sums of each row, added in the chunks' order
        meet(&ctrl[10], NC, lane);
        for (int r = tid; r < item_end - item0; r += 64 * NC) {
            float sum[RR];
#pragma unroll
            for (int t = 0; t < RR; t++) {
                float s = 0.f;
                for (int c = 0; c < sh.nchunks; c++) s = s + part[(r * RR + t) * sh.nchunks + c];
                sum[t] = s;
            }
            const int it = item0 + r;
            if (MODE == kRope) {
                q4_rope_store(job.rope, rope_pos, 0, 2 * it, sum[0], sum[RR - 1], y);
                continue;
            }
            float s = sum[0];
            if (job.resid) s = s + (r == tid ? tail_v[NTAIL - 1] : job.resid[it]);
            y[it] = s;
        }
    }
    if (STAMPS && tid == 0 && g_dma_stamps_dev) {
        long long* s = g_dma_stamps_dev + 5 * (int64_t)blockIdx.x;
        s[0] = t_entry; s[1] = t_staged; s[2] = t_first; s[3] = t_last; s[4] = wall_clock64();
    }
}

int dma_compute_units() {
    static std::once_flag once;
    static int n = 256;
    std::call_once(once, [] {
        int dev = 0, v = 0;
        if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) n = v;
    });
    return n;
}

std::atomic<int> g_dma_off{1};      // off unless "q4_0.stream" = 3: the kernel is the slower of the two whole-chip kernels (measured)
std::atomic<int> g_dma_feeders{8};  // "q4_0.feeders"
std::atomic<int> g_dma_window{3};  // "q4_0.feed_window": rows a feeder keeps under way
std::atomic<long long*> g_dma_stamps{nullptr};

struct DmaPlan {
    bool ok = false;
    int grid = 0, nit = 0, pieces = 0;
    size_t lds = 0;
    DmaShape sh{};
};

// How a product of `nitems` items (of rr rows each) over rows of `npairs` pairs of blocks is laid over the chip.
// min_waves: multiplying wavefronts the head needs; act_bytes: the converted row of x.
DmaPlan plan_dma(int nitems, int rr, int npairs, int min_waves, size_t act_bytes) {
    DmaPlan pl;
    if (nitems <= 0 || npairs <= 0) return pl;
    const int cus = dma_compute_units();
    const int nchunks = (npairs + 63) / 64;
    if (nchunks > 8 || npairs % nchunks != 0) return pl;  // equal chunks only
    const int ppc = npairs / nchunks;
    if (ppc % 4 != 0) return pl;  // a chunk is whole 16-byte pieces, 16-byte aligned within its row
    const int chunk_bytes = ppc * 36;
    const int pieces = (chunk_bytes + 1023) / 1024;
    if (pieces < 2) return pl;  // rows under 1 KB: not instantiated, the other kernels take them
    const int ipw = (nitems + cus - 1) / cus;
    const int grid = (nitems + ipw - 1) / ipw;
    if (grid > cus) return pl;  // one workgroup to a compute unit: LDS is the unit's
    int nl = g_dma_feeders.load(std::memory_order_relaxed);
    nl = nl < 1 ? 1 : nl > 8 ? 8 : nl;
    int window = g_dma_window.load(std::memory_order_relaxed);
    window = window < 1 ? 1 : window;
    while (window > 1 && (window - 1) * rr * pieces > 60) window--;  // what a wavefront's counter of loads can name
    const size_t part = nchunks > 1 ? (size_t)ipw * rr * nchunks * 4 : 0;
    const size_t slots_off = (kCtrlBytes + act_bytes + part + 15) / 16 * 16;
    int best_cost = 1 << 30, best_waves = 0, best_nit = 0;
    size_t best_lds = 0;
    for (int w = nchunks; w + nl <= 16; w += nchunks) {
        if (w < min_waves) continue;
        const int nrl = w / nchunks, nit = (ipw + nrl - 1) / nrl;
        if (nit > 8) continue;
        const size_t lds = slots_off + (size_t)w * nit * rr * chunk_bytes;
        if (lds > kDmaLdsMost) continue;
        const int cost = nit * ((w + 3) / 4);  // rows the busiest SIMD multiplies
        if (cost < best_cost || (cost == best_cost && w > best_waves)) best_cost = cost, best_waves = w, best_nit = nit, best_lds = lds;
    }
    if (best_waves == 0) return pl;
    pl.ok = true;
    pl.grid = grid;
    pl.nit = best_nit;
    pl.pieces = pieces;
    pl.lds = best_lds;
    pl.sh = DmaShape{ipw, nchunks, ppc, best_waves / nchunks, (int)slots_off, best_waves, nl, window};
    return pl;
}

// More dynamic LDS than a launch gets by default has to be asked for once per kernel.
template <int MODE, int HEAD, int NIT, int P, bool STAMPS>
hipError_t dma_kernel_ready() {
    static std::once_flag once;
    static hipError_t status = hipSuccess;
    std::call_once(once, [] {
        status = hipFuncSetAttribute((const void*)qgemv_q4_0_dma_kernel<MODE, HEAD, NIT, P, STAMPS>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kDmaLdsMost);
    });
    return status;
}

template <int MODE, int HEAD, int NIT, int P>
hipError_t launch_dma(const Q4Job& job, const void* act, float* y, int64_t K, const DmaPlan& pl, hipStream_t st) {
    const size_t act_bytes = q4_0_act_bytes(K);
    dim3 grid((unsigned)pl.grid), block((unsigned)(64 * (pl.sh.nc + pl.sh.nl)));
    note_kernel("qgemv_q4_0_dma_kernel<%d, %d, %d, %d>", MODE, HEAD, NIT, P);
    if constexpr (MODE == kPlain && HEAD == kHeadConvert) {
        if (g_dma_stamps.load(std::memory_order_relaxed)) {
            if (hipError_t e = dma_kernel_ready<MODE, HEAD, NIT, P, true>()) return e;
            hipLaunchKernelGGL((qgemv_q4_0_dma_kernel<MODE, HEAD, NIT, P, true>), grid, block, pl.lds, st, job, (const uint8_t*)act, y, (int)(K / 32),
                               (int64_t)act_bytes, pl.sh);
            return hipGetLastError();
        }
    }
    if (hipError_t e = dma_kernel_ready<MODE, HEAD, NIT, P, false>()) return e;
    hipEvent_t t0, t1;
    if (next_timing_events(&t0, &t1))  // a measurement is on: this launch's own begin and end
        hipExtLaunchKernelGGL((qgemv_q4_0_dma_kernel<MODE, HEAD, NIT, P, false>), grid, block, pl.lds, st, t0, t1, 0, job, (const uint8_t*)act, y,
                              (int)(K / 32), (int64_t)act_bytes, pl.sh);
    else
        hipLaunchKernelGGL((qgemv_q4_0_dma_kernel<MODE, HEAD, NIT, P, false>), grid, block, pl.lds, st, job, (const uint8_t*)act, y, (int)(K / 32),
                           (int64_t)act_bytes, pl.sh);
    return hipGetLastError();
}

template <int MODE, int HEAD, int P>
hipError_t launch_dma_nit(const Q4Job& job, const void* act, float* y, int64_t K, const DmaPlan& pl, hipStream_t st) {
    switch (pl.nit) {
    case 1: return launch_dma<MODE, HEAD, 1, P>(job, act, y, K, pl, st);
    case 2: return launch_dma<MODE, HEAD, 2, P>(job, act, y, K, pl, st);
    case 3: return launch_dma<MODE, HEAD, 3, P>(job, act, y, K, pl, st);
    case 4: return launch_dma<MODE, HEAD, 4, P>(job, act, y, K, pl, st);
    case 5: return launch_dma<MODE, HEAD, 5, P>(job, act, y, K, pl, st);
    case 6: return launch_dma<MODE, HEAD, 6, P>(job, act, y, K, pl, st);
    case 7: return launch_dma<MODE, HEAD, 7, P>(job, act, y, K, pl, st);
    case 8: return launch_dma<MODE, HEAD, 8, P>(job, act, y, K, pl, st);
    }
    return hipErrorInvalidValue;
}

template <int MODE, int HEAD>
hipError_t launch_dma_pieces(const Q4Job& job, const void* act, float* y, int64_t K, const DmaPlan& pl, hipStream_t st) {
    switch (pl.pieces) {
    case 2: return launch_dma_nit<MODE, HEAD, 2>(job, act, y, K, pl, st);
    case 3: return launch_dma_nit<MODE, HEAD, 3>(job, act, y, K, pl, st);
    }
    return hipErrorInvalidValue;
}

}  // namespace

void set_q4_dma_off(int v) { g_dma_off = v; }
void set_q4_dma_feed(int feeders, int window) {
    if (feeders > 0) g_dma_feeders = feeders;
    if (window > 0) g_dma_window = window;
}

// Where the next launches of the float32-x product leave five clock readings per workgroup (null: stop). Synchronous.
hipError_t set_q4_dma_stamps(long long* p) {
    g_dma_stamps = p;
    return hipMemcpyToSymbol(HIP_SYMBOL(g_dma_stamps_dev), &p, sizeof(p));
}

// Whether this kernel takes the product (then *err is the launch's status). One row of x; W, its rows and their
// chunks 16-byte aligned; x short enough for the head's threads.
bool q4_0_dma_dispatch(int mode, const Q4Job& job, const void* act, float* y, int64_t M, int64_t K, hipStream_t st, hipError_t* err) {
    if (g_dma_off.load(std::memory_order_relaxed) != 0 || M != 1 || K % 64 != 0) return false;
    if (mode != kPlain && mode != kRope) return false;
    const int npairs = (int)(K / 64);
    const int head = job.norm_w ? kHeadNorm : job.norm_x ? kHeadConvert : kHeadAct;
    const int nitems = mode == kRope ? job.total / 2 : job.total;
    if (mode == kRope && (job.total % 2 != 0 || job.n[0] % 2 != 0 || job.n[1] % 2 != 0)) return false;
    for (int i = 0; i < 3; i++)
        if (job.W[i] && ((uintptr_t)job.W[i] & 15) != 0) return false;
    if ((K / 32 * 18) % 16 != 0) return false;
    if (head == kHeadNorm && !q4_0_norm_head_ok(K)) return false;
    if (head != kHeadAct && ((uintptr_t)job.norm_x & 15) != 0) return false;
    if (head == kHeadNorm && ((uintptr_t)job.norm_w & 15) != 0) return false;
    if (head == kHeadAct && ((uintptr_t)act & 15) != 0) return false;
    const size_t act_bytes = q4_0_act_bytes(K);
    // multiplying wavefronts the head needs: an item of x a thread (kHeadConvert), four 16-byte pieces of the converted row a thread (kHeadAct)
    const int min_waves = head == kHeadNorm ? 4 : head == kHeadConvert ? (int)((K / 8 + 63) / 64) : (int)((act_bytes / 16 + 255) / 256);
    const DmaPlan pl = plan_dma(nitems, mode == kRope ? 2 : 1, npairs, min_waves, act_bytes);
    if (!pl.ok) return false;
#define DMA_CASE(MM, HH) \
    if (mode == MM && head == HH) { *err = launch_dma_pieces<MM, HH>(job, act, y, K, pl, st); return true; }
    DMA_CASE(kPlain, kHeadConvert) DMA_CASE(kPlain, kHeadAct)
    DMA_CASE(kRope, kHeadAct) DMA_CASE(kRope, kHeadNorm)
#undef DMA_CASE
    return false;
}

}  // namespace mimir
