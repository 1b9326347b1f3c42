// Attention of one query position per sequence (a decoding step) on gfx950:
// the same arithmetic as attention.hip (OpAttention, backend/op.go:117-129; the
// CPU's decode branch forwardFew, backend/cpu/attention.go:437-535) in one
// launch that is all latency at batch 1, so it is shaped for few, wide,
// independent loads and no second kernel.
//
// A workgroup of 256 threads takes one key head, up to four of its query heads
// and one share of the keys the step sees (the shares are equal: the number of
// keys may come from device memory, so that a replayed graph serves every
// position, and every workgroup of the grid has work at every position).
// Sixteen lanes share a key row, 16 or 32 bytes each, so a wavefront's load
// covers four whole rows; the sixteen key groups of the workgroup take
// consecutive keys. Scores go through LDS for the softmax, values are
// accumulated per key group and summed through LDS. The rows of a share are
// requested before the number of keys is read (shares are fixed ranges of the
// cache, rows past the end clamped), so that load's round trip runs beside the
// keys'. A share's (max, sum, weighted values) reach the combining workgroup one
// of two ways. With flag slots (the decoder's steps): every float travels as an
// 8-byte (value, flag) pair, stored and loaded as one word, so a pair that
// reads as flagged is complete without any fence; the first share's workgroup
// polls the other shares' slots (all of them requested in one trip, a bounded
// number of polls, the device's error word on a time-out), combines, and clears
// the slots for the next launch. The workgroups it waits for never wait
// themselves, and its own share is done before it polls. Without slots (the
// boundary's call with its own workspace): each workgroup takes a ticket
// (release-acquire at device scope) and the one that draws the last ticket of
// its heads combines, so no workgroup waits at all. Either can leave the
// result in the fixed-point form the Q4_0 product reads (q4_act.h), which
// saves the conversion launch before the output projection. The grid is
// (key head x query group, share, sequence): with eight key heads a head's
// shares have workgroup indices congruent modulo eight, i.e. they run on one
// die, and the head's rows and slots stay in that die's L2.
#include "device_util.h"
#include "kernels.h"
#include "kq_act.h"
#include "q4_rows_act.h"

namespace mimir {

namespace {

constexpr int kHeads = 4;      // query heads per workgroup
constexpr int kThreads = 256;
constexpr int kKeyGroups = 16;
constexpr int kCounterBytes = (int)kAttnTicketBytes;  // tickets at the front of the workspace

struct DecParams {
    int64_t q_b, q_h;
    int64_t k_b, k_h, k_p;
    int64_t v_b, v_h, v_p;
    int64_t o_b, o_h;
    int B, H, HK, K, kmax;
    float scale;
    int causal;
    int64_t causal_offset;
    int cmax, nsplit;
    const int32_t* dyn_k;
    int64_t act_row_bytes;
    int act_rows;  // the converted result in the form for a few rows of x (q4_rows_act.h), all sequences in one buffer
    int act_kq;    // the converted result as int8 super-blocks for Q4_K / Q6_K products (kq_act.h), rows act_row_bytes apart
    int fence;     // 1: the ticket is a release-acquire operation at device scope (the default); 0, 2: measurement aids, see the ticket
    unsigned long long* flagged;  // not null: shares travel as (value, flag) pairs and the first share's workgroup collects them (no ticket)
    uint32_t* err;                // the device's error word (a hand-over that never completes sets kErrInternal)
};

__device__ __forceinline__ float group16_sum(float v) {
    v += dpp_f32<0xb1>(v);   // quad_perm [1,0,3,2]
    v += dpp_f32<0x4e>(v);   // quad_perm [2,3,0,1]
    v += dpp_f32<0x141>(v);  // row_half_mirror
    v += dpp_f32<0x140>(v);  // row_mirror
    return v;
}

// Stores and loads that are coherent across the device on their own.
__device__ __forceinline__ void coherent_store(float* p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ float coherent_load(const float* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

// A value and the flag that says it is there, in one 8-byte store: whoever loads the pair sees both or neither.
constexpr uint32_t kShareReady = 1u;
constexpr int kGather = 16;           // shares whose values the collecting workgroup requests together
constexpr int kShareSpins = 1 << 18;  // polls of a slot before the collecting workgroup gives up (some tenths of a second)
__device__ __forceinline__ void flagged_store(unsigned long long* p, float v) {
    __hip_atomic_store(p, ((unsigned long long)kShareReady << 32) | __float_as_uint(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ unsigned long long flagged_load(const unsigned long long* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void flagged_clear(unsigned long long* p) { __hip_atomic_store(p, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

// FPL consecutive elements of a cache row as floats.
template <typename KV, int FPL>
__device__ __forceinline__ void load_row(const KV* p, float out[FPL]) {
    if constexpr (sizeof(KV) == 4) {
#pragma unroll
        for (int i = 0; i < FPL; i += 4) {
            f32x4 t;
            __builtin_memcpy(&t, __builtin_assume_aligned(p + i, 16), 16);
            out[i] = t[0]; out[i + 1] = t[1]; out[i + 2] = t[2]; out[i + 3] = t[3];
        }
    } else {
        uint32_t w[FPL / 2];
        __builtin_memcpy(w, __builtin_assume_aligned(p, FPL == 4 ? 8 : 16), FPL * 2);
#pragma unroll
        for (int i = 0; i < FPL / 2; i++) {
            out[2 * i] = f16_bits_to_f32((uint16_t)(w[i] & 0xffffu));
            out[2 * i + 1] = f16_bits_to_f32((uint16_t)(w[i] >> 16));
        }
    }
}

// The same, in two steps: the bytes as loaded (so that many rows can be in
// flight in few registers), and their values.
template <typename KV, int FPL>
struct RawRow {
    uint32_t w[FPL * sizeof(KV) / 4];
};
template <typename KV, int FPL>
__device__ __forceinline__ void load_raw(const KV* p, RawRow<KV, FPL>& r) {
    constexpr int kBytes = FPL * sizeof(KV);
    __builtin_memcpy(r.w, __builtin_assume_aligned(p, kBytes >= 16 ? 16 : 8), kBytes);
}
template <typename KV, int FPL>
__device__ __forceinline__ void raw_values(const RawRow<KV, FPL>& r, float out[FPL]) {
    if constexpr (sizeof(KV) == 4) {
#pragma unroll
        for (int i = 0; i < FPL; i++) out[i] = __uint_as_float(r.w[i]);
    } else {
#pragma unroll
        for (int i = 0; i < FPL / 2; i++) {
            out[2 * i] = f16_bits_to_f32((uint16_t)(r.w[i] & 0xffffu));
            out[2 * i + 1] = f16_bits_to_f32((uint16_t)(r.w[i] >> 16));
        }
    }
}

// UU: rows of keys (and of values) a thread has under way at a time: a batch is 16 UU keys.
template <typename KV, int FPL, int UU>
__global__ __launch_bounds__(kThreads) void attn_decode_kernel(const float* __restrict__ q, const KV* __restrict__ k,
                                                               const KV* __restrict__ v, float* __restrict__ ws,
                                                               uint32_t* __restrict__ counters, float* __restrict__ out,
                                                               float* __restrict__ lse, uint8_t* __restrict__ act, DecParams p) {
    constexpr int D = 16 * FPL;
    constexpr int OPL = D / 64;  // results a lane holds of its wavefront's head
    extern __shared__ float smem[];
    float* sc = smem;                  // [4][cmax] scores, then weights
    float* osl = sc + kHeads * p.cmax; // [16][4][D] values per key group; later the combine's factors and results
    __shared__ float red[2 * kHeads];
    __shared__ int s_last;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int part = tid & 15, kg = tid >> 4;
    // The grid's first dimension runs over the key heads (times the groups of four query heads), the second over the shares
    // of the keys: workgroups are handed to the chip's dies round robin by their linear index, so with eight key heads
    // every share of a head runs on the same die, whose L2 alone then holds the head's keys and values.
    const int split = blockIdx.y, nsplit = p.nsplit, cmax = p.cmax;
    const int group = blockIdx.x;
    const int G = p.H / p.HK, ngq = (G + kHeads - 1) / kHeads;
    const int hk = group / ngq, g0 = (group % ngq) * kHeads;
    const int ng = G - g0 < kHeads ? G - g0 : kHeads;
    const int b = blockIdx.z;

    // The shares are cmax keys each, fixed for the launch: share `split` takes keys [split cmax, (split + 1) cmax) of
    // those the step sees. How many it sees may come from device memory (p.dyn_k); nothing below waits for that
    // number before the queries, keys and values of the first batch have been requested (rows past the last key
    // seen are requested too, from within the caches, and ignored).
    const int j0 = split * cmax;
    float qr[kHeads][FPL];
#pragma unroll
    for (int g = 0; g < kHeads; g++) {
        if (g < ng) {
            load_row<float, FPL>(q + b * p.q_b + (int64_t)(hk * G + g0 + g) * p.q_h + part * FPL, qr[g]);
#pragma unroll
            for (int f = 0; f < FPL; f++) qr[g][f] = qr[g][f] * p.scale;
        } else {
#pragma unroll
            for (int f = 0; f < FPL; f++) qr[g][f] = 0.f;
        }
    }
    // rows of a head's keys and values lie within 2^31 elements and fewer than 2^23 apart (checked by the host): 24-bit multiplies
    // and 32-bit offsets in place of 64-bit address arithmetic per row
    const int kp = (int)p.k_p, vp = (int)p.v_p;
    const KV* kbase = k + b * p.k_b + (int64_t)hk * p.k_h + part * FPL;
    const KV* vbase = v + b * p.v_b + (int64_t)hk * p.v_h + part * FPL;

    // Rows in flight per thread: key j0 + jj with jj = jj0 + 16 u + kg. The first
    // batch of keys and of values is requested before anything is computed, so
    // that a share of up to 16 U keys costs one trip to memory for both.
    constexpr int U = UU;
    RawRow<KV, FPL> kraw[U], vraw[U];
    const int last_row = p.kmax - 1;  // the caches hold kmax rows
#pragma unroll
    for (int u = 0; u < U; u++) {
        const int jj = kKeyGroups * u + kg, row = j0 + (jj < cmax ? jj : 0);
        load_raw<KV, FPL>(kbase + (uint32_t)__mul24(row < last_row ? row : last_row, kp), kraw[u]);
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
        const int jj = kKeyGroups * u + kg, row = j0 + (jj < cmax ? jj : 0);
        load_raw<KV, FPL>(vbase + (uint32_t)__mul24(row < last_row ? row : last_row, vp), vraw[u]);
    }
    __builtin_amdgcn_sched_barrier(0);  // the requests above go out before the number of keys is waited for
    int64_t seen = (int64_t)p.K + (p.dyn_k ? *p.dyn_k : 0);
    if (p.causal) {
        int64_t c = p.causal_offset + 1;
        seen = c < seen ? c : seen;
    }
    seen = seen < 0 ? 0 : seen > p.kmax ? p.kmax : seen;
    const int nj = seen > j0 ? (int)(seen - j0 < cmax ? seen - j0 : cmax) : 0;
    for (int jj0 = 0; jj0 < nj; jj0 += U * kKeyGroups) {
        if (jj0 > 0) {
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int jj = jj0 + kKeyGroups * u + kg;
                load_raw<KV, FPL>(kbase + (uint32_t)__mul24(j0 + (jj < nj ? jj : 0), kp), kraw[u]);
            }
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int jj = jj0 + kKeyGroups * u + kg;
            float kf[FPL];
            raw_values<KV, FPL>(kraw[u], kf);
#pragma unroll
            for (int g = 0; g < kHeads; g++) {
                float s = 0.f;
#pragma unroll
                for (int f = 0; f < FPL; f++) s = fmaf(qr[g][f], kf[f], s);
                s = group16_sum(s);
                if (part == 0 && jj < nj) sc[g * cmax + jj] = s;
            }
        }
    }
    __syncthreads();

    // per head (wavefront g takes head g): max, exp, sum over the share's scores
    {
        float m = -__builtin_inff();
        for (int jj = lane; jj < nj; jj += 64) m = fmaxf(m, sc[wave * cmax + jj]);
        m = wave_max(m);
        float l = 0.f;
        if (nj > 0 && m > -__builtin_inff()) {
            for (int jj = lane; jj < nj; jj += 64) {
                float e = __builtin_expf(sc[wave * cmax + jj] - m);
                sc[wave * cmax + jj] = e;
                l += e;
            }
        } else {
            for (int jj = lane; jj < nj; jj += 64) sc[wave * cmax + jj] = 0.f;
        }
        l = wave_sum(l);
        if (lane == 0) {
            red[wave] = m;
            red[kHeads + wave] = l;
        }
    }
    __syncthreads();

    // values: key group kg sums its keys' rows, weighted, for the four heads
    float o[kHeads][FPL];
#pragma unroll
    for (int g = 0; g < kHeads; g++)
#pragma unroll
        for (int f = 0; f < FPL; f++) o[g][f] = 0.f;
    for (int jj0 = 0; jj0 < nj; jj0 += U * kKeyGroups) {
        if (jj0 > 0) {
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int jj = jj0 + kKeyGroups * u + kg;
                load_raw<KV, FPL>(vbase + (uint32_t)__mul24(j0 + (jj < nj ? jj : 0), vp), vraw[u]);
            }
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int jj = jj0 + kKeyGroups * u + kg;
            const bool live = jj < nj;
            float vf[FPL];
            raw_values<KV, FPL>(vraw[u], vf);
#pragma unroll
            for (int g = 0; g < kHeads; g++) {
                float pj = live ? sc[g * cmax + jj] : 0.f;
#pragma unroll
                for (int f = 0; f < FPL; f++) o[g][f] = fmaf(pj, live ? vf[f] : 0.f, o[g][f]);
            }
        }
    }
#pragma unroll
    for (int g = 0; g < kHeads; g++)
#pragma unroll
        for (int f = 0; f < FPL; f++) osl[(kg * kHeads + g) * D + part * FPL + f] = o[g][f];
    __syncthreads();
    // wavefront g now holds head g: lane takes features lane + 64 c
    const int g = wave, h = hk * G + g0 + g;
    float r[OPL];
#pragma unroll
    for (int c = 0; c < OPL; c++) {
        float s = 0.f;
#pragma unroll
        for (int x = 0; x < kKeyGroups; x++) s += osl[(x * kHeads + g) * D + lane + 64 * c];
        r[c] = s;
    }
    float M = red[g], L = red[kHeads + g];

    if (nsplit > 1 && p.flagged) {
        // The shares travel as (value, flag) pairs, each one 8-byte store that is coherent at device scope on its own:
        // a pair is seen whole or not at all, so nothing has to be waited for between the data and a signal that it
        // is there. The workgroups of shares 1.. store theirs and are done; the workgroup of share 0 keeps its own in
        // registers, polls the others' slots until every pair shows its flag (a bounded number of times: all
        // workgroups of a launch are resident together, the grid being far smaller than the chip), combines them in
        // the shares' order and clears the slots for the next launch on the stream.
        unsigned long long* slots = p.flagged + ((int64_t)b * p.H + h) * nsplit * (D + 2);
        if (split != 0) {
            if (g < ng) {
                unsigned long long* w = slots + (int64_t)split * (D + 2);
                if (lane == 0) {
                    flagged_store(w, M);
                    flagged_store(w + 1, L);
                }
#pragma unroll
                for (int c = 0; c < OPL; c++) flagged_store(w + 2 + lane + 64 * c, r[c]);
            }
            return;
        }
        bool late = false;
        float* fs = osl + g * 64;  // factor of share s of head g
        float own[OPL];
#pragma unroll
        for (int c = 0; c < OPL; c++) own[c] = r[c];
        const unsigned long long ready = (unsigned long long)kShareReady << 32;
        // Sixteen shares' values at a time, asked for again while any pair lacks its flag; with the first sixteen go the
        // (max, sum) of every share, so that one trip to memory brings all a short context needs.
        unsigned long long raw[kGather][OPL], mraw = ready | __float_as_uint(M), lraw = ready | __float_as_uint(L);
        auto gather = [&](int s0, bool with_sums) {
            bool all = g >= ng;  // a wavefront without a head has nothing to wait for
            for (int spin = 0; !all && spin < kShareSpins; spin++) {
                if (spin) __builtin_amdgcn_s_sleep(2);
                all = true;
                if (with_sums && lane < nsplit && lane > 0) {
                    mraw = flagged_load(slots + lane * (D + 2));
                    lraw = flagged_load(slots + lane * (D + 2) + 1);
                }
#pragma unroll
                for (int u = 0; u < kGather; u++) {
                    const int sidx = s0 + u < nsplit ? s0 + u : nsplit - 1;
#pragma unroll
                    for (int c = 0; c < OPL; c++)
                        raw[u][c] = sidx == 0 ? ready | __float_as_uint(own[c]) : flagged_load(slots + (int64_t)sidx * (D + 2) + 2 + lane + 64 * c);
                }
                all = (uint32_t)(mraw >> 32) == kShareReady && (uint32_t)(lraw >> 32) == kShareReady;
#pragma unroll
                for (int u = 0; u < kGather; u++)
#pragma unroll
                    for (int c = 0; c < OPL; c++) all = all && (uint32_t)(raw[u][c] >> 32) == kShareReady;
            }
            if (!all) late = true;
        };
        gather(0, true);
        float f = 0.f, ls = 0.f, ms = -__builtin_inff();
        if (g < ng && lane < nsplit) {
            ms = __uint_as_float((uint32_t)mraw);
            ls = __uint_as_float((uint32_t)lraw);
        }
        M = wave_max(ms);
        if (ls != 0.f && M > -__builtin_inff()) f = __builtin_expf(ms - M);
        L = wave_sum(ls * f);
        fs[lane] = f;
        __syncthreads();
#pragma unroll
        for (int c = 0; c < OPL; c++) r[c] = 0.f;
        if (g < ng) {
            for (int s0 = 0; s0 < nsplit; s0 += kGather) {
                if (s0 > 0) gather(s0, false);
#pragma unroll
                for (int u = 0; u < kGather; u++) {
                    const float fsv = s0 + u < nsplit ? fs[s0 + u] : 0.f;
#pragma unroll
                    for (int c = 0; c < OPL; c++) r[c] = fmaf(__uint_as_float((uint32_t)raw[u][c]), fsv, r[c]);
                }
            }
            // the slots are read: empty again for the next launch
            if (lane < nsplit && lane > 0) {
                flagged_clear(slots + lane * (D + 2));
                flagged_clear(slots + lane * (D + 2) + 1);
            }
            for (int sidx = 1; sidx < nsplit; sidx++)
#pragma unroll
                for (int c = 0; c < OPL; c++) flagged_clear(slots + (int64_t)sidx * (D + 2) + 2 + lane + 64 * c);
        }
        if (late && p.err) atomicOr(p.err, kErrInternal);
        __syncthreads();  // fs is read; the results go over it
    } else if (nsplit > 1) {
        // The shares travel between workgroups (and so between the L2 caches of
        // the chip's dies) through stores and loads that are coherent at device
        // scope by themselves (write-through stores, loads that bypass stale
        // lines). Ordering: every thread's stores have completed (the counters
        // are waited on, then the barrier) before thread 0 takes the ticket, a
        // release-acquire operation at device scope, and the combining loads are
        // issued only after the last ticket is known.
        if (g < ng) {
            float* w = ws + (((int64_t)b * p.H + h) * nsplit + split) * (D + 2);
            if (p.fence == 2) {  // measurement aid: plain stores, made visible by the ticket's release
                if (lane == 0) {
                    w[0] = M;
                    w[1] = L;
                }
#pragma unroll
                for (int c = 0; c < OPL; c++) w[2 + lane + 64 * c] = r[c];
            } else {
                if (lane == 0) {
                    coherent_store(w, M);
                    coherent_store(w + 1, L);
                }
#pragma unroll
                for (int c = 0; c < OPL; c++) coherent_store(w + 2 + lane + 64 * c, r[c]);
            }
        }
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        if (tid == 0) {
            uint32_t* ctr = counters + (int64_t)b * gridDim.x + group;
            // Release-acquire at device scope: the shares stored above (by operations that are coherent at that scope on their
            // own, and complete: the wait above counts them) happen before the ticket, and the combining loads below after it.
            // Measured against a relaxed ticket: no difference within the run-to-run spread of a decoding step (0.5 %).
            // p.fence 0: the relaxed ticket; 2: plain stores and loads of the shares under the same ticket (both to be measured).
            uint32_t ticket = p.fence != 0 ? __hip_atomic_fetch_add(ctr, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT)
                                           : __hip_atomic_fetch_add(ctr, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            s_last = ticket == (uint32_t)(nsplit - 1);
            if (s_last) __hip_atomic_store(ctr, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // for the next launch
        }
        __syncthreads();
        if (!s_last) return;
        // the last workgroup of these heads to get here combines the shares: their (max, sum) and the first eight shares'
        // values are requested together, one trip to memory for both
        float* fs = osl + g * 64;  // factor of share s of head g
        float f = 0.f, ls = 0.f, ms = -__builtin_inff();
        const float* w0 = ws + ((int64_t)b * p.H + h) * nsplit * (D + 2);
        if (g < ng && lane < nsplit) {
            ms = p.fence == 2 ? w0[lane * (D + 2)] : coherent_load(w0 + lane * (D + 2));
            ls = p.fence == 2 ? w0[lane * (D + 2) + 1] : coherent_load(w0 + lane * (D + 2) + 1);
        }
        float t[8][OPL];
        auto load_shares = [&](int s0) {
#pragma unroll
            for (int u = 0; u < 8; u++) {
                const int s = s0 + u < nsplit ? s0 + u : nsplit - 1;
#pragma unroll
                for (int c = 0; c < OPL; c++) t[u][c] = p.fence == 2 ? w0[s * (D + 2) + 2 + lane + 64 * c] : coherent_load(w0 + s * (D + 2) + 2 + lane + 64 * c);
            }
        };
        if (g < ng) load_shares(0);
        M = wave_max(ms);
        if (ls != 0.f && M > -__builtin_inff()) f = __builtin_expf(ms - M);
        L = wave_sum(ls * f);
        fs[lane] = f;
        __syncthreads();
#pragma unroll
        for (int c = 0; c < OPL; c++) r[c] = 0.f;
        if (g < ng) {
            for (int s0 = 0; s0 < nsplit; s0 += 8) {  // eight shares' loads in flight
                if (s0 > 0) load_shares(s0);
#pragma unroll
                for (int u = 0; u < 8; u++) {
                    const float fsv = s0 + u < nsplit ? fs[s0 + u] : 0.f;
#pragma unroll
                    for (int c = 0; c < OPL; c++) r[c] = fmaf(t[u][c], fsv, r[c]);
                }
            }
        }
        __syncthreads();  // fs is read; the results go over it
    }

    // (sum p v) * (1 / sum p); a row that sees no key gets zeros and -Inf
    const float inv = L == 0.f ? 0.f : 1.0f / L;
    float* fin = osl;  // [4][D]
#pragma unroll
    for (int c = 0; c < OPL; c++) {
        float val = L == 0.f ? 0.f : r[c] * inv;
        if (g < ng && out) out[b * p.o_b + (int64_t)h * p.o_h + lane + 64 * c] = val;
        if (act) fin[g * D + lane + 64 * c] = g < ng ? val : 0.f;
    }
    if (g < ng && lse && lane == 0) lse[(int64_t)b * p.H + h] = L == 0.f ? -__builtin_inff() : M + __builtin_logf(L);
    if (!act) return;
    __syncthreads();
    if (p.act_kq) {
        // the heads of this workgroup are whole super-blocks of 256 of the row (checked by the host): a wavefront each
        const int nsup = ng * D / 256, wv = tid >> 6;
        if (wv < nsup) {
            const f32x4 v = *(const f32x4*)(fin + 256 * wv + 4 * lane);
            kq_convert_superblock(v, (hk * G + g0) * D / 256 + wv, lane, p.H * D / 256, act + (int64_t)b * p.act_row_bytes);
        }
        return;
    }
    // item t: head t / (D/8), block (t % (D/8)) / 4 of the head, dword t % 4
    const int nit = ng * (D / 8);
    if (tid < nit) {
        const int gi = tid / (D / 8), rr = tid % (D / 8), blk = rr >> 2, dq = rr & 3;
        float lo[4], hi[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            lo[e] = fin[gi * D + blk * 32 + 4 * dq + e];
            hi[e] = fin[gi * D + blk * 32 + 16 + 4 * dq + e];
        }
        const int nb = p.H * D / 32, nbp = nb | 1;
        if (p.act_rows) {
            // sequence b: row b % 8 of its group of eight, which has a buffer of its own
            rows_convert_item(lo, hi, act + (int64_t)(b >> 3) * q4_0_rows_act_size((int64_t)nb * 32), nb, b & 7, (hk * G + g0 + gi) * (D / 32) + blk, dq);
        } else {
            u32x4* plane = (u32x4*)(act + (int64_t)b * p.act_row_bytes);
            float* xscale = (float*)(plane + kDigits * nbp);
            q4_convert_item(lo, hi, plane, xscale, nbp, (hk * G + g0 + gi) * (D / 32) + blk, dq);
        }
    }
}

}  // namespace

static std::atomic<int> g_share_keys{64};  // "attention.share": keys a share aims at (64 or 128)
void set_attention_decode_share(int n) { g_share_keys = n == 128 ? 128 : 64; }
static std::atomic<int> g_force_splits{0};  // measurement aid: a fixed number of shares
static std::atomic<int> g_fence{1};         // "attention.fence"
void set_attention_decode_splits(int n) { g_force_splits = n; }
void set_attention_decode_fence(int v) { g_fence = v; }

// Shares of the keys and the most keys a share can hold, for at most kmax keys.
void attention_decode_plan(int64_t B, int H, int HK, int64_t kmax, int* nsplit, int* cmax) {
    int G = H / HK, ngq = (G + kHeads - 1) / kHeads;
    int64_t rows = B * HK * ngq;
    int64_t ns = 512 / (rows > 0 ? rows : 1);
    ns = ns > 64 ? 64 : ns;
    // A share is one batch of loads per thread: 64 keys while that makes no more shares than the collecting workgroup
    // gathers in one trip to memory, 128 beyond ("attention.share" = 128: always). Measured at 768 keys against 128:
    // the scores and the weighted values of a share take half as long, the hand-over a little longer.
    const int64_t aim = g_share_keys.load(std::memory_order_relaxed);
    int64_t by_keys = (kmax + aim - 1) / aim;
    const bool short_shares = by_keys <= kGather;
    if (!short_shares) by_keys = (kmax + 127) / 128;
    // Shares of 64 keys are worth three workgroups a compute unit (eight sequences at 768 positions: 12 shares of 64 keys
    // decode 1.7 % faster than 8 of 96), longer ones are not (at 2048 positions 8 shares of 256 keys: 90 us a layer,
    // 12 of 171: 94, 16 of 128: 99).
    if (short_shares && rows * by_keys <= 768) ns = by_keys;
    ns = ns > by_keys ? by_keys : ns;
    ns = ns < 1 ? 1 : ns;
    if (g_force_splits > 0 && g_force_splits <= 64) ns = g_force_splits;
    *nsplit = (int)ns;
    int64_t c = (kmax + ns - 1) / ns;
    *cmax = (int)(c < 1 ? 1 : c);
}

size_t attention_decode_workspace_bytes(int64_t B, int H, int D, int nsplit) {
    return kCounterBytes + (nsplit <= 1 ? 0 : (size_t)(B * H * nsplit * (D + 2)) * sizeof(float));
}

// Whether the decode kernel takes this call: one query position, heads of 64
// or 128 features, rows of the caches and of q aligned for 16-byte loads.
bool attention_decode_ok(const AttnArgs& a, int64_t kmax) {
    if (a.Q != 1 || (a.D != 64 && a.D != 128) || a.B <= 0 || a.B > 65535) return false;
    if (a.mask || (a.DV > 0 && a.DV != a.D) || kmax <= 0 || !a.k || !a.v) return false;  // the general kernels take those
    int G = a.H / a.HK, ngq = (G + kHeads - 1) / kHeads;
    if (a.B * a.HK * ngq > kCounterBytes / 4 || (int64_t)a.HK * ngq > 65535) return false;
    const int es = a.kv_dtype == kF16 ? 2 : 4;
    const int fpl = a.D / 16;
    const int row_align = fpl * es >= 16 ? 16 : 8;
    for (int i = 0; i < 3; i++)
        if ((a.k_strides[i] * es) % row_align || (a.v_strides[i] * es) % row_align) return false;
    if (((uintptr_t)a.k | (uintptr_t)a.v) % row_align || (uintptr_t)a.q % 16 || a.q_strides[0] % 4 || a.q_strides[1] % 4) return false;
    int ns, cm;
    attention_decode_plan(a.B, a.H, a.HK, kmax, &ns, &cm);
    size_t lds = (size_t)(kHeads * cm + kKeyGroups * kHeads * a.D) * sizeof(float);
    if (a.k_strides[2] <= 0 || a.v_strides[2] <= 0 || a.k_strides[2] >= (1 << 23) || a.v_strides[2] >= (1 << 23) || kmax >= (1 << 23) ||
        kmax * a.k_strides[2] >= ((int64_t)1 << 31) || kmax * a.v_strides[2] >= ((int64_t)1 << 31))
        return false;
    return lds <= 60 * 1024 && kmax <= INT32_MAX / 2;
}

// Whether the result can leave in the K-quants' int8 form: the heads a workgroup finishes are whole super-blocks of the row.
bool attention_decode_kq_ok(const AttnArgs& a) {
    const int G = a.H / a.HK, per = G < kHeads ? G : kHeads;
    return (G <= kHeads || G % kHeads == 0) && (per * a.D) % 256 == 0 && (G * a.D) % 256 == 0;
}

// a.K keys (plus *a.dyn_k), at most kmax. workspace: attention_decode_workspace_bytes
// bytes whose first 4096 were zero before the first launch (the tickets reset
// themselves). act, if set, gets row b's result [H * D] in the Q4_0 product's
// fixed-point form, act_row_bytes apart; out may then be null.
// act_form: kAttnActQ4 that form; kAttnActRows the form for eight sequences together (q4_rows_act.h), a buffer per group of eight: row b's
// result as row b % 8 of group b / 8; kAttnActKQ int8 super-blocks for the K-quant products (where attention_decode_kq_ok).
size_t attention_decode_flagged_bytes(int64_t B, int H, int D, int nsplit) { return nsplit <= 1 ? 0 : (size_t)(B * H * nsplit * (D + 2)) * 8; }

static std::atomic<int> g_handover{0};  // "attention.handover": 1 keeps the ticket protocol although flagged slots are there
void set_attention_decode_handover(int v) { g_handover = v; }

hipError_t attention_decode(const AttnArgs& a, int64_t kmax, void* workspace, void* act, int64_t act_row_bytes, hipStream_t st, int act_form,
                            void* flagged, size_t flagged_bytes, uint32_t* err) {
    note_kernel("attn_decode_kernel");
    DecParams p;
    p.q_b = a.q_strides[0]; p.q_h = a.q_strides[1];
    p.k_b = a.k_strides[0]; p.k_h = a.k_strides[1]; p.k_p = a.k_strides[2];
    p.v_b = a.v_strides[0]; p.v_h = a.v_strides[1]; p.v_p = a.v_strides[2];
    p.o_b = a.o_strides[0]; p.o_h = a.o_strides[1];
    p.B = (int)a.B; p.H = a.H; p.HK = a.HK; p.K = (int)a.K; p.kmax = (int)kmax;
    p.scale = (float)a.scale;
    p.causal = a.causal;
    p.causal_offset = a.causal_offset;
    attention_decode_plan(a.B, a.H, a.HK, kmax, &p.nsplit, &p.cmax);
    p.dyn_k = a.dyn_k;
    p.act_row_bytes = act_row_bytes;
    p.act_rows = act_form == kAttnActRows ? 1 : 0;
    p.act_kq = act_form == kAttnActKQ ? 1 : 0;
    p.fence = g_fence.load(std::memory_order_relaxed);
    const bool flags_fit = flagged && attention_decode_flagged_bytes(a.B, a.H, a.D, p.nsplit) <= flagged_bytes;  // else the tickets
    p.flagged = g_handover.load(std::memory_order_relaxed) == 1 || !flags_fit ? nullptr : (unsigned long long*)flagged;
    p.err = err;
    int G = a.H / a.HK, ngq = (G + kHeads - 1) / kHeads;
    dim3 grid((unsigned)(a.HK * ngq), (unsigned)p.nsplit, (unsigned)a.B);
    size_t lds = (size_t)(kHeads * p.cmax + kKeyGroups * kHeads * a.D) * sizeof(float);
    uint32_t* counters = (uint32_t*)workspace;
    float* ws = (float*)((uint8_t*)workspace + kCounterBytes);
    // a thread keeps eight rows of binary16 keys (four of float32) under way, or half as many where a share is that short
#define DEC_LAUNCH(KV, FPL, UU)                                                                                                   \
    hipLaunchKernelGGL((attn_decode_kernel<KV, FPL, UU>), grid, dim3(kThreads), lds, st, a.q, (const KV*)a.k, (const KV*)a.v, ws, \
                       counters, a.out, a.lse, (uint8_t*)act, p)
    const bool short_share = p.cmax <= kKeyGroups * 4;
    if (a.kv_dtype == kF16) {
        if (a.D == 128) { if (short_share) DEC_LAUNCH(uint16_t, 8, 4); else DEC_LAUNCH(uint16_t, 8, 8); }
        else { if (short_share) DEC_LAUNCH(uint16_t, 4, 4); else DEC_LAUNCH(uint16_t, 4, 8); }
    } else {
        if (a.D == 128) DEC_LAUNCH(float, 8, 4); else DEC_LAUNCH(float, 4, 4);
    }
#undef DEC_LAUNCH
    return hipGetLastError();
}

}  // namespace mimir
