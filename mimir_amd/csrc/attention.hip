// Attention for decoding and prompts on gfx950: softmax(scale * q.k^T) . v per
// query row over a KV cache of float32 or binary16, with grouped query heads
// (OpAttention, backend/op.go:117-129; the CPU's decode branch is forwardFew,
// backend/cpu/attention.go:437-535; the replaced generated kernel is
// backend/internal/gen/attention.go:28-49, which at one query row launches one
// workgroup per query head, so the query heads of a key head each read the
// same keys and values).
//
// Here a workgroup takes one key head, one query position and a chunk of key
// positions, and serves up to four query heads of the group from one read of
// the chunk's keys and values (split-K: the chunks of a row are combined by a
// second small kernel, so even one sequence fills the chip). Scores: eight
// lanes share a key, each taking an eighth of its features, so a wavefront's
// load covers eight consecutive keys; values: lanes take consecutive features,
// so each load is one contiguous key row.
//
// As the reference: the query is scaled first; the additive mask [B, H, Q, K], if
// any, is added to the scores (backend/cpu/attention.go:268-292); p = exp(s -
// max); the result is (sum p v) * (1 / sum p); the logsumexp is max + log(sum p);
// a row that sees no key gets zeros and -Inf. Key j is hidden from query i when
// causal and j > i + causal_offset. Values may have another width (DV) than keys.
#include "device_util.h"
#include "kernels.h"

namespace mimir {

constexpr int kAttnHeads = 4;     // query heads served per workgroup
constexpr int kAttnMaxD = 256;
constexpr int kAttnThreads = 256;

template <typename KV>
__device__ __forceinline__ float kv_load(const KV* p);
template <>
__device__ __forceinline__ float kv_load<float>(const float* p) { return *p; }
template <>
__device__ __forceinline__ float kv_load<uint16_t>(const uint16_t* p) { return f16_bits_to_f32(*p); }

struct AttnParams {
    int64_t q_b, q_h, q_i;     // strides of q in floats
    int64_t k_b, k_h, k_p;     // strides of k in elements
    int64_t v_b, v_h, v_p;     // strides of v in elements
    int64_t o_b, o_h, o_i;     // strides of out in floats
    int64_t m_b, m_h, m_i, m_j; // strides of the mask in floats
    int B, H, HK, Q, K, D, DV;
    float scale;
    int causal;
    int64_t causal_offset;
    int chunk, nsplit;
    const int32_t* dyn_k;  // if set, *dyn_k more keys than K (a decoding step replayed at every position)
};

// Partial results of one (query row, head, split): m, l, then o[D].
template <typename KV>
__global__ __launch_bounds__(kAttnThreads) void attn_partial_kernel(const float* __restrict__ q, const KV* __restrict__ k,
                                                                    const KV* __restrict__ v, const float* __restrict__ mask,
                                                                    float* __restrict__ ws, float* __restrict__ out, float* __restrict__ lse,
                                                                    AttnParams p) {
    extern __shared__ float smem[];
    const int D = p.D, DV = p.DV, G = p.H / p.HK, chunk = p.chunk;
    float* qs = smem;                       // [4][D], scaled
    float* sc = qs + kAttnHeads * D;        // [4][chunk]
    float* red = sc + kAttnHeads * chunk;   // [4][kAttnThreads / 64 ... ] and slices of o: max(32, 4 * DV) floats
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int split = blockIdx.x;
    const int ngq = (G + kAttnHeads - 1) / kAttnHeads;
    const int hk = blockIdx.y / ngq, g0 = (blockIdx.y % ngq) * kAttnHeads;
    const int ng = G - g0 < kAttnHeads ? G - g0 : kAttnHeads;  // live query heads here
    const int b = blockIdx.z / p.Q, i = blockIdx.z % p.Q;

    const int64_t Kt = p.K + (p.dyn_k ? *p.dyn_k : 0);
    int64_t seen = Kt;
    if (p.causal) {
        seen = (int64_t)i + p.causal_offset + 1;
        seen = seen < 0 ? 0 : seen > Kt ? Kt : seen;
    }
    const int j0 = split * chunk;
    int j1 = j0 + chunk;
    j1 = j1 > seen ? (int)seen : j1;
    const int nj = j1 > j0 ? j1 - j0 : 0;

    for (int t = tid; t < kAttnHeads * D; t += kAttnThreads) {
        int g = t / D, d = t % D;
        qs[t] = g < ng ? q[b * p.q_b + (int64_t)(hk * G + g0 + g) * p.q_h + i * p.q_i + d] * p.scale : 0.f;
    }
    __syncthreads();

    // scores: lane (slot, part) takes features [part * dpl, ...) of key j0 + 8 * (4 * it + wave) + slot
    const int dpl = (D + 7) >> 3, part = lane & 7, slot = lane >> 3;
    const int d_lo = part * dpl, d_hi = d_lo + dpl < D ? d_lo + dpl : D;
    const KV* kbase = k + b * p.k_b + (int64_t)hk * p.k_h;
    for (int jj0 = wave * 8; jj0 < nj; jj0 += 8 * (kAttnThreads / 64)) {
        int jj = jj0 + slot;
        const bool live = jj < nj;
        const KV* kr = kbase + (int64_t)(j0 + (live ? jj : 0)) * p.k_p;
        float s[kAttnHeads] = {0.f, 0.f, 0.f, 0.f};
        for (int d = d_lo; d < d_hi; d++) {
            float kv = kv_load<KV>(kr + d);
#pragma unroll
            for (int g = 0; g < kAttnHeads; g++) s[g] = fmaf(qs[g * D + d], kv, s[g]);
        }
#pragma unroll
        for (int g = 0; g < kAttnHeads; g++) {
            float t = group8_sum(s[g]);
            if (part == 0 && live) {
                if (mask && g < ng) t = t + mask[b * p.m_b + (int64_t)(hk * G + g0 + g) * p.m_h + i * p.m_i + (int64_t)(j0 + jj) * p.m_j];
                sc[g * chunk + jj] = t;
            }
        }
    }
    __syncthreads();

    // per head: max, exp, sum over the chunk's scores (wave g takes head g)
    float m_g = -__builtin_inff(), l_g = 0.f;
    if (wave < kAttnHeads) {
        float m = -__builtin_inff();
        for (int jj = lane; jj < nj; jj += 64) m = fmaxf(m, sc[wave * chunk + jj]);
        m = wave_max(m);
        float l = 0.f;
        if (nj > 0 && m > -__builtin_inff()) {
            for (int jj = lane; jj < nj; jj += 64) {
                float e = __builtin_expf(sc[wave * chunk + jj] - m);
                sc[wave * chunk + jj] = e;
                l += e;
            }
        } else {
            for (int jj = lane; jj < nj; jj += 64) sc[wave * chunk + jj] = 0.f;
        }
        l = wave_sum(l);
        m_g = m;
        l_g = l;
        if (lane == 0) {
            red[wave] = m;
            red[kAttnHeads + wave] = l;
        }
    }
    __syncthreads();

    // values: thread (d, slice) sums the keys jj = slice, slice + nslice, ...
    const int nslice = kAttnThreads / DV > 0 ? kAttnThreads / DV : 1;  // DV <= 256
    const int d = tid % DV, slice = tid / DV;
    float o[kAttnHeads] = {0.f, 0.f, 0.f, 0.f};
    if (slice < nslice && tid < nslice * DV) {
        const KV* vbase = v + b * p.v_b + (int64_t)hk * p.v_h + d;
        for (int jj = slice; jj < nj; jj += nslice) {
            float vv = kv_load<KV>(vbase + (int64_t)(j0 + jj) * p.v_p);
#pragma unroll
            for (int g = 0; g < kAttnHeads; g++) o[g] = fmaf(sc[g * chunk + jj], vv, o[g]);
        }
    }
    float m4[kAttnHeads], l4[kAttnHeads];
#pragma unroll
    for (int g = 0; g < kAttnHeads; g++) {
        m4[g] = red[g];
        l4[g] = red[kAttnHeads + g];
    }
    __syncthreads();  // red is reused for the slices of o
    // combine slices through LDS: red[(slice * 4 + g) * D + d]
    float* oslices = red;
    if (nslice > 1) {
        if (slice > 0 && slice < nslice) {
#pragma unroll
            for (int g = 0; g < kAttnHeads; g++) oslices[((slice - 1) * kAttnHeads + g) * DV + d] = o[g];
        }
        __syncthreads();
        if (slice == 0) {
            for (int s2 = 1; s2 < nslice; s2++)
#pragma unroll
                for (int g = 0; g < kAttnHeads; g++) o[g] += oslices[((s2 - 1) * kAttnHeads + g) * DV + d];
        }
    }
    (void)m_g;
    (void)l_g;
    if (slice != 0 || tid >= DV) return;
#pragma unroll
    for (int g = 0; g < kAttnHeads; g++) {
        if (g >= ng) break;
        const int h = hk * G + g0 + g;
        if (p.nsplit == 1) {  // final
            float* orow = out + b * p.o_b + (int64_t)h * p.o_h + i * p.o_i;
            if (l4[g] == 0.f) {
                orow[d] = 0.f;
                if (lse && d == 0) lse[((int64_t)b * p.H + h) * p.Q + i] = -__builtin_inff();
            } else {
                orow[d] = o[g] * (1.0f / l4[g]);
                if (lse && d == 0) lse[((int64_t)b * p.H + h) * p.Q + i] = m4[g] + __builtin_logf(l4[g]);
            }
        } else {
            float* w = ws + ((((int64_t)b * p.Q + i) * p.H + h) * p.nsplit + split) * (DV + 2);
            if (d == 0) {
                w[0] = m4[g];
                w[1] = l4[g];
            }
            w[2 + d] = o[g];
        }
    }
}

// out = sum_s o_s e^(m_s - M) / sum_s l_s e^(m_s - M); one workgroup per (row, head).
__global__ __launch_bounds__(256) void attn_combine_kernel(const float* __restrict__ ws, float* __restrict__ out,
                                                           float* __restrict__ lse, AttnParams p) {
    const int D = p.DV, d = threadIdx.x;
    const int64_t rh = blockIdx.x;  // (b * Q + i) * H + h
    const int h = (int)(rh % p.H);
    const int64_t bi = rh / p.H;
    const int i = (int)(bi % p.Q);
    const int64_t b = bi / p.Q;
    const float* w = ws + rh * p.nsplit * (D + 2);
    float M = -__builtin_inff();
    for (int s = 0; s < p.nsplit; s++) M = fmaxf(M, w[s * (D + 2)]);
    float L = 0.f, o = 0.f;
    if (M > -__builtin_inff()) {
        for (int s = 0; s < p.nsplit; s++) {
            float ms = w[s * (D + 2)], ls = w[s * (D + 2) + 1];
            if (ls == 0.f) continue;
            float f = __builtin_expf(ms - M);
            L = fmaf(ls, f, L);
            if (d < D) o = fmaf(w[s * (D + 2) + 2 + d], f, o);
        }
    }
    if (d >= D) return;
    float* orow = out + b * p.o_b + (int64_t)h * p.o_h + i * p.o_i;
    if (L == 0.f) {
        orow[d] = 0.f;
        if (lse && d == 0) lse[(b * p.H + h) * p.Q + i] = -__builtin_inff();
    } else {
        orow[d] = o * (1.0f / L);
        if (lse && d == 0) lse[(b * p.H + h) * p.Q + i] = M + __builtin_logf(L);
    }
}

// D: the width of the values.
size_t attention_workspace_bytes(int64_t B, int H, int64_t Q, int D, int nsplit) {
    return nsplit <= 1 ? 0 : (size_t)(B * Q * H * nsplit * (D + 2)) * sizeof(float);
}

// Keys per workgroup: small enough that one sequence still spreads over the
// chip, large enough to amortise the combine.
void attention_plan(int64_t B, int H, int HK, int64_t Q, int64_t K, int* chunk, int* nsplit) {
    int G = H / HK, ngq = (G + kAttnHeads - 1) / kAttnHeads;
    int64_t rows = B * Q * HK * ngq;
    int c = 256;
    while (c > 32 && rows * ((K + c - 1) / c) < 512) c >>= 1;
    *chunk = c;
    *nsplit = (int)((K + c - 1) / c);
    if (*nsplit < 1) *nsplit = 1;
}

hipError_t attention(const AttnArgs& a, void* workspace, hipStream_t st) {
    if (attention_prompt_ok(a)) return attention_prompt(a, st);  // a prompt: tiles of rows on the matrix cores
    note_kernel("attn_partial_kernel");
    AttnParams p;
    p.q_b = a.q_strides[0]; p.q_h = a.q_strides[1]; p.q_i = a.q_strides[2];
    p.k_b = a.k_strides[0]; p.k_h = a.k_strides[1]; p.k_p = a.k_strides[2];
    p.v_b = a.v_strides[0]; p.v_h = a.v_strides[1]; p.v_p = a.v_strides[2];
    p.o_b = a.o_strides[0]; p.o_h = a.o_strides[1]; p.o_i = a.o_strides[2];
    const int DV = a.DV > 0 ? a.DV : a.D;
    p.m_b = a.m_strides[0]; p.m_h = a.m_strides[1]; p.m_i = a.m_strides[2]; p.m_j = a.m_strides[3];
    p.B = (int)a.B; p.H = a.H; p.HK = a.HK; p.Q = (int)a.Q; p.K = (int)a.K; p.D = a.D; p.DV = DV;
    p.scale = (float)a.scale;
    p.causal = a.causal;
    p.causal_offset = a.causal_offset;
    p.chunk = a.chunk;
    p.nsplit = a.nsplit;
    p.dyn_k = a.dyn_k;
    int G = a.H / a.HK, ngq = (G + kAttnHeads - 1) / kAttnHeads;
    dim3 grid((unsigned)a.nsplit, (unsigned)(a.HK * ngq), (unsigned)(a.B * a.Q));
    int redf = 4 * DV > 32 ? 4 * DV : 32;
    int nslice = kAttnThreads / DV > 0 ? kAttnThreads / DV : 1;
    if ((nslice - 1) * kAttnHeads * DV > redf) redf = (nslice - 1) * kAttnHeads * DV;
    size_t lds = (size_t)(kAttnHeads * a.D + kAttnHeads * a.chunk + redf) * sizeof(float);
    if (a.kv_dtype == kF16)
        hipLaunchKernelGGL(attn_partial_kernel<uint16_t>, grid, dim3(kAttnThreads), lds, st, a.q, (const uint16_t*)a.k,
                           (const uint16_t*)a.v, a.mask, (float*)workspace, a.out, a.lse, p);
    else
        hipLaunchKernelGGL(attn_partial_kernel<float>, grid, dim3(kAttnThreads), lds, st, a.q, (const float*)a.k, (const float*)a.v, a.mask,
                           (float*)workspace, a.out, a.lse, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || a.nsplit == 1) return e;
    hipLaunchKernelGGL(attn_combine_kernel, dim3((unsigned)(a.B * a.Q * a.H)), dim3(256), 0, st, (const float*)workspace, a.out,
                       a.lse, p);
    return hipGetLastError();
}

// No keys at all: every row gets zeros and a logsumexp of -Inf (backend/cpu/attention.go:472-476,494-497), and
// nothing reads k or v. One thread per output element.
__global__ __launch_bounds__(256) void attn_empty_kernel(float* __restrict__ out, float* __restrict__ lse, int64_t o_b, int64_t o_h, int64_t o_i,
                                                         int H, int Q, int DV, int64_t n) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n) return;
    const int d = (int)(t % DV);
    const int64_t row = t / DV;  // (b * H + h) * Q + i
    const int i = (int)(row % Q);
    const int h = (int)(row / Q % H);
    const int64_t b = row / Q / H;
    out[b * o_b + h * o_h + i * o_i + d] = 0.f;
    if (lse && d == 0) lse[row] = -__builtin_inff();
}

hipError_t attention_empty(const AttnArgs& a, hipStream_t st) {
    const int DV = a.DV > 0 ? a.DV : a.D;
    const int64_t n = a.B * a.H * a.Q * DV;
    hipLaunchKernelGGL(attn_empty_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, a.out, a.lse, a.o_strides[0], a.o_strides[1],
                       a.o_strides[2], a.H, (int)a.Q, DV, n);
    return hipGetLastError();
}

}  // namespace mimir
