// Attention for many query positions at once (a prompt) on the float32 matrix cores of gfx950: the semantics of
// attention.hip (softmax(scale * q.k^T) . v per query row, the query scaled first, p = exp(s - max), the result
// (sum p v) * (1 / sum p), the logsumexp max + log(sum p), a row that sees no key zeros and -Inf, key j hidden from
// query i when causal and j > i + causal_offset; backend/cpu/attention.go:268-292, 437-535), for the calls that kernel
// serves one query row a workgroup, re-reading every key and value for every row.
//
// Here a wavefront owns 32 query rows of one head and walks the keys in tiles of 32 with a running maximum and sum per
// row (a row's result is rescaled when its maximum grows), and both products of a tile are MFMAs on float32 operands
// (v_mfma_f32_32x32x2_f32), so that nothing is rounded that the other kernel does not round. Both are computed
// transposed, so that everything a row owns lives in one lane (and its partner 32 lanes on): scores^T = K . Q^T over the
// features, the tile's keys as the first operand from LDS and the lane's own row of Q (scaled, in registers for the
// whole walk, 64 a lane at 128 features) as the second, which leaves a lane 16 of its row's 32 scores in registers (the
// partner holds the other 16): maximum and sum are chains over those registers and one exchange with the partner; then
// result^T = V^T . P^T over the tile's keys, taken in the order the scores' registers hold them, so that p goes from the
// exponential straight into the MFMA's second operand, and the lane ends with 16 features of every 32 of its row. A
// workgroup is four wavefronts with consecutive rows of one head, which share the tile of keys and values in LDS
// (converted to float32 as they are loaded, the next tile's rows requested while this one is used; K's rows padded by a
// float so that 32 keys' equal feature falls on 32 banks).
//
// What differs from the other kernel is the order of the float32 sums (features and keys in pairs as the MFMA takes
// them, keys in tiles of 32 with rescaling), so results agree to float32 rounding, not bit for bit.
#include "device_util.h"
#include "kernels.h"

namespace mimir {

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kRows = 32;       // query rows a wavefront
// wavefronts a workgroup (WAVES below): four, 128 consecutive rows of one head, or two where four would leave the device short of workgroups
constexpr int kTile = 32;       // keys a tile

struct PromptParams {
    int64_t q_b, q_h, q_i, k_b, k_h, k_p, v_b, v_h, v_p, o_b, o_h, o_i;
    int B, H, HK, Q, K;
    float scale;
    int causal;
    int64_t causal_offset;
};

// Element e of a row part held as raw 32-bit words.
template <typename KV>
__device__ __forceinline__ float element(const uint32_t* raw, int e);
template <>
__device__ __forceinline__ float element<float>(const uint32_t* raw, int e) { return __builtin_bit_cast(float, raw[e]); }
template <>
__device__ __forceinline__ float element<uint16_t>(const uint32_t* raw, int e) { return f16_bits_to_f32((uint16_t)(raw[e >> 1] >> (16 * (e & 1)))); }

// The other half's value: lane ^ 32.
__device__ __forceinline__ float other_half(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((lane ^ 32) << 2, __builtin_bit_cast(int, v)));
}

template <typename KV, int D, int WAVES>
__global__ __launch_bounds__(64 * WAVES, (sizeof(KV) == 4 && D == 128 && WAVES == 2) ? 1 : 2) void attn_prompt_kernel(const float* __restrict__ q, const KV* __restrict__ k, const KV* __restrict__ v,
                                                                     float* __restrict__ out, float* __restrict__ lse, PromptParams p) {
    constexpr int KS = D + 1;            // floats between rows of the keys' tile
    constexpr int NT = D / 32;           // 32-feature tiles of the result
    constexpr int PER = D / 8;           // elements of a key (value) row a thread loads: eight threads a row
    constexpr int RP = 8 * WAVES;        // rows of a tile the workgroup loads at once
    constexpr int NP = kTile / RP;       // and how often
    __shared__ float ks[kTile * KS];
    __shared__ __align__(16) float vs[kTile * D];
    __shared__ int vbad[2];              // whether a tile's values hold a NaN or an infinity, for tiles of either parity
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r32 = lane & 31, hi = lane >> 5;
    // the grid is (head, sequence, block of rows), the last rows first: under causality they see the most keys, and
    // workgroups are handed out in this order
    const int b = blockIdx.y, h = blockIdx.x, hk = h / (p.H / p.HK), bx = (int)(gridDim.z - 1 - blockIdx.z);
    const int i0 = (bx * WAVES + wave) * kRows;  // this wavefront's first row
    const int64_t Kt = p.K;
    auto seen_of = [&](int i) -> int {  // keys row i sees
        int64_t s = Kt;
        if (p.causal) {
            s = (int64_t)i + p.causal_offset + 1;
            s = s < 0 ? 0 : s > Kt ? Kt : s;
        }
        return (int)s;
    };
    const int last_row_wg = (bx + 1) * WAVES * kRows - 1 < p.Q ? (bx + 1) * WAVES * kRows - 1 : p.Q - 1;
    const int last_row_wave = i0 + kRows - 1 < p.Q ? i0 + kRows - 1 : p.Q - 1;
    const int seen_wg = p.causal ? seen_of(last_row_wg) : (int)Kt;
    const int seen_wave = i0 < p.Q ? (p.causal ? seen_of(last_row_wave) : (int)Kt) : 0;

    // this lane's row, scaled, as the MFMA's second operand: lane (feature 2 s + hi, column r32) for s = 0 .. D / 2
    const int row = i0 + r32;
    float qreg[D / 2];
    {
        const int i = row < p.Q ? row : p.Q - 1;
        const float* qr = q + b * p.q_b + (int64_t)h * p.q_h + (int64_t)i * p.q_i + hi;
#pragma unroll
        for (int s = 0; s < D / 2; s++) qreg[s] = qr[2 * s] * p.scale;
    }
    const int seen = row < p.Q ? seen_of(row) : 0;
    float m = -__builtin_inff(), l = 0.f;  // the row's maximum so far; the sum over the keys this half of the lanes holds
    f32x16 o[NT];                          // the row's result, transposed: register e of tile t is feature 32 t + 8 (e / 4) + 4 hi + e % 4
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int e = 0; e < 16; e++) o[t][e] = 0.f;

    // a thread's part of a tile's keys and values: rows tid / 8 + RP n, elements [PER (tid % 8), + PER)
    const int lrow = tid >> 3, lpart = tid & 7;
    const KV* kbase = k + b * p.k_b + (int64_t)hk * p.k_h + PER * lpart;
    const KV* vbase = v + b * p.v_b + (int64_t)hk * p.v_h + PER * lpart;
    constexpr int VEC = PER * (int)sizeof(KV) / 16;  // 16-byte pieces of a thread's part (the host checks their alignment)
    uint32_t kreg[NP][4 * VEC], vreg[NP][4 * VEC];
    auto fetch = [&](int j0) {
#pragma unroll
        for (int n = 0; n < NP; n++) {
            int64_t j = j0 + lrow + RP * n;
            j = j < Kt ? j : Kt - 1;  // rows past the last key: never seen, loaded from the last one
#pragma unroll
            for (int c = 0; c < VEC; c++) {
                const u32x4 kw = ((const u32x4*)(kbase + j * p.k_p))[c], vw = ((const u32x4*)(vbase + j * p.v_p))[c];
#pragma unroll
                for (int w = 0; w < 4; w++) kreg[n][4 * c + w] = kw[w], vreg[n][4 * c + w] = vw[w];
            }
        }
    };
    auto stage = [&](int parity) {
        float chk = 0.f;  // 0 * value summed: NaN as soon as a value is a NaN or an infinity
#pragma unroll
        for (int n = 0; n < NP; n++) {
            const int r = lrow + RP * n;
#pragma unroll
            for (int e = 0; e < PER; e++) ks[r * KS + PER * lpart + e] = element<KV>(kreg[n], e);
#pragma unroll
            for (int e = 0; e < PER; e += 4) {
                const f32x4 f = {element<KV>(vreg[n], e), element<KV>(vreg[n], e + 1), element<KV>(vreg[n], e + 2), element<KV>(vreg[n], e + 3)};
                *(f32x4*)(vs + r * D + PER * lpart + e) = f;
#pragma unroll
                for (int c = 0; c < 4; c++) chk = __builtin_fmaf(f[c], 0.f, chk);
            }
        }
        if (__builtin_amdgcn_ballot_w64(chk != chk) != 0 && lane == 0) vbad[parity] = 1;
    };

    // The matrix cores multiply a whole tile of values by the rows' weights, zero for the keys a row does not see: fine
    // unless such a value is a NaN or an infinity, which the reference never reads for that row. A tile that holds one and
    // is not seen whole by every row of the wavefront takes the vector units for its second product instead, key by
    // key and only for the rows that see the key.
    const int seen_first = i0 < p.Q ? seen_of(i0) : 0;  // the fewest keys a row of this wavefront sees
    if (tid < 2) vbad[tid] = 0;
    if (seen_wg > 0) fetch(0);
    for (int j0 = 0; j0 < seen_wg; j0 += kTile) {
        const int parity = (j0 / kTile) & 1;
        __syncthreads();  // everyone has read the tile before
        stage(parity);
        __syncthreads();
        if (tid == 0) vbad[parity ^ 1] = 0;  // read last before the first barrier above, set next behind it a tile on
        if (j0 + kTile < seen_wg) fetch(j0 + kTile);
        if (j0 >= seen_wave) continue;  // nothing of this tile is seen by this wavefront's rows (uniform)
        const bool by_key = vbad[parity] != 0 && j0 + kTile > seen_first;

        // scores, transposed (K . Q^T): register e is key j0 + 8 (e / 4) + 4 hi + e % 4 against this lane's row
        f32x16 s;
#pragma unroll
        for (int e = 0; e < 16; e++) s[e] = 0.f;
#pragma unroll
        for (int f = 0; f < D / 2; f++) s = __builtin_amdgcn_mfma_f32_32x32x2f32(ks[r32 * KS + 2 * f + hi], qreg[f], s, 0, 0, 0);
        float mx = -__builtin_inff();
#pragma unroll
        for (int e = 0; e < 16; e++) {
            const int j = j0 + 8 * (e >> 2) + 4 * hi + (e & 3);
            s[e] = j < seen ? s[e] : -__builtin_inff();
            mx = fmaxf(mx, s[e]);
        }
        mx = fmaxf(mx, other_half(mx, lane));
        const float mn = fmaxf(m, mx);
        float al = 1.f, sum = 0.f;
        if (mn > -__builtin_inff()) {  // the row has seen a key by now
            al = __builtin_expf(m - mn);
#pragma unroll
            for (int e = 0; e < 16; e++) {
                s[e] = __builtin_expf(s[e] - mn);
                sum += s[e];
            }
        } else {
#pragma unroll
            for (int e = 0; e < 16; e++) s[e] = 0.f;
        }
        l = l * al + sum;
        m = mn;
#pragma unroll
        for (int t = 0; t < NT; t++)
#pragma unroll
            for (int e = 0; e < 16; e++) o[t][e] = o[t][e] * al;
        // result, transposed (V^T . P^T) over the tile's keys in the order the scores' registers hold them: step f takes
        // key 8 (f / 4) + 4 hi + f % 4 from each half, whose weight for this lane's row is register f
        if (!by_key) {
#pragma unroll
            for (int f = 0; f < kTile / 2; f++) {
                const int key = 8 * (f >> 2) + 4 * hi + (f & 3);
#pragma unroll
                for (int t = 0; t < NT; t++) o[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(vs[key * D + 32 * t + r32], s[f], o[t], 0, 0, 0);
            }
        } else {
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const float theirs = other_half(s[e], lane);
#pragma unroll
                for (int hk = 0; hk < 2; hk++) {  // the key that register e holds in the lanes of half hk
                    const int key = 8 * (e >> 2) + 4 * hk + (e & 3);
                    const float pk = hi == hk ? s[e] : theirs;
                    if (j0 + key < seen) {
#pragma unroll
                        for (int t = 0; t < NT; t++)
#pragma unroll
                            for (int g = 0; g < 4; g++) {
                                const f32x4 vv = *(const f32x4*)(vs + key * D + 32 * t + 8 * g + 4 * hi);
#pragma unroll
                                for (int c = 0; c < 4; c++) o[t][4 * g + c] = __builtin_fmaf(pk, vv[c], o[t][4 * g + c]);
                            }
                    }
                }
            }
        }
    }

    l += other_half(l, lane);
    if (row >= p.Q) return;
    float* orow = out + b * p.o_b + (int64_t)h * p.o_h + (int64_t)row * p.o_i;
    const float inv = l == 0.f ? 0.f : 1.0f / l;
    const bool wide = (((uintptr_t)orow) & 15) == 0;
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
            f32x4 r;
#pragma unroll
            for (int c = 0; c < 4; c++) r[c] = l == 0.f ? 0.f : o[t][4 * g + c] * inv;
            float* dst = orow + 32 * t + 8 * g + 4 * hi;
            if (wide) *(f32x4*)dst = r;
            else
#pragma unroll
                for (int c = 0; c < 4; c++) dst[c] = r[c];
        }
    if (lse && hi == 0) lse[((int64_t)b * p.H + h) * p.Q + row] = l == 0.f ? -__builtin_inff() : m + __builtin_logf(l);
}

std::atomic<int> g_prompt{1};  // measurement aid: 0 keeps every call on the kernel that takes a query row a workgroup

template <typename KV, int WAVES>
hipError_t launch(const AttnArgs& a, const PromptParams& p, hipStream_t st) {
    const dim3 grid((unsigned)a.H, (unsigned)a.B, (unsigned)((a.Q + WAVES * kRows - 1) / (WAVES * kRows)));
    if (a.D == 128)
        hipLaunchKernelGGL((attn_prompt_kernel<KV, 128, WAVES>), grid, dim3(64 * WAVES), 0, st, a.q, (const KV*)a.k, (const KV*)a.v, a.out, a.lse, p);
    else
        hipLaunchKernelGGL((attn_prompt_kernel<KV, 64, WAVES>), grid, dim3(64 * WAVES), 0, st, a.q, (const KV*)a.k, (const KV*)a.v, a.out, a.lse, p);
    return hipGetLastError();
}

}  // namespace

void set_attention_prompt(int v) { g_prompt = v; }

// Calls this kernel takes: at least 64 query positions, keys and values of 64 or 128 features in float32 or binary16
// whose rows start on 16 bytes (a thread loads an eighth of a row), no additive mask, no device-side key count.
bool attention_prompt_ok(const AttnArgs& a) {
    const int DV = a.DV > 0 ? a.DV : a.D;
    const int esz = a.kv_dtype == kF16 ? 2 : 4;
    if (g_prompt == 0 || a.mask || a.dyn_k || a.Q < 64 || a.K < 1 || DV != a.D || (a.D != 64 && a.D != 128) || (a.kv_dtype != kF16 && a.kv_dtype != kF32) ||
        a.HK <= 0 || a.H % a.HK != 0 || a.B <= 0 || a.B > 65535 || a.H > 65535 || a.Q > (1 << 22) || a.K > (1 << 30))
        return false;
    for (int s = 0; s < 3; s++)
        if ((a.k_strides[s] * esz) % 16 != 0 || (a.v_strides[s] * esz) % 16 != 0) return false;
    return ((uintptr_t)a.k & 15) == 0 && ((uintptr_t)a.v & 15) == 0;
}

hipError_t attention_prompt(const AttnArgs& a, hipStream_t st) {
    PromptParams p;
    p.q_b = a.q_strides[0]; p.q_h = a.q_strides[1]; p.q_i = a.q_strides[2];
    p.k_b = a.k_strides[0]; p.k_h = a.k_strides[1]; p.k_p = a.k_strides[2];
    p.v_b = a.v_strides[0]; p.v_h = a.v_strides[1]; p.v_p = a.v_strides[2];
    p.o_b = a.o_strides[0]; p.o_h = a.o_strides[1]; p.o_i = a.o_strides[2];
    p.B = (int)a.B; p.H = a.H; p.HK = a.HK; p.Q = (int)a.Q; p.K = (int)a.K;
    p.scale = (float)a.scale;
    p.causal = a.causal;
    p.causal_offset = a.causal_offset;
    // workgroups of two wavefronts where those of four would be fewer than the device holds at two a compute unit
    const bool two = a.B * a.H * ((a.Q + 4 * kRows - 1) / (4 * kRows)) < 512;
    note_kernel("attn_prompt_kernel");
    if (a.kv_dtype == kF16) return two ? launch<uint16_t, 2>(a, p, st) : launch<uint16_t, 4>(a, p, st);
    return two ? launch<float, 2>(a, p, st) : launch<float, 4>(a, p, st);
}

}  // namespace mimir
