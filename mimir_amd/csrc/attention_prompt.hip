// Attention for many query positions at once (a prompt) on the float32 matrix cores of gfx950: the semantics of
// attention.hip (softmax(scale * q.k^T) . v per query row, the query scaled first, p = exp(s - max), the result
// (sum p v) * (1 / sum p), the logsumexp max + log(sum p), a row that sees no key zeros and -Inf, key j hidden from
// query i when causal and j > i + causal_offset; backend/cpu/attention.go:268-292, 437-535), for the calls that kernel
// serves one query row a workgroup, re-reading every key and value for every row.
//
// Here a wavefront owns 32 query rows of one head and walks the keys in tiles of 32 with a running maximum and sum per
// row (the rows' results are rescaled when the maximum grows), and both products of a tile are MFMAs on float32
// operands, so that nothing is rounded that the other kernel does not round: scores = Q . K^T with
// v_mfma_f32_32x32x2_f32 over the features (Q's rows live in registers for the whole walk, 64 a lane at 128 features),
// then P . V with the same instruction over the tile's keys, P passing through LDS from the layout an MFMA leaves (a
// lane holds a key's column for 16 rows) to the one it takes (a lane holds a row). A workgroup is four wavefronts with
// consecutive rows of one head, which share the tile of keys and values in LDS (converted to float32 as they are
// loaded; K's rows padded by a float so that 32 keys' equal feature falls on 32 banks). Rows' maxima and sums over a
// tile are reductions over the 32 lanes that hold a row's columns.
//
// What differs from the other kernel is the order of the float32 sums (features and keys in pairs as the MFMA takes
// them, keys in tiles of 32 with rescaling), so results agree to float32 rounding, not bit for bit.
#include "device_util.h"
#include "kernels.h"

namespace mimir {

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kRows = 32;       // query rows a wavefront
constexpr int kWaves = 4;       // wavefronts a workgroup: 128 consecutive rows of one head
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

// Over the 32 lanes that share lane / 32: every lane gets the result.
__device__ __forceinline__ float half_max(float v) {
    v = fmaxf(v, dpp_f32<0xb1>(v));   // quad_perm [1,0,3,2]
    v = fmaxf(v, dpp_f32<0x4e>(v));   // quad_perm [2,3,0,1]
    v = fmaxf(v, dpp_f32<0x141>(v));  // row_half_mirror
    v = fmaxf(v, dpp_f32<0x140>(v));  // row_mirror
    return fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F)));  // lane ^ 16
}
__device__ __forceinline__ float half_sum(float v) {
    v = v + dpp_f32<0xb1>(v);
    v = v + dpp_f32<0x4e>(v);
    v = v + dpp_f32<0x141>(v);
    v = v + dpp_f32<0x140>(v);
    return v + __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F));
}

template <typename KV, int D>
__global__ __launch_bounds__(64 * kWaves) void attn_prompt_kernel(const float* __restrict__ q, const KV* __restrict__ k, const KV* __restrict__ v,
                                                                  float* __restrict__ out, float* __restrict__ lse, PromptParams p) {
    constexpr int KS = D + 1;            // floats between rows of the keys' tile
    constexpr int PS = kTile + 1;        // and of a wavefront's tile of p
    constexpr int NT = D / 32;           // 32-column tiles of the result
    constexpr int PER = D / 8;           // elements of a key (value) row a thread loads: eight threads a row
    __shared__ float ks[kTile * KS];
    __shared__ __align__(16) float vs[kTile * D];
    __shared__ float ps[kWaves * kRows * PS];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r32 = lane & 31, hi = lane >> 5;
    const int b = blockIdx.z, h = blockIdx.y, hk = h / (p.H / p.HK);
    const int i0 = ((int)blockIdx.x * kWaves + wave) * kRows;  // this wavefront's first row
    const int64_t Kt = p.K;
    auto seen_of = [&](int i) -> int {  // keys row i sees
        int64_t s = Kt;
        if (p.causal) {
            s = (int64_t)i + p.causal_offset + 1;
            s = s < 0 ? 0 : s > Kt ? Kt : s;
        }
        return (int)s;
    };
    const int last_row_wg = ((int)blockIdx.x + 1) * kWaves * kRows - 1 < p.Q ? ((int)blockIdx.x + 1) * kWaves * kRows - 1 : p.Q - 1;
    const int last_row_wave = i0 + kRows - 1 < p.Q ? i0 + kRows - 1 : p.Q - 1;
    const int seen_wg = p.causal ? seen_of(last_row_wg) : (int)Kt;
    const int seen_wave = i0 < p.Q ? (p.causal ? seen_of(last_row_wave) : (int)Kt) : 0;

    // Q's rows, scaled, as the MFMA's first operand: lane (row r32, feature 2 s + hi) for s = 0 .. D / 2
    float qreg[D / 2];
    {
        const int i = i0 + r32 < p.Q ? i0 + r32 : p.Q - 1;
        const float* qr = q + b * p.q_b + (int64_t)h * p.q_h + (int64_t)i * p.q_i + hi;
#pragma unroll
        for (int s = 0; s < D / 2; s++) qreg[s] = qr[2 * s] * p.scale;
    }
    // what a lane holds of its 16 rows (register e: row 8 (e / 4) + 4 hi + e % 4): the keys each sees, maximum, sum, result
    int seen[16];
    float m[16], l[16];
    f32x16 o[NT];
#pragma unroll
    for (int e = 0; e < 16; e++) {
        const int i = i0 + 8 * (e >> 2) + 4 * hi + (e & 3);
        seen[e] = i < p.Q ? seen_of(i) : 0;
        m[e] = -__builtin_inff();
        l[e] = 0.f;
    }
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int e = 0; e < 16; e++) o[t][e] = 0.f;

    // a thread's part of a tile's keys and values: row tid / 8, elements [PER (tid % 8), + PER)
    const int lrow = tid >> 3, lpart = tid & 7;
    const KV* kbase = k + b * p.k_b + (int64_t)hk * p.k_h + PER * lpart;
    const KV* vbase = v + b * p.v_b + (int64_t)hk * p.v_h + PER * lpart;
    constexpr int VEC = PER * (int)sizeof(KV) / 16;  // 16-byte pieces of a thread's part (the host checks their alignment)
    uint32_t kreg[4 * VEC], vreg[4 * VEC];
    auto fetch = [&](int j0) {
        int64_t j = j0 + lrow;
        j = j < Kt ? j : Kt - 1;  // rows past the last key: never seen, loaded from the last one
#pragma unroll
        for (int c = 0; c < VEC; c++) {
            const u32x4 kw = ((const u32x4*)(kbase + j * p.k_p))[c], vw = ((const u32x4*)(vbase + j * p.v_p))[c];
#pragma unroll
            for (int w = 0; w < 4; w++) kreg[4 * c + w] = kw[w], vreg[4 * c + w] = vw[w];
        }
    };
    auto stage = [&]() {
#pragma unroll
        for (int e = 0; e < PER; e++) ks[lrow * KS + PER * lpart + e] = element<KV>(kreg, e);
#pragma unroll
        for (int e = 0; e < PER; e += 4) {
            const f32x4 f = {element<KV>(vreg, e), element<KV>(vreg, e + 1), element<KV>(vreg, e + 2), element<KV>(vreg, e + 3)};
            *(f32x4*)(vs + lrow * D + PER * lpart + e) = f;
        }
    };

    float* pw = ps + wave * kRows * PS;
    if (seen_wg > 0) fetch(0);
    for (int j0 = 0; j0 < seen_wg; j0 += kTile) {
        __syncthreads();  // everyone has read the tile before
        stage();
        __syncthreads();
        if (j0 + kTile < seen_wg) fetch(j0 + kTile);
        if (j0 >= seen_wave) continue;  // nothing of this tile is seen by this wavefront's rows (uniform)

        // scores: lane (key j0 + r32) x 16 rows
        f32x16 s;
#pragma unroll
        for (int e = 0; e < 16; e++) s[e] = 0.f;
#pragma unroll
        for (int f = 0; f < D / 2; f++) s = __builtin_amdgcn_mfma_f32_32x32x2f32(qreg[f], ks[r32 * KS + 2 * f + hi], s, 0, 0, 0);
        const int j = j0 + r32;
        float alpha[16];
#pragma unroll
        for (int e = 0; e < 16; e++) {
            const float sc = j < seen[e] ? s[e] : -__builtin_inff();
            const float mx = half_max(sc);
            const float mn = fmaxf(m[e], mx);
            float pe = 0.f, al = 1.f;
            if (mn > -__builtin_inff()) {  // the row has seen a key by now (the same for all its lanes)
                pe = __builtin_expf(sc - mn);
                al = __builtin_expf(m[e] - mn);
            }
            l[e] = l[e] * al + half_sum(pe);
            m[e] = mn;
            alpha[e] = al;
            pw[(8 * (e >> 2) + 4 * hi + (e & 3)) * PS + r32] = pe;
        }
#pragma unroll
        for (int t = 0; t < NT; t++)
#pragma unroll
            for (int e = 0; e < 16; e++) o[t][e] = o[t][e] * alpha[e];
        // p . v: p as the first operand, lane (row r32, key 2 f + hi); a wavefront's LDS accesses complete in order
#pragma unroll
        for (int f = 0; f < kTile / 2; f++) {
            const float pa = pw[r32 * PS + 2 * f + hi];
#pragma unroll
            for (int t = 0; t < NT; t++) o[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(pa, vs[(2 * f + hi) * D + 32 * t + r32], o[t], 0, 0, 0);
        }
    }

#pragma unroll
    for (int e = 0; e < 16; e++) {
        const int i = i0 + 8 * (e >> 2) + 4 * hi + (e & 3);
        if (i >= p.Q) continue;
        float* orow = out + b * p.o_b + (int64_t)h * p.o_h + (int64_t)i * p.o_i;
        const float inv = l[e] == 0.f ? 0.f : 1.0f / l[e];
#pragma unroll
        for (int t = 0; t < NT; t++) orow[32 * t + r32] = l[e] == 0.f ? 0.f : o[t][e] * inv;
        if (lse && r32 == 0) lse[((int64_t)b * p.H + h) * p.Q + i] = l[e] == 0.f ? -__builtin_inff() : m[e] + __builtin_logf(l[e]);
    }
}

std::atomic<int> g_prompt{1};  // measurement aid: 0 keeps every call on the kernel that takes a query row a workgroup

template <typename KV>
hipError_t launch(const AttnArgs& a, const PromptParams& p, hipStream_t st) {
    const dim3 grid((unsigned)((a.Q + kWaves * kRows - 1) / (kWaves * kRows)), (unsigned)a.H, (unsigned)a.B);
    if (a.D == 128)
        hipLaunchKernelGGL((attn_prompt_kernel<KV, 128>), grid, dim3(64 * kWaves), 0, st, a.q, (const KV*)a.k, (const KV*)a.v, a.out, a.lse, p);
    else
        hipLaunchKernelGGL((attn_prompt_kernel<KV, 64>), grid, dim3(64 * kWaves), 0, st, a.q, (const KV*)a.k, (const KV*)a.v, a.out, a.lse, p);
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
        a.HK <= 0 || a.H % a.HK != 0 || a.B <= 0 || a.B > 65535 || a.H > 65535 || a.Q > (1 << 24) || a.K > (1 << 30))
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
    note_kernel("attn_prompt_kernel");
    return a.kv_dtype == kF16 ? launch<uint16_t>(a, p, st) : launch<float>(a, p, st);
}

}  // namespace mimir
