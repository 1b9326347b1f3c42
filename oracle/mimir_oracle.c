/*
 * TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A CPU restatement, in plain C, of the arithmetic of mimir's CPU backend on
 * the quantized-matmul decode path. Only tests, the smoke check and the
 * benchmark's cpu_baseline leg may load it, and only as the checker; the
 * product (the HIP library) never links or calls anything here.
 *
 * Every function cites the reference file:line it follows (paths relative to
 * the reference checkout). Build with -ffp-contract=off: the reference rounds
 * every product and sum to float32 on its own and never fuses them.
 *
 * What pins each function (beyond reading the reference):
 *   f16/bf16 conversions    exhaustive over 65 536 halves vs numpy.float16;
 *                           sampled float32 vs numpy / torch.bfloat16
 *   dequant Q8_0/Q4_K/Q6_K  bit-exact vs the reference's golden quant.mim
 *   quantize_row            tie and invariants cases of the reference's tests,
 *                           float64 twin
 *   qdot / qmatmul          golden quant.mim *_matmul (1e-5), float64 brute
 *                           force within the analytic bound, exact-row inputs
 *   rmsnorm, rope, attention golden attention.mim cases, brute force
 *   whole model             spm/bpe logits, tiny-q4km expected.json
 *   dequant Q4_0            PARITY UNPINNED: the reference holds no Q4_0
 *                           vector (its decoder lives in the external module
 *                           github.com/gsoultan/mimir-model v0.3.0, call site
 *                           io/mim/dtype.go:118-123). Restated from ggml's
 *                           published block_q4_0 (low nibbles are elements
 *                           0..15, high nibbles 16..31, value (n-8)*d) and
 *                           checked by closed form and brute force only.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define MO_EXPORT __attribute__((visibility("default")))

/* dtype codes shared with the device library (include/mimir_mi355x.h). */
enum { MO_F32 = 1, MO_I32 = 2, MO_BF16 = 3, MO_F16 = 4, MO_Q8_0 = 5, MO_Q4_K = 6, MO_Q6_K = 7, MO_Q4_0 = 8 };

static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint16_t le16(const uint8_t *b) { return (uint16_t)(b[0] | (uint16_t)b[1] << 8); }

/* ---- half conversions: backend/cpu/half.go:37-102 ---------------------- */

MO_EXPORT float mo_bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

/* half.go:42-51: RNE; a NaN keeps its sign and payload top, made quiet. */
MO_EXPORT uint16_t mo_f32_to_bf16(float f) {
    uint32_t b = f32_bits(f);
    if ((b & 0x7fffffffu) > 0x7f800000u) return (uint16_t)(b >> 16) | 0x0040;
    b += 0x7fffu + ((b >> 16) & 1u);
    return (uint16_t)(b >> 16);
}

/* half.go:54-74 */
MO_EXPORT float mo_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000) << 16;
    uint32_t exp = (h >> 10) & 0x1f;
    uint32_t mant = h & 0x3ff;
    if (exp == 0) {
        if (mant == 0) return bits_f32(sign);
        uint32_t shift = (uint32_t)__builtin_clz(mant) - 21;
        mant = (mant << shift) & 0x3ff;
        return bits_f32(sign | (113 - shift) << 23 | mant << 13);
    }
    if (exp == 0x1f) return bits_f32(sign | 0x7f800000u | mant << 13);
    return bits_f32(sign | (exp + 112) << 23 | mant << 13);
}

/* half.go:105-112 */
static inline uint32_t round_half_even(uint32_t h, uint32_t m, unsigned shift) {
    uint32_t rest = m & ((1u << shift) - 1);
    uint32_t half = 1u << (shift - 1);
    if (rest > half || (rest == half && (h & 1))) h++;
    return h;
}

/* half.go:80-103 */
MO_EXPORT uint16_t mo_f32_to_f16(float f) {
    uint32_t b = f32_bits(f);
    uint16_t sign = (uint16_t)(b >> 16) & 0x8000;
    b &= 0x7fffffffu;
    if (b > 0x7f800000u) return sign | 0x7e00 | ((uint16_t)(b >> 13) & 0x1ff);
    int exp = (int)(b >> 23) - 127;
    uint32_t mant = b & 0x7fffff;
    if (exp > 15) return sign | 0x7c00;
    if (exp >= -14) {
        uint32_t h = (uint32_t)(exp + 15) << 10 | mant >> 13;
        return sign | (uint16_t)round_half_even(h, mant, 13);
    }
    if (exp >= -25) {
        uint32_t m = mant | 0x800000;
        unsigned shift = (unsigned)(-exp - 1);
        return sign | (uint16_t)round_half_even(m >> shift, m, shift);
    }
    return sign;
}

MO_EXPORT void mo_f16_to_f32_n(const uint16_t *h, float *out, int64_t n) { for (int64_t i = 0; i < n; i++) out[i] = mo_f16_to_f32(h[i]); }
MO_EXPORT void mo_f32_to_f16_n(const float *f, uint16_t *out, int64_t n) { for (int64_t i = 0; i < n; i++) out[i] = mo_f32_to_f16(f[i]); }
MO_EXPORT void mo_bf16_to_f32_n(const uint16_t *h, float *out, int64_t n) { for (int64_t i = 0; i < n; i++) out[i] = mo_bf16_to_f32(h[i]); }
MO_EXPORT void mo_f32_to_bf16_n(const float *f, uint16_t *out, int64_t n) { for (int64_t i = 0; i < n; i++) out[i] = mo_f32_to_bf16(f[i]); }

/* ---- block accounting: backend/quant.go:18-59 (+ Q4_0, 32 per 18 bytes) -- */

MO_EXPORT int mo_block_size(int dt) {
    switch (dt) {
    case MO_Q8_0: case MO_Q4_0: return 32;
    case MO_Q4_K: case MO_Q6_K: return 256;
    default: return 1;
    }
}

MO_EXPORT int mo_block_bytes(int dt) {
    switch (dt) {
    case MO_Q8_0: return 34;
    case MO_Q4_0: return 18;
    case MO_Q4_K: return 144;
    case MO_Q6_K: return 210;
    case MO_F32: case MO_I32: return 4;
    case MO_BF16: case MO_F16: return 2;
    default: return 0;
    }
}

/* ---- dequantizers: backend/cpu/quant.go:113-181 ------------------------- */

/* quant.go:120-125 */
static void dequant_q8_0(float *dst, const uint8_t *b) {
    float d = mo_f16_to_f32(le16(b));
    for (int i = 0; i < 32; i++) dst[i] = (float)(int8_t)b[2 + i] * d;
}

/* ggml block_q4_0 (not in the reference; see the header): d f16 at 0, 16 bytes
 * of nibbles at 2; element j is the low nibble of byte j, element j+16 its
 * high nibble; value (n - 8) * d. */
static void dequant_q4_0(float *dst, const uint8_t *b) {
    float d = mo_f16_to_f32(le16(b));
    for (int j = 0; j < 16; j++) {
        dst[j] = (float)((int)(b[2 + j] & 0xf) - 8) * d;
        dst[j + 16] = (float)((int)(b[2 + j] >> 4) - 8) * d;
    }
}

/* quant.go:129-134 */
static inline void scale_min_k4(int j, const uint8_t *s, uint8_t *sc, uint8_t *m) {
    if (j < 4) { *sc = s[j] & 63; *m = s[j + 4] & 63; return; }
    *sc = (uint8_t)((s[j + 4] & 0xf) | (s[j - 4] >> 6) << 4);
    *m = (uint8_t)((s[j + 4] >> 4) | (s[j] >> 6) << 4);
}

/* quant.go:140-154 */
static void dequant_q4k(float *dst, const uint8_t *b) {
    float d = mo_f16_to_f32(le16(b)), dmin = mo_f16_to_f32(le16(b + 2));
    const uint8_t *scales = b + 4, *qs = b + 16;
    for (int j = 0; j < 4; j++) {
        const uint8_t *q = qs + 32 * j;
        float *y = dst + 64 * j;
        uint8_t sc, m;
        scale_min_k4(2 * j, scales, &sc, &m);
        float d1 = d * (float)sc, m1 = dmin * (float)m;
        scale_min_k4(2 * j + 1, scales, &sc, &m);
        float d2 = d * (float)sc, m2 = dmin * (float)m;
        for (int l = 0; l < 32; l++) {
            float t1 = d1 * (float)(q[l] & 0xf);
            float t2 = d2 * (float)(q[l] >> 4);
            y[l] = t1 - m1;
            y[l + 32] = t2 - m2;
        }
    }
}

/* quant.go:159-165 */
static inline int q6(const uint8_t *ql, const uint8_t *qh, int k, int l) {
    uint8_t lo = ql[l + 32 * (k & 1)];
    if (k >= 2) lo >>= 4;
    return (int)((lo & 0xf) | ((qh[l] >> (2 * k)) & 3) << 4);
}

/* quant.go:170-181 */
static void dequant_q6k(float *dst, const uint8_t *b) {
    float d = mo_f16_to_f32(le16(b + 208));
    for (int n = 0; n < 2; n++) {
        const uint8_t *ql = b + 64 * n, *qh = b + 128 + 32 * n, *sc = b + 192 + 8 * n;
        float *y = dst + 128 * n;
        for (int k = 0; k < 4; k++)
            for (int l = 0; l < 32; l++) {
                float s = d * (float)(int8_t)sc[l / 16 + 2 * k];
                y[32 * k + l] = s * (float)(q6(ql, qh, k, l) - 32);
            }
    }
}

static void dequant_block(int dt, float *dst, const uint8_t *b) {
    switch (dt) {
    case MO_Q8_0: dequant_q8_0(dst, b); break;
    case MO_Q4_0: dequant_q4_0(dst, b); break;
    case MO_Q4_K: dequant_q4k(dst, b); break;
    default: dequant_q6k(dst, b); break;
    }
}

/* quant.go:185-194, whole blocks. */
MO_EXPORT void mo_dequantize(int dt, const uint8_t *data, int64_t nblocks, float *out) {
    int bs = mo_block_size(dt), bb = mo_block_bytes(dt);
#pragma omp parallel for schedule(static) if (nblocks > 4096)
    for (int64_t i = 0; i < nblocks; i++) dequant_block(dt, out + i * bs, data + i * bb);
}

/* quant.go:198-218: one element, the per-element path of strided casts and
 * gathers. Note the Q4_K expression differs from the block form in where it
 * rounds: d*sc*q is (d*sc) then *q, the same two roundings. */
MO_EXPORT float mo_dequant_at(int dt, const uint8_t *data, int64_t i) {
    int bs = mo_block_size(dt), bb = mo_block_bytes(dt);
    const uint8_t *b = data + i / bs * bb;
    int j = (int)(i % bs);
    switch (dt) {
    case MO_Q8_0:
        return (float)(int8_t)b[2 + j] * mo_f16_to_f32(le16(b));
    case MO_Q4_0: {
        int n = j < 16 ? (b[2 + j] & 0xf) : (b[2 + j - 16] >> 4);
        return (float)(n - 8) * mo_f16_to_f32(le16(b));
    }
    case MO_Q4_K: {
        float d = mo_f16_to_f32(le16(b)), dmin = mo_f16_to_f32(le16(b + 2));
        int sub = j / 32, l = j % 32;
        uint8_t sc, m;
        scale_min_k4(sub, b + 4, &sc, &m);
        uint8_t v = b[16 + 32 * (sub / 2) + l];
        if (sub % 2 == 1) v >>= 4;
        float t = d * (float)sc;
        t = t * (float)(v & 0xf);
        float mm = dmin * (float)m;
        return t - mm;
    }
    default: {
        int n = j / 128, k = j % 128 / 32, l = j % 32;
        float s = mo_f16_to_f32(le16(b + 208)) * (float)(int8_t)b[192 + 8 * n + l / 16 + 2 * k];
        return s * (float)(q6(b + 64 * n, b + 128 + 32 * n, k, l) - 32);
    }
    }
}

/* quant.go:222-256 (OpCast of a block-quantized input): values rounded to
 * the output dtype with half.go's conversions. out_dt is MO_F32/BF16/F16. */
MO_EXPORT void mo_dequantize_to(int dt, const uint8_t *data, int64_t nblocks, void *out, int out_dt) {
    int bs = mo_block_size(dt), bb = mo_block_bytes(dt);
    if (out_dt == MO_F32) { mo_dequantize(dt, data, nblocks, (float *)out); return; }
    uint16_t *o = (uint16_t *)out;
    for (int64_t i = 0; i < nblocks; i++) {
        float tmp[256];
        dequant_block(dt, tmp, data + i * bb);
        for (int j = 0; j < bs; j++)
            o[i * bs + j] = out_dt == MO_BF16 ? mo_f32_to_bf16(tmp[j]) : mo_f32_to_f16(tmp[j]);
    }
}

/* quant.go:296-327 (OpGather, axis 0 of a [rows, k] table): out[r, :] =
 * dequant(table[idx[r], :]). Returns -1 on an index out of range (ErrIndex). */
MO_EXPORT int mo_gather_rows(int dt, const uint8_t *table, int64_t rows, int64_t k, const int32_t *idx, int64_t n, float *out) {
    for (int64_t r = 0; r < n; r++) {
        int64_t j = idx[r];
        if (j < 0 || j >= rows) return -1;
        for (int64_t c = 0; c < k; c++) out[r * k + c] = mo_dequant_at(dt, table, j * k + c);
    }
    return 0;
}

/* ---- activations: backend/cpu/qmatmul.go:202-262 ------------------------ */

/* qmatmul.go:259-262 */
static inline int32_t round_even(float f) {
    const float magic = 0x1.8p23f;
    volatile float t = f + magic; /* volatile: keep both float32 roundings */
    t = t - magic;
    return (int32_t)t;
}

/* qmatmul.go:208-254. dst blocks: f32 d | int8 q[bs] | (sums) int16 s[bs/16]. */
MO_EXPORT void mo_quantize_row(uint8_t *dst, const float *x, int64_t k, int bs, int sums) {
    int stride = 4 + bs + (sums ? 32 : 0);
    for (int64_t b = 0; b < k / bs; b++) {
        const float *v = x + b * bs;
        uint8_t *out = dst + b * stride;
        float amax = 0;
        int finite = 1;
        for (int i = 0; i < bs; i++) {
            uint32_t u = f32_bits(v[i]) & 0x7fffffffu;
            if (u >= 0x7f800000u) finite = 0;
            float a = bits_f32(u);
            if (a > amax) amax = a;
        }
        int8_t *q = (int8_t *)(out + 4);
        float d = 0;
        if (!finite) {
            d = bits_f32(0x7fc00000u);
            memset(q, 0, (size_t)bs);
        } else if (amax == 0) {
            memset(q, 0, (size_t)bs);
        } else {
            d = amax / 127;
            float id = 127 / amax;
            for (int i = 0; i < bs; i++) {
                int32_t r = round_even(v[i] * id);
                if (r > 127) r = 127;
                if (r < -127) r = -127;
                q[i] = (int8_t)r;
            }
        }
        memcpy(out, &d, 4);
        if (!sums) continue;
        uint8_t *s = out + 4 + bs;
        for (int g = 0; g < bs / 16; g++) {
            int32_t t = 0;
            for (int c = 0; c < 16; c++) t += q[16 * g + c];
            s[2 * g] = (uint8_t)t;
            s[2 * g + 1] = (uint8_t)(t >> 8);
        }
    }
}

static inline float f32_at(const uint8_t *b) { float f; memcpy(&f, b, 4); return f; }
static inline int32_t i16_at(const uint8_t *b) { return (int32_t)(int16_t)le16(b); }

/* ---- dot products: backend/cpu/qmatmul.go:119-200 ----------------------- */

/* qmatmul.go:125-139 */
MO_EXPORT float mo_qdot_q8_0(int64_t nb, const uint8_t *w, const uint8_t *x) {
    float acc[4] = {0, 0, 0, 0};
    for (int64_t b = 0; b < nb; b++) {
        const uint8_t *wb = w + 34 * b, *xb = x + 36 * b;
        int32_t s[4] = {0, 0, 0, 0};
        for (int p = 0; p < 32; p++) s[p / 4 % 4] += (int32_t)(int8_t)wb[2 + p] * (int32_t)(int8_t)xb[4 + p];
        float dd = mo_f16_to_f32(le16(wb)) * f32_at(xb);
        for (int l = 0; l < 4; l++) {
            float t = dd * (float)s[l];
            acc[l] += t;
        }
    }
    return (acc[0] + acc[2]) + (acc[1] + acc[3]);
}

/* qmatmul.go:148-172 */
MO_EXPORT float mo_qdot_q4k(int64_t nb, const uint8_t *w, const uint8_t *x) {
    float acc = 0, accm = 0;
    for (int64_t b = 0; b < nb; b++) {
        const uint8_t *wb = w + 144 * b, *xb = x + 292 * b;
        const uint8_t *scales = wb + 4, *sums = xb + 260;
        const int8_t *xq = (const int8_t *)(xb + 4);
        int32_t sumi = 0, summ = 0;
        for (int j = 0; j < 4; j++) {
            const uint8_t *q = wb + 16 + 32 * j;
            int32_t lo = 0, hi = 0;
            for (int l = 0; l < 32; l++) {
                lo += (int32_t)(q[l] & 0xf) * (int32_t)xq[64 * j + l];
                hi += (int32_t)(q[l] >> 4) * (int32_t)xq[64 * j + 32 + l];
            }
            uint8_t sc0, m0, sc1, m1;
            scale_min_k4(2 * j, scales, &sc0, &m0);
            scale_min_k4(2 * j + 1, scales, &sc1, &m1);
            sumi += (int32_t)sc0 * lo + (int32_t)sc1 * hi;
            summ += (int32_t)m0 * (i16_at(sums + 8 * j) + i16_at(sums + 8 * j + 2)) +
                    (int32_t)m1 * (i16_at(sums + 8 * j + 4) + i16_at(sums + 8 * j + 6));
        }
        float xd = f32_at(xb);
        float dd = mo_f16_to_f32(le16(wb)) * xd, dm = mo_f16_to_f32(le16(wb + 2)) * xd;
        float t = dd * (float)sumi;
        acc += t;
        float u = dm * (float)summ;
        accm += u;
    }
    return acc - accm;
}

/* qmatmul.go:180-200 */
MO_EXPORT float mo_qdot_q6k(int64_t nb, const uint8_t *w, const uint8_t *x) {
    float acc = 0;
    for (int64_t b = 0; b < nb; b++) {
        const uint8_t *wb = w + 210 * b, *xb = x + 292 * b;
        const int8_t *xq = (const int8_t *)(xb + 4);
        const uint8_t *sums = xb + 260;
        int32_t sumi = 0;
        for (int g = 0; g < 16; g++) {
            int n = g / 8, k = g % 8 / 2, l0 = 16 * (g % 2);
            const uint8_t *ql = wb + 64 * n, *qh = wb + 128 + 32 * n;
            int32_t s = 0;
            for (int l = l0; l < l0 + 16; l++) s += (int32_t)q6(ql, qh, k, l) * (int32_t)xq[128 * n + 32 * k + l];
            int32_t sc = (int32_t)(int8_t)wb[192 + g];
            sumi += sc * s - 32 * sc * i16_at(sums + 2 * g);
        }
        float dd = mo_f16_to_f32(le16(wb + 208)) * f32_at(xb);
        float t = dd * (float)sumi;
        acc += t;
    }
    return acc;
}

/* AVX2 twin of mo_qdot_q8_0 with the reference's instruction sequence,
 * vpsignb, vpmaddubsw, vpmaddwd, fold, cvt, mul, add
 * (tools/asmgen/qamd64/main.go:173-226); bit-identical to the scalar one by
 * construction (integer sums are exact; the float lanes and their order
 * match). Used for the CPU baseline timing. */
#if defined(__x86_64__)
#include <immintrin.h>
__attribute__((target("avx2,f16c")))
static float qdot_q8_0_avx2(int64_t nb, const uint8_t *w, const uint8_t *x) {
    __m128 acc = _mm_setzero_ps();
    const __m256i ones = _mm256_set1_epi16(1);
    for (int64_t b = 0; b < nb; b++) {
        const uint8_t *wb = w + 34 * b, *xb = x + 36 * b;
        __m256i q = _mm256_loadu_si256((const __m256i *)(wb + 2));
        __m256i aq = _mm256_sign_epi8(q, q);
        __m256i p = _mm256_loadu_si256((const __m256i *)(xb + 4));
        p = _mm256_sign_epi8(p, q);
        p = _mm256_maddubs_epi16(aq, p);
        p = _mm256_madd_epi16(ones, p);
        __m128i s = _mm_add_epi32(_mm256_extracti128_si256(p, 1), _mm256_castsi256_si128(p));
        __m128 sf = _mm_cvtepi32_ps(s);
        float dd = mo_f16_to_f32(le16(wb)) * f32_at(xb);
        sf = _mm_mul_ps(_mm_set1_ps(dd), sf);
        acc = _mm_add_ps(sf, acc);
    }
    float a[4];
    _mm_storeu_ps(a, acc);
    return (a[0] + a[2]) + (a[1] + a[3]);
}
static int have_avx2(void) { return __builtin_cpu_supports("avx2"); }
#else
static int have_avx2(void) { return 0; }
#endif

MO_EXPORT float mo_qdot_q8_0_simd(int64_t nb, const uint8_t *w, const uint8_t *x) {
#if defined(__x86_64__)
    if (have_avx2()) return qdot_q8_0_avx2(nb, w, x);
#endif
    return mo_qdot_q8_0(nb, w, x);
}

MO_EXPORT int mo_has_simd(void) { return have_avx2(); }

/* ---- float dot and GEMV: backend/cpu/gemv.go:110-148 -------------------- */

/* gemv.go:128-148, the portable dot: eight strided partial sums. */
MO_EXPORT float mo_dot(const float *a, const float *b, int64_t n) {
    float s0 = 0, s1 = 0, s2 = 0, s3 = 0, s4 = 0, s5 = 0, s6 = 0, s7 = 0;
    int64_t i = 0;
    for (; i + 8 <= n; i += 8) {
        s0 += a[i] * b[i];
        s1 += a[i + 1] * b[i + 1];
        s2 += a[i + 2] * b[i + 2];
        s3 += a[i + 3] * b[i + 3];
        s4 += a[i + 4] * b[i + 4];
        s5 += a[i + 5] * b[i + 5];
        s6 += a[i + 6] * b[i + 6];
        s7 += a[i + 7] * b[i + 7];
    }
    for (; i < n; i++) s0 += a[i] * b[i];
    return ((s0 + s1) + (s2 + s3)) + ((s4 + s5) + (s6 + s7));
}

/* gemv.go:73-104: out[i, c] = dot(x[i, :], w[c, :]) for few rows of x,
 * workers taking groups of four rows of w. threads <= 0 means all cores. */
MO_EXPORT void mo_sgemv(const float *w, const float *x, float *out, int64_t m, int64_t n, int64_t k, int threads) {
    int64_t groups = (n + 3) / 4;
#ifdef _OPENMP
    if (threads <= 0) threads = omp_get_max_threads();
#endif
#pragma omp parallel for schedule(static) num_threads(threads)
    for (int64_t g = 0; g < groups; g++)
        for (int64_t i = 0; i < m; i++)
            for (int64_t c = 4 * g; c < n && c < 4 * g + 4; c++) out[i * n + c] = mo_dot(x + i * k, w + c * k, k);
}

/* ---- products by quantized weights -------------------------------------- */

/* runQMatMul, backend/cpu/qmatmul.go:310-405, for contiguous rows of x
 * (x_row_stride elements apart): quantize each row of x, then one qdot per
 * output. Q8_0, Q4_K, Q6_K only. simd picks the AVX2 Q8_0 kernel. */
MO_EXPORT int mo_qmatmul(int dt, const uint8_t *w, const float *x, float *out, int64_t m, int64_t n, int64_t k,
                         int64_t x_row_stride, int simd, int threads) {
    if (dt != MO_Q8_0 && dt != MO_Q4_K && dt != MO_Q6_K) return -1;
    int bs = mo_block_size(dt), bb = mo_block_bytes(dt);
    if (k % bs) return -1;
    int abs_ = dt == MO_Q8_0 ? 32 : 256, abb = dt == MO_Q8_0 ? 36 : 292;
    int64_t xstride = k / abs_ * abb, nb = k / bs, wstride = nb * bb;
    uint8_t *xq = (uint8_t *)malloc((size_t)(m * xstride + 1));
    if (!xq) return -2;
    for (int64_t i = 0; i < m; i++) mo_quantize_row(xq + i * xstride, x + i * x_row_stride, k, abs_, abs_ == 256);
#ifdef _OPENMP
    if (threads <= 0) threads = omp_get_max_threads();
#endif
#pragma omp parallel for schedule(dynamic, 16) num_threads(threads)
    for (int64_t j = 0; j < n; j++) {
        const uint8_t *wrow = w + j * wstride;
        for (int64_t i = 0; i < m; i++) {
            const uint8_t *xr = xq + i * xstride;
            float r;
            if (dt == MO_Q8_0) r = simd ? mo_qdot_q8_0_simd(nb, wrow, xr) : mo_qdot_q8_0(nb, wrow, xr);
            else if (dt == MO_Q4_K) r = mo_qdot_q4k(nb, wrow, xr);
            else r = mo_qdot_q6k(nb, wrow, xr);
            out[i * n + j] = r;
        }
    }
    free(xq);
    return 0;
}

/* The reference's route for a Q4_0 linear: the file's blocks are decoded to
 * float32 when the model opens (io/mim/dtype.go:118-123) and the product is
 * the float32 one (tensor/quant.go:40-42 -> MatMul -> gemv.go:73-104). This
 * computes exactly that without keeping the float32 matrix: each row of W
 * is dequantized (exactly: (n-8)*d has 15 significant bits) into a scratch
 * row and multiplied with mo_dot. */
MO_EXPORT int mo_q4_0_matmul_f32(const uint8_t *w, const float *x, float *out, int64_t m, int64_t n, int64_t k,
                                 int64_t x_row_stride, int threads) {
    if (k % 32) return -1;
    int64_t nb = k / 32;
#ifdef _OPENMP
    if (threads <= 0) threads = omp_get_max_threads();
#endif
#pragma omp parallel num_threads(threads)
    {
        float *row = (float *)malloc((size_t)k * sizeof(float) + 4);
#pragma omp for schedule(static)
        for (int64_t j = 0; j < n; j++) {
            for (int64_t b = 0; b < nb; b++) dequant_q4_0(row + 32 * b, w + (j * nb + b) * 18);
            for (int64_t i = 0; i < m; i++) out[i * n + j] = mo_dot(x + i * x_row_stride, row, k);
        }
        free(row);
    }
    return 0;
}

/* The product a half x takes (tensor/quant.go:44-48): x is widened to
 * float32, multiplied as above, and the result rounded once to bf16. */
MO_EXPORT int mo_q4_0_matmul_bf16(const uint8_t *w, const uint16_t *x_bf16, uint16_t *out_bf16, int64_t m, int64_t n,
                                  int64_t k, int threads) {
    float *x = (float *)malloc((size_t)(m * k) * 4 + 4), *o = (float *)malloc((size_t)(m * n) * 4 + 4);
    if (!x || !o) { free(x); free(o); return -2; }
    mo_bf16_to_f32_n(x_bf16, x, m * k);
    int rc = mo_q4_0_matmul_f32(w, x, o, m, n, k, k, threads);
    if (rc == 0) mo_f32_to_bf16_n(o, out_bf16, m * n);
    free(x); free(o);
    return rc;
}

/* ---- RMSNorm: nn/transformer.go:50-61; llm/decode.go:376-385 ------------ */

/* y = cast(x * recip(sqrt(mean(x^2) + eps))) * w, normalised in float32.
 * The sum of squares runs in mo_dot's order (the decode twin computes it as
 * a product of x with itself); mean = sum * float32(1/d); eps is added as a
 * float32. w may be NULL. */
MO_EXPORT void mo_rmsnorm(const float *x, const float *w, float *y, int64_t rows, int64_t d, double eps) {
    float inv_d = (float)(1.0 / (double)d), e = (float)eps;
    for (int64_t r = 0; r < rows; r++) {
        const float *xr = x + r * d;
        float ss = mo_dot(xr, xr, d);
        float ms = ss * inv_d;
        float t = ms + e;
        t = sqrtf(t);
        float scale = 1.0f / t;
        for (int64_t i = 0; i < d; i++) {
            float v = xr[i] * scale;
            y[r * d + i] = w ? v * w[i] : v;
        }
    }
}

/* ---- RoPE: nn/transformer.go:146-257 ------------------------------------ */

/* scaling kinds */
enum { MO_ROPE_NONE = 0, MO_ROPE_LINEAR = 1, MO_ROPE_LLAMA3 = 2 };

/* transformer.go:146-164 (angles), :96-118 (scalings), llm/model.go:332-346
 * (linear scale and per-pair frequency factors). cos/sin are [n, dim/2].
 * p: linear -> p[0] = factor; llama3 -> p[0..3] = factor, low, high, original.
 * freq_factors (may be NULL): the pair's frequency is divided by its factor. */
MO_EXPORT void mo_rope_angles(int dim, double base, int scaling, const double *p, const float *freq_factors,
                              int64_t offset, int64_t n, float *cosv, float *sinv) {
    int half = dim / 2;
    double *inv = (double *)malloc(sizeof(double) * (size_t)(half + 1));
    for (int i = 0; i < half; i++) {
        double f = pow(base, -(double)(2 * i) / (double)dim);
        if (scaling == MO_ROPE_LINEAR) {
            f = f / p[0];
        } else if (scaling == MO_ROPE_LLAMA3) {
            double factor = p[0], low = p[1], high = p[2], original = p[3];
            double low_wave = original / low, high_wave = original / high;
            double wave = 2 * M_PI / f;
            if (wave < high_wave) {
            } else if (wave > low_wave) {
                f = f / factor;
            } else {
                double smooth = (original / wave - low) / (high - low);
                f = (1 - smooth) * f / factor + smooth * f;
            }
        }
        if (freq_factors) f /= (double)freq_factors[i];
        inv[i] = f;
    }
    for (int64_t q = 0; q < n; q++)
        for (int i = 0; i < half; i++) {
            double a = (double)(offset + q) * inv[i];
            cosv[q * half + i] = (float)cos(a);
            sinv[q * half + i] = (float)sin(a);
        }
    free(inv);
}

/* transformer.go:225-257 (Apply): x is [rows, S, head_dim]; the first dim
 * features of each head rotate by the angles of its position s, the rest
 * pass through. cos/sin are [S, dim/2]. a' = a*cos - b*sin, b' = a*sin +
 * b*cos for interleaved pairs (2i, 2i+1); for halves (i, i+dim/2):
 * a' = a*cos - b*sin, b' = b*cos + a*sin. Every product is rounded. */
MO_EXPORT void mo_rope_apply(const float *x, float *y, int64_t rows, int64_t s, int head_dim, int dim, int interleaved,
                             const float *cosv, const float *sinv) {
    int half = dim / 2;
    for (int64_t r = 0; r < rows; r++)
        for (int64_t q = 0; q < s; q++) {
            const float *xi = x + (r * s + q) * head_dim;
            float *yo = y + (r * s + q) * head_dim;
            for (int i = 0; i < half; i++) {
                int ia = interleaved ? 2 * i : i, ib = interleaved ? 2 * i + 1 : i + half;
                float a = xi[ia], b = xi[ib], c = cosv[q * half + i], sn = sinv[q * half + i];
                float ac = a * c, bs = b * sn, as = a * sn, bc = b * c;
                yo[ia] = ac - bs;
                yo[ib] = interleaved ? as + bc : bc + as;
            }
            for (int i = dim; i < head_dim; i++) yo[i] = xi[i];
        }
}

/* ---- attention: backend/op.go:117-129; backend/cpu/attention.go:437-535 -- */

/* softmax(scale*q.k^T + mask) . v per query row, with grouped query heads.
 * q [B, H, Q, D] contiguous float32. k, v: element (b, hk, j, :) at
 * b*kv_bstride + hk*kv_hstride + j*kv_pstride, float32 or (kv_dt = MO_F16)
 * binary16 widened on read (attention.go:93-115). Key j is hidden from
 * query i when causal and j > i + causal_offset. mask (may be NULL) is
 * additive float32 with strides mask_b, mask_h over [.., Q, K] (0 to
 * broadcast). out [B, H, Q, DV]; lse [B, H, Q]: max + log(sum). A row that
 * sees no key gets zeros and -Inf. As forwardFew: the query is scaled first,
 * scores are dot products, p = exp(s - max), o = (sum p*v) * (1/l). */
MO_EXPORT void mo_attention(const float *q, const void *k, const void *v, int kv_dt, float *out, float *lse, int64_t B,
                            int64_t H, int64_t HK, int64_t Q, int64_t K, int64_t D, int64_t DV, int64_t kv_bstride,
                            int64_t kv_hstride, int64_t kv_pstride, int64_t v_bstride, int64_t v_hstride,
                            int64_t v_pstride, double scale_d, int causal, int64_t causal_offset, const float *mask,
                            int64_t mask_b, int64_t mask_h) {
    float scale = (float)scale_d;
    int64_t group = H / HK;
#pragma omp parallel for schedule(static) collapse(2) if (B * H * K * D > (1 << 16))
    for (int64_t b = 0; b < B; b++)
        for (int64_t h = 0; h < H; h++) {
            int64_t hk = h / group;
            float *qs = (float *)malloc(sizeof(float) * (size_t)(D + 1));
            float *kr = (float *)malloc(sizeof(float) * (size_t)(D + 1));
            float *sc = (float *)malloc(sizeof(float) * (size_t)(K + 1));
            for (int64_t i = 0; i < Q; i++) {
                const float *qr = q + ((b * H + h) * Q + i) * D;
                float *o = out + ((b * H + h) * Q + i) * DV;
                for (int64_t p = 0; p < D; p++) qs[p] = qr[p] * scale;
                int64_t seen = K;
                if (causal) {
                    seen = i + causal_offset + 1;
                    if (seen > K) seen = K;
                    if (seen < 0) seen = 0;
                }
                float m = -INFINITY;
                for (int64_t j = 0; j < seen; j++) {
                    const float *kp;
                    if (kv_dt == MO_F16) {
                        const uint16_t *kh = (const uint16_t *)k + b * kv_bstride + hk * kv_hstride + j * kv_pstride;
                        for (int64_t p = 0; p < D; p++) kr[p] = mo_f16_to_f32(kh[p]);
                        kp = kr;
                    } else {
                        kp = (const float *)k + b * kv_bstride + hk * kv_hstride + j * kv_pstride;
                    }
                    float s = mo_dot(qs, kp, D);
                    if (mask) s += mask[b * mask_b + h * mask_h + i * K + j];
                    sc[j] = s;
                    if (s > m) m = s;
                }
                for (int64_t p = 0; p < DV; p++) o[p] = 0;
                if (seen == 0 || isinf(m)) {
                    if (lse) lse[(b * H + h) * Q + i] = -INFINITY;
                    continue;
                }
                float l = 0;
                for (int64_t j = 0; j < seen; j++) {
                    sc[j] = expf(sc[j] - m);
                    l += sc[j];
                }
                for (int64_t j = 0; j < seen; j++) {
                    float pj = sc[j];
                    if (pj == 0) continue;
                    if (kv_dt == MO_F16) {
                        const uint16_t *vh = (const uint16_t *)v + b * v_bstride + hk * v_hstride + j * v_pstride;
                        for (int64_t p = 0; p < DV; p++) o[p] += pj * mo_f16_to_f32(vh[p]);
                    } else {
                        const float *vp = (const float *)v + b * v_bstride + hk * v_hstride + j * v_pstride;
                        for (int64_t p = 0; p < DV; p++) o[p] += pj * vp[p];
                    }
                }
                float inv = 1 / l;
                for (int64_t p = 0; p < DV; p++) o[p] *= inv;
                if (lse) lse[(b * H + h) * Q + i] = m + (float)log((double)l);
            }
            free(qs); free(kr); free(sc);
        }
}

/* ---- SwiGLU: llm/model.go:446-448; tensor/elementwise.go:520-525,583-585 - */

/* out = (g * recip(1 + exp2(g * -log2e))) * u, each step a float32. */
MO_EXPORT void mo_silu_mul(const float *g, const float *u, float *out, int64_t n) {
    const float nl2e = (float)(-1.4426950408889634);
    for (int64_t i = 0; i < n; i++) {
        float t = g[i] * nl2e;
        t = exp2f(t);
        t = 1.0f + t;
        t = 1.0f / t;
        t = g[i] * t;
        out[i] = t * u[i];
    }
}

/* ---- greedy sampling: examples/llama/generate.go:44-53 ------------------ */

/* argmax with the first index winning ties (v > best). */
MO_EXPORT int32_t mo_argmax(const float *logits, int64_t n) {
    int64_t best = 0;
    for (int64_t i = 0; i < n; i++)
        if (logits[i] > logits[best]) best = i;
    return (int32_t)best;
}

/* ---- memory-bandwidth ceiling, as BenchmarkMemoryBandwidth -------------- */
/* backend/cpu/quant_test.go:455-488: every worker sums its share of a
 * buffer; returns the grand total so the reads are not optimised away. */
MO_EXPORT double mo_stream_sum(const float *p, int64_t n, int threads) {
    double total = 0;
#ifdef _OPENMP
    if (threads <= 0) threads = omp_get_max_threads();
#endif
#pragma omp parallel for schedule(static) reduction(+ : total) num_threads(threads)
    for (int64_t i = 0; i < n; i += 16) {
        float s = 0;
        for (int64_t j = i; j < i + 16 && j < n; j++) s += p[j];
        total += s;
    }
    return total;
}

MO_EXPORT int mo_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
