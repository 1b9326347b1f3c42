// Host-side entry points of the gfx950 kernels. Each launches on the given
// stream and returns the launch status; none of them synchronises.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <atomic>

namespace mimir {

// dtype codes: the reference's DType enumeration (backend/backend.go:72-90)
// with Q4_0 appended, so that IsQuantized stays the range test Q8_0..Q4_0.
enum DType : int { kInvalid = 0, kF32 = 1, kI32 = 2, kBF16 = 3, kF16 = 4, kQ8_0 = 5, kQ4_K = 6, kQ6_K = 7, kQ4_0 = 8 };

inline bool is_quantized(int dt) { return dt >= kQ8_0 && dt <= kQ4_0; }
inline int block_size(int dt) { return (dt == kQ8_0 || dt == kQ4_0) ? 32 : (dt == kQ4_K || dt == kQ6_K) ? 256 : 1; }
inline int block_bytes(int dt) {
    switch (dt) {
    case kQ8_0: return 34;
    case kQ4_0: return 18;
    case kQ4_K: return 144;
    case kQ6_K: return 210;
    case kF32: case kI32: return 4;
    case kBF16: case kF16: return 2;
    default: return 0;
    }
}

// y[m, :] = x[m, :] . W^T for m < M: W is [N, K] blocks read in place, x rows
// are x_row_stride floats apart, y rows N floats apart.
struct QGemvArgs {
    const void* W;
    const float* x;    // float32 activations, or
    const void* act;   // activations converted for the fixed-point Q4_0 kernel
    float* y;
    int64_t M, N, K;
    int64_t x_row_stride;
    int rows_per_wg;            // 0 = derived from the launch shape
    const float* resid = nullptr;  // [M, N] added to the product (fixed-point Q4_0 kernel only)
};

// The float32 Q4_0 product, any shape. tune: {rows, cols, waves, no_lds}; zeros
// pick the built-in plan.
hipError_t qgemv_q4_0(const QGemvArgs& a, const int* tune, hipStream_t st);

// The fixed-point Q4_0 product: x is converted once (q4_0_convert_act, into
// q4_0_act_bytes(K) bytes per row) and multiplied with v_dot8_i32_i4.
// q4_0_fixed_point_ok says whether a W and K qualify.
bool q4_0_fixed_point_ok(const void* W, int64_t K);
size_t q4_0_act_bytes(int64_t K);
hipError_t q4_0_convert_act(const float* x, int64_t M, int64_t K, int64_t x_row_stride, void* act, hipStream_t st);
hipError_t qgemv_q4_0_act(const QGemvArgs& a, const int* tune, hipStream_t st);
// Up to three matrices that share x and K in one launch, their rows
// concatenated in y; and a SwiGLU pair: y = SiLU(x . gate^T) * (x . up^T).
hipError_t qgemv_q4_0_act_multi(const void* const W[3], const int64_t n[3], const void* act, float* y, int64_t M, int64_t K,
                                const int* tune, hipStream_t st);
// The RMSNorm in front of a product as that product's first phase: with x and w set, every
// workgroup normalizes and converts row m of x [M, K] for itself and `act` is not read
// (q4_0_norm_head_ok(K) must hold); with w null the product reads `act` as usual.
struct Q4NormHead {
    const float* x = nullptr;
    const float* w = nullptr;
    double eps = 0;
};
bool q4_0_norm_head_ok(int64_t K);
void set_q4_batch_off(int v);  // 1: products of several rows of x stay on the one-row kernel
// The same products on the kernel shaped for the whole chip (qgemv_q4_0_stream.hip): one to four rows of x, a
// workgroup per compute unit, x kept in registers. Returns false where it does not take the shape (the caller then
// launches qgemv_q4_0_i4_kernel); otherwise *err is the launch's status. mode: a Q4Mode.
struct Q4Job;
bool q4_0_stream_dispatch(int mode, const Q4Job& job, const void* act, float* y, int64_t M, int64_t K, hipStream_t st, hipError_t* err);
void set_q4_stream_off(int v);             // measurement aid: 1 keeps every product off that kernel
// The same products with a compute unit's whole share of W requested at entry by loads that write LDS directly
// (qgemv_q4_0_dma.hip): one row of x, 16-byte aligned W and x. Tried before q4_0_stream_dispatch; same contract, same bits.
bool q4_0_dma_dispatch(int mode, const Q4Job& job, const void* act, float* y, int64_t M, int64_t K, hipStream_t st, hipError_t* err);
void set_q4_dma_off(int v);                // measurement aid: not 0 keeps every product off that kernel
void set_q4_dma_feed(int feeders, int window);  // its feeding wavefronts (1..4) and the rows each keeps under way; 0 leaves a value as it is
hipError_t set_q4_dma_stamps(long long* p);  // measurement aid: five timestamps per workgroup of its float32-x launches (null: none)
void set_q4_stream_waves(int v);           // measurement aid: wavefronts a workgroup of that kernel (0: its own choice)
hipError_t set_q4_stream_stamps(long long* p);   // measurement aid: device memory for five timestamps per workgroup of its launches (null: none)
bool q4_0_swiglu_convert_ok(int64_t N, int64_t K);
hipError_t qgemv_q4_0_act_swiglu_convert(const void* gate, const void* up, const void* act, void* act_out, int64_t M, int64_t N,
                                         int64_t K, const Q4NormHead& norm, const int* tune, hipStream_t st);
// What follows the q, k, v projections in a decoding step (rope_kv), as the tail of their fused product.
struct Q4RopeTail {
    const float* cosv = nullptr;   // [position][rope_dim / 2]
    const float* sinv = nullptr;
    const int32_t* pos = nullptr;  // the position, read on the device
    void* kcache = nullptr;        // [M, HK, cap, dim]
    void* vcache = nullptr;
    int cache_dt = 0, H = 0, HK = 0, dim = 0, rope_dim = 0;
    int64_t cap = 0;
};
hipError_t qgemv_q4_0_act_qkv_rope(const void* const W[3], const int64_t n[3], const void* act, float* y, int64_t M, int64_t K,
                                   const Q4RopeTail& rope, const Q4NormHead& norm, const int* tune, hipStream_t st);
// The same tail behind a Q4_K or Q6_K product (qgemv_kquant_rope_ok says whether the shape qualifies).
bool qgemv_kquant_rope_ok(int dt, const QGemvArgs& a);
hipError_t qgemv_kquant_act_rope(int dt, const QGemvArgs& a, const Q4RopeTail& rope, hipStream_t st);
hipError_t qgemv_q4_0_act_swiglu(const void* gate, const void* up, const void* act, float* y, int64_t M, int64_t N, int64_t K,
                                 const int* tune, hipStream_t st);

// The Q8_0 product as the reference's CPU computes it: x rounded to int8 per
// block of 32 (q8_convert_act, q8_act_bytes(K) bytes per row), integer dot
// products. q8_act_fits says whether the converted row fits the LDS.
bool q8_act_fits(int64_t K);
size_t q8_act_bytes(int64_t K);
hipError_t q8_convert_act(const float* x, int64_t M, int64_t K, int64_t x_row_stride, void* act, hipStream_t st);
hipError_t qgemv_q8_0_act(const QGemvArgs& a, const int* tune, hipStream_t st);
// Two or more rows of x against W read once (each sum formed as qgemv_q8_0_act forms it): rows converted beforehand,
// W 4-byte aligned, an even number of blocks a row, no residual.
bool qgemv_q8_0_rows_ok(const QGemvArgs& a);
hipError_t qgemv_q8_0_rows(const QGemvArgs& a, hipStream_t st);
// Two to eight rows of x on the int8 matrix cores (qgemv_q8_0_mfma.hip): the CPU's integer lane sums, the float32 sums
// of a row's blocks in another order than the kernels above add them. K a multiple of 256, W 16-byte aligned.
// qgemv_q8_0_mfma_pays: large enough a matrix for it to be the faster (or as "q8_0.mfma" says: 1 always, 2 never).
bool qgemv_q8_0_mfma_ok(const QGemvArgs& a);
bool qgemv_q8_0_mfma_pays(const QGemvArgs& a);
void set_q8_mfma(int v);
hipError_t qgemv_q8_0_mfma(const QGemvArgs& a, hipStream_t st);

// The Q4_K and Q6_K products as the reference's CPU computes them: x rounded
// to int8 in super-blocks of 256 with the sums of each 16 quants
// (kq_convert_act, kq_act_bytes(K) bytes per row), integer dot products.
size_t kq_act_bytes(int64_t K);
hipError_t kq_convert_act(const float* x, int64_t M, int64_t K, int64_t x_row_stride, void* act, hipStream_t st);
// RMSNorm then conversion, and SiLU(g) * u then conversion, each in one launch and with the separate
// kernels' arithmetic (d and n multiples of 256; x, w, g, u 16-byte aligned).
hipError_t rmsnorm_kq_act(const float* x, const float* w, void* act, int64_t rows, int64_t d, double eps, hipStream_t st);
hipError_t swiglu_kq_act(const float* g, const float* u, void* act, int64_t rows, int64_t n, int64_t stride, hipStream_t st);
// The same from bfloat16 rows (8-byte aligned, a multiple of 4 elements apart).
hipError_t kq_convert_act_bf16(const void* x, int64_t M, int64_t K, int64_t x_row_stride, void* act, hipStream_t st);
// With a.act null and qgemv_kquant_rope_ok(dt, a): one launch from float32 a.x (16-byte aligned rows), rounded by every workgroup.
hipError_t qgemv_kquant_act(int dt, const QGemvArgs& a, hipStream_t st);
// The same products for many rows of x on the matrix cores (qgemm_kquant.hip); qgemv_kquant_act
// hands over to it where qgemm_kquant_pays says it is the faster of the two.
bool qgemm_kquant_pays(int dt, const QGemvArgs& a);
bool qgemm_kquant_ok(int dt, const QGemvArgs& a);
// y float32, or with out_bf16 each result rounded once to bfloat16 into y taken as uint16_t*.
hipError_t qgemm_kquant(int dt, const QGemvArgs& a, hipStream_t st, bool out_bf16 = false);
// which 0: rows of W per wavefront (1, 2, 4; 0 = by shape); which 1: value 1 = always the kernels that keep x in
// global memory, 2 = never the matrix-core kernel, 3 = always the matrix-core kernel.
void set_kquant_tune(int which, int value);
// Two rows of x or more against Q4_K or Q6_K weights, eight to a pass over W, on the int8 matrix cores with the CPU's bits
// (qgemv_kquant_rows.hip); qgemv_kquant_act hands over where qgemv_kquant_rows_pays says so ("kquant.mfma_rows": 1 never, 2 wherever
// the kernel takes the shape).
bool qgemv_kquant_rows_ok(int dt, const QGemvArgs& a);
bool qgemv_kquant_rows_pays(int dt, const QGemvArgs& a);
hipError_t qgemv_kquant_rows(int dt, const QGemvArgs& a, hipStream_t st);
// With the rotation and the cache writes of a decoding step as its tail (y receives the rotated queries only).
bool qgemv_kquant_rows_rope_ok(int dt, const QGemvArgs& a);
hipError_t qgemv_kquant_rows_rope(int dt, const QGemvArgs& a, const Q4RopeTail& rope, hipStream_t st);
void set_kquant_rows(int v);
void set_kquant_rows_waves(int v);

// y = x . W^T for a float32, binary16 or bfloat16 W [N, K].
hipError_t gemv_float(int dt, const void* W, const float* x, float* y, int64_t M, int64_t N, int64_t K, int64_t x_row_stride,
                      hipStream_t st);

// ---- the other kernels of a decoding step ------------------------------------
hipError_t rmsnorm(const float* x, const float* w, float* y, int64_t rows, int64_t d, double eps, hipStream_t st);
// period > 0: the s positions are those of s / period sequences one behind the other, position p turned by the angles of
// offset + p % period (0: of offset + p).
hipError_t rope(const float* x, float* y, int64_t rows, int64_t s, int head_dim, int dim, int interleaved, int64_t x_row_stride,
                int64_t x_pos_stride, int64_t y_row_stride, int64_t y_pos_stride, const float* cosv, const float* sinv,
                int64_t offset, hipStream_t st, int64_t period = 0);
hipError_t kv_write(const float* src, void* cache, int cache_dt, int64_t B, int heads, int64_t s, int dim, int64_t cap,
                    int64_t pos, int64_t src_b, int64_t src_h, int64_t src_p, hipStream_t st);
// RMSNorm that also writes the row converted for the Q4_0 kernel (y may be
// null); rmsnorm_q4act_ok says whether a row length qualifies.
bool rmsnorm_q4act_ok(int64_t d);
hipError_t rmsnorm_q4act(const float* x, const float* w, float* y, void* act, int64_t rows, int64_t d, double eps, hipStream_t st);
// One decoding position: rotates the queries of qkv [B, (H + 2 HK) * dim] in
// place, rotates and caches its keys, caches its values, at position *pos_dev.
// bias, if not null: [(H + 2 HK) * dim] float32 added to every row before that (the q, k, v biases of qwen2, concatenated).
hipError_t rope_kv(float* qkv, void* kcache, void* vcache, int cache_dt, int64_t B, int H, int HK, int dim, int rope_dim,
                   int interleaved, int64_t cap, const float* cosv, const float* sinv, const int32_t* pos_dev, hipStream_t st,
                   const float* bias = nullptr);
// The same for q [B, H dim], k and v [B, HK dim] in buffers of their own.
hipError_t rope_kv_split(float* q, const float* k, const float* v, void* kcache, void* vcache, int cache_dt, int64_t B, int H, int HK, int dim,
                         int rope_dim, int interleaved, int64_t cap, const float* cosv, const float* sinv, const int32_t* pos_dev,
                         hipStream_t st, const float* bias = nullptr);
// state = {position, steps}: record[steps] = next_tok [B], then steps += 1 and
// position += pos_inc.
hipError_t advance(int32_t* state, const int32_t* next_tok, int32_t* record, int B, int pos_inc, hipStream_t st);
hipError_t set_state(int32_t* state, int pos, int step, hipStream_t st);
hipError_t swiglu(const float* g, const float* u, float* out, int64_t rows, int64_t n, int64_t stride, hipStream_t st);
hipError_t add(const float* a, const float* b, float* out, int64_t n, hipStream_t st);
hipError_t add_bias(float* y, const float* bias, int64_t rows, int64_t n, hipStream_t st);  // y[r, :] += bias
// workspace: argmax_workspace_bytes(rows) bytes, the first kArgmaxTicketBytes zero
// before the first launch (they restore themselves), or null for one workgroup a row.
constexpr size_t kArgmaxTicketBytes = 4096;
size_t argmax_workspace_bytes(int64_t rows);
hipError_t argmax(const float* logits, int64_t rows, int64_t n, int32_t* out, void* workspace, hipStream_t st);

// Attention of queries [B, H, Q, D] over keys and values [B, HK, K, D], each
// read through strides {batch, head, position} (features contiguous). chunk
// and nsplit come from attention_plan; workspace holds
// attention_workspace_bytes(...) bytes when nsplit > 1.
struct AttnArgs {
    const float* q;
    const void *k, *v;
    int kv_dtype;  // kF32 or kF16
    float* out;
    float* lse;    // [B, H, Q] contiguous, or null
    int64_t q_strides[3], k_strides[3], v_strides[3], o_strides[3];
    int64_t B, Q, K;
    int H, HK, D;
    double scale;
    int causal;
    int64_t causal_offset;
    int chunk, nsplit;
    const int32_t* dyn_k = nullptr;  // device int: that many more keys than K
    int DV = 0;                      // features of a value (0: D)
    const float* mask = nullptr;     // added to the scores, [B, H, Q, K] read through m_strides {batch, head, query, key}
    int64_t m_strides[4] = {0, 0, 0, 0};
};
void attention_plan(int64_t B, int H, int HK, int64_t Q, int64_t K, int* chunk, int* nsplit);
size_t attention_workspace_bytes(int64_t B, int H, int64_t Q, int D, int nsplit);
hipError_t attention(const AttnArgs& a, void* workspace, hipStream_t st);
// Many query positions at once on the float32 matrix cores (attention_prompt.hip), which attention() takes for the calls
// attention_prompt_ok names: the same results up to the order of the float32 sums.
bool attention_prompt_ok(const AttnArgs& a);
hipError_t attention_prompt(const AttnArgs& a, hipStream_t st);
void set_attention_prompt(int v);  // measurement aid: 0 keeps every call on the kernel that takes a query row a workgroup
// K == 0: zeros and a logsumexp of -Inf for every row; reads neither keys nor values.
hipError_t attention_empty(const AttnArgs& a, hipStream_t st);

// One query position per sequence in a single launch (attention_decode.hip).
// The workspace begins with kAttnTicketBytes of tickets that must be zero before
// the first launch and restore themselves; a.K keys plus *a.dyn_k, at most kmax.
// act, if set, receives the result in the Q4_0 product's fixed-point form
// (out may then be null; needs o_strides {H * D, D, .}).
constexpr size_t kAttnTicketBytes = 4096;
bool attention_decode_ok(const AttnArgs& a, int64_t kmax);
void set_attention_decode_splits(int n);
void set_attention_decode_share(int n);  // keys a share of decode attention aims at: 64 or 128
void set_attention_decode_fence(int v);  // 1 (default): the hand-over's ticket is a release-acquire operation at device scope; 0 relaxed, 2 plain share accesses (measurement)
void attention_decode_plan(int64_t B, int H, int HK, int64_t kmax, int* nsplit, int* cmax);
size_t attention_decode_workspace_bytes(int64_t B, int H, int D, int nsplit);
enum { kAttnActQ4 = 0, kAttnActRows = 1, kAttnActKQ = 2 };
// flagged, if not null: flagged_bytes bytes (at least attention_decode_flagged_bytes, else the tickets are used), zero before the first launch and left zero by every launch, that no
// other kernel writes: the shares of the keys then travel as (value, flag) pairs to the first share's workgroup, which polls for
// them (a bounded number of times; a pair that never arrives sets kErrInternal in *err), instead of through tickets.
size_t attention_decode_flagged_bytes(int64_t B, int H, int D, int nsplit);
void set_attention_decode_handover(int v);  // measurement aid: 1 keeps the ticket protocol
hipError_t attention_decode(const AttnArgs& a, int64_t kmax, void* workspace, void* act, int64_t act_row_bytes, hipStream_t st,
                            int act_form = kAttnActQ4, void* flagged = nullptr, size_t flagged_bytes = 0, uint32_t* err = nullptr);
bool attention_decode_kq_ok(const AttnArgs& a);

// The fixed-point Q4_0 product of a few rows of float32 x that reads W once per eight of them (qgemv_q4_0_rows.hip,
// int8 matrix cores): each group of eight rows is converted together by q4_0_rows_convert_act into q4_0_rows_act_bytes(K) bytes,
// group after group; the plain product takes any number of groups in one launch, its tails and shapes without whole runs one
// (x 16-byte aligned rows, K a multiple of 64).
size_t q4_0_rows_act_bytes(int64_t K);
hipError_t q4_0_rows_convert_act(const float* x, int64_t M, int64_t K, int64_t x_row_stride, void* act, hipStream_t st);
bool qgemv_q4_0_rows_ok(const void* W, int64_t M, int64_t N, int64_t K);
double qgemv_q4_0_rows_cost_us(int64_t M, int64_t N, int64_t K);  // about what M rows take, conversion included
// shares > 1 (qgemv_q4_0_rows_shares_ok; no resid): K is cut into that many shares, whose sums go to y[shares, M, N]
// for a later kernel to add in their order.
bool qgemv_q4_0_rows_shares_ok(const void* W, int64_t M, int64_t N, int64_t K, int shares);
hipError_t qgemv_q4_0_rows(const void* W, const void* act, float* y, const float* resid, int64_t M, int64_t N, int64_t K, int shares,
                           hipStream_t st);
// Up to three matrices (n[i] = 0: none) that share act and K in one launch, their rows one after the other in
// y[shares, M, n[0] + n[1] + n[2]]: each must satisfy qgemv_q4_0_rows_shares_ok, all but the last with a multiple of 32 rows.
hipError_t qgemv_q4_0_rows_multi(const void* const W[3], const int64_t n[3], const void* act, float* y, const float* resid, int64_t M,
                                 int64_t K, int shares, hipStream_t st);
// q, k and v in one launch with the rotation and the cache writes of a decoding step as its tail (y [M, n[0] + n[1] + n[2]]
// receives the rotated queries only; interleaved pairs, rows in multiples of 32); and gate and up [N, K] in one launch that
// leaves SiLU(x . gate^T) * (x . up^T) converted in act_out as the x of a product over N (N a multiple of 32).
hipError_t qgemv_q4_0_rows_qkv_rope(const void* const W[3], const int64_t n[3], const void* act, float* y, int64_t M, int64_t K,
                                    const Q4RopeTail& rope, hipStream_t st);
hipError_t qgemv_q4_0_rows_swiglu_act(const void* gate, const void* up, const void* act, void* act_out, int64_t M, int64_t N, int64_t K,
                                      hipStream_t st);
// Around that product in a decoding step of up to eight sequences, each leaving its result in the converted form:
// RMSNorm (with shares > 0, x += parts[0] + parts[1] + ... first, parts [shares, rows, d], written back to x: the
// residual connection behind a product cut into shares), SiLU(g) * u, and the addition of the shares alone.
hipError_t rows_norm_act(float* x, const float* parts, int shares, const float* w, void* act, int64_t rows, int64_t d, double eps,
                         hipStream_t st);
hipError_t rows_swiglu_act(const float* g, const float* u, void* act, int64_t rows, int64_t n, int64_t stride, hipStream_t st);
hipError_t rows_add_parts(float* x, const float* parts, int shares, int64_t n, hipStream_t st);
void set_q4_rows_waves(int v);   // measurement aid: 4 or 8 wavefronts a workgroup, 0 by shape
void set_q4_rows_direct(int v);  // measurement aid: 1 = its kernel that loads each lane's block where it lies
// The fixed-point Q4_0 product for many rows of float32 x on the matrix cores: x converted by q4_0_fx_convert_act
// (q4_0_fx_act_bytes(K) bytes a row), K a multiple of 128. On the int8 matrix cores (qgemm_q4_0_fx.hip), or, with
// `pairs` and a workspace (some hundreds of rows and more: qgemm_q4_0_fx16_pays says when), x converted into pairs
// of 12-bit digits (q4_0_fx16_act_bytes(K) bytes a row) and the product on the binary16 matrix cores with the same
// bits (qgemm_q4_0_fx16.hip): ws qgemm_q4_0_fx16_ws_bytes(N, K) bytes, 16-byte aligned; ws null: act holds the int8 form.
size_t q4_0_fx_act_bytes(int64_t K);
hipError_t q4_0_fx_convert_act(const float* x, int64_t M, int64_t K, int64_t x_row_stride, void* act, bool pairs, hipStream_t st);
bool qgemm_q4_0_fx_ok(const void* W, int64_t M, int64_t N, int64_t K);
bool qgemm_q4_0_fx_pays(const void* W, int64_t M, int64_t N, int64_t K);  // and is the faster choice against the one-row kernels
double qgemm_q4_0_fx_cost_us(int64_t M, int64_t N, int64_t K);           // about what it takes, conversion aside
hipError_t qgemm_q4_0_fx(const void* W, const void* act, float* y, const float* resid, int64_t M, int64_t N, int64_t K, void* ws, hipStream_t st);
bool qgemm_q4_0_fx16_pays(int64_t M, int64_t N, int64_t K);  // against the int8 form, its pass over W included
size_t q4_0_fx16_act_bytes(int64_t K);
hipError_t q4_0_fx16_convert_act(const float* x, int64_t M, int64_t K, int64_t x_row_stride, void* act, hipStream_t st);
size_t qgemm_q4_0_fx16_ws_bytes(int64_t N, int64_t K);
hipError_t qgemm_q4_0_fx16(const void* W, const void* act, float* y, const float* resid, int64_t M, int64_t N, int64_t K, void* ws, hipStream_t st);
void set_q4_0_fx16(int v);  // measurement aid: 0 keeps every product on the int8 form

// Prompt-sized Q4_0 product on the matrix cores (qgemm_q4_0.hip): X [M, K]
// bfloat16, Y [M, N] bfloat16 or float32. Exact up to the order of the float32 sums when half_ws is null; with
// half_ws (qgemm_q4_0_half_ws_bytes(M, N, K, panel) bytes of device memory, 256-byte aligned) the weights are rounded to
// binary16 (2^-11 of each) and X goes through half_ws as row-scaled binary16. With `panel` (the same value in both
// calls) the products that qgemm_f16_panel_pays names write W to half_ws once as a binary16 panel and multiply from it.
bool qgemm_q4_0_ok(const void* W, const void* X, int64_t M, int64_t N, int64_t K, int64_t x_row_stride);
size_t qgemm_q4_0_half_ws_bytes(int64_t M, int64_t N, int64_t K, bool panel);
hipError_t qgemm_q4_0_bf16(const void* W, const void* X, void* Y, int64_t M, int64_t N, int64_t K, int64_t x_row_stride, bool out_f32,
                           void* half_ws, bool panel, hipStream_t st);
// The exact form from a panel of the weights' integers (qgemm_q4_0_blocks.hip): block sums on the bfloat16 matrix
// cores, one FMA per output and block with the block's scale; X as for qgemm_q4_0_bf16, ws qgemm_q4_0_blocks_ws_bytes(N, K)
// bytes of device memory, 16-byte aligned.
size_t qgemm_q4_0_blocks_ws_bytes(int64_t N, int64_t K);
bool qgemm_q4_0_blocks_pays(int64_t M, int64_t N, int64_t K);  // against the tile kernel, its pass over W included
hipError_t qgemm_q4_0_blocks(const void* W, const void* X, int64_t x_row_stride, void* Y, int64_t M, int64_t N, int64_t K, bool out_f32, void* ws,
                             hipStream_t st);
void set_q4_0_blocks(int v);  // measurement aid: 0 keeps every product on the tile kernel, 2 takes this route whatever the shape
// The panel route (qgemm_f16_panel.hip): X [M, K] bfloat16 goes to X16 [M, K] binary16 with row_scale[m] to multiply row
// m's results by (both written here), W Q4_0 to `panel` (qgemm_f16_panel_bytes(N, K) bytes of device memory, 256-byte aligned).
size_t qgemm_f16_panel_bytes(int64_t N, int64_t K);
bool qgemm_f16_panel_pays(int64_t M, int64_t N, int64_t K);
hipError_t qgemm_f16_panel(const void* W, const void* X, int64_t x_row_stride, void* X16, float* row_scale, void* Y, int64_t M, int64_t N, int64_t K,
                           bool out_f32, void* panel, hipStream_t st);
hipError_t bf16_rows_to_f32(const void* x, float* y, int64_t M, int64_t K, int64_t x_row_stride, hipStream_t st);
hipError_t f32_to_bf16(const float* x, void* y, int64_t n, hipStream_t st);

// A plain streaming read of `bytes` bytes, summed into out[0..grid): the
// practical ceiling of HBM reads to compare the products against.
// While a measurement is on (capi.hip), hands out the next pair of events for a
// launch to be bracketed by; false otherwise.
bool next_timing_events(hipEvent_t* start, hipEvent_t* stop);
// Records which kernel the calling thread's latest Q4_0 product (of one row of x, or prompt-sized with bfloat16 x) or attention call launched (printf-style), for mi355x_last_kernel.
void note_kernel(const char* fmt, ...);
hipError_t stream_read(const void* p, size_t bytes, float* out, int grid, int threads, hipStream_t st);
int stream_read_out_len(int grid, int threads);

// p[i] = v for i < n 32-bit words, as a kernel.
hipError_t fill_u32(void* p, uint32_t v, int64_t n, hipStream_t st);

// Bits a kernel ORs into the device error word, read back at sync, as the
// reference's kernels report theirs (backend/rocm/rocm_linux.go:349-375).
enum : uint32_t { kErrIndex = 1u, kErrInternal = 2u };

// out[i] = element first + i of the blocks at data, i < n, as out_dt
// (kF32, kBF16 or kF16): OpCast of a contiguous view.
hipError_t dequantize(int dt, const void* data, int64_t first, int64_t n, void* out, int out_dt, hipStream_t st);

// How a kernel reads a buffer (backend.View, backend/view.go:23-27), by value.
constexpr int kMaxRank = 8;
struct ViewArg {
    int rank;
    int64_t shape[kMaxRank], strides[kMaxRank];
    int64_t offset;
};
hipError_t dequantize_view(int dt, const void* data, const ViewArg& v, int64_t n, void* out, int out_dt, hipStream_t st);
hipError_t gather_view(int dt, const void* table, const ViewArg& tv, const int32_t* idx, const ViewArg& iv, int axis, int64_t n, float* out,
                       uint32_t* err, hipStream_t st);
hipError_t copy_view32(const void* src, const ViewArg& v, int64_t n, void* out, hipStream_t st);

// out[r, :] = dequantized row idx[r] of a [rows, k] table: OpGather on axis 0.
hipError_t gather_rows(int dt, const void* table, int64_t rows, int64_t k, const int32_t* idx, int64_t n, float* out,
                       uint32_t* err, hipStream_t st);

}  // namespace mimir
