// Host-side decoder of the llama architecture over the kernels of this
// library: the counterpart of the reference's llm.Model (llm/model.go:216-455:
// Load, NewCaches, Logits, project, mlp), nn.KVCache (nn/transformer.go:348-423)
// and the greedy loop of examples/llama (generate.go:44-53,162-202), with the
// same error behaviour (shape and index errors before anything is queued).
//
// Differences that are the point of this build: weights stay in their block
// dtypes on the device, Q4_0 included (the reference decodes Q4_0 to float32
// when the model opens); a step is queued as a fixed run of launches with no
// host synchronisation in between (the reference's GPU path realizes and
// syncs twice per block, llm/model.go:409-427); the next token is chosen on
// the device and fed to the next step's embedding lookup from device memory,
// so generation downloads nothing until it ends; several sequences may be
// decoded in lockstep (llm fixes batch 1, llm/model.go:378-385,408).
#include "../../include/mimir_mi355x.h"

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "kernels.h"

namespace mimir {

mi355x_status capi_fail(mi355x_status code, const char* fmt, ...);  // capi.hip

namespace {

#define LLM_HIP(expr, what)                                                          \
    do {                                                                             \
        hipError_t e_ = (expr);                                                      \
        if (e_ != hipSuccess) return capi_fail((mi355x_status)e_, "mi355x: llama: %s: %s", what, hipGetErrorName(e_)); \
    } while (0)

struct DevBuf {
    void* p = nullptr;
    size_t bytes = 0;
    bool view = false;  // p points into another buffer's memory
    ~DevBuf() { release(); }
    void release() {
        if (p && !view) (void)hipFree(p);
        p = nullptr;
        view = false;
    }
    hipError_t alloc(size_t n) {
        release();
        bytes = n;
        return hipMalloc(&p, n < 4 ? 4 : n);
    }
    void point_at(void* q, size_t n) {
        release();
        p = q;
        bytes = n;
        view = true;
    }
    template <typename T>
    T* as() const { return (T*)p; }
};

struct Weight {
    int dtype = 0;
    int64_t n = 0, k = 0;
    DevBuf buf;
    bool set() const { return buf.p != nullptr; }
};

// The form of converted activations a weight's product reads.
// kActFx: Q4_0 by many rows of x, on the int8 matrix cores; kActFxPairs: the same product through the binary16 ones
enum ActClass { kActNone = 0, kActQ4 = 1, kActQ8 = 2, kActKQ = 3, kActFx = 4, kActFxPairs = 5, kActClasses = 6 };

// qkv and gate_up: where q, k, v (gate, up) share a block dtype, finalize also keeps their rows in one
// buffer, which a decoding step multiplies in one product (the reference concatenates the same
// weights for its recorded step, fusedFor, llm/decode.go:240-266). Models that take step_fast do
// not need them (its kernels read the three matrices where they are).
struct Block {
    Weight attn_norm, ffn_norm, q, k, v, o, gate, up, down, qkv, gate_up;
    Weight q_bias, k_bias, v_bias;  // qwen2's (llm/model.go:251-258): float32 [n], all three or none
    DevBuf qkv_bias;                // the three in one row, beside qkv
    bool biased() const { return q_bias.set(); }
};

struct Model {
    mi355x_llama_config c{};
    Weight embed, norm, output;
    bool tied = false;
    std::vector<Block> blocks;
    std::vector<float> rope_factors;
    bool ready = false;

    DevBuf cos_t, sin_t;                 // [context, rope_dim/2]
    DevBuf attn_flags;                   // decode attention's (value, flag) slots: zero between launches
    std::vector<DevBuf> keys, values;    // per block: [batch, kv_heads, context, head_dim]
    int64_t cache_len = 0;

    // activations of up to max_rows rows (batch x tokens of one call)
    int64_t max_rows = 0;
    DevBuf x, h, q, k, v, a, o, gate, up, s, xlast, hlast, logits, act[kActClasses], act2, tokens_dev, next_tok;
    DevBuf fx_panel;  // the workspace of the fixed-point Q4_0 product of a prompt's rows in its binary16 form: the largest matrix's
    hipStream_t stream = nullptr;

    // The decoding step as a fixed run of launches that read the position from
    // the device: state = {position, steps taken}; record holds the tokens
    // chosen so far, [max_new, batch]. `fast` says the blocks qualify (Q4_0
    // linears that the fixed-point kernel takes); step_graph replays the run.
    bool fast = false;
    DevBuf state, record, qkv, gu, argmax_ws;  // gu: gate|up of a step, [batch, 2 hidden]
    // `rows`: a fast model with two to sixty-four sequences, whose step reads every weight once per eight of them
    // (step_rows): the sequences' activations converted together, and the two shares of K of the output and
    // down projections, [2, batch, embed].
    bool rows = false;
    DevBuf rows_act, rows_act2, parts;
    hipGraphExec_t step_graph = nullptr;
    int graph_rows = 0;  // which step the graph holds: 0 step_fast or step_any, 1 step_rows, 2 step_rows without its riders

    ~Model() {
        if (step_graph) (void)hipGraphExecDestroy(step_graph);
        if (stream) (void)hipStreamDestroy(stream);
    }
};

// panel_bytes: what the model holds as workspace for the fixed-point product's binary16 form (0: that form is not taken)
int act_class(const Weight& w, int64_t rows = 1, size_t panel_bytes = 0) {
    switch (w.dtype) {
    case kQ4_0:
        if (qgemm_q4_0_fx_pays(w.buf.p, rows, w.n, w.k))
            return panel_bytes >= qgemm_q4_0_fx16_ws_bytes(w.n, w.k) && qgemm_q4_0_fx16_pays(rows, w.n, w.k) ? kActFxPairs : kActFx;
        return q4_0_fixed_point_ok(w.buf.p, w.k) ? kActQ4 : kActNone;
    case kQ8_0: return q8_act_fits(w.k) ? kActQ8 : kActNone;
    case kQ4_K: case kQ6_K: return kActKQ;
    default: return kActNone;
    }
}

size_t act_row_bytes(int cls, int64_t K) {
    switch (cls) {
    case kActQ4: return q4_0_act_bytes(K);
    case kActQ8: return q8_act_bytes(K);
    case kActKQ: return kq_act_bytes(K);
    case kActFx: return q4_0_fx_act_bytes(K);
    case kActFxPairs: return q4_0_fx16_act_bytes(K);
    default: return 0;
    }
}

const int kNoTune[5] = {0, 0, 0, 0, 0};

// Converts rows of x once for every activation form that `ws` need.
mi355x_status convert_for(Model& m, const float* x, int64_t rows, int64_t K, std::initializer_list<const Weight*> ws, bool done[kActClasses]) {
    for (int i = 0; i < kActClasses; i++) done[i] = false;
    for (const Weight* w : ws) {
        int cls = act_class(*w, rows, m.fx_panel.bytes);
        if (cls == kActNone || done[cls]) continue;
        size_t need = act_row_bytes(cls, K) * (size_t)rows;
        if (m.act[cls].bytes < need) return capi_fail(MI355X_ERR_INTERNAL, "mi355x: llama: activation scratch of %zu bytes, need %zu", m.act[cls].bytes, need);
        hipError_t e = cls == kActQ4   ? q4_0_convert_act(x, rows, K, K, m.act[cls].p, m.stream)
                       : cls == kActQ8 ? q8_convert_act(x, rows, K, K, m.act[cls].p, m.stream)
                       : cls == kActFx || cls == kActFxPairs ? q4_0_fx_convert_act(x, rows, K, K, m.act[cls].p, cls == kActFxPairs, m.stream)
                                       : kq_convert_act(x, rows, K, K, m.act[cls].p, m.stream);
        LLM_HIP(e, "convert activations");
        done[cls] = true;
    }
    return MI355X_OK;
}

// y[rows, n] = x[rows, k] . W^T (nn/layers.go:49-55 -> tensor/quant.go:35-56).
// With resid, y = product + resid (which may be y); only the row kernels of the quantized dtypes add it.
mi355x_status linear(Model& m, const Weight& w, const float* x, float* y, int64_t rows, const float* resid = nullptr) {
    int cls = act_class(w, rows, m.fx_panel.bytes);
    if (resid && cls == kActNone) return capi_fail(MI355X_ERR_INTERNAL, "mi355x: llama: no residual epilogue for this product");
    QGemvArgs a{w.buf.p, x, m.act[cls].p, y, rows, w.n, w.k, w.k, 0};
    a.resid = resid;
    hipError_t e;
    switch (w.dtype) {
    case kQ4_0:
        e = cls == kActFx || cls == kActFxPairs
                ? qgemm_q4_0_fx(w.buf.p, m.act[cls].p, y, resid, rows, w.n, w.k, cls == kActFxPairs ? m.fx_panel.p : nullptr, m.stream)
            : cls == kActQ4 ? qgemv_q4_0_act(a, kNoTune, m.stream)
                            : qgemv_q4_0(a, kNoTune, m.stream);
        break;
    case kQ8_0:
        if (cls != kActQ8) return capi_fail(MI355X_ERR_SHAPE, "mi355x: llama: q8_0 rows of %lld are too long", (long long)w.k);
        // several rows: W read once, on the matrix cores where the matrix is large
        e = qgemv_q8_0_mfma_pays(a) ? qgemv_q8_0_mfma(a, m.stream) : qgemv_q8_0_rows_ok(a) ? qgemv_q8_0_rows(a, m.stream) : qgemv_q8_0_act(a, kNoTune, m.stream);
        break;
    case kQ4_K: case kQ6_K: e = qgemv_kquant_act(w.dtype, a, m.stream); break;
    case kF32: case kF16: case kBF16: e = gemv_float(w.dtype, w.buf.p, x, y, rows, w.n, w.k, w.k, m.stream); break;
    default: return capi_fail(MI355X_ERR_DTYPE, "mi355x: llama: a linear weight of dtype %d", w.dtype);
    }
    LLM_HIP(e, "linear");
    return MI355X_OK;
}

mi355x_status embed_rows(Model& m, const int32_t* idx_dev, int64_t rows, float* out, uint32_t* err) {
    const Weight& w = m.embed;
    if (is_quantized(w.dtype)) {
        LLM_HIP(gather_rows(w.dtype, w.buf.p, w.n, w.k, idx_dev, rows, out, err, m.stream), "embedding");
        return MI355X_OK;
    }
    return capi_fail(MI355X_ERR_DTYPE, "mi355x: llama: token_embd.weight of dtype %d (block-quantized tables only)", w.dtype);
}

}  // namespace

uint32_t* device_error_word();  // capi.hip

// One pass of s tokens per sequence over the blocks (llm/model.go:391-437),
// tokens already on the device at m.tokens_dev [batch, s]. Leaves the final
// hidden state in m.x; advances the caches.
static mi355x_status forward(Model& m, int64_t s) {
    const auto& c = m.c;
    const int64_t B = c.batch, rows = B * s, past = m.cache_len;
    const int64_t qd = (int64_t)c.heads * c.head_dim, kvd = (int64_t)c.kv_heads * c.head_dim;
    float *x = m.x.as<float>(), *h = m.h.as<float>(), *q = m.q.as<float>(), *k = m.k.as<float>(), *v = m.v.as<float>();
    float *a = m.a.as<float>(), *o = m.o.as<float>(), *gate = m.gate.as<float>(), *up = m.up.as<float>(), *sw = m.s.as<float>();
    bool done[kActClasses];
    if (mi355x_status st = embed_rows(m, m.tokens_dev.as<int32_t>(), rows, x, device_error_word())) return st;
    // x += in . W^T: the prompt-sized fixed-point products add x as they store, the others leave it to a launch
    auto onto_x = [&](const Weight& w, const float* in) -> mi355x_status {
        const int cls = act_class(w, rows, m.fx_panel.bytes);
        if (cls == kActFx || cls == kActFxPairs) return linear(m, w, in, x, rows, x);
        if (mi355x_status st = linear(m, w, in, o, rows)) return st;
        LLM_HIP(add(x, o, x, rows * c.embed, m.stream), "residual");
        return MI355X_OK;
    };
    for (int i = 0; i < c.layers; i++) {
        Block& b = m.blocks[i];
        LLM_HIP(rmsnorm(x, b.attn_norm.buf.as<float>(), h, rows, c.embed, c.eps, m.stream), "attn_norm");
        if (mi355x_status st = convert_for(m, h, rows, c.embed, {&b.q, &b.k, &b.v}, done)) return st;
        if (mi355x_status st = linear(m, b.q, h, q, rows)) return st;
        if (mi355x_status st = linear(m, b.k, h, k, rows)) return st;
        if (mi355x_status st = linear(m, b.v, h, v, rows)) return st;
        if (b.biased()) {  // Linear.Forward: the bias behind the product, before the rotation (nn/layers.go:49-55)
            LLM_HIP(add_bias(q, b.q_bias.buf.as<float>(), rows, qd, m.stream), "q bias");
            LLM_HIP(add_bias(k, b.k_bias.buf.as<float>(), rows, kvd, m.stream), "k bias");
            LLM_HIP(add_bias(v, b.v_bias.buf.as<float>(), rows, kvd, m.stream), "v bias");
        }
        // q and k are [B, s, heads, dim]. One position: every head of every
        // sequence is a row `dim` apart. More: per sequence, heads are rows
        // `dim` apart and positions heads * dim apart.
        if (s == 1) {
            LLM_HIP(rope(q, q, B * c.heads, 1, c.head_dim, c.rope_dim, c.interleaved, c.head_dim, qd, c.head_dim, qd,
                         m.cos_t.as<float>(), m.sin_t.as<float>(), past, m.stream), "rope q");
            LLM_HIP(rope(k, k, B * c.kv_heads, 1, c.head_dim, c.rope_dim, c.interleaved, c.head_dim, kvd, c.head_dim, kvd,
                         m.cos_t.as<float>(), m.sin_t.as<float>(), past, m.stream), "rope k");
        } else {
            // the sequences' positions follow one another at the same distance: one launch, each sequence counting from `past`
            LLM_HIP(rope(q, q, c.heads, B * s, c.head_dim, c.rope_dim, c.interleaved, c.head_dim, qd, c.head_dim, qd,
                         m.cos_t.as<float>(), m.sin_t.as<float>(), past, m.stream, s), "rope q");
            LLM_HIP(rope(k, k, c.kv_heads, B * s, c.head_dim, c.rope_dim, c.interleaved, c.head_dim, kvd, c.head_dim, kvd,
                         m.cos_t.as<float>(), m.sin_t.as<float>(), past, m.stream, s), "rope k");
        }
        LLM_HIP(kv_write(k, m.keys[i].p, c.cache_dtype, B, c.kv_heads, s, c.head_dim, c.context, past, s * kvd, c.head_dim, kvd, m.stream), "cache keys");
        LLM_HIP(kv_write(v, m.values[i].p, c.cache_dtype, B, c.kv_heads, s, c.head_dim, c.context, past, s * kvd, c.head_dim, kvd, m.stream), "cache values");
        AttnArgs at;
        at.q = q; at.k = m.keys[i].p; at.v = m.values[i].p; at.kv_dtype = c.cache_dtype; at.out = a; at.lse = nullptr;
        at.q_strides[0] = s * qd; at.q_strides[1] = c.head_dim; at.q_strides[2] = qd;
        at.k_strides[0] = at.v_strides[0] = (int64_t)c.kv_heads * c.context * c.head_dim;
        at.k_strides[1] = at.v_strides[1] = (int64_t)c.context * c.head_dim;
        at.k_strides[2] = at.v_strides[2] = c.head_dim;
        for (int j = 0; j < 3; j++) at.o_strides[j] = at.q_strides[j];
        at.B = B; at.Q = s; at.K = past + s; at.H = c.heads; at.HK = c.kv_heads; at.D = c.head_dim;
        at.scale = 1.0 / std::sqrt((double)c.head_dim);
        at.causal = 1; at.causal_offset = past;
        attention_plan(B, c.heads, c.kv_heads, s, at.K, &at.chunk, &at.nsplit);
        size_t need = attention_workspace_bytes(B, c.heads, s, c.head_dim, at.nsplit);
        if (need + kAttnTicketBytes > m.act[0].bytes) return capi_fail(MI355X_ERR_INTERNAL, "mi355x: llama: attention scratch of %zu bytes, need %zu", m.act[0].bytes, need);
        LLM_HIP(attention(at, (uint8_t*)m.act[0].p + kAttnTicketBytes, m.stream), "attention");
        if (mi355x_status st = convert_for(m, a, rows, qd, {&b.o}, done)) return st;
        if (mi355x_status st = onto_x(b.o, a)) return st;
        LLM_HIP(rmsnorm(x, b.ffn_norm.buf.as<float>(), h, rows, c.embed, c.eps, m.stream), "ffn_norm");
        if (mi355x_status st = convert_for(m, h, rows, c.embed, {&b.gate, &b.up}, done)) return st;
        if (mi355x_status st = linear(m, b.gate, h, gate, rows)) return st;
        if (mi355x_status st = linear(m, b.up, h, up, rows)) return st;
        LLM_HIP(swiglu(gate, up, sw, rows, c.hidden, c.hidden, m.stream), "swiglu");
        if (mi355x_status st = convert_for(m, sw, rows, c.hidden, {&b.down}, done)) return st;
        if (mi355x_status st = onto_x(b.down, sw)) return st;
    }
    m.cache_len = past + s;
    return MI355X_OK;
}

// One decoding step of every sequence (llm/decode.go:188-227, stepGraph), for
// blocks whose linears are Q4_0: the tokens come from m.next_tok and the
// position from m.state, both on the device, so the same run of launches
// serves every position and can be replayed as a graph. Per block: norm with
// the activation conversion fused, q|k|v in one product, rotation and cache
// write in one launch, split attention, conversion, output projection with the
// residual added, norm, gate|up with SwiGLU in one product, conversion, down
// projection with the residual added.
static mi355x_status step_fast(Model& m) {
    const auto& c = m.c;
    const int64_t B = c.batch;
    const int64_t qd = (int64_t)c.heads * c.head_dim, kvd = (int64_t)c.kv_heads * c.head_dim, row = qd + 2 * kvd;
    float *x = m.x.as<float>(), *qkv = m.qkv.as<float>(), *a = m.a.as<float>(), *sw = m.s.as<float>();
    void* act = m.act[kActQ4].p;
    const int32_t* pos = m.state.as<int32_t>();
    if (mi355x_status st = embed_rows(m, m.next_tok.as<int32_t>(), B, x, device_error_word())) return st;
    AttnArgs at;
    at.q = qkv; at.kv_dtype = c.cache_dtype; at.out = a; at.lse = nullptr;
    at.q_strides[0] = row; at.q_strides[1] = c.head_dim; at.q_strides[2] = 0;
    at.k_strides[0] = at.v_strides[0] = (int64_t)c.kv_heads * c.context * c.head_dim;
    at.k_strides[1] = at.v_strides[1] = (int64_t)c.context * c.head_dim;
    at.k_strides[2] = at.v_strides[2] = c.head_dim;
    at.o_strides[0] = qd; at.o_strides[1] = c.head_dim; at.o_strides[2] = 0;
    at.B = B; at.Q = 1; at.K = 1; at.H = c.heads; at.HK = c.kv_heads; at.D = c.head_dim;
    at.scale = 1.0 / std::sqrt((double)c.head_dim);
    at.causal = 0; at.causal_offset = 0;
    at.dyn_k = pos;  // position p holds p keys before this step's own
    at.k = m.keys[0].p; at.v = m.values[0].p;  // every layer's caches are allocated alike
    const bool one_launch = attention_decode_ok(at, c.context);
    // one sequence: the norms ride on the products; with several, norms of their own are the faster (measured at 8)
    const bool norm_head = q4_0_norm_head_ok(c.embed) && B == 1;
    if (!one_launch) attention_plan(B, c.heads, c.kv_heads, 1, c.context, &at.chunk, &at.nsplit);
    for (int i = 0; i < c.layers; i++) {
        Block& b = m.blocks[i];
        const void* w3[3] = {b.q.buf.p, b.k.buf.p, b.v.buf.p};
        const int64_t n3[3] = {qd, kvd, kvd};
        if (c.interleaved && c.head_dim % 2 == 0 && c.rope_dim % 2 == 0) {  // the rotation and the cache writes ride on the product
            Q4RopeTail tail;
            tail.cosv = m.cos_t.as<float>(); tail.sinv = m.sin_t.as<float>(); tail.pos = pos;
            tail.kcache = m.keys[i].p; tail.vcache = m.values[i].p;
            tail.cache_dt = c.cache_dtype; tail.H = c.heads; tail.HK = c.kv_heads; tail.dim = c.head_dim; tail.rope_dim = c.rope_dim;
            tail.cap = c.context;
            Q4NormHead head;  // and the norm in front of it is its first phase
            if (norm_head) {
                head.x = x; head.w = b.attn_norm.buf.as<float>(); head.eps = c.eps;
            } else {
                LLM_HIP(rmsnorm_q4act(x, b.attn_norm.buf.as<float>(), nullptr, act, B, c.embed, c.eps, m.stream), "attn_norm");
            }
            LLM_HIP(qgemv_q4_0_act_qkv_rope(w3, n3, act, qkv, B, c.embed, tail, head, kNoTune, m.stream), "norm, q|k|v, rope and cache");
        } else {
            LLM_HIP(rmsnorm_q4act(x, b.attn_norm.buf.as<float>(), nullptr, act, B, c.embed, c.eps, m.stream), "attn_norm");
            LLM_HIP(qgemv_q4_0_act_multi(w3, n3, act, qkv, B, c.embed, kNoTune, m.stream), "q|k|v");
            LLM_HIP(rope_kv(qkv, m.keys[i].p, m.values[i].p, c.cache_dtype, B, c.heads, c.kv_heads, c.head_dim, c.rope_dim, c.interleaved,
                            c.context, m.cos_t.as<float>(), m.sin_t.as<float>(), pos, m.stream), "rope and cache");
        }
        at.k = m.keys[i].p; at.v = m.values[i].p;
        if (one_launch) {  // leaves its result converted for the output projection
            at.out = nullptr;
            LLM_HIP(attention_decode(at, c.context, m.act[0].p, act, (int64_t)q4_0_act_bytes(qd), m.stream, kAttnActQ4, m.attn_flags.p, m.attn_flags.bytes, device_error_word()), "attention");
        } else {
            LLM_HIP(attention(at, (uint8_t*)m.act[0].p + kAttnTicketBytes, m.stream), "attention");
            LLM_HIP(q4_0_convert_act(a, B, qd, qd, act, m.stream), "convert");
        }
        QGemvArgs o{b.o.buf.p, nullptr, act, x, B, c.embed, qd, 0, 0};
        o.resid = x;
        LLM_HIP(qgemv_q4_0_act(o, kNoTune, m.stream), "attn_output");
        void* act_down = act;
        if (q4_0_swiglu_convert_ok(c.hidden, c.embed)) {  // the conversion rides on the product, into a buffer of its own
            act_down = m.act2.p;
            Q4NormHead head;
            if (norm_head) {
                head.x = x; head.w = b.ffn_norm.buf.as<float>(); head.eps = c.eps;
            } else {
                LLM_HIP(rmsnorm_q4act(x, b.ffn_norm.buf.as<float>(), nullptr, act, B, c.embed, c.eps, m.stream), "ffn_norm");
            }
            LLM_HIP(qgemv_q4_0_act_swiglu_convert(b.gate.buf.p, b.up.buf.p, act, act_down, B, c.hidden, c.embed, head, kNoTune, m.stream),
                    "norm, gate|up, conversion");
        } else {
            LLM_HIP(rmsnorm_q4act(x, b.ffn_norm.buf.as<float>(), nullptr, act, B, c.embed, c.eps, m.stream), "ffn_norm");
            LLM_HIP(qgemv_q4_0_act_swiglu(b.gate.buf.p, b.up.buf.p, act, sw, B, c.hidden, c.embed, kNoTune, m.stream), "gate|up");
            LLM_HIP(q4_0_convert_act(sw, B, c.hidden, c.hidden, act, m.stream), "convert");
        }
        QGemvArgs d{b.down.buf.p, nullptr, act_down, x, B, c.embed, c.hidden, 0, 0};
        d.resid = x;
        LLM_HIP(qgemv_q4_0_act(d, kNoTune, m.stream), "ffn_down");
    }
    return MI355X_OK;
}

static std::atomic<int> g_llama_rows_off{0};  // measurement aid: 1 = several sequences take step_fast as one does
static std::atomic<int> g_llama_rows_plain{0};  // measurement aid: 1 = step_rows with the rotation and SwiGLU as launches of their own
void set_llama_rows_off(int v) { g_llama_rows_off = v == 1; g_llama_rows_plain = v >= 2 ? v : 0; }

// One decoding step of two to sixty-four sequences with Q4_0 linears (the case of step_fast): the same
// operations, but every product reads its weights once per eight sequences (from HBM once), on the int8 matrix cores
// (qgemv_q4_0_rows.hip), where step_fast's products read them once per sequence. Nine launches a block:
// norm (adding the shares of the product before it into x) with conversion, q|k|v, rotation and cache
// write, attention with conversion, output projection in two shares of K, norm, gate|up, SiLU * up with
// conversion, down projection in two shares. The shares of the last down projection are added at the end.
static mi355x_status step_rows(Model& m) {
    const auto& c = m.c;
    const int64_t B = c.batch;
    const int64_t qd = (int64_t)c.heads * c.head_dim, kvd = (int64_t)c.kv_heads * c.head_dim, row = qd + 2 * kvd;
    float *x = m.x.as<float>(), *qkv = m.qkv.as<float>(), *gu = m.gu.as<float>(), *parts = m.parts.as<float>();
    void* act = m.rows_act.p;
    const int32_t* pos = m.state.as<int32_t>();
    if (mi355x_status st = embed_rows(m, m.next_tok.as<int32_t>(), B, x, device_error_word())) return st;
    AttnArgs at;
    at.q = qkv; at.kv_dtype = c.cache_dtype; at.out = nullptr; at.lse = nullptr;
    at.q_strides[0] = row; at.q_strides[1] = c.head_dim; at.q_strides[2] = 0;
    at.k_strides[0] = at.v_strides[0] = (int64_t)c.kv_heads * c.context * c.head_dim;
    at.k_strides[1] = at.v_strides[1] = (int64_t)c.context * c.head_dim;
    at.k_strides[2] = at.v_strides[2] = c.head_dim;
    at.o_strides[0] = qd; at.o_strides[1] = c.head_dim; at.o_strides[2] = 0;
    at.B = B; at.Q = 1; at.K = 1; at.H = c.heads; at.HK = c.kv_heads; at.D = c.head_dim;
    at.scale = 1.0 / std::sqrt((double)c.head_dim);
    at.causal = 0; at.causal_offset = 0;
    at.dyn_k = pos;  // position p holds p keys before this step's own
    const int shares = 2;  // of K, for the two products with 4096 rows of W: measured against 1, 3 and 4
    for (int i = 0; i < c.layers; i++) {
        Block& b = m.blocks[i];
        LLM_HIP(rows_norm_act(x, parts, i == 0 ? 0 : shares, b.attn_norm.buf.as<float>(), act, B, c.embed, c.eps, m.stream), "attn_norm");
        const void* w3[3] = {b.q.buf.p, b.k.buf.p, b.v.buf.p};
        const int64_t n3[3] = {qd, kvd, kvd};
        if (c.interleaved && c.head_dim % 2 == 0 && c.rope_dim % 2 == 0 && g_llama_rows_plain != 2 && g_llama_rows_plain != 4) {  // the rotation and the cache writes ride on the product
            Q4RopeTail tail;
            tail.cosv = m.cos_t.as<float>(); tail.sinv = m.sin_t.as<float>(); tail.pos = pos;
            tail.kcache = m.keys[i].p; tail.vcache = m.values[i].p;
            tail.cache_dt = c.cache_dtype; tail.H = c.heads; tail.HK = c.kv_heads; tail.dim = c.head_dim; tail.rope_dim = c.rope_dim;
            tail.cap = c.context;
            LLM_HIP(qgemv_q4_0_rows_qkv_rope(w3, n3, act, qkv, B, c.embed, tail, m.stream), "q|k|v, rope and cache");
        } else {
            LLM_HIP(qgemv_q4_0_rows_multi(w3, n3, act, qkv, nullptr, B, c.embed, 1, m.stream), "q|k|v");
            LLM_HIP(rope_kv(qkv, m.keys[i].p, m.values[i].p, c.cache_dtype, B, c.heads, c.kv_heads, c.head_dim, c.rope_dim, c.interleaved,
                            c.context, m.cos_t.as<float>(), m.sin_t.as<float>(), pos, m.stream), "rope and cache");
        }
        at.k = m.keys[i].p; at.v = m.values[i].p;
        LLM_HIP(attention_decode(at, c.context, m.act[0].p, act, 0, m.stream, kAttnActRows, m.attn_flags.p, m.attn_flags.bytes, device_error_word()), "attention");
        LLM_HIP(qgemv_q4_0_rows(b.o.buf.p, act, parts, nullptr, B, c.embed, qd, shares, m.stream), "attn_output");
        LLM_HIP(rows_norm_act(x, parts, shares, b.ffn_norm.buf.as<float>(), act, B, c.embed, c.eps, m.stream), "ffn_norm");
        if (g_llama_rows_plain != 2 && g_llama_rows_plain != 3) {  // SiLU * up and the conversion ride on the product, into a buffer of their own
            LLM_HIP(qgemv_q4_0_rows_swiglu_act(b.gate.buf.p, b.up.buf.p, act, m.rows_act2.p, B, c.hidden, c.embed, m.stream), "gate|up, conversion");
            LLM_HIP(qgemv_q4_0_rows(b.down.buf.p, m.rows_act2.p, parts, nullptr, B, c.embed, c.hidden, shares, m.stream), "ffn_down");
        } else {
            const void* w2[3] = {b.gate.buf.p, b.up.buf.p, nullptr};
            const int64_t n2[3] = {c.hidden, c.hidden, 0};
            LLM_HIP(qgemv_q4_0_rows_multi(w2, n2, act, gu, nullptr, B, c.embed, 1, m.stream), "gate|up");
            LLM_HIP(rows_swiglu_act(gu, gu + c.hidden, act, B, c.hidden, 2 * (int64_t)c.hidden, m.stream), "swiglu");
            LLM_HIP(qgemv_q4_0_rows(b.down.buf.p, act, parts, nullptr, B, c.embed, c.hidden, shares, m.stream), "ffn_down");
        }
    }
    LLM_HIP(rows_add_parts(x, parts, shares, B * c.embed, m.stream), "residual");
    return MI355X_OK;
}

// One decoding step of every sequence for blocks of any supported dtypes: the per-operator launches of
// forward() for one position, but with the position read from m.state on the device (rotation, cache
// write, number of keys), so that the step can be captured once and replayed as a graph like step_fast
// (the reference records its decoding step for the same reason, llm/decode.go:79-160).
static mi355x_status step_any(Model& m) {
    const auto& c = m.c;
    const int64_t B = c.batch;
    const int64_t qd = (int64_t)c.heads * c.head_dim, kvd = (int64_t)c.kv_heads * c.head_dim;
    float *x = m.x.as<float>(), *h = m.h.as<float>(), *q = m.q.as<float>(), *k = m.k.as<float>(), *v = m.v.as<float>();
    float *a = m.a.as<float>(), *o = m.o.as<float>(), *gate = m.gate.as<float>(), *up = m.up.as<float>(), *sw = m.s.as<float>();
    float *qkv = m.qkv.as<float>(), *gu = m.gu.as<float>();
    const int32_t* pos = m.state.as<int32_t>();
    bool done[kActClasses];
    if (mi355x_status st = embed_rows(m, m.next_tok.as<int32_t>(), B, x, device_error_word())) return st;
    AttnArgs at;
    at.q = q; at.kv_dtype = c.cache_dtype; at.out = a; at.lse = nullptr;
    at.q_strides[0] = qd; at.q_strides[1] = c.head_dim; at.q_strides[2] = 0;
    at.k_strides[0] = at.v_strides[0] = (int64_t)c.kv_heads * c.context * c.head_dim;
    at.k_strides[1] = at.v_strides[1] = (int64_t)c.context * c.head_dim;
    at.k_strides[2] = at.v_strides[2] = c.head_dim;
    at.o_strides[0] = qd; at.o_strides[1] = c.head_dim; at.o_strides[2] = 0;
    at.B = B; at.Q = 1; at.K = 1; at.H = c.heads; at.HK = c.kv_heads; at.D = c.head_dim;
    at.scale = 1.0 / std::sqrt((double)c.head_dim);
    at.causal = 0; at.causal_offset = 0;
    at.dyn_k = pos;  // position p holds p keys before this step's own
    at.k = m.keys[0].p; at.v = m.values[0].p;
    const bool one_launch = attention_decode_ok(at, c.context);
    if (!one_launch) attention_plan(B, c.heads, c.kv_heads, 1, c.context, &at.chunk, &at.nsplit);
    for (int i = 0; i < c.layers; i++) {
        Block& b = m.blocks[i];
        const bool qkv_kq = b.qkv.set() && act_class(b.qkv, B) == kActKQ;
        if (qkv_kq) {  // norm and conversion in one launch
            LLM_HIP(rmsnorm_kq_act(x, b.attn_norm.buf.as<float>(), m.act[kActKQ].p, B, c.embed, c.eps, m.stream), "attn_norm");
        } else {
            LLM_HIP(rmsnorm(x, b.attn_norm.buf.as<float>(), h, B, c.embed, c.eps, m.stream), "attn_norm");
            if (b.qkv.set())
                if (mi355x_status st = convert_for(m, h, B, c.embed, {&b.qkv}, done)) return st;
        }
        if (b.qkv.set()) {  // one product into [B, q | k | v]
            QGemvArgs qa{b.qkv.buf.p, nullptr, m.act[kActKQ].p, qkv, B, b.qkv.n, b.qkv.k, b.qkv.k, 0};
            // From three sequences on, where W can be read once for eight of them, that beats the tail that saves a launch.
            const bool read_once = B >= 3 && qkv_kq && qgemv_kquant_rows_pays(b.qkv.dtype, qa);
            const bool pairs = c.interleaved && c.head_dim % 2 == 0 && c.rope_dim % 2 == 0;
            const bool once_rope = read_once && pairs && qgemv_kquant_rows_rope_ok(b.qkv.dtype, qa);
            if (!b.biased() && (once_rope || (qkv_kq && !read_once && pairs && qgemv_kquant_rope_ok(b.qkv.dtype, qa)))) {
                Q4RopeTail tail;  // the rotation and the cache writes ride on the product
                tail.cosv = m.cos_t.as<float>(); tail.sinv = m.sin_t.as<float>(); tail.pos = pos;
                tail.kcache = m.keys[i].p; tail.vcache = m.values[i].p;
                tail.cache_dt = c.cache_dtype; tail.H = c.heads; tail.HK = c.kv_heads; tail.dim = c.head_dim; tail.rope_dim = c.rope_dim;
                tail.cap = c.context;
                if (once_rope) LLM_HIP(qgemv_kquant_rows_rope(b.qkv.dtype, qa, tail, m.stream), "q|k|v, rope and cache");
                else LLM_HIP(qgemv_kquant_act_rope(b.qkv.dtype, qa, tail, m.stream), "q|k|v, rope and cache");
            } else {
                // with biases (qwen2): one product, then the biases, the rotation and the cache writes in one launch
                if (mi355x_status st = linear(m, b.qkv, h, qkv, B)) return st;
                LLM_HIP(rope_kv(qkv, m.keys[i].p, m.values[i].p, c.cache_dtype, B, c.heads, c.kv_heads, c.head_dim, c.rope_dim, c.interleaved,
                                c.context, m.cos_t.as<float>(), m.sin_t.as<float>(), pos, m.stream,
                                b.biased() ? b.qkv_bias.as<float>() : nullptr), "biases, rope and cache");
            }
            at.q = qkv; at.q_strides[0] = qd + 2 * kvd;
        } else {
            if (mi355x_status st = convert_for(m, h, B, c.embed, {&b.q, &b.k, &b.v}, done)) return st;
            if (mi355x_status st = linear(m, b.q, h, q, B)) return st;
            if (mi355x_status st = linear(m, b.k, h, k, B)) return st;
            if (mi355x_status st = linear(m, b.v, h, v, B)) return st;
            // biases (qwen2), rotation and cache writes in one launch
            LLM_HIP(rope_kv_split(q, k, v, m.keys[i].p, m.values[i].p, c.cache_dtype, B, c.heads, c.kv_heads, c.head_dim, c.rope_dim,
                                  c.interleaved, c.context, m.cos_t.as<float>(), m.sin_t.as<float>(), pos, m.stream,
                                  b.biased() ? b.qkv_bias.as<float>() : nullptr), "biases, rope and cache");
            at.q = q; at.q_strides[0] = qd;
        }
        at.k = m.keys[i].p; at.v = m.values[i].p;
        // K-quant output projection: attention leaves its result as the int8 super-blocks that product reads
        const bool a_kq = one_launch && act_class(b.o, B) == kActKQ && attention_decode_kq_ok(at);
        if (a_kq) {
            LLM_HIP(attention_decode(at, c.context, m.act[0].p, m.act[kActKQ].p, (int64_t)kq_act_bytes(qd), m.stream, kAttnActKQ, m.attn_flags.p, m.attn_flags.bytes, device_error_word()), "attention");
        } else {
            if (one_launch) LLM_HIP(attention_decode(at, c.context, m.act[0].p, nullptr, 0, m.stream, kAttnActQ4, m.attn_flags.p, m.attn_flags.bytes, device_error_word()), "attention");
            else LLM_HIP(attention(at, (uint8_t*)m.act[0].p + kAttnTicketBytes, m.stream), "attention");
            if (mi355x_status st = convert_for(m, a, B, qd, {&b.o}, done)) return st;
        }
        if (act_class(b.o, B) != kActNone) {  // the residual rides on the product
            if (mi355x_status st = linear(m, b.o, a, x, B, x)) return st;
        } else {
            if (mi355x_status st = linear(m, b.o, a, o, B)) return st;
            LLM_HIP(add(x, o, x, B * c.embed, m.stream), "residual");
        }
        const bool down_kq = act_class(b.down, B) == kActKQ;  // then SwiGLU leaves its result converted
        if (b.gate_up.set() && act_class(b.gate_up, B) == kActKQ) {
            LLM_HIP(rmsnorm_kq_act(x, b.ffn_norm.buf.as<float>(), m.act[kActKQ].p, B, c.embed, c.eps, m.stream), "ffn_norm");
            if (mi355x_status st = linear(m, b.gate_up, h, gu, B)) return st;
            if (down_kq) LLM_HIP(swiglu_kq_act(gu, gu + c.hidden, m.act[kActKQ].p, B, c.hidden, 2 * (int64_t)c.hidden, m.stream), "swiglu");
            else LLM_HIP(swiglu(gu, gu + c.hidden, sw, B, c.hidden, 2 * (int64_t)c.hidden, m.stream), "swiglu");
        } else if (b.gate_up.set()) {  // one product into [B, gate | up]
            LLM_HIP(rmsnorm(x, b.ffn_norm.buf.as<float>(), h, B, c.embed, c.eps, m.stream), "ffn_norm");
            if (mi355x_status st = convert_for(m, h, B, c.embed, {&b.gate_up}, done)) return st;
            if (mi355x_status st = linear(m, b.gate_up, h, gu, B)) return st;
            if (down_kq) LLM_HIP(swiglu_kq_act(gu, gu + c.hidden, m.act[kActKQ].p, B, c.hidden, 2 * (int64_t)c.hidden, m.stream), "swiglu");
            else LLM_HIP(swiglu(gu, gu + c.hidden, sw, B, c.hidden, 2 * (int64_t)c.hidden, m.stream), "swiglu");
        } else {
            LLM_HIP(rmsnorm(x, b.ffn_norm.buf.as<float>(), h, B, c.embed, c.eps, m.stream), "ffn_norm");
            if (mi355x_status st = convert_for(m, h, B, c.embed, {&b.gate, &b.up}, done)) return st;
            if (mi355x_status st = linear(m, b.gate, h, gate, B)) return st;
            if (mi355x_status st = linear(m, b.up, h, up, B)) return st;
            if (down_kq) LLM_HIP(swiglu_kq_act(gate, up, m.act[kActKQ].p, B, c.hidden, c.hidden, m.stream), "swiglu");
            else LLM_HIP(swiglu(gate, up, sw, B, c.hidden, c.hidden, m.stream), "swiglu");
        }
        if (!down_kq)
            if (mi355x_status st = convert_for(m, sw, B, c.hidden, {&b.down}, done)) return st;
        if (act_class(b.down, B) != kActNone) {
            if (mi355x_status st = linear(m, b.down, sw, x, B, x)) return st;
        } else {
            if (mi355x_status st = linear(m, b.down, sw, o, B)) return st;
            LLM_HIP(add(x, o, x, B * c.embed, m.stream), "residual");
        }
    }
    return MI355X_OK;
}

// Norm and output projection of `rows` rows of hidden states at xin, which are
// row_stride floats apart, into m.logits [rows, vocab].
static mi355x_status head(Model& m, const float* xin, int64_t rows, int64_t row_stride) {
    const auto& c = m.c;
    float* hl = m.hlast.as<float>();
    if (row_stride == c.embed) {
        LLM_HIP(rmsnorm(xin, m.norm.buf.as<float>(), hl, rows, c.embed, c.eps, m.stream), "output_norm");
    } else {
        for (int64_t r = 0; r < rows; r++)
            LLM_HIP(rmsnorm(xin + r * row_stride, m.norm.buf.as<float>(), hl + r * c.embed, 1, c.embed, c.eps, m.stream), "output_norm");
    }
    const Weight& w = m.tied ? m.embed : m.output;
    bool done[kActClasses];
    if (mi355x_status st = convert_for(m, hl, rows, c.embed, {&w}, done)) return st;
    return linear(m, w, hl, m.logits.as<float>(), rows);
}

}  // namespace mimir

using mimir::Model;

// How mi355x_llama_generate runs its decoding steps: 0 the fused launches
// replayed as a graph where the model qualifies, 1 the same launches issued one
// by one, 2 the general per-operator path.
static std::atomic<int> g_llama_step_mode{0};
namespace mimir {
void set_llama_step_mode(int mode) { g_llama_step_mode = mode; }
}

extern "C" {

mi355x_status mi355x_llama_create(const mi355x_llama_config* cfg, void** out) {
    using namespace mimir;
    if (!cfg || !out) return capi_fail(MI355X_ERR_INTERNAL, "mi355x: llama_create: null pointer");
    const auto& c = *cfg;
    // readConfig's checks (llm/model.go:97-171)
    if (c.embed <= 0 || c.hidden <= 0 || c.layers <= 0 || c.layers > 1024 || c.heads <= 0 || c.kv_heads <= 0 || c.heads % c.kv_heads != 0 ||
        c.head_dim <= 0 || c.head_dim > 256 || c.rope_dim <= 0 || c.rope_dim > c.head_dim || c.rope_dim % 2 != 0 || c.vocab <= 0 || c.context <= 0 ||
        c.batch <= 0 || !(c.rope_base > 1) || !(c.rope_scale > 0) || !(c.eps > 0))
        return capi_fail(MI355X_ERR_SHAPE, "mi355x: llama: model hyperparameters: %d layers, %d heads and %d key heads of %d features, %d rotated",
                         c.layers, c.heads, c.kv_heads, c.head_dim, c.rope_dim);
    if (c.cache_dtype != MI355X_F32 && c.cache_dtype != MI355X_F16) return capi_fail(MI355X_ERR_DTYPE, "mi355x: llama: KV cache of dtype %d", c.cache_dtype);
    auto m = std::make_unique<Model>();
    m->c = c;
    m->blocks.resize(c.layers);
    *out = m.release();
    return MI355X_OK;
}

mi355x_status mi355x_llama_destroy(void* model) {
    delete (Model*)model;
    return MI355X_OK;
}

// Names are llama.cpp's, as the reference reads them (llm/model.go:268-310).
mi355x_status mi355x_llama_set_tensor(void* model, const char* name, int dtype, const void* host, int64_t n_elems) {
    using namespace mimir;
    Model* m = (Model*)model;
    if (!m || !name || !host) return capi_fail(MI355X_ERR_INTERNAL, "mi355x: llama_set_tensor: null pointer");
    const auto& c = m->c;
    const int64_t qd = (int64_t)c.heads * c.head_dim, kvd = (int64_t)c.kv_heads * c.head_dim;
    Weight* w = nullptr;
    int64_t n = 0, k = 0;
    std::string s(name);
    if (s == "token_embd.weight") { w = &m->embed; n = c.vocab; k = c.embed; }
    else if (s == "output_norm.weight") { w = &m->norm; n = 1; k = c.embed; }
    else if (s == "output.weight") { w = &m->output; n = c.vocab; k = c.embed; }
    else if (s.rfind("blk.", 0) == 0) {
        size_t dot = s.find('.', 4);
        int i = atoi(s.substr(4, dot - 4).c_str());
        if (dot == std::string::npos || i < 0 || i >= c.layers) return capi_fail(MI355X_ERR_SHAPE, "mi355x: llama: tensor %s of a model of %d blocks", name, c.layers);
        std::string leaf = s.substr(dot + 1);
        Block& b = m->blocks[i];
        if (leaf == "attn_norm.weight") { w = &b.attn_norm; n = 1; k = c.embed; }
        else if (leaf == "ffn_norm.weight") { w = &b.ffn_norm; n = 1; k = c.embed; }
        else if (leaf == "attn_q.weight") { w = &b.q; n = qd; k = c.embed; }
        else if (leaf == "attn_k.weight") { w = &b.k; n = kvd; k = c.embed; }
        else if (leaf == "attn_v.weight") { w = &b.v; n = kvd; k = c.embed; }
        else if (leaf == "attn_output.weight") { w = &b.o; n = c.embed; k = qd; }
        else if (leaf == "ffn_gate.weight") { w = &b.gate; n = c.hidden; k = c.embed; }
        else if (leaf == "ffn_up.weight") { w = &b.up; n = c.hidden; k = c.embed; }
        else if (leaf == "ffn_down.weight") { w = &b.down; n = c.embed; k = c.hidden; }
        else if (leaf == "attn_q.bias") { w = &b.q_bias; n = 1; k = qd; }
        else if (leaf == "attn_k.bias") { w = &b.k_bias; n = 1; k = kvd; }
        else if (leaf == "attn_v.bias") { w = &b.v_bias; n = 1; k = kvd; }
    }
    if (!w) return capi_fail(MI355X_ERR_SHAPE, "mi355x: llama: unknown tensor %s", name);
    if (n * k != n_elems) return capi_fail(MI355X_ERR_SHAPE, "mi355x: llama: %s of %lld elements, want [%lld, %lld]", name, (long long)n_elems, (long long)n, (long long)k);
    int bs = block_size(dtype), bb = block_bytes(dtype);
    if (bb == 0 || k % bs != 0) return capi_fail(MI355X_ERR_DTYPE, "mi355x: llama: %s of dtype %d", name, dtype);
    if ((w == &m->norm || s.find("_norm.weight") != std::string::npos || s.find(".bias") != std::string::npos) && dtype != kF32)
        return capi_fail(MI355X_ERR_DTYPE, "mi355x: llama: %s of dtype %d, want float32", name, dtype);
    size_t bytes = (size_t)(n_elems / bs) * bb;
    LLM_HIP(w->buf.alloc(bytes), "hipMalloc(weight)");
    LLM_HIP(hipMemcpy(w->buf.p, host, bytes, hipMemcpyHostToDevice), "hipMemcpy(weight)");
    w->dtype = dtype; w->n = n; w->k = k;
    m->ready = false;
    return MI355X_OK;
}

// Divisors of each pair's frequency (rope_freqs.weight, llm/model.go:318-346).
mi355x_status mi355x_llama_set_rope_factors(void* model, const float* factors, int32_t n) {
    using namespace mimir;
    Model* m = (Model*)model;
    if (!m || (n > 0 && !factors)) return capi_fail(MI355X_ERR_INTERNAL, "mi355x: llama_set_rope_factors: null pointer");
    if (n != 0 && n != m->c.rope_dim / 2) return capi_fail(MI355X_ERR_SHAPE, "mi355x: llama: %d rope frequency factors, want %d", n, m->c.rope_dim / 2);
    for (int i = 0; i < n; i++)
        if (!(factors[i] > 0) || std::isinf(factors[i])) return capi_fail(MI355X_ERR_SHAPE, "mi355x: llama: rope frequency factor %g", factors[i]);
    m->rope_factors.assign(factors, factors + n);
    m->ready = false;
    return MI355X_OK;
}

// Checks that every tensor is there, builds the rotary table and allocates
// the caches and the activations of calls of up to max_tokens tokens per
// sequence.
mi355x_status mi355x_llama_finalize(void* model, int64_t max_tokens) {
    using namespace mimir;
    Model* m = (Model*)model;
    if (!m || max_tokens <= 0) return capi_fail(MI355X_ERR_INTERNAL, "mi355x: llama_finalize: bad arguments");
    const auto& c = m->c;
    if (!m->embed.set() || !m->norm.set()) return capi_fail(MI355X_ERR_SHAPE, "mi355x: llama: token_embd.weight or output_norm.weight missing");
    m->tied = !m->output.set();  // llm/model.go:283-288
    for (int i = 0; i < c.layers; i++) {
        Block& b = m->blocks[i];
        for (const Weight* w : {&b.attn_norm, &b.ffn_norm, &b.q, &b.k, &b.v, &b.o, &b.gate, &b.up, &b.down})
            if (!w->set()) return capi_fail(MI355X_ERR_SHAPE, "mi355x: llama: block %d is missing a tensor", i);
        if (b.q_bias.set() != b.k_bias.set() || b.q_bias.set() != b.v_bias.set())
            return capi_fail(MI355X_ERR_SHAPE, "mi355x: llama: block %d has some of attn_{q,k,v}.bias, want all three or none", i);
    }
    // nn/transformer.go:146-164 with llm/model.go:332-346: float64 angles, rounded to float32
    const int half = c.rope_dim / 2;
    std::vector<float> cosv((size_t)c.context * half), sinv((size_t)c.context * half);
    std::vector<double> inv(half);
    for (int i = 0; i < half; i++) {
        double f = std::pow(c.rope_base, -(double)(2 * i) / (double)c.rope_dim);
        f = f / c.rope_scale;
        if (!m->rope_factors.empty()) f /= (double)m->rope_factors[i];
        inv[i] = f;
    }
    for (int64_t p = 0; p < c.context; p++)
        for (int i = 0; i < half; i++) {
            double ang = (double)p * inv[i];
            cosv[p * half + i] = (float)std::cos(ang);
            sinv[p * half + i] = (float)std::sin(ang);
        }
    LLM_HIP(m->cos_t.alloc(cosv.size() * 4), "hipMalloc(rope table)");
    LLM_HIP(m->sin_t.alloc(sinv.size() * 4), "hipMalloc(rope table)");
    LLM_HIP(hipMemcpy(m->cos_t.p, cosv.data(), cosv.size() * 4, hipMemcpyHostToDevice), "hipMemcpy(rope table)");
    LLM_HIP(hipMemcpy(m->sin_t.p, sinv.data(), sinv.size() * 4, hipMemcpyHostToDevice), "hipMemcpy(rope table)");

    const size_t esz = c.cache_dtype == kF32 ? 4 : 2;
    const size_t cache_bytes = (size_t)c.batch * c.kv_heads * c.context * c.head_dim * esz;
    m->keys.clear(); m->values.clear();
    m->keys.resize(c.layers); m->values.resize(c.layers);
    for (int i = 0; i < c.layers; i++) {
        LLM_HIP(m->keys[i].alloc(cache_bytes), "hipMalloc(KV cache)");
        LLM_HIP(m->values[i].alloc(cache_bytes), "hipMalloc(KV cache)");
        LLM_HIP(hipMemset(m->keys[i].p, 0, cache_bytes), "hipMemset(KV cache)");    // NewKVCache starts from zeros
        LLM_HIP(hipMemset(m->values[i].p, 0, cache_bytes), "hipMemset(KV cache)");
    }
    m->cache_len = 0;
    const int64_t rows = (int64_t)c.batch * max_tokens;
    const int64_t qd = (int64_t)c.heads * c.head_dim, kvd = (int64_t)c.kv_heads * c.head_dim;
    m->max_rows = rows;
    LLM_HIP(m->x.alloc(rows * c.embed * 4), "hipMalloc"); LLM_HIP(m->h.alloc(rows * c.embed * 4), "hipMalloc");
    LLM_HIP(m->q.alloc(rows * qd * 4), "hipMalloc"); LLM_HIP(m->k.alloc(rows * kvd * 4), "hipMalloc"); LLM_HIP(m->v.alloc(rows * kvd * 4), "hipMalloc");
    LLM_HIP(m->a.alloc(rows * qd * 4), "hipMalloc"); LLM_HIP(m->o.alloc(rows * c.embed * 4), "hipMalloc");
    LLM_HIP(m->gate.alloc(rows * c.hidden * 4), "hipMalloc"); LLM_HIP(m->up.alloc(rows * c.hidden * 4), "hipMalloc"); LLM_HIP(m->s.alloc(rows * c.hidden * 4), "hipMalloc");
    LLM_HIP(m->hlast.alloc(rows * c.embed * 4), "hipMalloc");
    LLM_HIP(m->logits.alloc((size_t)rows * c.vocab * 4), "hipMalloc(logits)");
    LLM_HIP(m->tokens_dev.alloc(rows * 4), "hipMalloc"); LLM_HIP(m->next_tok.alloc(c.batch * 4), "hipMalloc");
    const int64_t kmax = c.hidden > qd ? (c.hidden > c.embed ? c.hidden : c.embed) : (qd > c.embed ? qd : c.embed);
    for (int cls = 1; cls < kActClasses; cls++) {
        int64_t kk = cls == kActKQ ? (kmax + 255) / 256 * 256 : cls == kActFx || cls == kActFxPairs ? (kmax + 127) / 128 * 128 : (kmax + 63) / 64 * 64;
        LLM_HIP(m->act[cls].alloc(act_row_bytes(cls, kk) * rows + 64), "hipMalloc(activations)");
    }
    LLM_HIP(m->act2.alloc(q4_0_act_bytes((c.hidden + 63) / 64 * 64) * c.batch + 64), "hipMalloc(activations)");
    {
        // the workspace of the fixed-point product's binary16 form, which calls of some hundreds of rows take: the largest matrix's
        size_t panel = 0;
        for (const Block& b : m->blocks)
            for (const Weight* w : {&b.q, &b.k, &b.v, &b.o, &b.gate, &b.up, &b.down, &b.qkv, &b.gate_up})
                if (w->set() && w->dtype == kQ4_0 && qgemm_q4_0_fx16_ws_bytes(w->n, w->k) > panel) panel = qgemm_q4_0_fx16_ws_bytes(w->n, w->k);
        m->fx_panel.release();
        m->fx_panel.bytes = 0;
        if (panel && rows >= 256) LLM_HIP(m->fx_panel.alloc(panel), "hipMalloc(fixed-point product workspace)");
    }
    int chunk, nsplit;
    attention_plan(c.batch, c.heads, c.kv_heads, max_tokens, c.context, &chunk, &nsplit);
    size_t attn_ws = 0;  // the most splits come from the smallest chunk
    for (int cc = 32; cc <= 256; cc <<= 1) {
        size_t b = attention_workspace_bytes(c.batch, c.heads, max_tokens, c.head_dim, (int)((c.context + cc - 1) / cc));
        attn_ws = b > attn_ws ? b : attn_ws;
    }
    {
        int ns, cm;
        attention_decode_plan(c.batch, c.heads, c.kv_heads, c.context, &ns, &cm);
        size_t b = attention_decode_workspace_bytes(c.batch, c.heads, c.head_dim, ns);
        attn_ws = (b > attn_ws ? b : attn_ws) + kAttnTicketBytes;
    }
    LLM_HIP(m->act[0].alloc(attn_ws + 64), "hipMalloc(attention scratch)");
    LLM_HIP(hipMemset(m->act[0].p, 0, kAttnTicketBytes), "hipMemset(attention tickets)");
    {
        int ns = 1, cm = 1;
        attention_decode_plan(c.batch, c.heads, c.kv_heads, c.context, &ns, &cm);
        const size_t fb = attention_decode_flagged_bytes(c.batch, c.heads, c.head_dim, ns);
        LLM_HIP(m->attn_flags.alloc(fb + 64), "hipMalloc(attention hand-over)");
        LLM_HIP(hipMemset(m->attn_flags.p, 0, fb + 64), "hipMemset(attention hand-over)");
    }
    if (!m->stream) LLM_HIP(hipStreamCreate(&m->stream), "hipStreamCreate");
    if (m->step_graph) {
        (void)hipGraphExecDestroy(m->step_graph);
        m->step_graph = nullptr;
    }
    LLM_HIP(m->state.alloc(256), "hipMalloc");
    if (c.batch <= (int)(kArgmaxTicketBytes / 4)) {
        LLM_HIP(m->argmax_ws.alloc(argmax_workspace_bytes(c.batch)), "hipMalloc");
        LLM_HIP(hipMemset(m->argmax_ws.p, 0, kArgmaxTicketBytes), "hipMemset");
    }
    LLM_HIP(m->record.alloc(((size_t)c.context + 1) * c.batch * 4), "hipMalloc");  // a graph keeps its address
    LLM_HIP(m->qkv.alloc((size_t)c.batch * (qd + 2 * kvd) * 4), "hipMalloc");
    m->fast = rmsnorm_q4act_ok(c.embed) && c.head_dim % 2 == 0;
    bool biased = false;  // q, k, v with biases: the generic step, whose rotation launch adds them first
    for (int i = 0; i < c.layers; i++) biased = biased || m->blocks[i].biased();
    if (biased) m->fast = false;
    for (int i = 0; i < c.layers && m->fast; i++) {
        Block& b = m->blocks[i];
        for (const Weight* w : {&b.q, &b.k, &b.v, &b.o, &b.gate, &b.up, &b.down})
            if (act_class(*w) != kActQ4) m->fast = false;
    }
    for (int i = 0; i < c.layers; i++) {
        Block& b = m->blocks[i];
        b.qkv.buf.release();
        b.gate_up.buf.release();
        if (m->fast) continue;
        auto fuse = [&](std::initializer_list<const Weight*> parts, Weight& into) -> mi355x_status {
            const Weight* first = *parts.begin();
            size_t total = 0;
            int64_t n = 0;
            for (const Weight* p : parts) {
                // a part that is not a multiple of 16 bytes long would leave the next one misaligned for the kernels' wide loads
                if (!is_quantized(p->dtype) || p->dtype != first->dtype || p->k != first->k || p->buf.bytes % 16) return MI355X_OK;
                total += p->buf.bytes;
                n += p->n;
            }
            LLM_HIP(into.buf.alloc(total), "hipMalloc(fused weights)");
            size_t off = 0;
            for (const Weight* p : parts) {
                LLM_HIP(hipMemcpy((uint8_t*)into.buf.p + off, p->buf.p, p->buf.bytes, hipMemcpyDeviceToDevice), "hipMemcpy(fused weights)");
                off += p->buf.bytes;
            }
            into.dtype = first->dtype; into.n = n; into.k = first->k;
            return MI355X_OK;
        };
        if (mi355x_status st = fuse({&b.q, &b.k, &b.v}, b.qkv)) return st;
        if (b.biased()) {  // the three biases in one row, as the three matrices are where they share a block dtype
            LLM_HIP(b.qkv_bias.alloc((size_t)(qd + 2 * kvd) * 4), "hipMalloc(fused biases)");
            size_t off = 0;
            for (const Weight* p : {&b.q_bias, &b.k_bias, &b.v_bias}) {
                LLM_HIP(hipMemcpy((uint8_t*)b.qkv_bias.p + off, p->buf.p, p->buf.bytes, hipMemcpyDeviceToDevice), "hipMemcpy(fused biases)");
                off += p->buf.bytes;
            }
        }
        if (mi355x_status st = fuse({&b.gate, &b.up}, b.gate_up)) return st;
    }
    LLM_HIP(m->gu.alloc((size_t)c.batch * 2 * c.hidden * 4), "hipMalloc");
    // several sequences: every product of a step on the kernels that read W once for up to eight rows of x
    m->rows = m->fast && c.batch >= 2 && c.batch <= 64 && qd % 32 == 0 && kvd % 32 == 0 && c.hidden % 32 == 0 && c.embed <= 8192;
    if (m->rows) {
        AttnArgs at;  // the shape of a step's attention, as step_rows sets it up
        at.q = m->qkv.as<float>(); at.k = m->keys[0].p; at.v = m->values[0].p; at.kv_dtype = c.cache_dtype;
        at.q_strides[0] = qd + 2 * kvd; at.q_strides[1] = c.head_dim; at.q_strides[2] = 0;
        at.k_strides[0] = at.v_strides[0] = (int64_t)c.kv_heads * c.context * c.head_dim;
        at.k_strides[1] = at.v_strides[1] = (int64_t)c.context * c.head_dim;
        at.k_strides[2] = at.v_strides[2] = c.head_dim;
        at.B = c.batch; at.Q = 1; at.K = 1; at.H = c.heads; at.HK = c.kv_heads; at.D = c.head_dim;
        m->rows = attention_decode_ok(at, c.context);
    }
    for (int i = 0; i < c.layers && m->rows; i++) {
        Block& b = m->blocks[i];
        for (const Weight* w : {&b.q, &b.k, &b.v, &b.gate, &b.up})
            if (!qgemv_q4_0_rows_shares_ok(w->buf.p, c.batch, w->n, w->k, 1)) m->rows = false;
        for (const Weight* w : {&b.o, &b.down})
            if (!qgemv_q4_0_rows_shares_ok(w->buf.p, c.batch, w->n, w->k, 2)) m->rows = false;
    }
    if (m->rows) {
        const size_t ab = q4_0_rows_act_bytes(kmax) * (size_t)((c.batch + 7) / 8);  // a buffer per group of eight sequences
        LLM_HIP(m->rows_act.alloc(ab), "hipMalloc(activations)");
        LLM_HIP(hipMemset(m->rows_act.p, 0, ab), "hipMemset(activations)");  // rows past the batch stay zero
        LLM_HIP(m->rows_act2.alloc(ab), "hipMalloc(activations)");
        LLM_HIP(hipMemset(m->rows_act2.p, 0, ab), "hipMemset(activations)");
        LLM_HIP(m->parts.alloc((size_t)2 * c.batch * c.embed * 4), "hipMalloc");
    }
    m->ready = true;
    return MI355X_OK;
}

mi355x_status mi355x_llama_reset(void* model) {
    Model* m = (Model*)model;
    if (!m) return mimir::capi_fail(MI355X_ERR_INTERNAL, "mi355x: llama_reset: null pointer");
    m->cache_len = 0;  // KVCache.Reset (nn/transformer.go:377)
    return MI355X_OK;
}

// Loads positions [0, n) of one block's caches from the host (keys and values
// [batch, kv_heads, n, head_dim] in the cache's dtype) and makes n the length
// of every cache: KVCache contents as a prompt would have left them
// (nn/transformer.go:348-423), for callers that keep caches of their own.
mi355x_status mi355x_llama_set_cache(void* model, int32_t layer, const void* keys, const void* values, int64_t n) {
    using namespace mimir;
    Model* m = (Model*)model;
    if (!m || !keys || !values) return capi_fail(MI355X_ERR_INTERNAL, "mi355x: llama_set_cache: null pointer");
    const auto& c = m->c;
    if (!m->ready) return capi_fail(MI355X_ERR_INTERNAL, "mi355x: llama: model is not finalized");
    if (layer < 0 || layer >= c.layers || n < 0 || n > c.context)
        return capi_fail(MI355X_ERR_SHAPE, "mi355x: llama: %lld positions of block %d into caches of %d blocks and %d positions", (long long)n, layer,
                         c.layers, c.context);
    const size_t esz = c.cache_dtype == kF32 ? 4 : 2;
    const size_t row = (size_t)n * c.head_dim * esz, pitch = (size_t)c.context * c.head_dim * esz;
    if (n > 0) {
        LLM_HIP(hipMemcpy2D(m->keys[layer].p, pitch, keys, row, row, (size_t)c.batch * c.kv_heads, hipMemcpyHostToDevice), "hipMemcpy2D(keys)");
        LLM_HIP(hipMemcpy2D(m->values[layer].p, pitch, values, row, row, (size_t)c.batch * c.kv_heads, hipMemcpyHostToDevice), "hipMemcpy2D(values)");
    }
    m->cache_len = n;
    return MI355X_OK;
}

int64_t mi355x_llama_cache_len(void* model) { return model ? ((Model*)model)->cache_len : -1; }

static mi355x_status check_tokens(Model* m, const int32_t* tokens, int64_t n) {
    using namespace mimir;
    const auto& c = m->c;
    if (!m->ready) return capi_fail(MI355X_ERR_INTERNAL, "mi355x: llama: model is not finalized");
    // llm/model.go:393-400
    if (n <= 0 || (int64_t)c.batch * n > m->max_rows) return capi_fail(MI355X_ERR_SHAPE, "mi355x: llama: %lld tokens a sequence, at most %lld a call", (long long)n, (long long)(m->max_rows / c.batch));
    if (m->cache_len + n > c.context)
        return capi_fail(MI355X_ERR_SHAPE, "mi355x: llama: append %lld positions to a cache holding %lld of %d", (long long)n, (long long)m->cache_len, c.context);
    for (int64_t i = 0; i < (int64_t)c.batch * n; i++)
        if (tokens[i] < 0 || tokens[i] >= c.vocab) return capi_fail(MI355X_ERR_INDEX, "mi355x: llama: token %d of a vocabulary of %d", tokens[i], c.vocab);
    return MI355X_OK;
}

// Model.Logits (llm/model.go:391-437): runs tokens [batch, n], which follow the
// positions the caches hold, and copies to the host the logits of the last
// token, [batch, vocab], or of every token, [batch, n, vocab], if all is set.
mi355x_status mi355x_llama_logits(void* model, const int32_t* tokens, int64_t n, int all, float* logits_host) {
    using namespace mimir;
    Model* m = (Model*)model;
    if (!m || !tokens || !logits_host) return capi_fail(MI355X_ERR_INTERNAL, "mi355x: llama_logits: null pointer");
    if (mi355x_status st = check_tokens(m, tokens, n)) return st;
    const auto& c = m->c;
    const int64_t rows = (int64_t)c.batch * n;
    LLM_HIP(hipMemcpyAsync(m->tokens_dev.p, tokens, rows * 4, hipMemcpyHostToDevice, m->stream), "upload tokens");
    if (mi355x_status st = forward(*m, n)) return st;
    int64_t out_rows = all ? rows : c.batch;
    if (mi355x_status st = all ? head(*m, m->x.as<float>(), rows, c.embed) : head(*m, m->x.as<float>() + (n - 1) * c.embed, c.batch, n * c.embed)) return st;
    LLM_HIP(hipMemcpyAsync(logits_host, m->logits.p, (size_t)out_rows * c.vocab * 4, hipMemcpyDeviceToHost, m->stream), "download logits");
    return mi355x_sync(m->stream);
}

// Greedy generation (examples/llama/generate.go:162-202 with Sample at :44-53):
// the prompt [batch, n_prompt], then n_new steps. Each step's token is chosen on
// the device and read by the next step's embedding lookup from device memory;
// out_tokens [batch, n_new] comes back once at the end. seconds, if not NULL,
// gets the wall time of the prompt pass and of the n_new - 1 decoding steps.
mi355x_status mi355x_llama_generate(void* model, const int32_t* prompt, int64_t n_prompt, int64_t n_new, int32_t* out_tokens, double* seconds) {
    using namespace mimir;
    Model* m = (Model*)model;
    if (!m || !prompt || !out_tokens || n_new <= 0) return capi_fail(MI355X_ERR_INTERNAL, "mi355x: llama_generate: bad arguments");
    if (mi355x_status st = check_tokens(m, prompt, n_prompt)) return st;
    const auto& c = m->c;
    if (m->cache_len + n_prompt + n_new - 1 > c.context)
        return capi_fail(MI355X_ERR_SHAPE, "mi355x: llama: %lld positions for a context of %d", (long long)(m->cache_len + n_prompt + n_new - 1), c.context);
    const int64_t B = c.batch;
    const bool use_graph = g_llama_step_mode == 0, use_fast = g_llama_step_mode != 2;  // 2: forward() with the position from the host
    DevBuf picked;  // [n_new, batch]
    LLM_HIP(picked.alloc((size_t)n_new * B * 4), "hipMalloc(tokens)");
    hipEvent_t e0, e1, e2;
    LLM_HIP(hipEventCreate(&e0), "hipEventCreate"); LLM_HIP(hipEventCreate(&e1), "hipEventCreate"); LLM_HIP(hipEventCreate(&e2), "hipEventCreate");
    LLM_HIP(hipMemcpyAsync(m->tokens_dev.p, prompt, B * n_prompt * 4, hipMemcpyHostToDevice, m->stream), "upload tokens");
    LLM_HIP(hipEventRecord(e0, m->stream), "hipEventRecord");
    mi355x_status st = forward(*m, n_prompt);
    if (!st) st = head(*m, m->x.as<float>() + (n_prompt - 1) * c.embed, B, n_prompt * c.embed);
    if (!st) {
        hipError_t e = argmax(m->logits.as<float>(), B, c.vocab, picked.as<int32_t>(), m->argmax_ws.p, m->stream);
        if (e != hipSuccess) st = capi_fail((mi355x_status)e, "mi355x: llama: argmax: %s", hipGetErrorName(e));
    }
    if (!st) (void)hipEventRecord(e1, m->stream);
    if (!st && use_fast) {
        // record[0] is the prompt's choice; each step then reads next_tok and the
        // position from the device, and leaves its own choice in both places
        hipError_t e = hipSuccess;  // n_new <= context: the record holds it
        if (!st) e = hipMemcpyAsync(m->next_tok.p, picked.p, B * 4, hipMemcpyDeviceToDevice, m->stream);
        if (!st && e == hipSuccess) e = set_state(m->state.as<int32_t>(), (int)m->cache_len, 0, m->stream);
        if (!st && e == hipSuccess) e = advance(m->state.as<int32_t>(), m->next_tok.as<int32_t>(), m->record.as<int32_t>(), (int)B, 0, m->stream);
        if (!st && e != hipSuccess) st = capi_fail((mi355x_status)e, "mi355x: llama: step state: %s", hipGetErrorName(e));
        auto one_step = [&]() -> mi355x_status {
            if (mi355x_status s2 = m->rows && !g_llama_rows_off ? step_rows(*m) : m->fast ? step_fast(*m) : step_any(*m)) return s2;
            if (mi355x_status s2 = head(*m, m->x.as<float>(), B, c.embed)) return s2;
            LLM_HIP(argmax(m->logits.as<float>(), B, c.vocab, m->next_tok.as<int32_t>(), m->argmax_ws.p, m->stream), "argmax");
            LLM_HIP(advance(m->state.as<int32_t>(), m->next_tok.as<int32_t>(), m->record.as<int32_t>(), (int)B, 1, m->stream), "advance");
            return MI355X_OK;
        };
        const int rows_now = m->rows && !g_llama_rows_off ? 1 + g_llama_rows_plain : 0;
        if (m->step_graph && m->graph_rows != rows_now) {  // the measurement aid changed which step runs
            (void)hipGraphExecDestroy(m->step_graph);
            m->step_graph = nullptr;
        }
        if (!st && n_new > 1 && !m->step_graph && use_graph) {
            m->graph_rows = rows_now;
            hipGraph_t g = nullptr;
            e = hipStreamBeginCapture(m->stream, hipStreamCaptureModeThreadLocal);
            if (e != hipSuccess) st = capi_fail((mi355x_status)e, "mi355x: llama: begin capture: %s", hipGetErrorName(e));
            if (!st) {
                mi355x_status cst = one_step();
                e = hipStreamEndCapture(m->stream, &g);
                if (cst) st = cst;
                else if (e != hipSuccess) st = capi_fail((mi355x_status)e, "mi355x: llama: end capture: %s", hipGetErrorName(e));
            }
            if (!st) {
                e = hipGraphInstantiate(&m->step_graph, g, nullptr, nullptr, 0);
                if (e != hipSuccess) st = capi_fail((mi355x_status)e, "mi355x: llama: instantiate graph: %s", hipGetErrorName(e));
            }
            if (g) (void)hipGraphDestroy(g);
        }
        for (int64_t t = 1; t < n_new && !st; t++) {
            if (m->step_graph && use_graph) {
                e = hipGraphLaunch(m->step_graph, m->stream);
                if (e != hipSuccess) st = capi_fail((mi355x_status)e, "mi355x: llama: graph launch: %s", hipGetErrorName(e));
            } else {
                st = one_step();
            }
            if (!st) m->cache_len += 1;
        }
        if (!st) {
            e = hipMemcpyAsync(picked.p, m->record.p, (size_t)n_new * B * 4, hipMemcpyDeviceToDevice, m->stream);
            if (e != hipSuccess) st = capi_fail((mi355x_status)e, "mi355x: llama: copy record: %s", hipGetErrorName(e));
        }
    } else
    for (int64_t t = 1; t < n_new && !st; t++) {
        // the step reads its tokens where the last step's argmax wrote them
        hipError_t e = hipMemcpyAsync(m->tokens_dev.p, picked.as<int32_t>() + (t - 1) * B, B * 4, hipMemcpyDeviceToDevice, m->stream);
        if (e != hipSuccess) { st = capi_fail((mi355x_status)e, "mi355x: llama: token copy: %s", hipGetErrorName(e)); break; }
        st = forward(*m, 1);
        if (!st) st = head(*m, m->x.as<float>(), B, c.embed);
        if (!st) {
            e = argmax(m->logits.as<float>(), B, c.vocab, picked.as<int32_t>() + t * B, m->argmax_ws.p, m->stream);
            if (e != hipSuccess) st = capi_fail((mi355x_status)e, "mi355x: llama: argmax: %s", hipGetErrorName(e));
        }
    }
    if (!st) (void)hipEventRecord(e2, m->stream);
    std::vector<int32_t> host((size_t)n_new * B);
    if (!st) {
        hipError_t e = hipMemcpyAsync(host.data(), picked.p, host.size() * 4, hipMemcpyDeviceToHost, m->stream);
        if (e != hipSuccess) st = capi_fail((mi355x_status)e, "mi355x: llama: download tokens: %s", hipGetErrorName(e));
    }
    if (!st) st = mi355x_sync(m->stream);
    if (!st) {
        for (int64_t t = 0; t < n_new; t++)
            for (int64_t b = 0; b < B; b++) out_tokens[b * n_new + t] = host[t * B + b];
        if (seconds) {
            float ms01 = 0, ms12 = 0;
            (void)hipEventElapsedTime(&ms01, e0, e1);
            (void)hipEventElapsedTime(&ms12, e1, e2);
            seconds[0] = ms01 * 1e-3;
            seconds[1] = ms12 * 1e-3;
        }
    }
    (void)hipEventDestroy(e0); (void)hipEventDestroy(e1); (void)hipEventDestroy(e2);
    return st;
}

}  // extern "C"
