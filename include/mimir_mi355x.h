/*
 * C ABI of libmimir_mi355x.so: the MI355X (gfx950) implementation of mimir's
 * quantized-matmul decode path. A host binds these symbols with dlopen/dlsym
 * (purego's Dlopen + RegisterFunc in Go, ctypes in Python); the signatures use
 * plain pointers and integers only.
 *
 * Conventions
 *  - Every function returns a status word: 0 on success, a hipError_t value
 *    (1..1999) when the HIP runtime failed, or one of the MI355X_ERR_* codes,
 *    which map one to one onto the reference's sentinel errors
 *    (backend/backend.go:31-54). mi355x_last_error gives the message of the
 *    calling thread's last failure.
 *  - Device pointers come from mi355x_alloc or from any other HIP allocation
 *    of the same process (hipMalloc, a torch tensor's data_ptr).
 *  - `stream` is a hipStream_t passed as a pointer; NULL is the device's
 *    default stream. Launches return once queued, like Backend.Run
 *    (backend/backend.go:152-168); mi355x_sync waits and reports device-side
 *    errors, like Backend.Sync (backend/rocm/rocm_linux.go:349-375).
 *  - Entry points that need memory beyond their arguments (mi355x_qgemv,
 *    mi355x_qgemm_bf16, mi355x_attention, mi355x_argmax) keep it per device and
 *    stream: calls on different streams share nothing, calls on one stream are
 *    ordered by it. Such a block grows on demand with hipMalloc, which HIP
 *    refuses while the stream is being captured: run a call once at its
 *    largest size before recording it into a graph (the block a graph was
 *    recorded with is never freed, so the graph stays valid however the
 *    scratch grows afterwards), or use mi355x_qgemv_noalloc.
 *  - dtype codes are the reference's DType enumeration
 *    (backend/backend.go:72-90) with Q4_0 appended.
 *  - Block-quantized buffers hold ggml's block layout unchanged
 *    (backend/backend.go:66-71); kernels read it in place.
 */
#ifndef MIMIR_MI355X_H
#define MIMIR_MI355X_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Exported from the shared library, whose other symbols are hidden. */
#define MI355X_API __attribute__((visibility("default")))

typedef uint32_t mi355x_status;

enum {
    MI355X_OK = 0,
    MI355X_ERR_OUT_OF_MEMORY = 2,     /* hipErrorOutOfMemory -> backend.ErrOutOfMemory (rocm_linux.go:194-203) */
    MI355X_ERR_SHAPE = 0x1001,        /* backend.ErrShape */
    MI355X_ERR_DTYPE = 0x1002,        /* backend.ErrDType */
    MI355X_ERR_INDEX = 0x1003,        /* backend.ErrIndex */
    MI355X_ERR_INTERNAL = 0x1005      /* backend.ErrInternal */
};

enum {
    MI355X_F32 = 1, MI355X_I32 = 2, MI355X_BF16 = 3, MI355X_F16 = 4,
    MI355X_Q8_0 = 5, MI355X_Q4_K = 6, MI355X_Q6_K = 7, MI355X_Q4_0 = 8
};

/* ---- device, memory, ordering: Backend.Alloc/Free/Upload/Download/Sync ----
 * (backend/backend.go:141-171; backend/rocm/rocm_linux.go:88,220-375) */

/* Selects the device, creates the library's state on it (once per device) and
 * checks that it is a gfx950. */
MI355X_API mi355x_status mi355x_init(int device);
/* Copies the calling thread's last error message into buf (NUL-terminated,
 * truncated to n); returns its length. */
MI355X_API size_t mi355x_last_error(char* buf, size_t n);
/* Elements per block and bytes per block of a dtype (backend/quant.go:24-48);
 * 0 bytes for an unknown dtype. */
MI355X_API int mi355x_block_size(int dtype);
MI355X_API int mi355x_block_bytes(int dtype);
/* Bytes of n elements of dtype, or -1 when n is not whole blocks
 * (backend/quant.go:53-59). */
MI355X_API int64_t mi355x_bytes(int dtype, int64_t n);

MI355X_API mi355x_status mi355x_alloc(void** out, size_t bytes);
MI355X_API mi355x_status mi355x_free(void* ptr);
MI355X_API mi355x_status mi355x_upload(void* dst, const void* src, size_t bytes, void* stream);
MI355X_API mi355x_status mi355x_download(void* dst, const void* src, size_t bytes, void* stream);
/* Waits for the stream, then reports and clears the device error word:
 * MI355X_ERR_INDEX if a gather read an index out of range. */
MI355X_API mi355x_status mi355x_sync(void* stream);
/* Frees the scratch memory the library keeps for `stream` on the current device: converted activations,
 * attention's and argmax's partial results and tickets, qgemm_bf16's float32 copies, and the blocks kept aside
 * when one of them grew. Waits for the stream first. For hosts that create and destroy streams (the library
 * otherwise keeps a stream's scratch, some 5 MiB and up, for the life of the process). After it, no HIP graph
 * recorded over this library's calls on that stream may be replayed: such a graph points into these blocks.
 * No counterpart in the reference, whose backend owns one stream for its whole life
 * (backend/rocm/rocm_linux.go:34-40). */
MI355X_API mi355x_status mi355x_stream_release(void* stream);

/* ---- the hot path: OpQMatMul ------------------------------------------------
 * y[m, :] = x[m, :] . W^T for m < M. W is [N, K] of a block-quantized dtype,
 * contiguous from a block boundary (any 2-byte aligned address); x rows are
 * x_row_stride floats apart; y is [M, N] float32, contiguous.
 * Replaces the generated kernel of backend/internal/gen/quant.go:163-209 and
 * computes what the CPU backend's runQMatMul computes
 * (backend/cpu/qmatmul.go:310-405): for Q8_0, Q4_K and Q6_K each block of a
 * row of x is rounded to int8 first and the dot products are integer; for
 * Q4_0 it is the float32 product with the dequantized weights, the route the
 * reference takes for that file dtype (io/mim/dtype.go:118-123).
 * One entry point for every M, as OpQMatMul is one operation: by dtype and
 * shape the library runs row kernels (few rows of x; one launch for one row of
 * x by Q4_0 or by a small Q8_0, Q4_K or Q6_K matrix; Q8_0 weights are read
 * once for up to eight rows) or kernels on the int8 matrix cores (Q4_0 from two
 * rows on: up to some tens of rows a kernel that reads W once per eight rows,
 * beyond them a tiled one, and from some hundreds of rows by a large matrix the
 * same integers through the binary16 matrix cores, with the tiled one's bits,
 * which takes a workspace of 2 N K bytes in the stream's scratch; two to eight
 * rows by a large Q8_0
 * matrix; Q4_K, Q6_K from enough rows on); which one ran changes the results
 * only by the order of float32 additions (Q4_0, Q8_0), or not at all (Q8_0
 * among its row kernels, Q4_K, Q6_K). */
MI355X_API mi355x_status mi355x_qgemv(int dtype, const void* W, const float* x, float* y, int64_t M, int64_t N, int64_t K,
                           int64_t x_row_stride, void* stream);

/* mi355x_qgemv for callers that cannot allocate device memory: code under HIP
 * graph capture, serving loops and harnesses that forbid hipMalloc. It has no
 * counterpart in the reference. Same arguments, kernels and results as
 * mi355x_qgemv, but the converted activations go to a fixed block of 1 MiB inside
 * the library's code object instead of a scratch buffer that grows, and nothing
 * is allocated or freed: mi355x_init must have run on the device, and a product
 * whose converted activations exceed the block (M * mi355x_act_bytes(dtype, K),
 * for Q4_0 rounded up to groups of eight rows where W is read once per eight)
 * fails with MI355X_ERR_SHAPE. Every call on a device uses that device's one
 * block: calls that overlap on one device (two streams) race on it. */
MI355X_API mi355x_status mi355x_qgemv_noalloc(int dtype, const void* W, const float* x, float* y, int64_t M, int64_t N, int64_t K,
                                   int64_t x_row_stride, void* stream);

/* The product in two steps, for callers that multiply one x by several
 * matrices (q, k and v; gate and up). mi355x_convert_act turns each row of x
 * into the form the kernels of `dtype` read, mi355x_act_bytes(dtype, K) bytes
 * per row at a 16-byte aligned `act` (0 when that dtype and K have no such
 * form); mi355x_qgemv_act multiplies by W. mi355x_qgemv does both through a
 * scratch buffer of its own.
 *   Q8_0: quantizeRow's int8 blocks (backend/cpu/qmatmul.go:208-254).
 *   Q4_K, Q6_K: quantizeRow's int8 super-blocks of 256 with their sums.
 *   Q4_0: 24-bit fixed point per block of 32 (K a multiple of 64, W dword
 *         aligned); no counterpart in the reference, whose kernels take
 *         float32 activations only. Block floating point, not float32: an
 *         element is held to 2^-23 of its block's largest magnitude amax_b, so
 *         y[m, n] is within 2^-23 * sum_b amax_b * sum|w_b| of the float32
 *         product (b over the blocks of row n), beside the float32 sums' own
 *         2e-6 * sum|x||w|. For activations of even magnitude that is 1e-6 of
 *         the result; next to an element 1e6 times the rest of its block the
 *         small ones keep three of their bits. mi355x_tune("q4_0.path", 1)
 *         keeps every Q4_0 product on the float32 kernel instead. */
MI355X_API size_t mi355x_act_bytes(int dtype, int64_t K);
MI355X_API mi355x_status mi355x_convert_act(int dtype, const float* x, int64_t M, int64_t K, int64_t x_row_stride, void* act, void* stream);
MI355X_API mi355x_status mi355x_qgemv_act(int dtype, const void* W, const void* act, float* y, int64_t M, int64_t N, int64_t K, void* stream);

/* The same product for prompt-sized M with bfloat16 activations, as
 * Tensor.MatMulT computes it for a half-precision x and a block-quantized w
 * (tensor/quant.go:45-48: x cast to float32, the product accumulated in float32,
 * one rounding to x's dtype): X [M, K] bfloat16 with rows x_row_stride elements
 * apart, W [N, K] of any block dtype, Y [M, N] contiguous of out_dtype
 * MI355X_BF16 (the reference's result) or MI355X_F32 (the same sums before the
 * rounding). Q4_0 runs on the bfloat16 matrix cores without rounding any
 * operand (each weight as two bfloat16 halves; or, for large products, the
 * weights' integers against x block by block and one float32 FMA per block with
 * the block's scale, which takes a workspace of 2 N K bytes in the stream's
 * scratch), when K is a multiple of 256, X and W are 16-byte aligned
 * and rows of X are a multiple of 8 elements apart; otherwise, and for the other
 * dtypes, X goes through mi355x_qgemv as float32. Q4_K and Q6_K then run on
 * the int8 matrix cores from a few rows of X on, with the CPU's results bit for
 * bit (backend/cpu/qtile.go:51-54 claims the same of the reference's tiles). */
MI355X_API mi355x_status mi355x_qgemm_bf16(int dtype, const void* W, const void* X, void* Y, int64_t M, int64_t N, int64_t K,
                                           int64_t x_row_stride, int out_dtype, void* stream);

/* The fused products of a decoding step, over converted activations (Q4_0
 * weights that qualify for mi355x_qgemv_act). The reference fuses the same
 * products on its CPU path by concatenating the weights (fusedFor,
 * llm/decode.go:240-266); here the matrices stay where they are.
 *   _add     y = resid + x . W^T                     (attn_output, ffn_down + residual)
 *   _multi   y = x . [W0; W1; W2]^T, rows n0+n1+n2   (attn_q, attn_k, attn_v)
 *   _swiglu  y = SiLU(x . gate^T) * (x . up^T)        (Block.mlp, llm/model.go:446-448) */
MI355X_API mi355x_status mi355x_qgemv_act_add(int dtype, const void* W, const void* act, const float* resid, float* y, int64_t M, int64_t N, int64_t K, void* stream);
MI355X_API mi355x_status mi355x_qgemv_act_multi(int dtype, const void* W0, const void* W1, const void* W2, int64_t n0, int64_t n1, int64_t n2,
                                     const void* act, float* y, int64_t M, int64_t K, void* stream);
MI355X_API mi355x_status mi355x_qgemv_act_swiglu(int dtype, const void* gate, const void* up, const void* act, float* y, int64_t M, int64_t N, int64_t K, void* stream);

/* ---- OpCast / OpGather of a block-quantized input ---------------------------
 * (backend/cpu/quant.go:198-327; replaced kernels gen/quant.go:140-150 and
 * gen/gen.go:751-756). Bit-exact with the CPU backend. */
/* out[i] = element first + i of the blocks at W, i < n, rounded to out_dtype
 * (F32, BF16 or F16). */
MI355X_API mi355x_status mi355x_dequant(int dtype, const void* W, int64_t first, int64_t n, void* out, int out_dtype, void* stream);
/* out[r, :] = row idx[r] of the [rows, K] table, dequantized; an index outside
 * [0, rows) writes zeros and makes the next mi355x_sync fail with
 * MI355X_ERR_INDEX. */
MI355X_API mi355x_status mi355x_gather_rows(int dtype, const void* table, int64_t rows, int64_t K, const int32_t* idx, int64_t n,
                                 float* out, void* stream);

/* ---- the other kernels of a decoding step -----------------------------------
 * On the reference these are runs of generated elementwise and reduction
 * kernels plus OpAttention; each is one launch here, so a whole step is queued
 * without a host round trip. */

/* RMSNorm.Forward (nn/transformer.go:50-61; llm/decode.go:376-385):
 * y[r, :] = (x[r, :] * recip(sqrt(mean(x[r, :]^2) + eps))) * w; w may be NULL. */
MI355X_API mi355x_status mi355x_rmsnorm(const float* x, const float* w, float* y, int64_t rows, int64_t d, double eps, void* stream);
/* RotaryEmbedding.Apply (nn/transformer.go:225-257). x is [rows, S, head_dim]
 * read with strides in floats; position s of every row turns by row
 * offset + s of cos_table and sin_table, [table_len, rope_dim/2] float32, which
 * the host computes in float64 as the reference does (transformer.go:146-164).
 * interleaved pairs features (2i, 2i+1), else (i, i + rope_dim/2). y may be x. */
MI355X_API mi355x_status mi355x_rope(const float* x, float* y, int64_t rows, int64_t S, int head_dim, int rope_dim, int interleaved,
                          int64_t x_row_stride, int64_t x_pos_stride, int64_t y_row_stride, int64_t y_pos_stride,
                          const float* cos_table, const float* sin_table, int64_t table_len, int64_t offset, void* stream);
/* KVCache.Append's write (nn/transformer.go:397-423): src [B, heads, S, dim],
 * read with strides, lands at positions [pos, pos + S) of cache
 * [B, heads, capacity, dim], cast to cache_dtype (F32 or F16). */
MI355X_API mi355x_status mi355x_kv_write(const float* src, void* cache, int cache_dtype, int64_t B, int heads, int64_t S, int dim,
                              int64_t capacity, int64_t pos, int64_t src_b_stride, int64_t src_h_stride, int64_t src_p_stride,
                              void* stream);
/* OpAttention (backend/op.go:117-129; backend/attention.go:25-143):
 * softmax(scale * q . k^T + mask) . v. Queries [B, H, Q, D], keys [B, HK, K, D]
 * and values [B, HK, K, DV] of kv_dtype (F32 or F16), out [B, H, Q, DV], each
 * read through its strides {batch, head, position} in elements with contiguous
 * features; lse, if not NULL, [B, H, Q] contiguous: the logsumexp of each row's
 * scores. mask, if not NULL, is float32 [B, H, Q, K] read through mask_strides
 * {batch, head, query, key} (0 broadcasts a dimension) and added to the scores;
 * key j is also hidden from query i when causal and j > i + causal_offset. A
 * row that sees no key gets zeros and -Inf; with K == 0 that is every row, and
 * k, v and their strides may be NULL. D and DV at most 256. A NaN or an
 * infinity in the values of a key reaches the rows that see the key and no
 * other, as in the reference, which reads a row's visible keys only. */
MI355X_API mi355x_status mi355x_attention(const float* q, const int64_t* q_strides, const void* k, const int64_t* k_strides, const void* v,
                               const int64_t* v_strides, int kv_dtype, const float* mask, const int64_t* mask_strides, float* out,
                               const int64_t* out_strides, float* lse, int64_t B, int H, int HK, int64_t Q, int64_t K, int D, int DV, double scale,
                               int causal, int64_t causal_offset, void* stream);
/* mi355x_attention with its arguments in one structure, for hosts whose foreign-function layer limits the number of
 * parameters of a call (purego's RegisterFunc in Go): the same operation, checks and results. Strides as above;
 * mask_strides is read only when mask is not NULL. */
typedef struct mi355x_attention_desc {
    const float* q;
    const void* k;
    const void* v;
    const float* mask;
    float* out;
    float* lse;
    int64_t q_strides[3], k_strides[3], v_strides[3], out_strides[3], mask_strides[4];
    int64_t B, Q, K, causal_offset;
    double scale;
    int32_t kv_dtype, H, HK, D, DV, causal;
} mi355x_attention_desc;
MI355X_API mi355x_status mi355x_attention_d(const mi355x_attention_desc* desc, void* stream);
/* Block.mlp's activation (llm/model.go:446-448): out = SiLU(gate) * up, rows of
 * gate and up in_row_stride floats apart, out contiguous. */
MI355X_API mi355x_status mi355x_swiglu(const float* gate, const float* up, float* out, int64_t rows, int64_t n, int64_t in_row_stride, void* stream);
MI355X_API mi355x_status mi355x_add(const float* a, const float* b, float* out, int64_t n, void* stream);
/* Sampler.Sample at temperature 0 (examples/llama/generate.go:44-53): the first
 * index of each row's largest value, into device memory. */
MI355X_API mi355x_status mi355x_argmax(const float* logits, int64_t rows, int64_t n, int32_t* out, void* stream);

/* ---- the decoder: llm.Model, its caches and the greedy loop ------------------
 * (llm/model.go:216-455; nn/transformer.go:348-423;
 * examples/llama/generate.go:44-53,162-202). Weights keep their block dtypes on
 * the device, a step is queued without host synchronisation, and the next
 * token is chosen on the device. batch sequences are decoded in lockstep (the
 * reference's llm fixes batch 1). */
typedef struct mi355x_llama_config {
    int32_t embed, hidden, layers, heads, kv_heads, head_dim, rope_dim, vocab;
    int32_t context;      /* capacity of the KV caches, in positions */
    int32_t interleaved;  /* rotate pairs (2i, 2i+1): arch "llama"; else halves: "qwen2" (llm/model.go:321) */
    int32_t cache_dtype;  /* MI355X_F32 or MI355X_F16 */
    int32_t batch;
    double rope_base, rope_scale, eps;
} mi355x_llama_config;

MI355X_API mi355x_status mi355x_llama_create(const mi355x_llama_config* cfg, void** model);
MI355X_API mi355x_status mi355x_llama_destroy(void* model);
/* Uploads one tensor from host bytes in its file layout (ggml blocks for the
 * quantized dtypes). Names are llama.cpp's, as llm.Load reads them
 * (llm/model.go:268-310): token_embd.weight, output_norm.weight, output.weight
 * (absent: tied to the embeddings), blk.N.{attn_norm,attn_q,attn_k,attn_v,
 * attn_output,ffn_norm,ffn_gate,ffn_up,ffn_down}.weight, and the float32 biases
 * blk.N.{attn_q,attn_k,attn_v}.bias that qwen2 gives its queries, keys and
 * values (llm/model.go:251-258; Linear.Forward adds them behind the product,
 * before the rotation: nn/layers.go:49-55). A block carries all three or none
 * (mi355x_llama_finalize returns MI355X_ERR_SHAPE otherwise). A model with biases
 * decodes with one launch per operator: the fused decoding launches are built
 * for models without them. */
MI355X_API mi355x_status mi355x_llama_set_tensor(void* model, const char* name, int dtype, const void* host_data, int64_t n_elems);
/* rope_freqs.weight: divisors of each pair's frequency (llm/model.go:318-346). */
MI355X_API mi355x_status mi355x_llama_set_rope_factors(void* model, const float* factors, int32_t n);
/* Checks the tensors, builds the rotary table, allocates the caches (zeroed)
 * and the activations of calls of up to max_tokens tokens per sequence. */
MI355X_API mi355x_status mi355x_llama_finalize(void* model, int64_t max_tokens);
/* Empties the caches (KVCache.Reset). */
MI355X_API mi355x_status mi355x_llama_reset(void* model);
MI355X_API int64_t mi355x_llama_cache_len(void* model);
/* Loads positions [0, n) of block `layer`'s caches from host arrays [batch,
 * kv_heads, n, head_dim] of the cache's dtype and makes n the caches' length
 * (what KVCache.Append would have left, nn/transformer.go:397-423). */
MI355X_API mi355x_status mi355x_llama_set_cache(void* model, int32_t layer, const void* keys, const void* values, int64_t n);
/* Model.Logits: runs tokens [batch, n], which follow the positions the caches
 * hold, appends their keys and values, and copies to the host the logits of the
 * last token [batch, vocab], or of every token [batch, n, vocab] if all. */
MI355X_API mi355x_status mi355x_llama_logits(void* model, const int32_t* tokens, int64_t n, int all, float* logits_host);
/* Greedy generation: prompt [batch, n_prompt], then n_new tokens a sequence into
 * out_tokens [batch, n_new]. seconds, if not NULL, gets the device time of the
 * prompt pass (with the first token) and of the n_new - 1 decoding steps. */
MI355X_API mi355x_status mi355x_llama_generate(void* model, const int32_t* prompt, int64_t n_prompt, int64_t n_new, int32_t* out_tokens, double* seconds);

/* ---- the reference's operator interface for this path ---------------------------
 * backend.Backend and backend.Batcher (backend/backend.go:141-171,
 * backend/batch.go:46-52) over this library: buffers that belong to their
 * backend, kernels described by an operation, the output's dtype and shape, and
 * one view per input (backend.Kernel and backend.View, backend.go:174-180,
 * view.go:23-27), checked by CheckRun (check.go:29-74) before they run.
 * Operations: MI355X_OP_QMATMUL (In[0] float32 [..., K] through any view, In[1]
 * block-quantized [N, K] read contiguously from a block boundary),
 * MI355X_OP_CAST and MI355X_OP_GATHER of a block-quantized In[0] through any
 * view, MI355X_OP_ATTENTION (q, k, v and the optional additive mask In[3]
 * [B..., H, Q, K]; the output holds the result [B..., H, Q, DV] followed by the
 * logsumexp [B..., H, Q]). Anything else fails with
 * MI355X_ERR_INTERNAL. Errors: a foreign or freed buffer is MI355X_ERR_DTYPE, a
 * size that does not match MI355X_ERR_SHAPE, a gather index out of range
 * MI355X_ERR_INDEX at the next sync (rocm_linux.go:275-375).
 * mi355x_backend_last_error has the message. A batch that is run again with the
 * same kernels and buffers is recorded into a HIP graph on its second run and
 * replayed from its third (rocm/batch_linux.go:115-203). */
#define MI355X_MAX_RANK 8
#define MI355X_MAX_INPUTS 4
enum { MI355X_OP_CAST = 1, MI355X_OP_GATHER = 2, MI355X_OP_QMATMUL = 3, MI355X_OP_ATTENTION = 4 };
typedef struct mi355x_view {
    int32_t rank;
    int64_t shape[MI355X_MAX_RANK], strides[MI355X_MAX_RANK]; /* in elements */
    int64_t offset;
} mi355x_view;
typedef struct mi355x_kernel {
    int32_t op, dtype, rank;
    int64_t shape[MI355X_MAX_RANK];
    int32_t n_in;
    mi355x_view in[MI355X_MAX_INPUTS];
    int32_t axis;          /* Attrs.Axis */
    double scale;          /* Attrs.Scale */
    int32_t causal;        /* Attrs.Causal */
    int64_t causal_offset; /* Attrs.CausalOffset */
} mi355x_kernel;
MI355X_API size_t mi355x_backend_last_error(char* buf, size_t n);
MI355X_API mi355x_status mi355x_backend_open(int device, void** backend);
MI355X_API mi355x_status mi355x_backend_close(void* backend);
MI355X_API mi355x_status mi355x_backend_alloc(void* backend, int dtype, int64_t n, void** buffer);
MI355X_API mi355x_status mi355x_backend_free(void* backend, void* buffer);
MI355X_API mi355x_status mi355x_backend_upload(void* backend, void* dst, const void* src, size_t bytes);
MI355X_API mi355x_status mi355x_backend_download(void* backend, void* dst, size_t bytes, void* src);
MI355X_API mi355x_status mi355x_backend_sync(void* backend);
MI355X_API mi355x_status mi355x_backend_run(void* backend, const mi355x_kernel* k, void* const* outs, int n_outs, void* const* ins, int n_ins);
MI355X_API mi355x_status mi355x_batch_new(const mi355x_kernel* kernels, int n, void* const* const* outs, const int* n_outs,
                                          void* const* const* ins, const int* n_ins, void** batch);
MI355X_API mi355x_status mi355x_batch_free(void* batch);
MI355X_API mi355x_status mi355x_backend_run_batch(void* backend, void* batch);
MI355X_API int64_t mi355x_backend_graph_replays(void* backend);

/* ---- measurement aids (no counterpart in the reference) ---------------------
 * Overrides the launch plan of mi355x_qgemv for sweeps: key is one of
 * "q4_0.rows", "q4_0.cols", "q4_0.waves", "q4_0.no_lds", "q4_0.path" (1 forces
 * the float32 kernel, 2 the fixed-point one); 0 restores the built-in choice.
 * "q4_0.stream" = 1 keeps Q4_0 products of one to four rows of x off the kernel
 * that runs one workgroup per compute unit (the older, finer-grained launch shape
 * then takes them); 3 sends products of one row of x to that kernel's variant whose
 * weights reach LDS by loads that write it directly, requested by "q4_0.feeders"
 * (1 to 8) wavefronts of their own that keep "q4_0.feed_window" rows each under way
 * (same bits; slower on this device, kept to be measured). "q4_0.stream_waves" = n
 * fixes the wavefronts a workgroup of the whole-chip kernel where the shape allows.
 * "q4_0.batch_off" = 1 keeps products of several rows of x on the one-row
 * kernel, 2 puts them all on the kernel that shares W among rows of x.
 * "q4_0.rows_path" = 1 keeps Q4_0 and Q8_0 products of a few rows of x off the
 * kernels that read W once for eight rows, 2 selects the Q4_0 one's variant
 * without the pass through LDS; "q4_0.rows_waves" = 4 or 8 fixes its wavefronts
 * a workgroup; "q4_0.rows_max" = n sends Q4_0 products of fewer than n rows to
 * it (0: up to where the tiled kernel's cost model undercuts its own).
 * "q8_0.mfma" = 1 sends every Q8_0 product of two to eight rows of x that the
 * matrix-core kernel takes to it, 2 none (0: matrices of 64 M weights or more).
 * "attention.splits" = n fixes the shares of the keys in decode attention; "attention.share" = 128 makes it aim at
 * shares of 128 keys whatever their number (otherwise 64 while there are at most sixteen shares);
 * "attention.handover" = 1 makes its shares travel through a ticket per head instead of as (value, flag) pairs;
 * "attention.fence" = 0 makes the ticket that hands its shares over a relaxed operation instead of a
 * release-acquire one at device scope, 2 also stores and loads the shares plainly (both to be measured; 1 restores).
 * "q4_0.fx_rows" = n sends Q4_0 products of at least n rows of float32 x to the
 * int8 matrix cores whatever the shape (0: the built-in cost model);
 * "q4_0.fx_pairs" = 0 keeps those products off the binary16 form of that
 * kernel, 2 sends them all there (1: its cost model).
 * "qgemm.blocks" = 0 keeps the exact Q4_0 products of mi355x_qgemm_bf16 on the
 * kernel that needs no workspace, 2 sends them all through the panel of the
 * weights' integers (1: by shape).
 * "kquant.rows" = 1, 2 or 4 fixes the rows of W a wavefront of the Q4_K / Q6_K
 * kernels takes; "kquant.path" = 1 forces their variant that reads x from
 * global memory (otherwise used only for rows of x too long for the LDS), 2
 * keeps them off the matrix cores whatever M is, 3 puts them there for any M.
 * "kquant.mfma_rows" = 1 keeps Q4_K / Q6_K products of a few rows of x off the
 * kernel that reads W once per eight rows, 2 sends them there for any number of
 * rows from two on; "kquant.mfma_rows_waves" = 4 or 8 fixes its wavefronts a
 * workgroup, 1 keeps its partial sums in LDS whatever K is (0: both by shape).
 * "qgemm.path" = 1 makes mi355x_qgemm_bf16 take its general route for every shape.
 * "qgemm.f16" = 1 makes mi355x_qgemm_bf16's Q4_0 matrix-core kernel round every
 * weight once to binary16 instead of multiplying it exactly (each weight within
 * 2^-11 of itself; at K = 4096 the results are off by about 2e-4 of their root mean
 * square, 1e-3 of it at worst; block scales beyond 8188 in magnitude overflow):
 * no vector arithmetic per block, 862 against the exact form's 757 TFLOP/s at
 * 2048 x 14336 x 4096. From 1024 rows of X on
 * (and enough of Y for three quarters of the device in tiles of 256 x 256) this form
 * first writes W once as a binary16 panel into the call's scratch (2 N K bytes) and
 * multiplies from it; = 2 keeps it on the one launch whose tiles convert W for
 * themselves. Off by default; the setting is process-wide.
 * "attention.path" = 1 makes mi355x_attention use its general kernels also for
 * one query position (which otherwise takes a single-launch kernel).
 * "attention.prompt" = 0 makes it use them also for 64 and more query positions
 * (which otherwise, without a mask, at 64 or 128 features and key rows that start
 * on 16 bytes, take a kernel that shares tiles of keys among 128 query rows on the
 * float32 matrix cores: the same sums in another order).
 * "llama.step" chooses how mi355x_llama_generate runs its decoding steps: 0 the
 * fused launches replayed as a HIP graph where every block's linears are Q4_0
 * (else the per-operator path), 1 the same launches without the graph, 2 the
 * per-operator path always. "llama.rows" = 1 makes two to eight sequences decode
 * with the one-sequence kernels run per sequence instead of the step that reads
 * every weight once for all of them, 2 keeps that step but runs the rotation
 * and SwiGLU as launches of their own (3, 4: only SwiGLU, only the rotation). */
MI355X_API mi355x_status mi355x_tune(const char* key, int value);
#ifdef __cplusplus
}
#endif
#endif /* MIMIR_MI355X_H */
