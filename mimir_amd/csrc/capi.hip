// The C ABI declared in include/mimir_mi355x.h: argument checks on the host
// (so that a launch never sees a shape its kernel does not expect), the
// per-device state, and the mapping of failures onto status codes.
#include "../../include/mimir_mi355x.h"
#include "../../include/mimir_mi355x_measure.h"

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <map>
#include <mutex>
#include <vector>
#include <string>

#include "kernels.h"

namespace {

thread_local std::string g_last_error;

mi355x_status fail(mi355x_status code, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return code;
}

mi355x_status hip_fail(hipError_t e, const char* what) {
    return fail((mi355x_status)e, "mi355x: %s: %s", what, hipGetErrorName(e));
}

#define HIP_TRY(expr, what)                         \
    do {                                            \
        hipError_t e_ = (expr);                     \
        if (e_ != hipSuccess) return hip_fail(e_, what); \
    } while (0)

constexpr int kMaxDevices = 16;

// The converted activations of mi355x_qgemv_noalloc: a fixed block in the code object's own
// device memory, so that the entry point allocates nothing. Every device the library runs on
// holds its own copy at its own address (DeviceState::fixed, looked up when the device's state
// is created); in host code the array's name is only a handle for that lookup, never an address.
constexpr size_t kNoallocScratchBytes = (size_t)1 << 20;
static __device__ __align__(256) unsigned char g_noalloc_scratch[kNoallocScratchBytes];

// Scratch memory of the entry points that need some beyond their arguments (converted activations,
// partial results and tickets of split attention and argmax, float32 copies of qgemm_bf16's general
// route). One set per device and stream: calls on different streams never share a block, calls on one
// stream are ordered by it. A block that has become too small is replaced by a larger one and kept
// aside: work already queued, and HIP graphs a caller has instantiated over an entry point, may still
// read and write it, tickets included (a graph keeps the block it was recorded with and stays valid).
// Growth at least doubles a block, so what is kept aside stays below the size of the live block.
// mi355x_stream_release frees everything a stream holds, live and kept aside.
struct ScratchBlock {
    void* p = nullptr;
    size_t bytes = 0;
};
struct StreamScratch {
    ScratchBlock act, attn, attn_flags, gemm, argmax;
    std::vector<void*> retired;  // outgrown blocks
};

// Per-device state: the error word kernels OR bits into, read back at sync.
struct DeviceState {
    bool ready = false;
    uint32_t* err_dev = nullptr;
    uint32_t* err_host = nullptr;  // pinned
    std::map<void*, StreamScratch> scratch;  // by stream handle
    void* fixed = nullptr;                   // this device's copy of g_noalloc_scratch
};

std::mutex g_mu;
DeviceState g_dev[kMaxDevices];
std::atomic<int> g_tune_q4_live[5] = {{0}, {0}, {0}, {0}, {0}};
// A call's own copy of the launch-plan overrides, so that one call sees one plan.
struct TuneQ4 {
    int v[5];
    TuneQ4() { for (int i = 0; i < 5; i++) v[i] = g_tune_q4_live[i].load(std::memory_order_relaxed); }
    operator const int*() const { return v; }
    int operator[](int i) const { return v[i]; }
};
// Up to this many rows of x the Q4_0 product converts x inside its own launch (each workgroup
// for itself); beyond, one conversion launch serves all workgroups.
constexpr int64_t kConvertInProductRows = 8;
// Rows of x from which the Q4_0 product of float32 x goes to the int8 matrix cores: 16 means wherever its
// cost model says it pays; "q4_0.fx_rows" sets another threshold, which then holds for every shape.
std::atomic<int> g_fx_min_rows{16};
std::atomic<int> g_rows_max{0};    // "q4_0.rows_max" n: Q4_0 products of fewer than n rows of x take the kernel that reads W once per eight rows (0: by cost)
std::atomic<int> g_rows_path{0};  // "q4_0.rows_path" 1: no matrix-core kernel for two to fifteen rows of x
std::atomic<int> g_tune_gemm{0};  // 1: qgemm_bf16 always takes its general route
std::atomic<int> g_tune_gemm_f16{0};  // 1: the Q4_0 matrix-core product with weights rounded to binary16
std::atomic<int> g_tune_attn{0};  // 1: the general kernels also for one query position
}
thread_local char t_last_kernel[160] = "";
thread_local std::vector<hipEvent_t> t_events;
thread_local size_t t_events_used = 0;
namespace mimir {
void set_llama_step_mode(int mode);  // llm.hip
void set_llama_rows_off(int v);      // llm.hip
void note_kernel(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(t_last_kernel, sizeof t_last_kernel, fmt, ap);
    va_end(ap);
}
bool next_timing_events(hipEvent_t* start, hipEvent_t* stop) {
    if (t_events_used + 2 > t_events.size()) return false;
    *start = t_events[t_events_used];
    *stop = t_events[t_events_used + 1];
    t_events_used += 2;
    return true;
}
}
namespace {

mi355x_status current_state(DeviceState** out) {
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev), "hipGetDevice");
    if (dev < 0 || dev >= kMaxDevices) return fail(MI355X_ERR_INTERNAL, "mi355x: device %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_mu);
    DeviceState& s = g_dev[dev];
    if (!s.ready) {
        hipDeviceProp_t prop;
        HIP_TRY(hipGetDeviceProperties(&prop, dev), "hipGetDeviceProperties");
        if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
            return fail(MI355X_ERR_INTERNAL, "mi355x: device %d is %s; this library holds gfx950 code only", dev, prop.gcnArchName);
        // the lookup first: if it fails nothing has been allocated that a later call would allocate again
        HIP_TRY(hipGetSymbolAddress(&s.fixed, HIP_SYMBOL(g_noalloc_scratch)), "hipGetSymbolAddress(fixed scratch)");
        if (!s.err_dev) {
            HIP_TRY(hipMalloc((void**)&s.err_dev, 256), "hipMalloc(error word)");
            HIP_TRY(hipMemset(s.err_dev, 0, 256), "hipMemset(error word)");
        }
        if (!s.err_host) HIP_TRY(hipHostMalloc((void**)&s.err_host, 256, hipHostMallocDefault), "hipHostMalloc(error word)");
        s.ready = true;
    }
    *out = &s;
    return MI355X_OK;
}

// Returns the calling stream's block `which` of the current device, at least `bytes` long (at least `floor`
// when it has to be allocated); the first `zero_prefix` bytes of a new block are zeroed (tickets).
// Allocates, so it fails under stream capture when the block has to grow: a caller that records a
// graph runs the call once beforehand, as run_batch does.
mi355x_status stream_scratch(void* stream, ScratchBlock StreamScratch::*which, size_t bytes, size_t floor, size_t zero_prefix, const char* what,
                             void** out) {
    DeviceState* s;
    if (mi355x_status st = current_state(&s)) return st;
    std::lock_guard<std::mutex> lock(g_mu);
    StreamScratch& mine = s->scratch[stream];
    ScratchBlock& b = mine.*which;
    if (b.bytes < bytes) {
        size_t want = bytes < floor ? floor : bytes;
        if (want < 2 * b.bytes) want = 2 * b.bytes;
        void* p = nullptr;
        hipError_t e = hipMalloc(&p, want);
        if (e != hipSuccess) return fail((mi355x_status)e, "mi355x: hipMalloc(%s scratch, %zu bytes): %s", what, want, hipGetErrorName(e));
        if (zero_prefix) {
            // on the calling stream, so that the zeros are in place before the first kernel that takes a ticket there
            // (never under capture: the allocation above fails first)
            e = hipMemsetAsync(p, 0, zero_prefix < want ? zero_prefix : want, (hipStream_t)stream);
            if (e != hipSuccess) {
                (void)hipFree(p);  // nothing has seen it yet
                return fail((mi355x_status)e, "mi355x: hipMemset(%s tickets): %s", what, hipGetErrorName(e));
            }
        }
        if (b.p) mine.retired.push_back(b.p);
        b.p = p;
        b.bytes = want;
    }
    *out = b.p;
    return MI355X_OK;
}

mi355x_status act_scratch(void* stream, size_t bytes, void** out) {
    return stream_scratch(stream, &StreamScratch::act, bytes, 1u << 20, 0, "activation", out);
}
// Where a product's converted activations go: the stream's growing block, or a fixed block of
// fixed_bytes bytes (then nothing is allocated and a larger need is an error).
struct ActSource {
    void* stream;
    void* fixed;
    size_t fixed_bytes;
};
mi355x_status act_for(const ActSource& src, size_t bytes, void** out) {
    if (!src.fixed) return act_scratch(src.stream, bytes, out);
    if (bytes > src.fixed_bytes)
        return fail(MI355X_ERR_SHAPE, "mi355x: qgemv_noalloc: the converted activations take %zu bytes, the fixed scratch holds %zu", bytes, src.fixed_bytes);
    *out = src.fixed;
    return MI355X_OK;
}
mi355x_status attn_scratch(void* stream, size_t bytes, void** out) {
    return stream_scratch(stream, &StreamScratch::attn, bytes, 4u << 20, mimir::kAttnTicketBytes, "attention", out);
}
// The (value, flag) slots of decode attention's hand-over: all zero when handed out, and nobody else's.
mi355x_status attn_flags_scratch(void* stream, size_t bytes, void** out) {
    return stream_scratch(stream, &StreamScratch::attn_flags, bytes, 1u << 20, (size_t)-1 /* all of it */, "attention hand-over", out);
}
mi355x_status gemm_scratch(void* stream, size_t bytes, void** out) {
    return stream_scratch(stream, &StreamScratch::gemm, bytes, 0, 0, "gemm", out);
}
mi355x_status argmax_scratch(void* stream, size_t bytes, void** out) {
    return stream_scratch(stream, &StreamScratch::argmax, bytes, 0, mimir::kArgmaxTicketBytes, "argmax", out);
}

}  // namespace

// For the other host files of the library.
namespace mimir {
mi355x_status capi_fail(mi355x_status code, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return code;
}
uint32_t* device_error_word() {
    DeviceState* s;
    return current_state(&s) == MI355X_OK ? s->err_dev : nullptr;
}
}  // namespace mimir

extern "C" {

mi355x_status mi355x_init(int device) {
    int n = 0;
    HIP_TRY(hipGetDeviceCount(&n), "hipGetDeviceCount");
    if (device < 0 || device >= n) return fail(MI355X_ERR_INTERNAL, "mi355x: device %d of %d", device, n);
    HIP_TRY(hipSetDevice(device), "hipSetDevice");
    DeviceState* s;
    return current_state(&s);
}

size_t mi355x_last_error(char* buf, size_t n) {
    if (buf && n) {
        size_t c = g_last_error.size() < n - 1 ? g_last_error.size() : n - 1;
        memcpy(buf, g_last_error.data(), c);
        buf[c] = 0;
    }
    return g_last_error.size();
}

int mi355x_block_size(int dtype) { return mimir::block_size(dtype); }
int mi355x_block_bytes(int dtype) { return mimir::block_bytes(dtype); }

int64_t mi355x_bytes(int dtype, int64_t n) {
    int bs = mimir::block_size(dtype), bb = mimir::block_bytes(dtype);
    if (bb == 0 || n < 0 || n % bs != 0 || n / bs > INT64_MAX / bb) return -1;
    return n / bs * bb;
}

mi355x_status mi355x_alloc(void** out, size_t bytes) {
    if (!out) return fail(MI355X_ERR_INTERNAL, "mi355x: alloc: null result pointer");
    *out = nullptr;
    // at least 4 bytes, as the reference's Alloc (backend/rocm/rocm_linux.go:220-240)
    hipError_t e = hipMalloc(out, bytes < 4 ? 4 : bytes);
    if (e != hipSuccess) return hip_fail(e, "hipMalloc");
    return MI355X_OK;
}

mi355x_status mi355x_free(void* ptr) {
    if (!ptr) return MI355X_OK;
    HIP_TRY(hipFree(ptr), "hipFree");
    return MI355X_OK;
}

mi355x_status mi355x_upload(void* dst, const void* src, size_t bytes, void* stream) {
    if (bytes == 0) return MI355X_OK;
    if (!dst || !src) return fail(MI355X_ERR_INTERNAL, "mi355x: upload: null pointer");
    HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, (hipStream_t)stream), "hipMemcpyAsync(H2D)");
    return MI355X_OK;
}

mi355x_status mi355x_download(void* dst, const void* src, size_t bytes, void* stream) {
    if (bytes == 0) return MI355X_OK;
    if (!dst || !src) return fail(MI355X_ERR_INTERNAL, "mi355x: download: null pointer");
    HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, (hipStream_t)stream), "hipMemcpyAsync(D2H)");
    HIP_TRY(hipStreamSynchronize((hipStream_t)stream), "hipStreamSynchronize");
    return MI355X_OK;
}

mi355x_status mi355x_sync(void* stream) {
    DeviceState* s;
    if (mi355x_status st = current_state(&s)) return st;
    HIP_TRY(hipMemcpyAsync(s->err_host, s->err_dev, 4, hipMemcpyDeviceToHost, (hipStream_t)stream), "hipMemcpyAsync(error word)");
    HIP_TRY(hipStreamSynchronize((hipStream_t)stream), "hipStreamSynchronize");
    uint32_t bits = *s->err_host;
    if (bits) {
        HIP_TRY(hipMemsetAsync(s->err_dev, 0, 4, (hipStream_t)stream), "hipMemsetAsync(error word)");
        HIP_TRY(hipStreamSynchronize((hipStream_t)stream), "hipStreamSynchronize");
        if (bits & mimir::kErrIndex) return fail(MI355X_ERR_INDEX, "mi355x: a gather read an index out of range");
        return fail(MI355X_ERR_INTERNAL, "mi355x: device error bits %#x", bits);
    }
    return MI355X_OK;
}

// Tensor.MatMulT with bfloat16 activations (tensor/quant.go:45-48): float32
// product, one rounding to the output's dtype.
mi355x_status mi355x_qgemm_bf16(int dtype, const void* W, const void* X, void* Y, int64_t M, int64_t N, int64_t K, int64_t x_row_stride,
                                int out_dtype, void* stream) {
    if (!mimir::is_quantized(dtype)) return fail(MI355X_ERR_DTYPE, "mi355x: qgemm_bf16 by weights of dtype %d", dtype);
    if (out_dtype != MI355X_BF16 && out_dtype != MI355X_F32) return fail(MI355X_ERR_DTYPE, "mi355x: qgemm_bf16 into dtype %d", out_dtype);
    if (M < 0 || N < 0 || K < 0 || K % mimir::block_size(dtype) != 0)
        return fail(MI355X_ERR_INTERNAL, "mi355x: qgemm_bf16 of [%lld, %lld] by [%lld, %lld] in blocks of %d", (long long)M, (long long)K,
                    (long long)N, (long long)K, mimir::block_size(dtype));
    if (M == 0 || N == 0) return MI355X_OK;
    if (!W || !X || !Y) return fail(MI355X_ERR_INTERNAL, "mi355x: qgemm_bf16: null pointer");
    if (M > 65535 || N > (int64_t)1 << 24 || K > (int64_t)1 << 24)
        return fail(MI355X_ERR_SHAPE, "mi355x: qgemm_bf16 of %lld rows by [%lld, %lld]: too large", (long long)M, (long long)N, (long long)K);
    if (M > 1 && x_row_stride < K) return fail(MI355X_ERR_SHAPE, "mi355x: qgemm_bf16: rows of x %lld apart overlap (K = %lld)", (long long)x_row_stride, (long long)K);
    hipStream_t st = (hipStream_t)stream;
    const bool f32 = out_dtype == MI355X_F32;
    if (K == 0) {
        HIP_TRY(mimir::fill_u32(Y, 0, f32 ? M * N : (M * N + 1) / 2, st), "launch fill");
        return MI355X_OK;
    }
    void* ws;
    if (dtype == MI355X_Q4_0 && g_tune_gemm != 1 && mimir::qgemm_q4_0_ok(W, X, M, N, K, x_row_stride)) {
        if (g_tune_gemm_f16 == 0 && mimir::qgemm_q4_0_blocks_pays(M, N, K)) {
            // the exact form of a large product: W's integers once as a bfloat16 panel, then one MFMA a weight
            if (mi355x_status s2 = gemm_scratch(stream, mimir::qgemm_q4_0_blocks_ws_bytes(N, K), &ws)) return s2;
            HIP_TRY(mimir::qgemm_q4_0_blocks(W, X, x_row_stride, Y, M, N, K, f32, ws, st), "launch qgemm_q4_0_blocks");
            return MI355X_OK;
        }
        void* half_ws = nullptr;
        const bool panel = g_tune_gemm_f16 == 1;  // 2: the binary16 form without the panel route
        if (g_tune_gemm_f16 == 1 || g_tune_gemm_f16 == 2)
            if (mi355x_status s2 = gemm_scratch(stream, mimir::qgemm_q4_0_half_ws_bytes(M, N, K, panel), &half_ws)) return s2;
        HIP_TRY(mimir::qgemm_q4_0_bf16(W, X, Y, M, N, K, x_row_stride, f32, half_ws, panel, st), "launch qgemm_q4_0");
        return MI355X_OK;
    }
    if ((dtype == MI355X_Q4_K || dtype == MI355X_Q6_K) && g_tune_gemm != 1 && ((uintptr_t)X & 7) == 0 && x_row_stride % 4 == 0) {
        // the int8 rounding reads the bfloat16 rows directly and the matrix-core kernel rounds its results
        void* act;
        if (mi355x_status s2 = act_scratch(stream, mimir::kq_act_bytes(K) * (size_t)M, &act)) return s2;
        mimir::QGemvArgs a{W, nullptr, act, (float*)Y, M, N, K, 0, 0};
        if (mimir::qgemv_kquant_rows_pays(dtype, a)) {  // a few rows: W read once per eight of them, the same bits, one rounding after
            float* yf = (float*)Y;
            if (!f32) {
                if (mi355x_status s2 = gemm_scratch(stream, ((size_t)M * N * 4 + 255) & ~(size_t)255, &ws)) return s2;
                yf = (float*)ws;
            }
            a.y = yf;
            HIP_TRY(mimir::kq_convert_act_bf16(X, M, K, x_row_stride, act, st), "launch kq_convert_act");
            HIP_TRY(mimir::qgemv_kquant_rows(dtype, a, st), "launch qgemv_kquant_rows");
            if (!f32) HIP_TRY(mimir::f32_to_bf16(yf, Y, M * N, st), "launch cast");
            return MI355X_OK;
        }
        if (mimir::qgemm_kquant_ok(dtype, a) && mimir::qgemm_kquant_pays(dtype, a)) {
            HIP_TRY(mimir::kq_convert_act_bf16(X, M, K, x_row_stride, act, st), "launch kq_convert_act");
            HIP_TRY(mimir::qgemm_kquant(dtype, a, st, !f32), "launch qgemm_kquant");
            return MI355X_OK;
        }
    }
    // Any other shape or dtype: the activations as float32 through mi355x_qgemv, then one rounding. For
    // Q8_0, Q4_K and Q6_K that is the reference's own sequence (cast, int8 rounding of x, integer dot
    // products, cast), and the K-quants take their matrix-core kernel from a few rows on.
    const size_t xb = ((size_t)M * K * 4 + 255) & ~(size_t)255, yb = ((size_t)M * N * 4 + 255) & ~(size_t)255;
    if (mi355x_status s2 = gemm_scratch(stream, xb + yb, &ws)) return s2;
    float* xf = (float*)ws;
    float* yf = f32 ? (float*)Y : (float*)((uint8_t*)ws + xb);
    HIP_TRY(mimir::bf16_rows_to_f32(X, xf, M, K, x_row_stride, st), "launch cast");
    if (mi355x_status s2 = mi355x_qgemv(dtype, W, xf, yf, M, N, K, K, stream)) return s2;
    if (!f32) HIP_TRY(mimir::f32_to_bf16(yf, Y, M * N, st), "launch cast");
    return MI355X_OK;
}

static mi355x_status qgemv_impl(int dtype, const void* W, const float* x, float* y, int64_t M, int64_t N, int64_t K, int64_t x_row_stride,
                                void* stream, const ActSource& src) {
    const TuneQ4 g_tune_q4;  // this call's copy of the launch-plan overrides
    if (!mimir::is_quantized(dtype)) return fail(MI355X_ERR_DTYPE, "mi355x: qgemv by weights of dtype %d", dtype);
    int bs = mimir::block_size(dtype);
    if (M < 0 || N < 0 || K < 0 || K % bs != 0)
        return fail(MI355X_ERR_INTERNAL, "mi355x: qgemv of [%lld, %lld] by [%lld, %lld] in blocks of %d", (long long)M,
                    (long long)K, (long long)N, (long long)K, bs);
    if (M == 0 || N == 0) return MI355X_OK;
    if (!W || !x || !y) return fail(MI355X_ERR_INTERNAL, "mi355x: qgemv: null pointer");
    if (M > 65535 || N > (int64_t)1 << 30 || K > (int64_t)1 << 30)
        return fail(MI355X_ERR_SHAPE, "mi355x: qgemv of %lld rows by [%lld, %lld]: too large", (long long)M, (long long)N,
                    (long long)K);
    if (M > 1 && x_row_stride < K && x_row_stride != 0)
        return fail(MI355X_ERR_SHAPE, "mi355x: qgemv: rows of x %lld apart overlap (K = %lld)", (long long)x_row_stride, (long long)K);
    if (K == 0) {  // an empty sum: zeros (backend/cpu/qmatmul.go:336-339)
        HIP_TRY(mimir::fill_u32(y, 0, M * N, (hipStream_t)stream), "launch fill");
        return MI355X_OK;
    }
    mimir::QGemvArgs a{W, x, nullptr, y, M, N, K, x_row_stride, 0};
    switch (dtype) {
    case MI355X_Q4_0:
        if (g_tune_q4[4] != 1 && mimir::q4_0_fixed_point_ok(W, K)) {
            // A few rows (the decoding step of a batch): W read once per eight rows of x, on the int8 matrix cores; up to
            // where the tiled kernel for many rows is the faster by both kernels' measured costs (some tens of rows).
            const bool wide_x = ((uintptr_t)x & 15) == 0 && x_row_stride % 4 == 0;
            const bool fx_forced = g_fx_min_rows != 16 && M >= g_fx_min_rows;
            bool rows = M >= 2 && g_rows_path != 1 && g_tune_q4[4] != 2 && wide_x && !fx_forced && mimir::qgemv_q4_0_rows_ok(W, 1, N, K);
            if (rows && g_rows_max > 0) rows = M < g_rows_max;
            else if (rows && M >= 16 && mimir::qgemm_q4_0_fx_ok(W, M, N, K))
                rows = mimir::qgemv_q4_0_rows_cost_us(M, N, K) < mimir::qgemm_q4_0_fx_cost_us(M, N, K);
            if (rows) {
                const bool one_launch = mimir::qgemv_q4_0_rows_shares_ok(W, M, N, K, 1);  // else the variant that takes eight rows a launch
                const int64_t groups = (M + 7) / 8;
                void* act;
                if (mi355x_status st = act_for(src, mimir::q4_0_rows_act_bytes(K) * (size_t)(one_launch ? groups : 1), &act)) return st;
                if (one_launch) {
                    HIP_TRY(mimir::q4_0_rows_convert_act(x, M, K, x_row_stride, act, (hipStream_t)stream), "launch q4_0_rows_convert_act");
                    HIP_TRY(mimir::qgemv_q4_0_rows(W, act, y, nullptr, M, N, K, 1, (hipStream_t)stream), "launch qgemv_q4_0_rows");
                    return MI355X_OK;
                }
                for (int64_t m0 = 0; m0 < M; m0 += 8) {
                    const int64_t mm = M - m0 < 8 ? M - m0 : 8;
                    HIP_TRY(mimir::q4_0_rows_convert_act(x + m0 * x_row_stride, mm, K, x_row_stride, act, (hipStream_t)stream), "launch q4_0_rows_convert_act");
                    HIP_TRY(mimir::qgemv_q4_0_rows(W, act, y + m0 * N, nullptr, mm, N, K, 1, (hipStream_t)stream), "launch qgemv_q4_0_rows");
                }
                return MI355X_OK;
            }
            if (g_tune_q4[4] != 2 && M >= g_fx_min_rows && (g_fx_min_rows != 16 ? mimir::qgemm_q4_0_fx_ok(W, M, N, K) : mimir::qgemm_q4_0_fx_pays(W, M, N, K)) &&
                ((uintptr_t)x & 15) == 0 && x_row_stride % 4 == 0) {
                // many rows: the same fixed-point arithmetic on the int8 matrix cores
                void* act;
                // from some hundreds of rows on as pairs of 12-bit digits on the binary16 matrix cores, which want a
                // workspace behind the activations (not from a fixed scratch, which is too small for it)
                const bool pairs = !src.fixed && mimir::qgemm_q4_0_fx16_pays(M, N, K);
                const size_t act_bytes = ((pairs ? mimir::q4_0_fx16_act_bytes(K) : mimir::q4_0_fx_act_bytes(K)) * (size_t)M + 255) / 256 * 256;
                if (mi355x_status st = act_for(src, act_bytes + (pairs ? mimir::qgemm_q4_0_fx16_ws_bytes(N, K) : 0), &act)) return st;
                HIP_TRY(mimir::q4_0_fx_convert_act(x, M, K, x_row_stride, act, pairs, (hipStream_t)stream), "launch q4_0_fx_convert_act");
                HIP_TRY(mimir::qgemm_q4_0_fx(W, act, y, nullptr, M, N, K, pairs ? (uint8_t*)act + act_bytes : nullptr, (hipStream_t)stream),
                        "launch qgemm_q4_0_fx");
                return MI355X_OK;
            }
            if (M == 1 && ((uintptr_t)x & 15) == 0) {
                // one row: one launch, every workgroup converts x for itself (several rows: converted once, multiplied together)
                HIP_TRY(mimir::qgemv_q4_0_act(a, g_tune_q4, (hipStream_t)stream), "launch qgemv_q4_0");
                return MI355X_OK;
            }
            void* act;
            if (mi355x_status st = act_for(src, mimir::q4_0_act_bytes(K) * (size_t)M, &act)) return st;
            HIP_TRY(mimir::q4_0_convert_act(x, M, K, x_row_stride, act, (hipStream_t)stream), "launch q4_0_convert_act");
            a.act = act;
            HIP_TRY(mimir::qgemv_q4_0_act(a, g_tune_q4, (hipStream_t)stream), "launch qgemv_q4_0_act");
            return MI355X_OK;
        }
        HIP_TRY(mimir::qgemv_q4_0(a, g_tune_q4, (hipStream_t)stream), "launch qgemv_q4_0");
        return MI355X_OK;
    case MI355X_Q8_0: {
        if (!mimir::q8_act_fits(K)) return fail(MI355X_ERR_SHAPE, "mi355x: qgemv by q8_0 with K = %lld: rows longer than 57344 are not supported", (long long)K);
        // Small products in one launch (a.act stays null: every workgroup rounds x for itself); this kernel does not
        // request its weights ahead of that, so on large ones a conversion launch of its own is the faster (measured).
        if (M <= kConvertInProductRows && N * K <= (int64_t)24 << 20 && ((uintptr_t)x & 15) == 0 && (M == 1 || x_row_stride % 4 == 0)) {
            HIP_TRY(mimir::qgemv_q8_0_act(a, g_tune_q4, (hipStream_t)stream), "launch qgemv_q8_0");
            return MI355X_OK;
        }
        void* act;
        if (mi355x_status st = act_for(src, mimir::q8_act_bytes(K) * (size_t)M, &act)) return st;
        HIP_TRY(mimir::q8_convert_act(x, M, K, x_row_stride, act, (hipStream_t)stream), "launch q8_convert_act");
        a.act = act;
        if (g_rows_path != 1 && mimir::qgemv_q8_0_mfma_pays(a)) {  // a large matrix and two to eight rows: the int8 matrix cores
            HIP_TRY(mimir::qgemv_q8_0_mfma(a, (hipStream_t)stream), "launch qgemv_q8_0_mfma");
            return MI355X_OK;
        }
        if (g_rows_path != 1 && mimir::qgemv_q8_0_rows_ok(a)) {  // several rows: W read once for up to eight of them, the same sums
            HIP_TRY(mimir::qgemv_q8_0_rows(a, (hipStream_t)stream), "launch qgemv_q8_0_rows");
            return MI355X_OK;
        }
        HIP_TRY(mimir::qgemv_q8_0_act(a, g_tune_q4, (hipStream_t)stream), "launch qgemv_q8_0_act");
        return MI355X_OK;
    }
    case MI355X_Q4_K:
    case MI355X_Q6_K: {
        // One row against a small matrix: one launch, every workgroup rounding x itself (a.act stays null). Measured at
        // K = 4096: 4.7 against 6.5 us at N = 1024, level at N = 4096, 2 us behind at N = 14336.
        if (M == 1 && N * K <= (8ll << 20) && ((uintptr_t)x & 15) == 0 && mimir::qgemv_kquant_rope_ok(dtype, a)) {
            HIP_TRY(mimir::qgemv_kquant_act(dtype, a, (hipStream_t)stream), "launch qgemv_kquant");
            return MI355X_OK;
        }
        void* act;
        if (mi355x_status st = act_for(src, mimir::kq_act_bytes(K) * (size_t)M, &act)) return st;
        HIP_TRY(mimir::kq_convert_act(x, M, K, x_row_stride, act, (hipStream_t)stream), "launch kq_convert_act");
        a.act = act;
        HIP_TRY(mimir::qgemv_kquant_act(dtype, a, (hipStream_t)stream), "launch qgemv_kquant_act");
        return MI355X_OK;
    }
    default:
        return fail(MI355X_ERR_DTYPE, "mi355x: qgemv by weights of dtype %d", dtype);
    }
}

mi355x_status mi355x_qgemv(int dtype, const void* W, const float* x, float* y, int64_t M, int64_t N, int64_t K,
                           int64_t x_row_stride, void* stream) {
    return qgemv_impl(dtype, W, x, y, M, N, K, x_row_stride, stream, ActSource{stream, nullptr, 0});
}

// mi355x_qgemv without an allocation: the device's state must exist already (mi355x_init), and the
// converted activations go to the device's fixed block.
mi355x_status mi355x_qgemv_noalloc(int dtype, const void* W, const float* x, float* y, int64_t M, int64_t N, int64_t K,
                                   int64_t x_row_stride, void* stream) {
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev), "hipGetDevice");
    void* fixed = nullptr;
    if (dev >= 0 && dev < kMaxDevices) {
        std::lock_guard<std::mutex> lock(g_mu);
        if (g_dev[dev].ready) fixed = g_dev[dev].fixed;
    }
    if (!fixed) return fail(MI355X_ERR_INTERNAL, "mi355x: qgemv_noalloc: call mi355x_init(%d) first (creating the device's state allocates)", dev);
    return qgemv_impl(dtype, W, x, y, M, N, K, x_row_stride, stream, ActSource{stream, fixed, kNoallocScratchBytes});
}

size_t mi355x_act_bytes(int dtype, int64_t K) {
    if (K <= 0) return 0;
    if (dtype == MI355X_Q4_0 && K % 64 == 0) return mimir::q4_0_act_bytes(K);
    if (dtype == MI355X_Q8_0 && K % 32 == 0) return mimir::q8_act_bytes(K);
    if ((dtype == MI355X_Q4_K || dtype == MI355X_Q6_K) && K % 256 == 0) return mimir::kq_act_bytes(K);
    return 0;
}

mi355x_status mi355x_convert_act(int dtype, const float* x, int64_t M, int64_t K, int64_t x_row_stride, void* act, void* stream) {
    if (mi355x_act_bytes(dtype, K) == 0 || M < 0 || M > 65535)
        return fail(MI355X_ERR_SHAPE, "mi355x: convert activations [%lld, %lld] for weights of dtype %d", (long long)M, (long long)K, dtype);
    if (M == 0) return MI355X_OK;
    if (!x || !act || ((uintptr_t)act & 15)) return fail(MI355X_ERR_INTERNAL, "mi355x: convert activations: null or misaligned pointer");
    if (dtype == MI355X_Q4_0)
        HIP_TRY(mimir::q4_0_convert_act(x, M, K, x_row_stride, act, (hipStream_t)stream), "launch q4_0_convert_act");
    else if (dtype == MI355X_Q8_0)
        HIP_TRY(mimir::q8_convert_act(x, M, K, x_row_stride, act, (hipStream_t)stream), "launch q8_convert_act");
    else
        HIP_TRY(mimir::kq_convert_act(x, M, K, x_row_stride, act, (hipStream_t)stream), "launch kq_convert_act");
    return MI355X_OK;
}

mi355x_status mi355x_qgemv_act(int dtype, const void* W, const void* act, float* y, int64_t M, int64_t N, int64_t K, void* stream) {
    const TuneQ4 g_tune_q4;  // this call's copy of the launch-plan overrides
    if (M < 0 || N < 0 || K <= 0 || M > 65535 || N > (int64_t)1 << 30)
        return fail(MI355X_ERR_SHAPE, "mi355x: qgemv_act of %lld rows by [%lld, %lld]", (long long)M, (long long)N, (long long)K);
    if (M == 0 || N == 0) return MI355X_OK;
    if (!W || !act || !y || ((uintptr_t)act & 15)) return fail(MI355X_ERR_INTERNAL, "mi355x: qgemv_act: null or misaligned pointer");
    mimir::QGemvArgs a{W, nullptr, act, y, M, N, K, 0, 0};
    if (dtype == MI355X_Q4_0) {
        if (!mimir::q4_0_fixed_point_ok(W, K))
            return fail(MI355X_ERR_SHAPE, "mi355x: qgemv_act by q4_0 needs K a multiple of 64 up to 20928 and W dword aligned (K = %lld)", (long long)K);
        HIP_TRY(mimir::qgemv_q4_0_act(a, g_tune_q4, (hipStream_t)stream), "launch qgemv_q4_0_act");
    } else if (dtype == MI355X_Q8_0) {
        if (K % 32 != 0 || !mimir::q8_act_fits(K))
            return fail(MI355X_ERR_SHAPE, "mi355x: qgemv_act by q8_0 needs K a multiple of 32 up to 57344 (K = %lld)", (long long)K);
        HIP_TRY(mimir::qgemv_q8_0_act(a, g_tune_q4, (hipStream_t)stream), "launch qgemv_q8_0_act");
    } else if (dtype == MI355X_Q4_K || dtype == MI355X_Q6_K) {
        if (K % 256 != 0) return fail(MI355X_ERR_SHAPE, "mi355x: qgemv_act by a K-quant needs K a multiple of 256 (K = %lld)", (long long)K);
        HIP_TRY(mimir::qgemv_kquant_act(dtype, a, (hipStream_t)stream), "launch qgemv_kquant_act");
    } else {
        return fail(MI355X_ERR_DTYPE, "mi355x: qgemv_act by dtype %d", dtype);
    }
    return MI355X_OK;
}

// The fused products of a decoding step. The reference fuses the same ones on
// its CPU path by concatenating weights (fusedFor, llm/decode.go:240-266).
static mi355x_status fused_args_ok(const char* what, int dtype, const void* act, const float* y, int64_t M, int64_t K) {
    if (dtype != MI355X_Q4_0) return fail(MI355X_ERR_DTYPE, "mi355x: %s by weights of dtype %d (q4_0 only)", what, dtype);
    if (M < 0 || M > 65535 || K <= 0) return fail(MI355X_ERR_SHAPE, "mi355x: %s of [%lld, %lld]", what, (long long)M, (long long)K);
    if (!act || !y || ((uintptr_t)act & 15)) return fail(MI355X_ERR_INTERNAL, "mi355x: %s: null or misaligned pointer", what);
    return MI355X_OK;
}

mi355x_status mi355x_qgemv_act_add(int dtype, const void* W, const void* act, const float* resid, float* y, int64_t M, int64_t N, int64_t K, void* stream) {
    const TuneQ4 g_tune_q4;  // this call's copy of the launch-plan overrides
    if (mi355x_status st = fused_args_ok("qgemv_act_add", dtype, act, y, M, K)) return st;
    if (N < 0 || N > (int64_t)1 << 30) return fail(MI355X_ERR_SHAPE, "mi355x: qgemv_act_add of %lld rows", (long long)N);
    if (M == 0 || N == 0) return MI355X_OK;
    if (!W || !resid || !mimir::q4_0_fixed_point_ok(W, K)) return fail(MI355X_ERR_SHAPE, "mi355x: qgemv_act_add needs K a multiple of 64 up to 20928 and W dword aligned");
    mimir::QGemvArgs a{W, nullptr, act, y, M, N, K, 0, 0};
    a.resid = resid;
    HIP_TRY(mimir::qgemv_q4_0_act(a, g_tune_q4, (hipStream_t)stream), "launch qgemv_q4_0_act");
    return MI355X_OK;
}

mi355x_status mi355x_qgemv_act_multi(int dtype, const void* W0, const void* W1, const void* W2, int64_t n0, int64_t n1, int64_t n2,
                                     const void* act, float* y, int64_t M, int64_t K, void* stream) {
    const TuneQ4 g_tune_q4;  // this call's copy of the launch-plan overrides
    if (mi355x_status st = fused_args_ok("qgemv_act_multi", dtype, act, y, M, K)) return st;
    const void* W[3] = {W0, W1, W2};
    const int64_t n[3] = {n0, n1, n2};
    for (int i = 0; i < 3; i++) {
        if (n[i] < 0 || n[i] > (int64_t)1 << 28) return fail(MI355X_ERR_SHAPE, "mi355x: qgemv_act_multi: matrix %d of %lld rows", i, (long long)n[i]);
        if (n[i] > 0 && (!W[i] || !mimir::q4_0_fixed_point_ok(W[i], K)))
            return fail(MI355X_ERR_SHAPE, "mi355x: qgemv_act_multi needs K a multiple of 64 up to 20928 and every W dword aligned");
    }
    if (n0 == 0 && (n1 > 0 || n2 > 0)) return fail(MI355X_ERR_SHAPE, "mi355x: qgemv_act_multi: the first matrix is empty");
    if (n1 == 0 && n2 > 0) return fail(MI355X_ERR_SHAPE, "mi355x: qgemv_act_multi: the second matrix is empty");
    if (M == 0 || n0 + n1 + n2 == 0) return MI355X_OK;
    HIP_TRY(mimir::qgemv_q4_0_act_multi(W, n, act, y, M, K, g_tune_q4, (hipStream_t)stream), "launch qgemv_q4_0_act_multi");
    return MI355X_OK;
}

mi355x_status mi355x_qgemv_act_swiglu(int dtype, const void* gate, const void* up, const void* act, float* y, int64_t M, int64_t N, int64_t K, void* stream) {
    const TuneQ4 g_tune_q4;  // this call's copy of the launch-plan overrides
    if (mi355x_status st = fused_args_ok("qgemv_act_swiglu", dtype, act, y, M, K)) return st;
    if (N < 0 || N > (int64_t)1 << 28) return fail(MI355X_ERR_SHAPE, "mi355x: qgemv_act_swiglu of %lld rows", (long long)N);
    if (M == 0 || N == 0) return MI355X_OK;
    if (!gate || !up || !mimir::q4_0_fixed_point_ok(gate, K) || !mimir::q4_0_fixed_point_ok(up, K))
        return fail(MI355X_ERR_SHAPE, "mi355x: qgemv_act_swiglu needs K a multiple of 64 up to 20928 and both W dword aligned");
    HIP_TRY(mimir::qgemv_q4_0_act_swiglu(gate, up, act, y, M, N, K, g_tune_q4, (hipStream_t)stream), "launch qgemv_q4_0_act_swiglu");
    return MI355X_OK;
}

mi355x_status mi355x_dequant(int dtype, const void* W, int64_t first, int64_t n, void* out, int out_dtype, void* stream) {
    if (!mimir::is_quantized(dtype)) return fail(MI355X_ERR_DTYPE, "mi355x: dequantize dtype %d", dtype);
    if (out_dtype != MI355X_F32 && out_dtype != MI355X_BF16 && out_dtype != MI355X_F16)
        return fail(MI355X_ERR_DTYPE, "mi355x: dequantize into dtype %d", out_dtype);  // backend/cpu/quant.go:288-290
    if (first < 0 || n < 0) return fail(MI355X_ERR_INTERNAL, "mi355x: dequantize elements [%lld, +%lld)", (long long)first, (long long)n);
    if (n == 0) return MI355X_OK;
    if (!W || !out) return fail(MI355X_ERR_INTERNAL, "mi355x: dequantize: null pointer");
    HIP_TRY(mimir::dequantize(dtype, W, first, n, out, out_dtype, (hipStream_t)stream), "launch dequantize");
    return MI355X_OK;
}

mi355x_status mi355x_gather_rows(int dtype, const void* table, int64_t rows, int64_t K, const int32_t* idx, int64_t n,
                                 float* out, void* stream) {
    if (!mimir::is_quantized(dtype)) return fail(MI355X_ERR_DTYPE, "mi355x: gather from dtype %d", dtype);
    if (rows < 0 || K < 0 || n < 0 || K % mimir::block_size(dtype) != 0 || n > 65535)
        return fail(MI355X_ERR_SHAPE, "mi355x: gather %lld rows of [%lld, %lld]", (long long)n, (long long)rows, (long long)K);
    if (n == 0 || K == 0) return MI355X_OK;
    if (!table || !idx || !out) return fail(MI355X_ERR_INTERNAL, "mi355x: gather: null pointer");
    DeviceState* s;
    if (mi355x_status st = current_state(&s)) return st;
    HIP_TRY(mimir::gather_rows(dtype, table, rows, K, idx, n, out, s->err_dev, (hipStream_t)stream), "launch gather_rows");
    return MI355X_OK;
}

mi355x_status mi355x_rmsnorm(const float* x, const float* w, float* y, int64_t rows, int64_t d, double eps, void* stream) {
    if (rows < 0 || d < 0 || rows > INT32_MAX || d > INT32_MAX) return fail(MI355X_ERR_SHAPE, "mi355x: rmsnorm of [%lld, %lld]", (long long)rows, (long long)d);
    if (rows == 0 || d == 0) return MI355X_OK;
    if (!x || !y) return fail(MI355X_ERR_INTERNAL, "mi355x: rmsnorm: null pointer");
    HIP_TRY(mimir::rmsnorm(x, w, y, rows, d, eps, (hipStream_t)stream), "launch rmsnorm");
    return MI355X_OK;
}

mi355x_status mi355x_rope(const float* x, float* y, int64_t rows, int64_t S, int head_dim, int rope_dim, int interleaved,
                          int64_t x_row_stride, int64_t x_pos_stride, int64_t y_row_stride, int64_t y_pos_stride,
                          const float* cos_table, const float* sin_table, int64_t table_len, int64_t offset, void* stream) {
    // nn/transformer.go:229-231
    if (rows < 0 || S < 0 || head_dim <= 0 || rope_dim <= 0 || rope_dim % 2 != 0 || rope_dim > head_dim || offset < 0 ||
        offset + S > table_len)
        return fail(MI355X_ERR_SHAPE, "mi355x: rotary embedding of %d of %d features at positions [%lld, %lld) of a table of %lld",
                    rope_dim, head_dim, (long long)offset, (long long)(offset + S), (long long)table_len);
    if (rows == 0 || S == 0) return MI355X_OK;
    if (!x || !y || !cos_table || !sin_table) return fail(MI355X_ERR_INTERNAL, "mi355x: rope: null pointer");
    HIP_TRY(mimir::rope(x, y, rows, S, head_dim, rope_dim, interleaved, x_row_stride, x_pos_stride, y_row_stride, y_pos_stride,
                        cos_table, sin_table, offset, (hipStream_t)stream), "launch rope");
    return MI355X_OK;
}

mi355x_status mi355x_kv_write(const float* src, void* cache, int cache_dtype, int64_t B, int heads, int64_t S, int dim,
                              int64_t capacity, int64_t pos, int64_t src_b_stride, int64_t src_h_stride, int64_t src_p_stride,
                              void* stream) {
    if (cache_dtype != MI355X_F32 && cache_dtype != MI355X_F16) return fail(MI355X_ERR_DTYPE, "mi355x: KV cache of dtype %d", cache_dtype);
    // nn/transformer.go:405-411
    if (B < 0 || heads <= 0 || S < 0 || dim <= 0 || pos < 0 || pos + S > capacity)
        return fail(MI355X_ERR_SHAPE, "mi355x: write %lld positions at %lld to a cache of %lld", (long long)S, (long long)pos, (long long)capacity);
    if (B == 0 || S == 0) return MI355X_OK;
    if (!src || !cache) return fail(MI355X_ERR_INTERNAL, "mi355x: kv_write: null pointer");
    HIP_TRY(mimir::kv_write(src, cache, cache_dtype, B, heads, S, dim, capacity, pos, src_b_stride, src_h_stride, src_p_stride,
                            (hipStream_t)stream), "launch kv_write");
    return MI355X_OK;
}

mi355x_status mi355x_attention(const float* q, const int64_t* q_strides, const void* k, const int64_t* k_strides, const void* v,
                               const int64_t* v_strides, int kv_dtype, const float* mask, const int64_t* mask_strides, float* out,
                               const int64_t* out_strides, float* lse, int64_t B, int H, int HK, int64_t Q, int64_t K, int D, int DV, double scale,
                               int causal, int64_t causal_offset, void* stream) {
    if (kv_dtype != MI355X_F32 && kv_dtype != MI355X_F16) return fail(MI355X_ERR_DTYPE, "mi355x: attention over keys of dtype %d", kv_dtype);
    // backend/attention.go:36-62
    if (B < 0 || Q < 0 || K < 0 || H <= 0 || HK <= 0 || H % HK != 0 || D <= 0 || D > 256 || DV <= 0 || DV > 256)
        return fail(MI355X_ERR_SHAPE, "mi355x: attention of %d heads on %d key heads of %d features and values of %d (at most 256)", H, HK, D, DV);
    if (B == 0 || Q == 0) return MI355X_OK;
    if (B * Q > 65535 || (int64_t)HK * ((H / HK + 3) / 4) > 65535)
        return fail(MI355X_ERR_SHAPE, "mi355x: attention of %lld query rows: too many for one launch", (long long)(B * Q));
    if (!q || !out || !q_strides || !out_strides || (K > 0 && (!k || !v || !k_strides || !v_strides)) || (mask && !mask_strides))
        return fail(MI355X_ERR_INTERNAL, "mi355x: attention: null pointer");
    mimir::AttnArgs a;
    a.q = q; a.k = k; a.v = v; a.kv_dtype = kv_dtype; a.out = out; a.lse = lse;
    for (int i = 0; i < 3; i++) {
        a.q_strides[i] = q_strides[i];
        a.k_strides[i] = K > 0 ? k_strides[i] : 0;
        a.v_strides[i] = K > 0 ? v_strides[i] : 0;
        a.o_strides[i] = out_strides[i];
    }
    a.B = B; a.Q = Q; a.K = K; a.H = H; a.HK = HK; a.D = D; a.DV = DV;
    a.scale = scale; a.causal = causal; a.causal_offset = causal_offset;
    a.mask = K > 0 ? mask : nullptr;
    if (a.mask)
        for (int i = 0; i < 4; i++) a.m_strides[i] = mask_strides[i];
    if (K == 0) {  // no row sees a key: zeros and -Inf, and nothing reads k or v (which may be null)
        HIP_TRY(mimir::attention_empty(a, (hipStream_t)stream), "launch attention_empty");
        return MI355X_OK;
    }
    void* ws = nullptr;
    if (g_tune_attn != 1 && mimir::attention_decode_ok(a, K)) {  // one query position: a single launch
        int cmax;
        mimir::attention_decode_plan(B, H, HK, K, &a.nsplit, &cmax);
        if (mi355x_status st = attn_scratch(stream, mimir::attention_decode_workspace_bytes(B, H, D, a.nsplit), &ws)) return st;
        void* flags = nullptr;
        const size_t flag_bytes = mimir::attention_decode_flagged_bytes(B, H, D, a.nsplit);
        if (a.nsplit > 1)
            if (mi355x_status st = attn_flags_scratch(stream, flag_bytes, &flags)) return st;
        HIP_TRY(mimir::attention_decode(a, K, ws, nullptr, 0, (hipStream_t)stream, mimir::kAttnActQ4, flags, flag_bytes, mimir::device_error_word()), "launch attention_decode");
        return MI355X_OK;
    }
    if (mimir::attention_prompt_ok(a)) {  // many query positions: tiles of rows on the matrix cores, no scratch
        HIP_TRY(mimir::attention_prompt(a, (hipStream_t)stream), "launch attention_prompt");
        return MI355X_OK;
    }
    mimir::attention_plan(B, H, HK, Q, K, &a.chunk, &a.nsplit);
    // the scratch begins with the decode kernel's tickets
    if (mi355x_status st = attn_scratch(stream, mimir::kAttnTicketBytes + mimir::attention_workspace_bytes(B, H, Q, DV, a.nsplit), &ws)) return st;
    HIP_TRY(mimir::attention(a, (uint8_t*)ws + mimir::kAttnTicketBytes, (hipStream_t)stream), "launch attention");
    return MI355X_OK;
}

mi355x_status mi355x_attention_d(const mi355x_attention_desc* d, void* stream) {
    if (!d) return fail(MI355X_ERR_INTERNAL, "mi355x: attention_d: null descriptor");
    return mi355x_attention(d->q, d->q_strides, d->k, d->k_strides, d->v, d->v_strides, d->kv_dtype, d->mask, d->mask_strides, d->out, d->out_strides, d->lse,
                            d->B, d->H, d->HK, d->Q, d->K, d->D, d->DV, d->scale, d->causal, d->causal_offset, stream);
}

mi355x_status mi355x_swiglu(const float* gate, const float* up, float* out, int64_t rows, int64_t n, int64_t in_row_stride, void* stream) {
    if (rows < 0 || n < 0) return fail(MI355X_ERR_SHAPE, "mi355x: swiglu of [%lld, %lld]", (long long)rows, (long long)n);
    if (rows == 0 || n == 0) return MI355X_OK;
    if (!gate || !up || !out) return fail(MI355X_ERR_INTERNAL, "mi355x: swiglu: null pointer");
    HIP_TRY(mimir::swiglu(gate, up, out, rows, n, in_row_stride, (hipStream_t)stream), "launch swiglu");
    return MI355X_OK;
}

mi355x_status mi355x_add(const float* a, const float* b, float* out, int64_t n, void* stream) {
    if (n < 0) return fail(MI355X_ERR_SHAPE, "mi355x: add of %lld elements", (long long)n);
    if (n == 0) return MI355X_OK;
    if (!a || !b || !out) return fail(MI355X_ERR_INTERNAL, "mi355x: add: null pointer");
    HIP_TRY(mimir::add(a, b, out, n, (hipStream_t)stream), "launch add");
    return MI355X_OK;
}

mi355x_status mi355x_argmax(const float* logits, int64_t rows, int64_t n, int32_t* out, void* stream) {
    if (rows < 0 || n <= 0 || n > INT32_MAX || rows > 65535) return fail(MI355X_ERR_SHAPE, "mi355x: argmax of [%lld, %lld]", (long long)rows, (long long)n);
    if (rows == 0) return MI355X_OK;
    if (!logits || !out) return fail(MI355X_ERR_INTERNAL, "mi355x: argmax: null pointer");
    void* ws = nullptr;
    if (rows <= 1024)
        if (mi355x_status st = argmax_scratch(stream, mimir::argmax_workspace_bytes(1024), &ws)) return st;
    HIP_TRY(mimir::argmax(logits, rows, n, out, ws, (hipStream_t)stream), "launch argmax");
    return MI355X_OK;
}

// Frees the scratch memory the library holds for `stream` on the current device (converted activations, attention's
// and argmax's partial results and tickets, qgemm_bf16's float32 copies), blocks kept aside after growth included.
// Waits for the stream first. The caller promises that no HIP graph recorded over this library's calls on that
// stream will be replayed afterwards: such a graph points into these blocks.
mi355x_status mi355x_stream_release(void* stream) {
    DeviceState* s;
    if (mi355x_status st = current_state(&s)) return st;
    HIP_TRY(hipStreamSynchronize((hipStream_t)stream), "hipStreamSynchronize");
    std::lock_guard<std::mutex> lock(g_mu);
    auto it = s->scratch.find(stream);
    if (it == s->scratch.end()) return MI355X_OK;
    StreamScratch& m = it->second;
    hipError_t first = hipSuccess;
    for (void* p : {m.act.p, m.attn.p, m.attn_flags.p, m.gemm.p, m.argmax.p})
        if (p) { hipError_t e = hipFree(p); if (first == hipSuccess) first = e; }
    for (void* p : m.retired) { hipError_t e = hipFree(p); if (first == hipSuccess) first = e; }
    s->scratch.erase(it);
    HIP_TRY(first, "hipFree(stream scratch)");
    return MI355X_OK;
}

mi355x_status mi355x_tune(const char* key, int value) {
    static const char* keys[5] = {"q4_0.rows", "q4_0.cols", "q4_0.waves", "q4_0.no_lds", "q4_0.path"};
    for (int i = 0; i < 5; i++)
        if (key && strcmp(key, keys[i]) == 0) {
            g_tune_q4_live[i] = value;
            return MI355X_OK;
        }
    if (key && (strcmp(key, "kquant.rows") == 0 || strcmp(key, "kquant.path") == 0)) {
        mimir::set_kquant_tune(key[7] == 'p', value);
        return MI355X_OK;
    }
    if (key && strcmp(key, "qgemm.path") == 0) {
        g_tune_gemm = value;
        return MI355X_OK;
    }
    if (key && strcmp(key, "qgemm.blocks") == 0) {  // 0: the exact form always on the tile kernel; 2: always from the panel of integers; 1: by shape
        mimir::set_q4_0_blocks(value);
        return MI355X_OK;
    }
    if (key && strcmp(key, "qgemm.f16") == 0) {
        g_tune_gemm_f16 = value == 1 || value == 2 ? value : 0;
        return MI355X_OK;
    }
    if (key && strcmp(key, "q4_0.fx_pairs") == 0) {  // 0: every product of many rows on the int8 form; 2: on the binary16 form; 1: by cost
        mimir::set_q4_0_fx16(value);
        return MI355X_OK;
    }
    if (key && strcmp(key, "q4_0.fx_rows") == 0) {
        g_fx_min_rows = value > 0 ? value : 16;
        return MI355X_OK;
    }
    if (key && strcmp(key, "q4_0.rows_path") == 0) {  // 1: off; 2: its kernel without the LDS pass
        g_rows_path = value == 1 ? 1 : 0;
        mimir::set_q4_rows_direct(value == 2);
        return MI355X_OK;
    }
    if (key && strcmp(key, "q8_0.mfma") == 0) {
        mimir::set_q8_mfma(value);
        return MI355X_OK;
    }
    if (key && strcmp(key, "kquant.mfma_rows_waves") == 0) {
        mimir::set_kquant_rows_waves(value);
        return MI355X_OK;
    }
    if (key && strcmp(key, "kquant.mfma_rows") == 0) {
        mimir::set_kquant_rows(value);
        return MI355X_OK;
    }
    if (key && strcmp(key, "q4_0.rows_max") == 0) {
        g_rows_max = value > 0 ? value : 0;
        return MI355X_OK;
    }
    if (key && strcmp(key, "q4_0.rows_waves") == 0) {
        mimir::set_q4_rows_waves(value);
        return MI355X_OK;
    }
    if (key && strcmp(key, "q4_0.stream") == 0) {  // 1: the whole-chip kernel off; 3: its variant that feeds W through LDS (slower, measured) where it takes the shape
        mimir::set_q4_stream_off(value == 1);
        mimir::set_q4_dma_off(value != 3);
        return MI355X_OK;
    }
    if (key && strcmp(key, "q4_0.stream_waves") == 0) {
        mimir::set_q4_stream_waves(value);
        return MI355X_OK;
    }
    if (key && strcmp(key, "q4_0.feeders") == 0) {
        mimir::set_q4_dma_feed(value, 0);
        return MI355X_OK;
    }
    if (key && strcmp(key, "q4_0.feed_window") == 0) {
        mimir::set_q4_dma_feed(0, value);
        return MI355X_OK;
    }
    if (key && strcmp(key, "q4_0.batch_off") == 0) {
        mimir::set_q4_batch_off(value);
        return MI355X_OK;
    }
    if (key && strcmp(key, "attention.splits") == 0) {
        mimir::set_attention_decode_splits(value);
        return MI355X_OK;
    }
    if (key && strcmp(key, "attention.share") == 0) {
        mimir::set_attention_decode_share(value);
        return MI355X_OK;
    }
    if (key && strcmp(key, "attention.handover") == 0) {
        mimir::set_attention_decode_handover(value);
        return MI355X_OK;
    }
    if (key && strcmp(key, "attention.fence") == 0) {
        mimir::set_attention_decode_fence(value);
        return MI355X_OK;
    }
    if (key && strcmp(key, "attention.prompt") == 0) {  // 0: calls of many query positions on the kernel that takes a row a workgroup too
        mimir::set_attention_prompt(value);
        return MI355X_OK;
    }
    if (key && strcmp(key, "attention.path") == 0) {
        g_tune_attn = value;
        return MI355X_OK;
    }
    if (key && strcmp(key, "llama.rows") == 0) {  // 1: a batch of sequences decodes with the one-sequence kernels; 2: the batch step without its riders
        mimir::set_llama_rows_off(value);
        return MI355X_OK;
    }
    if (key && strcmp(key, "llama.step") == 0 && value >= 0 && value <= 2) {
        mimir::set_llama_step_mode(value);
        return MI355X_OK;
    }
    return fail(MI355X_ERR_INTERNAL, "mi355x: unknown tuning key %s", key ? key : "(null)");
}

// Per-launch timing of the fixed-point Q4_0 kernel: between timed_begin and
// timed_end every such launch of this thread carries its own pair of events.
mi355x_status mi355x_timed_begin(int max_launches) {
    if (max_launches <= 0 || max_launches > (1 << 20) || !t_events.empty()) return fail(MI355X_ERR_INTERNAL, "mi355x: timed_begin(%d)", max_launches);
    t_events.resize(2 * (size_t)max_launches);
    for (auto& e : t_events) HIP_TRY(hipEventCreate(&e), "hipEventCreate");
    t_events_used = 0;
    return MI355X_OK;
}

mi355x_status mi355x_timed_end(float* ms_each, int* n_launches) {
    if (!ms_each || !n_launches) return fail(MI355X_ERR_INTERNAL, "mi355x: timed_end: null pointer");
    hipError_t e = hipDeviceSynchronize();
    size_t n = t_events_used / 2;
    for (size_t i = 0; i < n && e == hipSuccess; i++) e = hipEventElapsedTime(&ms_each[i], t_events[2 * i], t_events[2 * i + 1]);
    for (auto& ev : t_events) (void)hipEventDestroy(ev);
    t_events.clear();
    t_events_used = 0;
    *n_launches = (int)n;
    HIP_TRY(e, "timed_end");
    return MI355X_OK;
}

// Where the launches of the Q4_0 product's whole-chip kernel leave five timestamps per workgroup
// (qgemv_q4_0_stream.hip), or null to stop.
mi355x_status mi355x_gemv_stamps(void* stamps) {
    HIP_TRY(mimir::set_q4_stream_stamps((long long*)stamps), "gemv_stamps");
    HIP_TRY(mimir::set_q4_dma_stamps((long long*)stamps), "gemv_stamps");
    return MI355X_OK;
}

// The kernel (name and template arguments) that the calling thread's latest Q4_0 product (one row of x, or prompt-sized) launched.
mi355x_status mi355x_last_kernel(char* buf, size_t n) {
    if (!buf || n == 0) return fail(MI355X_ERR_INTERNAL, "mi355x: last_kernel: no buffer");
    snprintf(buf, n, "%s", t_last_kernel);
    return MI355X_OK;
}

mi355x_status mi355x_stream_read(const void* p, size_t bytes, float* scratch, int grid, int threads, void* stream) {
    if (!p || !scratch || grid <= 0 || threads <= 0 || threads > 1024 || threads % 64 != 0 || ((uintptr_t)p & 15))
        return fail(MI355X_ERR_INTERNAL, "mi355x: stream_read: bad arguments");
    HIP_TRY(mimir::stream_read(p, bytes, scratch, grid, threads, (hipStream_t)stream), "launch stream_read");
    return MI355X_OK;
}

}  // extern "C"
