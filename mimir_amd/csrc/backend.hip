// The reference's Backend and Batcher for the quantized path, on this library's
// kernels (see backend.h), and their C ABI (mi355x_backend_*).
#include "backend.h"

#include <cstdarg>
#include <cstdio>
#include <cstring>

#include "kernels.h"

namespace mimir {
uint32_t* device_error_word();  // capi.hip

namespace backend {

namespace {

// Scratch for a run of kernels: the same requests in the same order get the
// same memory again after rewind(), which is what a replayed graph needs.
struct Arena {
    std::vector<std::pair<void*, size_t>> blocks;
    size_t next = 0;
    ~Arena() {
        for (auto& b : blocks) (void)hipFree(b.first);
    }
    void rewind() { next = 0; }
    hipError_t get(size_t bytes, void** out) {
        if (bytes < 256) bytes = 256;
        if (next < blocks.size() && blocks[next].second >= bytes) {
            *out = blocks[next++].first;
            return hipSuccess;
        }
        void* p = nullptr;
        hipError_t e = hipMalloc(&p, bytes);
        if (e != hipSuccess) return e;
        if (next < blocks.size()) {  // too small: replace (nothing queued reads it once the stream is drained)
            (void)hipDeviceSynchronize();
            (void)hipFree(blocks[next].first);
            blocks[next] = {p, bytes};
        } else {
            blocks.push_back({p, bytes});
        }
        next++;
        *out = p;
        return hipSuccess;
    }
};

struct BatchState {
    Arena arena;
    std::vector<const void*> signature;  // kernels and buffers of the run it was built for
    hipGraphExec_t exec = nullptr;
    int runs = 0;
    ~BatchState() {
        if (exec) (void)hipGraphExecDestroy(exec);
    }
};

Status from_code(mi355x_status s, const char* what) {
    if (s == MI355X_OK) return {};
    char msg[600];
    mi355x_last_error(msg, sizeof msg);
    Err kind = s == MI355X_ERR_OUT_OF_MEMORY ? Err::OutOfMemory
               : s == MI355X_ERR_SHAPE       ? Err::Shape
               : s == MI355X_ERR_DTYPE       ? Err::DType
               : s == MI355X_ERR_INDEX       ? Err::Index
                                             : Err::Internal;
    return Status::fail(kind, "mi355x: %s: %s", what, msg);
}

Status from_hip(hipError_t e, const char* what) {
    if (e == hipSuccess) return {};
    return Status::fail(e == hipErrorOutOfMemory ? Err::OutOfMemory : Err::Internal, "mi355x: %s: %s", what, hipGetErrorName(e));
}

bool num_elements(const std::vector<int64_t>& shape, int64_t* n) {
    int64_t t = 1;
    for (int64_t d : shape) {
        if (d < 0) return false;
        if (d != 0 && t > INT64_MAX / d) return false;
        t *= d;
    }
    *n = t;
    return true;
}

std::string shape_str(const std::vector<int64_t>& s) {
    std::string out = "[";
    for (size_t i = 0; i < s.size(); i++) out += (i ? " " : "") + std::to_string(s[i]);
    return out + "]";
}

bool to_arg(const View& v, ViewArg* a) {
    if (v.shape.size() > (size_t)kMaxRank) return false;
    a->rank = (int)v.shape.size();
    for (int d = 0; d < a->rank; d++) {
        a->shape[d] = v.shape[d];
        a->strides[d] = v.strides[d];
    }
    a->offset = v.offset;
    return true;
}

// Whether the dimensions before the last `keep` are one run of equally spaced
// items (or a single item): their count and spacing.
bool leading_rows(const View& v, int keep, int64_t* count, int64_t* stride) {
    int r = (int)v.shape.size() - keep;
    int64_t n = 1, s = 0;
    bool have = false;
    for (int d = r - 1; d >= 0; d--) {
        if (v.shape[d] == 1) continue;
        if (!have) {
            s = v.strides[d];
            have = true;
        } else if (v.strides[d] != s * n) {
            return false;
        }
        n *= v.shape[d];
    }
    *count = n;
    *stride = s;
    return true;
}

}  // namespace

Status Status::fail(Err kind, const char* fmt, ...) {
    char buf[700];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    Status s;
    s.kind = kind;
    s.message = buf;
    return s;
}

const char* op_name(Op op) {
    switch (op) {
    case Op::Cast: return "cast";
    case Op::Gather: return "gather";
    case Op::QMatMul: return "qmatmul";
    case Op::Attention: return "attention";
    }
    return "op";
}

// ---- View: backend/view.go ---------------------------------------------------
View View::contiguous(const std::vector<int64_t>& shape) {
    View v;
    v.shape = shape;
    v.strides.assign(shape.size(), 0);
    int64_t s = 1;
    for (int i = (int)shape.size() - 1; i >= 0; i--) {
        v.strides[i] = s;
        s *= shape[i];
    }
    return v;
}

int64_t View::size() const {
    int64_t n = 0;
    return num_elements(shape, &n) ? n : 0;
}

bool View::is_contiguous() const {
    int64_t want = 1;
    for (int i = (int)shape.size() - 1; i >= 0; i--) {
        if (shape[i] == 1) continue;
        if (shape[i] == 0) return true;
        if (strides[i] != want) return false;
        want *= shape[i];
    }
    return true;
}

View View::permute(const std::vector<int>& perm) const {
    View out;
    out.offset = offset;
    for (int p : perm) {
        out.shape.push_back(shape[p]);
        out.strides.push_back(strides[p]);
    }
    return out;
}

View View::expand(const std::vector<int64_t>& to) const {
    View out = *this;
    out.shape = to;
    for (size_t i = 0; i < to.size(); i++)
        if (shape[i] == 1 && to[i] != 1) out.strides[i] = 0;
    return out;
}

View View::shrink(const std::vector<std::pair<int64_t, int64_t>>& ranges) const {
    View out = *this;
    for (size_t i = 0; i < ranges.size(); i++) {
        out.shape[i] = ranges[i].second - ranges[i].first;
        if (out.shape[i] > 0) out.offset += ranges[i].first * strides[i];
    }
    return out;
}

size_t Buffer::bytes() const {
    int bs = block_size(dtype_), bb = block_bytes(dtype_);
    return bs ? (size_t)(len_ / bs) * bb : 0;
}

// ---- CheckRun: backend/check.go:29-74 -------------------------------------------
Status check_run(const Kernel& k, const std::vector<Buffer*>& outs, const std::vector<Buffer*>& ins) {
    if (ins.size() != k.in.size())
        return Status::fail(Err::Internal, "%s: %zu buffers for %zu views", op_name(k.op), ins.size(), k.in.size());
    int64_t n = 0;
    if (!num_elements(k.shape, &n) || outs.size() != 1)
        return Status::fail(Err::Internal, "%s: %zu outputs for 0 stored values", op_name(k.op), outs.size());
    for (size_t i = 0; i < outs.size(); i++)
        if (!outs[i] || outs[i]->len() != n || outs[i]->dtype() != k.dtype)
            return Status::fail(Err::Internal, "%s: output %zu of dtype %d[%lld] for dtype %d%s", op_name(k.op), i, outs[i] ? outs[i]->dtype() : 0,
                                (long long)(outs[i] ? outs[i]->len() : 0), k.dtype, shape_str(k.shape).c_str());
    for (size_t i = 0; i < k.in.size(); i++) {
        const View& v = k.in[i];
        if (v.shape.size() != v.strides.size()) return Status::fail(Err::Internal, "%s: input %zu view rank mismatch", op_name(k.op), i);
        if (!ins[i]) return Status::fail(Err::Internal, "%s: input %zu is nil", op_name(k.op), i);
        int64_t lo = v.offset, hi = v.offset;
        bool empty = false;
        for (size_t d = 0; d < v.shape.size(); d++) {
            if (v.shape[d] == 0) {
                empty = true;
                break;
            }
            int64_t span = (v.shape[d] - 1) * v.strides[d];
            if (span < 0) lo += span; else hi += span;
        }
        if (!empty && (lo < 0 || hi >= ins[i]->len()))
            return Status::fail(Err::Internal, "%s: input %zu view [%lld, %lld] outside buffer of %lld", op_name(k.op), i, (long long)lo,
                                (long long)hi, (long long)ins[i]->len());
    }
    for (size_t i = 0; i < ins.size(); i++) {
        bool shared = false;
        for (Buffer* o : outs) shared = shared || o == ins[i];
        if (!shared) continue;
        // only elementwise kernels may write over an input they read whole (OpCast here)
        const View& v = k.in[i];
        bool in_place = k.op == Op::Cast;
        if (!in_place || !v.is_contiguous() || v.offset != 0 || v.shape != k.shape)
            return Status::fail(Err::Internal, "%s: input %zu is also an output", op_name(k.op), i);
    }
    return {};
}

// ---- Backend -------------------------------------------------------------------
Status Backend::open(int device, std::unique_ptr<Backend>* out) {
    if (Status s = from_code(mi355x_init(device), "init"); !s.ok()) return s;
    std::unique_ptr<Backend> b(new Backend());
    b->device_ = device;
    if (Status s = from_hip(hipStreamCreate(&b->stream_), "hipStreamCreate"); !s.ok()) return s;
    b->arena_ = std::make_shared<Arena>();
    *out = std::move(b);
    return {};
}

Backend::~Backend() {
    (void)hipSetDevice(device_);
    if (stream_) {
        (void)hipStreamSynchronize(stream_);
        (void)hipStreamDestroy(stream_);
    }
    for (auto& b : buffers_)
        if (b->ptr_) (void)hipFree(b->ptr_);
}

// rocm_linux.go:220-251.
Status Backend::alloc(int dtype, int64_t n, Buffer** out) {
    if (n < 0 || n > ((int64_t)1 << 40)) return Status::fail(Err::Shape, "mi355x: alloc %lld elements", (long long)n);
    int bs = block_size(dtype), bb = block_bytes(dtype);
    if (bb == 0) return Status::fail(Err::DType, "mi355x: alloc dtype %d", dtype);
    if (n % bs != 0) return Status::fail(Err::Shape, "mi355x: alloc %lld elements of dtype %d, in blocks of %d", (long long)n, dtype, bs);
    size_t bytes = (size_t)(n / bs) * bb;
    if (bytes < 4) bytes = 4;
    std::lock_guard<std::mutex> lock(mu_);
    (void)hipSetDevice(device_);
    void* p = nullptr;
    if (Status s = from_hip(hipMalloc(&p, bytes), "alloc"); !s.ok()) return s;
    auto b = std::make_unique<Buffer>();
    b->owner_ = this;
    b->ptr_ = p;
    b->dtype_ = dtype;
    b->len_ = n;
    *out = b.get();
    buffers_.push_back(std::move(b));
    return {};
}

// rocm_linux.go:265-273: freeing twice, or a foreign buffer, does nothing.
void Backend::free(Buffer* b) {
    if (!b || b->owner_ != this || !b->ptr_) return;
    std::lock_guard<std::mutex> lock(mu_);
    (void)hipSetDevice(device_);
    (void)hipStreamSynchronize(stream_);  // queued work that uses it runs first
    (void)hipFree(b->ptr_);
    b->ptr_ = nullptr;
}

// rocm_linux.go:275-281.
Status Backend::own(Buffer* b, void** ptr) {
    if (!b || b->owner_ != this || !b->ptr_) return Status::fail(Err::DType, "mi355x: foreign or freed buffer");
    *ptr = b->ptr_;
    return {};
}

Status Backend::upload(Buffer* dst, const void* src, size_t bytes) {
    void* p;
    if (Status s = own(dst, &p); !s.ok()) return s;
    if (bytes != dst->bytes()) return Status::fail(Err::Shape, "mi355x: upload %zu bytes into %zu-byte buffer", bytes, dst->bytes());
    std::lock_guard<std::mutex> lock(mu_);
    (void)hipSetDevice(device_);
    if (bytes == 0) return {};
    return from_code(mi355x_upload(p, src, bytes, stream_), "upload");
}

Status Backend::download(void* dst, size_t bytes, Buffer* src) {
    void* p;
    if (Status s = own(src, &p); !s.ok()) return s;
    if (bytes != src->bytes()) return Status::fail(Err::Shape, "mi355x: download %zu bytes from %zu-byte buffer", bytes, src->bytes());
    std::lock_guard<std::mutex> lock(mu_);
    (void)hipSetDevice(device_);
    if (bytes == 0) return {};
    if (Status s = from_code(mi355x_download(dst, p, bytes, stream_), "download"); !s.ok()) return s;
    return from_code(mi355x_sync(stream_), "download");
}

// rocm_linux.go:335-375: waits, then reports what kernels flagged on the device.
Status Backend::sync() {
    std::lock_guard<std::mutex> lock(mu_);
    (void)hipSetDevice(device_);
    Status s = from_code(mi355x_sync(stream_), "sync");
    static_cast<Arena*>(arena_.get())->rewind();  // nothing queued reads the scratch any more
    return s;
}

Status Backend::scratch(size_t bytes, void** out) { return from_hip(static_cast<Arena*>(arena_.get())->get(bytes, out), "scratch"); }

Status Backend::run(const Kernel& k, const std::vector<Buffer*>& outs, const std::vector<Buffer*>& ins) {
    if (Status s = check_run(k, outs, ins); !s.ok()) return s;  // rocm_linux.go:382
    std::lock_guard<std::mutex> lock(mu_);
    (void)hipSetDevice(device_);
    return issue(k, outs, ins);
}

namespace {
thread_local Arena* t_arena = nullptr;  // the running batch's scratch, if any
}

Status Backend::issue(const Kernel& k, const std::vector<Buffer*>& outs, const std::vector<Buffer*>& ins) {
    void* out;
    if (Status s = own(outs[0], &out); !s.ok()) return s;
    std::vector<void*> in(ins.size());
    for (size_t i = 0; i < ins.size(); i++)
        if (Status s = own(ins[i], &in[i]); !s.ok()) return s;
    int64_t n_out = 0;
    num_elements(k.shape, &n_out);
    auto temp = [&](size_t bytes, void** p) -> Status {
        if (t_arena) return from_hip(t_arena->get(bytes, p), "scratch");
        return scratch(bytes, p);
    };

    switch (k.op) {
    case Op::QMatMul: {
        // runQMatMul's checks (backend/cpu/qmatmul.go:318-332)
        if (k.in.size() != 2) return Status::fail(Err::Internal, "qmatmul: %zu inputs", k.in.size());
        const View &vx = k.in[0], &vw = k.in[1];
        const int r = (int)vx.shape.size(), wdt = ins[1]->dtype();
        if (!is_quantized(wdt) || ins[0]->dtype() != MI355X_F32) return Status::fail(Err::DType, "qmatmul: x of dtype %d by weights of dtype %d", ins[0]->dtype(), wdt);
        if (k.dtype != MI355X_F32 || r == 0 || vw.shape.size() != 2 || (int)k.shape.size() != r)
            return Status::fail(Err::Internal, "product of %s by dtype %d%s", shape_str(vx.shape).c_str(), wdt, shape_str(vw.shape).c_str());
        const int64_t N = vw.shape[0], K = vw.shape[1], bs = block_size(wdt);
        bool lead = true;
        for (int d = 0; d < r - 1; d++) lead = lead && k.shape[d] == vx.shape[d];
        if (vx.shape[r - 1] != K || k.shape[r - 1] != N || !lead || K % bs != 0 || !vw.is_contiguous() || vw.offset % bs != 0)
            return Status::fail(Err::Internal, "product of %s by dtype %d%s into %s", shape_str(vx.shape).c_str(), wdt, shape_str(vw.shape).c_str(),
                                shape_str(k.shape).c_str());
        if (n_out == 0) return {};
        const int64_t M = n_out / N;
        const uint8_t* W = (const uint8_t*)in[1] + (vw.offset / bs) * block_bytes(wdt);
        const float* x = (const float*)in[0] + vx.offset;
        int64_t rows = 0, stride = 0;
        bool direct = (K <= 1 || vx.strides[r - 1] == 1) && leading_rows(vx, 1, &rows, &stride) && (rows == 1 || stride >= K);
        if (!direct) {  // any other view: its elements gathered into rows first (OpContiguous)
            ViewArg va;
            if (!to_arg(vx, &va)) return Status::fail(Err::Internal, "qmatmul: x of rank %d", r);
            void* tmp;
            if (Status s = temp((size_t)M * K * 4, &tmp); !s.ok()) return s;
            if (Status s = from_hip(copy_view32(in[0], va, M * K, tmp, stream_), "contiguous"); !s.ok()) return s;
            x = (const float*)tmp;
            stride = K;
        }
        if (M == 1) stride = K;
        return from_code(mi355x_qgemv(wdt, W, x, (float*)out, M, N, K, stride, stream_), "qmatmul");
    }
    case Op::Cast: {
        if (k.in.size() != 1) return Status::fail(Err::Internal, "cast: %zu inputs", k.in.size());
        const int dt = ins[0]->dtype();
        if (!is_quantized(dt)) return Status::fail(Err::Internal, "cast of dtype %d: only block-quantized inputs are on this path", dt);
        if (k.dtype != MI355X_F32 && k.dtype != MI355X_F16 && k.dtype != MI355X_BF16) return Status::fail(Err::DType, "dequantize into dtype %d", k.dtype);
        if (k.in[0].shape != k.shape) return Status::fail(Err::Internal, "cast of %s into %s", shape_str(k.in[0].shape).c_str(), shape_str(k.shape).c_str());
        if (k.in[0].is_contiguous()) return from_code(mi355x_dequant(dt, in[0], k.in[0].offset, n_out, out, k.dtype, stream_), "dequantize");
        ViewArg va;
        if (!to_arg(k.in[0], &va)) return Status::fail(Err::Internal, "cast: rank %zu", k.in[0].shape.size());
        return from_hip(dequantize_view(dt, in[0], va, n_out, out, k.dtype, stream_), "dequantize");
    }
    case Op::Gather: {
        if (k.in.size() != 2) return Status::fail(Err::Internal, "gather: %zu inputs", k.in.size());
        const int dt = ins[0]->dtype();
        const View &vt = k.in[0], &vi = k.in[1];
        if (!is_quantized(dt)) return Status::fail(Err::Internal, "gather from dtype %d: only block-quantized tables are on this path", dt);
        if (ins[1]->dtype() != MI355X_I32 || k.dtype != MI355X_F32) return Status::fail(Err::DType, "gather by dtype %d into dtype %d", ins[1]->dtype(), k.dtype);
        const int r = (int)vt.shape.size(), axis = k.attrs.axis;
        if (vi.shape != k.shape || (int)vi.shape.size() != r || axis < 0 || axis >= r)
            return Status::fail(Err::Internal, "gather of %s by %s on axis %d into %s", shape_str(vt.shape).c_str(), shape_str(vi.shape).c_str(), axis,
                                shape_str(k.shape).c_str());
        for (int d = 0; d < r; d++)
            if (d != axis && vi.shape[d] > vt.shape[d])
                return Status::fail(Err::Internal, "gather of %s by %s on axis %d", shape_str(vt.shape).c_str(), shape_str(vi.shape).c_str(), axis);
        if (n_out == 0) return {};
        // an embedding's lookup: whole rows of a contiguous table, one index a row
        if (r == 2 && axis == 0 && vt.is_contiguous() && vt.offset == 0 && vi.shape[1] == vt.shape[1] && vi.strides[1] == 0 &&
            (vi.strides[0] == 1 || vi.shape[0] == 1))
            return from_code(mi355x_gather_rows(dt, in[0], vt.shape[0], vt.shape[1], (const int32_t*)in[1] + vi.offset, vi.shape[0], (float*)out, stream_),
                             "gather");
        ViewArg ta, ia;
        if (!to_arg(vt, &ta) || !to_arg(vi, &ia)) return Status::fail(Err::Internal, "gather: rank %d", r);
        return from_hip(gather_view(dt, in[0], ta, (const int32_t*)in[1], ia, axis, n_out, (float*)out, device_error_word(), stream_), "gather");
    }
    case Op::Attention: {
        // NewAttentionShape (backend/attention.go:36-62)
        if (k.in.size() != 3 && k.in.size() != 4) return Status::fail(Err::Internal, "attention: %zu inputs", k.in.size());
        const bool masked = k.in.size() == 4;
        const View &vq = k.in[0], &vk = k.in[1], &vv = k.in[2];
        const int r = (int)vq.shape.size();
        bool ok = r >= 3 && (int)vk.shape.size() == r && (int)vv.shape.size() == r;
        for (int d = 0; ok && d < r - 3; d++) ok = vq.shape[d] == vk.shape[d];
        for (int d = 0; ok && d < r - 1; d++) ok = vk.shape[d] == vv.shape[d];
        if (!ok) return Status::fail(Err::Shape, "attention of queries %s, keys %s, values %s", shape_str(vq.shape).c_str(), shape_str(vk.shape).c_str(),
                                     shape_str(vv.shape).c_str());
        const int64_t H = vq.shape[r - 3], HK = vk.shape[r - 3], Q = vq.shape[r - 2], Kn = vk.shape[r - 2], D = vq.shape[r - 1], DV = vv.shape[r - 1];
        if (vk.shape[r - 1] != D || HK < 1 || H % HK != 0)
            return Status::fail(Err::Shape, "attention of queries %s, keys %s, values %s", shape_str(vq.shape).c_str(), shape_str(vk.shape).c_str(),
                                shape_str(vv.shape).c_str());
        if (masked) {  // [B..., H, Q, K] (backend/attention.go:53-55)
            const View& vm = k.in[3];
            bool mok = (int)vm.shape.size() == r && vm.shape[r - 3] == H && vm.shape[r - 2] == Q && vm.shape[r - 1] == Kn;
            for (int d = 0; mok && d < r - 3; d++) mok = vm.shape[d] == vq.shape[d];
            if (!mok) return Status::fail(Err::Shape, "attention of queries %s, keys %s and mask %s", shape_str(vq.shape).c_str(), shape_str(vk.shape).c_str(),
                                          shape_str(vm.shape).c_str());
            if (ins[3]->dtype() != MI355X_F32) return Status::fail(Err::DType, "attention with a mask of dtype %d", ins[3]->dtype());
        }
        if (ins[0]->dtype() != MI355X_F32 || k.dtype != MI355X_F32 || ins[1]->dtype() != ins[2]->dtype() ||
            (ins[1]->dtype() != MI355X_F32 && ins[1]->dtype() != MI355X_F16))
            return Status::fail(Err::DType, "attention of dtype %d over keys of dtype %d", ins[0]->dtype(), ins[1]->dtype());
        int64_t B = 0, qb = 0, kb = 0, vb = 0, mb = 0, B2 = 0, B3 = 0, B4 = 0;
        if (!leading_rows(vq, 3, &B, &qb) || !leading_rows(vk, 3, &B2, &kb) || !leading_rows(vv, 3, &B3, &vb) ||
            (masked && !leading_rows(k.in[3], 3, &B4, &mb)) ||
            (D > 1 && (vq.strides[r - 1] != 1 || vk.strides[r - 1] != 1)) || (DV > 1 && vv.strides[r - 1] != 1))
            return Status::fail(Err::Internal, "attention: views of this layout are not on this path");
        if (n_out != B * H * Q * (DV + 1)) return Status::fail(Err::Internal, "attention into %s", shape_str(k.shape).c_str());
        if (n_out == 0) return {};
        int64_t qs[3] = {qb, vq.strides[r - 3], vq.strides[r - 2]}, ks[3] = {kb, vk.strides[r - 3], vk.strides[r - 2]};
        int64_t vs[3] = {vb, vv.strides[r - 3], vv.strides[r - 2]};
        int64_t os[3] = {H * Q * DV, Q * DV, DV}, ms[4] = {0, 0, 0, 0};
        const float* mask = nullptr;
        if (masked) {
            const View& vm = k.in[3];
            ms[0] = mb; ms[1] = vm.strides[r - 3]; ms[2] = vm.strides[r - 2]; ms[3] = vm.strides[r - 1];
            mask = (const float*)in[3] + vm.offset;
        }
        const size_t esz = ins[1]->dtype() == MI355X_F16 ? 2 : 4;
        float* o = (float*)out;
        return from_code(mi355x_attention((const float*)in[0] + vq.offset, qs, (const uint8_t*)in[1] + vk.offset * esz, ks,
                                          (const uint8_t*)in[2] + vv.offset * esz, vs, ins[1]->dtype(), mask, ms, o, os, o + B * H * Q * DV, B, (int)H,
                                          (int)HK, Q, Kn, (int)D, (int)DV, k.attrs.scale, k.attrs.causal ? 1 : 0, k.attrs.causal_offset, stream_),
                         "attention");
    }
    }
    return Status::fail(Err::Internal, "mi355x: operation %d is not on this path", (int)k.op);
}

// rocm/batch_linux.go:115-203: a schedule that repeats with the same kernels and
// buffers is recorded into a graph on its second run and replayed from then on.
Status Backend::run_batch(Batch& b) {
    if (b.outs.size() != b.kernels.size() || b.ins.size() != b.kernels.size())
        return Status::fail(Err::Internal, "mi355x: batch of %zu kernels with %zu and %zu buffer lists", b.kernels.size(), b.outs.size(), b.ins.size());
    std::vector<const void*> sig;
    for (size_t i = 0; i < b.kernels.size(); i++) {
        if (Status s = check_run(*b.kernels[i], b.outs[i], b.ins[i]); !s.ok()) return s;
        sig.push_back(b.kernels[i]);
        for (Buffer* o : b.outs[i]) sig.push_back(o->ptr_);
        for (Buffer* in : b.ins[i]) sig.push_back(in->ptr_);
    }
    std::lock_guard<std::mutex> lock(mu_);
    (void)hipSetDevice(device_);
    auto st = std::static_pointer_cast<BatchState>(b.state);
    if (!st || st->signature != sig) {
        st = std::make_shared<BatchState>();
        st->signature = sig;
        b.state = st;
    }
    auto issue_all = [&]() -> Status {
        st->arena.rewind();
        t_arena = &st->arena;
        Status s;
        for (size_t i = 0; i < b.kernels.size() && s.ok(); i++) s = issue(*b.kernels[i], b.outs[i], b.ins[i]);
        t_arena = nullptr;
        return s;
    };
    st->runs++;
    if (st->exec) {
        graph_replays_++;
        return from_hip(hipGraphLaunch(st->exec, stream_), "graph launch");
    }
    if (st->runs < 2) return issue_all();  // the first run also grows the library's own scratch to size
    hipGraph_t g = nullptr;
    if (Status s = from_hip(hipStreamBeginCapture(stream_, hipStreamCaptureModeThreadLocal), "begin capture"); !s.ok()) return s;
    Status s = issue_all();
    hipError_t e = hipStreamEndCapture(stream_, &g);
    if (s.ok()) s = from_hip(e, "end capture");
    if (s.ok()) s = from_hip(hipGraphInstantiate(&st->exec, g, nullptr, nullptr, 0), "instantiate graph");
    if (g) (void)hipGraphDestroy(g);
    if (!s.ok()) return s;
    graph_replays_++;
    return from_hip(hipGraphLaunch(st->exec, stream_), "graph launch");
}

}  // namespace backend
}  // namespace mimir

// ---- C ABI ----------------------------------------------------------------------
using mimir::backend::Backend;
using mimir::backend::Buffer;
using mimir::backend::Status;

namespace {

thread_local std::string t_backend_error;

mi355x_status done(const Status& s) {
    if (s.ok()) return MI355X_OK;
    t_backend_error = s.message;
    return (mi355x_status)s.kind;
}

mimir::backend::Kernel to_kernel(const mi355x_kernel* k) {
    mimir::backend::Kernel out;
    out.op = (mimir::backend::Op)k->op;
    out.dtype = k->dtype;
    out.shape.assign(k->shape, k->shape + k->rank);
    for (int i = 0; i < k->n_in; i++) {
        mimir::backend::View v;
        v.shape.assign(k->in[i].shape, k->in[i].shape + k->in[i].rank);
        v.strides.assign(k->in[i].strides, k->in[i].strides + k->in[i].rank);
        v.offset = k->in[i].offset;
        out.in.push_back(v);
    }
    out.attrs.axis = k->axis;
    out.attrs.scale = k->scale;
    out.attrs.causal = k->causal != 0;
    out.attrs.causal_offset = k->causal_offset;
    return out;
}

bool kernel_ok(const mi355x_kernel* k) {
    if (!k || k->rank < 0 || k->rank > MI355X_MAX_RANK || k->n_in < 0 || k->n_in > MI355X_MAX_INPUTS) return false;
    for (int i = 0; i < k->n_in; i++)
        if (k->in[i].rank < 0 || k->in[i].rank > MI355X_MAX_RANK) return false;
    return true;
}

struct BatchHandle {
    std::vector<mimir::backend::Kernel> kernels;
    mimir::backend::Batch batch;
};

}  // namespace

extern "C" {

size_t mi355x_backend_last_error(char* buf, size_t n) {
    if (buf && n) {
        size_t c = t_backend_error.size() < n - 1 ? t_backend_error.size() : n - 1;
        memcpy(buf, t_backend_error.data(), c);
        buf[c] = 0;
    }
    return t_backend_error.size();
}

mi355x_status mi355x_backend_open(int device, void** backend) {
    if (!backend) return done(Status::fail(mimir::backend::Err::Internal, "mi355x: backend_open: null pointer"));
    std::unique_ptr<Backend> b;
    Status s = Backend::open(device, &b);
    if (s.ok()) *backend = b.release();
    return done(s);
}

mi355x_status mi355x_backend_close(void* backend) {
    delete (Backend*)backend;
    return MI355X_OK;
}

mi355x_status mi355x_backend_alloc(void* backend, int dtype, int64_t n, void** buffer) {
    if (!backend || !buffer) return done(Status::fail(mimir::backend::Err::Internal, "mi355x: backend_alloc: null pointer"));
    Buffer* b = nullptr;
    Status s = ((Backend*)backend)->alloc(dtype, n, &b);
    if (s.ok()) *buffer = b;
    return done(s);
}

mi355x_status mi355x_backend_free(void* backend, void* buffer) {
    if (backend) ((Backend*)backend)->free((Buffer*)buffer);
    return MI355X_OK;
}

mi355x_status mi355x_backend_upload(void* backend, void* dst, const void* src, size_t bytes) {
    if (!backend) return done(Status::fail(mimir::backend::Err::Internal, "mi355x: backend_upload: null pointer"));
    return done(((Backend*)backend)->upload((Buffer*)dst, src, bytes));
}

mi355x_status mi355x_backend_download(void* backend, void* dst, size_t bytes, void* src) {
    if (!backend) return done(Status::fail(mimir::backend::Err::Internal, "mi355x: backend_download: null pointer"));
    return done(((Backend*)backend)->download(dst, bytes, (Buffer*)src));
}

mi355x_status mi355x_backend_sync(void* backend) {
    if (!backend) return done(Status::fail(mimir::backend::Err::Internal, "mi355x: backend_sync: null pointer"));
    return done(((Backend*)backend)->sync());
}

mi355x_status mi355x_backend_run(void* backend, const mi355x_kernel* k, void* const* outs, int n_outs, void* const* ins, int n_ins) {
    if (!backend || !kernel_ok(k) || n_outs < 0 || n_ins < 0 || (n_outs && !outs) || (n_ins && !ins))
        return done(Status::fail(mimir::backend::Err::Internal, "mi355x: backend_run: bad arguments"));
    std::vector<Buffer*> o((Buffer* const*)outs, (Buffer* const*)outs + n_outs), i((Buffer* const*)ins, (Buffer* const*)ins + n_ins);
    return done(((Backend*)backend)->run(to_kernel(k), o, i));
}

mi355x_status mi355x_batch_new(const mi355x_kernel* kernels, int n, void* const* const* outs, const int* n_outs, void* const* const* ins,
                               const int* n_ins, void** batch) {
    if (!batch || n < 0 || (n && (!kernels || !outs || !n_outs || !ins || !n_ins)))
        return done(Status::fail(mimir::backend::Err::Internal, "mi355x: batch_new: bad arguments"));
    auto h = std::make_unique<BatchHandle>();
    h->kernels.reserve(n);
    for (int i = 0; i < n; i++) {
        if (!kernel_ok(&kernels[i])) return done(Status::fail(mimir::backend::Err::Internal, "mi355x: batch_new: kernel %d", i));
        h->kernels.push_back(to_kernel(&kernels[i]));
        h->batch.outs.emplace_back((Buffer* const*)outs[i], (Buffer* const*)outs[i] + n_outs[i]);
        h->batch.ins.emplace_back((Buffer* const*)ins[i], (Buffer* const*)ins[i] + n_ins[i]);
    }
    for (auto& k : h->kernels) h->batch.kernels.push_back(&k);
    *batch = h.release();
    return MI355X_OK;
}

mi355x_status mi355x_batch_free(void* batch) {
    delete (BatchHandle*)batch;
    return MI355X_OK;
}

mi355x_status mi355x_backend_run_batch(void* backend, void* batch) {
    if (!backend || !batch) return done(Status::fail(mimir::backend::Err::Internal, "mi355x: run_batch: null pointer"));
    return done(((Backend*)backend)->run_batch(((BatchHandle*)batch)->batch));
}

int64_t mi355x_backend_graph_replays(void* backend) { return backend ? ((Backend*)backend)->graph_replays() : -1; }

}  // extern "C"
