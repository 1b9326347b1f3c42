// The reference's operator interface for this path, in C++: Backend, Buffer,
// Kernel, View, Attrs, CheckRun and Batch as backend/backend.go:131-180,
// backend/view.go:23-27, backend/check.go:29-74 and backend/batch.go:22-52
// declare them, with the same names, argument meaning and error kinds. It sits
// on the kernels of this library the way the reference's rocm backend sits on
// its generated ones (backend/rocm/rocm_linux.go:220-412), and takes the
// operations of the quantized path: OpQMatMul, OpCast and OpGather of a
// block-quantized input, and OpAttention. Any other operation is not this
// backend's to run and fails with ErrInternal, where a deployment would
// delegate to the general backend.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "../../include/mimir_mi355x.h"

namespace mimir {
namespace backend {

// backend/backend.go:31-54: every failure carries one of these kinds.
enum class Err : uint32_t {
    None = 0,
    OutOfMemory = MI355X_ERR_OUT_OF_MEMORY,
    Shape = MI355X_ERR_SHAPE,
    DType = MI355X_ERR_DTYPE,
    Index = MI355X_ERR_INDEX,
    Internal = MI355X_ERR_INTERNAL,
};

struct Status {
    Err kind = Err::None;
    std::string message;
    bool ok() const { return kind == Err::None; }
    static Status fail(Err kind, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
};

// backend/op.go, the operations of this path only.
enum class Op : int32_t { Cast = 1, Gather = 2, QMatMul = 3, Attention = 4 };
const char* op_name(Op op);

// backend/view.go:23-165.
struct View {
    std::vector<int64_t> shape, strides;
    int64_t offset = 0;

    static View contiguous(const std::vector<int64_t>& shape);
    int64_t size() const;
    bool is_contiguous() const;
    View permute(const std::vector<int>& perm) const;
    View expand(const std::vector<int64_t>& shape) const;
    View shrink(const std::vector<std::pair<int64_t, int64_t>>& ranges) const;
};

// backend/backend.go:184-222, the fields this path reads.
struct Attrs {
    int axis = 0;
    double scale = 0;
    bool causal = false;
    int64_t causal_offset = 0;
};

// backend/backend.go:174-180.
struct Kernel {
    Op op;
    int dtype;                   // element type of the output (MI355X_F32 ...)
    std::vector<int64_t> shape;  // shape of the contiguous output
    std::vector<View> in;        // how each input buffer is read
    Attrs attrs;
};

class Backend;

// backend/backend.go:131-134: device memory holding len elements of one dtype,
// created by and valid only with its backend.
class Buffer {
public:
    int dtype() const { return dtype_; }
    int64_t len() const { return len_; }
    size_t bytes() const;

private:
    friend class Backend;
    Backend* owner_ = nullptr;
    void* ptr_ = nullptr;  // null once freed
    int dtype_ = 0;
    int64_t len_ = 0;
};

// backend/batch.go:22-41: the kernels of one schedule with their buffers.
struct Batch {
    std::vector<const Kernel*> kernels;
    std::vector<std::vector<Buffer*>> outs, ins;
    std::shared_ptr<void> state;  // the backend's: what it resolved on an earlier run
};

// backend/check.go:29-74.
Status check_run(const Kernel& k, const std::vector<Buffer*>& outs, const std::vector<Buffer*>& ins);

// backend/backend.go:141-171 and backend/batch.go:46-52.
class Backend {
public:
    static Status open(int device, std::unique_ptr<Backend>* out);
    ~Backend();
    const char* name() const { return "mi355x"; }
    Status alloc(int dtype, int64_t n, Buffer** out);
    void free(Buffer* b);
    Status upload(Buffer* dst, const void* src, size_t bytes);
    Status download(void* dst, size_t bytes, Buffer* src);
    Status run(const Kernel& k, const std::vector<Buffer*>& outs, const std::vector<Buffer*>& ins);
    Status run_batch(Batch& b);
    Status sync();
    int64_t graph_replays() const { return graph_replays_; }

private:
    Backend() = default;
    Status own(Buffer* b, void** ptr);
    Status issue(const Kernel& k, const std::vector<Buffer*>& outs, const std::vector<Buffer*>& ins);
    Status scratch(size_t bytes, void** out);

    int device_ = 0;
    hipStream_t stream_ = nullptr;
    std::mutex mu_;
    std::vector<std::unique_ptr<Buffer>> buffers_;
    std::shared_ptr<void> arena_;  // scratch of runs outside batches, reused after every sync
    int64_t graph_replays_ = 0;
};

}  // namespace backend
}  // namespace mimir
