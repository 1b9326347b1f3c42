// Package mi355x is a mimir backend for AMD Instinct MI355X (gfx950) that
// runs the block-quantized product and the operators around it in a decoding
// step through libmimir_mi355x.so, and everything else through the rocm
// backend it embeds.
//
// It belongs at backend/mi355x of github.com/gsoultan/mimir. The shared
// library is bound with purego, as backend/rocm binds the HIP runtime
// (backend/rocm/driver_linux.go:58-195): no cgo. Its C interface is
// include/mimir_mi355x.h of the library's repository; driver_linux.go holds
// one Go function variable per entry point it uses, with the parameter list of
// the header's declaration.
//
// This package has not been compiled: the image it was written in has no Go
// toolchain. Its table of entry points is held to the header by a test of the
// library's repository (parameter counts and kinds), nothing more.
//
// The backend shares the rocm backend's buffers and stream, so both sides see
// the same memory in the same order. That needs two accessors from
// backend/rocm, one line each beside the unexported fields they read (the
// only symbols this package uses that the reference does not export today:
// DevicePointer, Stream):
//
//	// DevicePointer returns the device address of a buffer of b.
//	func (b *Backend) DevicePointer(buf backend.Buffer) (uint64, error) { rb, err := b.own(buf); if err != nil { return 0, err }; return rb.ptr, nil }
//	// Stream returns the HIP stream b queues its work on.
//	func (b *Backend) Stream() uintptr { return b.stream }
//
// and one more block dtype in backend/backend.go and backend/quant.go for
// models whose linears stay Q4_0 (Q4_0: blocks of 32 in 18 bytes; the
// reference decodes it to float32 at load, io/mim/dtype.go:118-123).
//
// Operations taken here (the rest goes to the embedded backend unchanged):
//
//   - OpQMatMul (backend/op.go:107-115): In[0] float32 [..., K] whose leading
//     dimensions share one row stride, In[1] Q8_0, Q4_K, Q6_K or Q4_0 [N, K].
//   - OpCast of a block-quantized input read contiguously (dequantize) and
//     OpGather of rows of a block-quantized table along axis 0 (embedding
//     lookup): backend/cpu/quant.go:198-327.
//   - OpAttention (backend/op.go:117-129) with float32 queries, float32 or
//     binary16 keys and values, an optional additive mask.
//
// A Batch (backend/batch.go:22-52) keeps in its State the call each kernel
// resolved to; when a schedule repeats with the same buffers, as a decoding
// step does, the calls are captured on the stream into a HIP graph and
// replayed (backend/rocm/batch_linux.go:115-203 does the same for its
// launches). The library never allocates, frees, copies or memsets inside a
// launch once its per-stream scratch has its size, which one run before the
// capture guarantees.
package mi355x
