//go:build linux

package mi355x

import (
	"context"
	"fmt"
	"slices"
	"sync"

	"github.com/gsoultan/mimir/backend"
	"github.com/gsoultan/mimir/backend/rocm"
)

// Q4_0 is the block dtype this backend adds to the reference's enum: the
// value after Q6_K, as the library numbers it. A mimir that keeps Q4_0
// tensors as blocks declares it in backend/backend.go.
const Q4_0 = backend.Q6_K + 1

// Backend runs the hot operators through the library and the rest through
// the rocm backend it embeds.
type Backend struct {
	*rocm.Backend
	stream uintptr

	mu sync.Mutex // serializes the library's calls, which share the stream's scratch
}

var _ backend.Backend = (*Backend)(nil)

// New returns the backend of the first ROCm device, the one rocm.New opens
// (backend/rocm/rocm_linux.go:86-97).
func New() (*Backend, error) {
	if err := load(); err != nil {
		return nil, fmt.Errorf("mi355x: %w", err)
	}
	rb, err := rocm.New()
	if err != nil {
		return nil, err
	}
	if err := check(miInit(0), "init"); err != nil {
		return nil, err
	}
	return &Backend{Backend: rb, stream: rb.Stream()}, nil
}

// Close gives back the scratch memory the library keeps for this backend's stream; graphs recorded
// over it (a Batch's State) must not be replayed afterwards.
func (b *Backend) Close() error {
	b.mu.Lock()
	defer b.mu.Unlock()
	return check(miStreamFree(b.stream), "release stream scratch")
}

// Name identifies the device.
func (b *Backend) Name() string { return "mi355x" }

// Sync waits for the stream and reports what the kernels of either side left
// in their error words (a gather index out of range is ErrIndex).
func (b *Backend) Sync(ctx context.Context) error {
	if err := b.Backend.Sync(ctx); err != nil {
		return err
	}
	return check(miSync(b.stream), "sync")
}

// code returns the library's code of a dtype.
func code(dt backend.DType) (int32, bool) {
	switch dt {
	case backend.Float32:
		return codeF32, true
	case backend.Int32:
		return codeI32, true
	case backend.BFloat16:
		return codeBF16, true
	case backend.Float16:
		return codeF16, true
	case backend.Q8_0:
		return codeQ8_0, true
	case backend.Q4_K:
		return codeQ4_K, true
	case backend.Q6_K:
		return codeQ6_K, true
	case Q4_0:
		return codeQ4_0, true
	}
	return 0, false
}

// quantized reports whether dt is a block dtype.
func quantized(dt backend.DType) bool { return dt.Size() == 0 && dt != backend.Invalid }

// call is one operator resolved to an entry point of the library: issue
// queues it over the device addresses of the kernel's buffers, outputs
// first. A nil issue means the embedded backend runs the kernel.
type call struct {
	issue func(ptrs []uint64) status
	what  string
}

// rowsOf returns how many rows of k elements v holds and their stride, if
// its leading dimensions collapse into rows one stride apart and its last
// dimension is contiguous.
func rowsOf(v backend.View, k int) (rows, stride int, ok bool) {
	r := len(v.Shape)
	if r == 0 || v.Shape[r-1] != k || (k > 1 && v.Strides[r-1] != 1) {
		return 0, 0, false
	}
	rows, stride = 1, k
	first := true
	for i := r - 2; i >= 0; i-- {
		if v.Shape[i] == 1 {
			continue
		}
		if first {
			stride, first = v.Strides[i], false
		} else if v.Strides[i] != stride*rows {
			return 0, 0, false
		}
		rows *= v.Shape[i]
	}
	if stride < k {
		return 0, 0, false // overlapping or broadcast rows: the general kernel reads them
	}
	return rows, stride, true
}

// plan resolves k over buffers of the dtypes of outs and ins. The result
// depends on the kernel, the dtypes and the lengths alone, so a Batch keeps
// it between runs.
func (b *Backend) plan(k *backend.Kernel, outs, ins []backend.Buffer) call {
	stream := b.stream
	switch k.Op {
	case backend.OpQMatMul: // In[0] float32 [..., K], In[1] block-quantized [N, K] (backend/op.go:107-115)
		x, w := k.In[0], k.In[1]
		wc, ok := code(ins[1].DType())
		if !ok || !quantized(ins[1].DType()) || ins[0].DType() != backend.Float32 || len(w.Shape) != 2 {
			break
		}
		n, kk := w.Shape[0], w.Shape[1]
		rows, stride, ok := rowsOf(x, kk)
		// W from a block boundary, rows one after another (backend/cpu/qmatmul.go:323-332)
		if !ok || w.Strides[1] != 1 || w.Strides[0] != kk || w.Offset%ins[1].DType().BlockSize() != 0 {
			break
		}
		wbytes, _ := ins[1].DType().Bytes(w.Offset) // whole blocks: the offset was just checked
		woff := uint64(wbytes)
		xoff := 4 * uint64(x.Offset)
		return call{what: "qmatmul", issue: func(p []uint64) status {
			return miQGemv(wc, p[2]+woff, p[1]+xoff, p[0], int64(rows), int64(n), int64(kk), int64(stride), stream)
		}}
	case backend.OpCast: // a block-quantized In[0] read contiguously dequantizes (backend/cpu/quant.go:198-256)
		src := k.In[0]
		sc, ok := code(ins[0].DType())
		oc, ok2 := code(k.DType)
		if !ok || !ok2 || !quantized(ins[0].DType()) || !k.DType.IsFloat() || !slices.Equal(src.Strides, backend.ContiguousStrides(src.Shape)) {
			break
		}
		n, _ := backend.NumElements(k.Shape)
		first := int64(src.Offset)
		return call{what: "dequantize", issue: func(p []uint64) status {
			return miDequant(sc, p[1], first, int64(n), p[0], oc, stream)
		}}
	case backend.OpGather: // rows of a block-quantized table (backend/cpu/quant.go:296-327)
		table, idx := k.In[0], k.In[1]
		tc, ok := code(ins[0].DType())
		if !ok || !quantized(ins[0].DType()) || k.Attrs.Axis != 0 || len(table.Shape) != 2 || k.DType != backend.Float32 ||
			table.Offset != 0 || !slices.Equal(table.Strides, backend.ContiguousStrides(table.Shape)) ||
			ins[1].DType() != backend.Int32 || len(idx.Shape) != 2 || idx.Strides[1] != 0 || idx.Shape[1] != table.Shape[1] {
			break // an index per element rather than per row: the general kernel
		}
		rows, kk, n := table.Shape[0], table.Shape[1], idx.Shape[0]
		ioff := 4 * uint64(idx.Offset)
		istride := idx.Strides[0]
		if istride != 1 && n > 1 {
			break
		}
		return call{what: "gather", issue: func(p []uint64) status {
			return miGatherRows(tc, p[1], int64(rows), int64(kk), p[2]+ioff, int64(n), p[0], stream)
		}}
	case backend.OpAttention: // backend/op.go:117-129
		if c, ok := b.planAttention(k, ins); ok {
			return c
		}
	}
	return call{}
}

// planAttention resolves an OpAttention whose leading dimensions collapse
// into one batch stride per input.
func (b *Backend) planAttention(k *backend.Kernel, ins []backend.Buffer) (call, bool) {
	var maskShape []int
	if len(k.In) == 4 {
		maskShape = k.In[3].Shape
	}
	s, err := backend.NewAttentionShape(k.In[0].Shape, k.In[1].Shape, k.In[2].Shape, maskShape)
	if err != nil || ins[0].DType() != backend.Float32 || k.DType != backend.Float32 || ins[1].DType() != ins[2].DType() ||
		(ins[1].DType() != backend.Float32 && ins[1].DType() != backend.Float16) || s.D > 256 || s.DV > 256 {
		return call{}, false
	}
	kv, _ := code(ins[1].DType())
	// The leading dimensions as one batch stride, then the strides of the last `keep` dimensions but the features'.
	strides := func(v backend.View, keep int, features bool) ([]int64, bool) {
		r := len(v.Shape)
		if features && v.Shape[r-1] > 1 && v.Strides[r-1] != 1 {
			return nil, false
		}
		lead := r - keep
		if features {
			lead--
		}
		batch, n := 0, 1
		for i := lead - 1; i >= 0; i-- { // row-major among themselves, whatever follows them
			if v.Shape[i] == 1 {
				continue
			}
			if n == 1 {
				batch = v.Strides[i]
			} else if v.Strides[i] != batch*n {
				return nil, false
			}
			n *= v.Shape[i]
		}
		out := []int64{int64(batch)}
		for i := lead; i < lead+keep; i++ {
			out = append(out, int64(v.Strides[i]))
		}
		return out, true
	}
	qs, ok1 := strides(k.In[0], 2, true) // {batch, head, position}
	ks, ok2 := strides(k.In[1], 2, true)
	vs, ok3 := strides(k.In[2], 2, true)
	if !ok1 || !ok2 || !ok3 {
		return call{}, false
	}
	var ms []int64
	if maskShape != nil {
		var ok bool
		if ms, ok = strides(k.In[3], 3, false); !ok || ins[3].DType() != backend.Float32 { // {batch, head, query, key}
			return call{}, false
		}
	}
	bsz := int64(s.Batches())
	os := []int64{int64(s.Heads * s.Q * s.DV), int64(s.Q * s.DV), int64(s.DV)}
	lseOff := 4 * uint64(s.Batches()*s.Heads*s.Q*s.DV) // the logsumexp follows the result in the output
	offs := [4]uint64{4 * uint64(k.In[0].Offset), uint64(ins[1].DType().Size() * k.In[1].Offset), uint64(ins[2].DType().Size() * k.In[2].Offset), 0}
	if maskShape != nil {
		offs[3] = 4 * uint64(k.In[3].Offset)
	}
	causal := int32(0)
	if k.Attrs.Causal {
		causal = 1
	}
	scale, coff, stream := k.Attrs.Scale, int64(k.Attrs.CausalOffset), b.stream
	desc := attentionDesc{b: bsz, nq: int64(s.Q), nk: int64(s.K), causalOffset: coff, scale: scale, kvDType: kv,
		heads: int32(s.Heads), kvHeads: int32(s.KVHeads), d: int32(s.D), dv: int32(s.DV), causal: causal}
	copy(desc.qStrides[:], qs)
	copy(desc.kStrides[:], ks)
	copy(desc.vStrides[:], vs)
	copy(desc.outStrides[:], os)
	copy(desc.maskStrides[:], ms)
	return call{what: "attention", issue: func(p []uint64) status {
		d := desc // the descriptor of this issue: the same shape, this run's buffers
		d.q, d.k, d.v, d.out, d.lse = p[1]+offs[0], p[2]+offs[1], p[3]+offs[2], p[0], p[0]+lseOff
		if ms != nil {
			d.mask = p[4] + offs[3]
		}
		return miAttention(&d, stream)
	}}, true
}

// pointers appends the device addresses of outs, then ins, to dst.
func (b *Backend) pointers(dst []uint64, outs, ins []backend.Buffer) ([]uint64, error) {
	for _, buf := range slices.Concat(outs, ins) {
		p, err := b.Backend.DevicePointer(buf)
		if err != nil {
			return nil, err
		}
		dst = append(dst, p)
	}
	return dst, nil
}

// Run queues k on the stream.
func (b *Backend) Run(ctx context.Context, k *backend.Kernel, outs []backend.Buffer, ins []backend.Buffer) error {
	if err := ctx.Err(); err != nil {
		return err
	}
	if err := backend.CheckRun(k, outs, ins); err != nil { // backend/check.go:29-74
		return fmt.Errorf("mi355x: %w", err)
	}
	c := b.plan(k, outs, ins)
	if c.issue == nil {
		return b.Backend.Run(ctx, k, outs, ins)
	}
	ptrs, err := b.pointers(nil, outs, ins)
	if err != nil {
		return err
	}
	b.mu.Lock()
	defer b.mu.Unlock()
	return check(c.issue(ptrs), c.what)
}
