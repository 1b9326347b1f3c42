//go:build linux

package mi355x

import (
	"context"
	"fmt"
	"runtime"
	"slices"

	"github.com/gsoultan/mimir/backend"
)

var _ backend.Batcher = (*Backend)(nil)

// maxBackoff bounds how long a batch whose buffers moved under a graph waits
// before it is captured again: 1<<maxBackoff repeated runs
// (backend/rocm/batch_linux.go:67-69).
const maxBackoff = 6

// batchState is what the backend keeps of a batch between runs
// (Batch.State, backend/batch.go:37-40).
type batchState struct {
	calls []batchCall
	graph *graphHandles
	// repeats counts the runs in a row with the last run's buffers, moved the
	// times the buffers moved under a graph.
	repeats, moved int
	noGraph        bool // a capture failed: the calls run one by one
	args, ptrs     []uint64
}

// batchCall is one kernel of a batch and the call it resolved to.
type batchCall struct {
	call
	k    *backend.Kernel
	args []uint64     // k's arguments in the last run (Kernel.AppendArgs)
	bufs []bufferKind // its buffers when it was planned, outputs first
	ptrs []uint64     // their device addresses in this run
}

type bufferKind struct {
	dt backend.DType
	n  int
}

type graphHandles struct{ graph, exec uintptr }

func (g *graphHandles) live() bool { return g != nil && g.exec != 0 }

func (g *graphHandles) destroy() {
	if g.exec != 0 {
		hipGraphExecDestroy(g.exec)
	}
	if g.graph != 0 {
		hipGraphDestroy(g.graph)
	}
	g.graph, g.exec = 0, 0
}

// planned reports whether the call was planned for buffers like outs and ins.
func (c *batchCall) planned(outs, ins []backend.Buffer) bool {
	if len(c.bufs) != len(outs)+len(ins) {
		return false
	}
	for j, buf := range slices.Concat(outs, ins) {
		if c.bufs[j] != (bufferKind{buf.DType(), buf.Len()}) {
			return false
		}
	}
	return true
}

// RunBatch queues the kernels of bt in order, as one HIP graph once its
// runs repeat with the same buffers and arguments.
func (b *Backend) RunBatch(ctx context.Context, bt *backend.Batch) error {
	if err := ctx.Err(); err != nil {
		return err
	}
	st, _ := bt.State.(*batchState)
	if st == nil || len(st.calls) != len(bt.Kernels) {
		st = &batchState{calls: make([]batchCall, len(bt.Kernels))}
		bt.State = st
	}
	b.mu.Lock()
	defer b.mu.Unlock()
	moved := false // a buffer, an argument or a kernel differs from the last run's: a captured graph no longer holds
	for i, k := range bt.Kernels {
		c, outs, ins := &st.calls[i], bt.Outs[i], bt.Ins[i]
		st.args = k.AppendArgs(st.args[:0])
		if c.k != k || !c.planned(outs, ins) {
			if err := backend.CheckRun(k, outs, ins); err != nil {
				return fmt.Errorf("mi355x: %w", err)
			}
			c.call = b.plan(k, outs, ins)
			c.k = k
			c.bufs = c.bufs[:0]
			for _, buf := range slices.Concat(outs, ins) {
				c.bufs = append(c.bufs, bufferKind{buf.DType(), buf.Len()})
			}
			moved = true
		}
		if !slices.Equal(c.args, st.args) {
			c.args = append(c.args[:0], st.args...)
			moved = true
		}
		var err error
		if st.ptrs, err = b.pointers(st.ptrs[:0], outs, ins); err != nil {
			return err
		}
		if !slices.Equal(st.ptrs, c.ptrs) {
			c.ptrs = append(c.ptrs[:0], st.ptrs...)
			moved = true
		}
	}
	if moved {
		st.repeats = 0
		if st.graph.live() {
			st.graph.destroy()
			st.moved++
		}
	} else {
		st.repeats++
	}
	if !st.noGraph {
		if st.graph.live() {
			return checkHIP(hipGraphLaunch(st.graph.exec, b.stream), "launch graph")
		}
		if st.repeats >= 1<<min(st.moved, maxBackoff) {
			// This run's scratch sizes are the last run's: the capture records
			// launches alone.
			if err := b.capture(ctx, bt, st); err != nil {
				st.noGraph = true
			} else {
				return checkHIP(hipGraphLaunch(st.graph.exec, b.stream), "launch graph")
			}
		}
	}
	return b.direct(ctx, bt, st)
}

// direct queues the calls one by one.
func (b *Backend) direct(ctx context.Context, bt *backend.Batch, st *batchState) error {
	for i := range st.calls {
		c := &st.calls[i]
		if c.issue == nil {
			// the embedded backend takes its own lock; ours only orders the library's calls
			if err := b.Backend.Run(ctx, c.k, bt.Outs[i], bt.Ins[i]); err != nil {
				return err
			}
			continue
		}
		if err := check(c.issue(c.ptrs), c.what); err != nil {
			return err
		}
	}
	return nil
}

// capture records the batch's calls on the stream as a HIP graph and
// instantiates it (backend/rocm/batch_linux.go:258-310). The embedded
// backend's launches on the same stream are recorded with the library's.
func (b *Backend) capture(ctx context.Context, bt *backend.Batch, st *batchState) error {
	if st.graph == nil {
		st.graph = &graphHandles{}
		runtime.AddCleanup(st, func(g *graphHandles) { g.destroy() }, st.graph)
	}
	st.graph.destroy()
	if err := checkHIP(hipStreamBeginCapture(b.stream, captureModeThreadLocal), "begin capture"); err != nil {
		return err
	}
	err := b.direct(ctx, bt, st)
	var graph uintptr
	r := hipStreamEndCapture(b.stream, &graph)
	if err == nil {
		err = checkHIP(r, "end capture")
	}
	if err == nil {
		st.graph.graph = graph
		err = checkHIP(hipGraphInstantiate(&st.graph.exec, graph, 0), "instantiate graph")
	} else if graph != 0 {
		hipGraphDestroy(graph)
	}
	if err != nil {
		st.graph.destroy()
	}
	return err
}
