//go:build linux

package mi355x

import (
	"errors"
	"fmt"
	"os"
	"strings"
	"sync"
	"unsafe"

	"github.com/ebitengine/purego"

	"github.com/gsoultan/mimir/backend"
)

// status is an mi355x_status: 0 on success, a hipError_t below 0x1000, or one
// of the library's own codes.
type status uint32

const (
	statusOK          status = 0
	statusOutOfMemory status = 2 // hipErrorOutOfMemory
	statusShape       status = 0x1001
	statusDType       status = 0x1002
	statusIndex       status = 0x1003
	statusInternal    status = 0x1005
)

// DType codes of the library (mimir_mi355x.h): the reference's enum
// (backend/backend.go:72-92) with Q4_0 behind it.
const (
	codeF32  int32 = 1
	codeI32  int32 = 2
	codeBF16 int32 = 3
	codeF16  int32 = 4
	codeQ8_0 int32 = 5
	codeQ4_K int32 = 6
	codeQ6_K int32 = 7
	codeQ4_0 int32 = 8
)

// Loaded functions of libmimir_mi355x.so, named and typed as in
// mimir_mi355x.h. Device addresses are uint64, as the rocm backend keeps
// them; a stream is the uintptr of a hipStream_t.
var (
	libOnce sync.Once
	libErr  error

	miInit       func(device int32) status
	miLastError  func(buf *byte, n uintptr) uintptr
	miSync       func(stream uintptr) status
	miQGemv      func(dtype int32, w, x, y uint64, m, n, k, xRowStride int64, stream uintptr) status
	miQGemmBF16  func(dtype int32, w, x, y uint64, m, n, k, xRowStride int64, outDType int32, stream uintptr) status
	miDequant    func(dtype int32, w uint64, first, n int64, out uint64, outDType int32, stream uintptr) status
	miGatherRows func(dtype int32, table uint64, rows, k int64, idx uint64, n int64, out uint64, stream uintptr) status
	miAttention  func(desc *attentionDesc, stream uintptr) status
	miStreamFree func(stream uintptr) status
	miTune func(key string, value int32) status
)

// HIP graph functions, loaded from the runtime the rocm backend has loaded.
var (
	hipStreamBeginCapture func(stream uintptr, mode int32) uint32
	hipStreamEndCapture   func(stream uintptr, graph *uintptr) uint32
	hipGraphInstantiate   func(exec *uintptr, graph uintptr, flags uint64) uint32
	hipGraphLaunch        func(exec uintptr, stream uintptr) uint32
	hipGraphExecDestroy   func(exec uintptr) uint32
	hipGraphDestroy       func(graph uintptr) uint32
)

const captureModeThreadLocal = 1 // hipStreamCaptureModeThreadLocal

// attentionDesc is mi355x_attention_desc, field for field: six device addresses, the strides of queries, keys,
// values and result ({batch, head, position}) and of the mask ({batch, head, query, key}), the sizes, the scale and
// the 32-bit fields. One pointer to it keeps the call within what purego.RegisterFunc takes as parameters.
type attentionDesc struct {
	q, k, v, mask, out, lse                              uint64
	qStrides, kStrides, vStrides, outStrides             [3]int64
	maskStrides                                          [4]int64
	b, nq, nk, causalOffset                              int64
	scale                                                float64
	kvDType, heads, kvHeads, d, dv, causal               int32
}

// binding is one row of a table that load fills in: where the function goes and what the library calls it.
type binding struct {
	target any
	symbol string
}

// dlopenFirst opens the library a host names in the environment variable override, or else the first of
// candidates that the dynamic loader can open, and says why each one failed when none does.
func dlopenFirst(override string, candidates ...string) (uintptr, error) {
	if forced, ok := os.LookupEnv(override); ok && forced != "" {
		candidates = []string{forced}
	}
	var why []string
	for _, path := range candidates {
		handle, err := purego.Dlopen(path, purego.RTLD_NOW|purego.RTLD_GLOBAL)
		if err == nil {
			return handle, nil
		}
		why = append(why, path+": "+err.Error())
	}
	return 0, errors.New("no library could be opened (" + strings.Join(why, "; ") + ")")
}

// bindAll resolves every row of table in handle. All rows are tried, so that the error names every symbol the
// library lacks at once (a library older than this package shows up as such a list).
func bindAll(handle uintptr, table []binding) error {
	var absent []string
	for _, row := range table {
		addr, err := purego.Dlsym(handle, row.symbol)
		if err != nil {
			absent = append(absent, row.symbol)
			continue
		}
		purego.RegisterFunc(row.target, addr)
	}
	if len(absent) != 0 {
		return fmt.Errorf("symbols not found: %s", strings.Join(absent, ", "))
	}
	return nil
}

// load loads the library and the HIP graph API once.
func load() error {
	libOnce.Do(func() {
		lib, err := dlopenFirst("MIMIR_MI355X_LIB", "libmimir_mi355x.so")
		if err != nil {
			libErr = err
			return
		}
		if libErr = bindAll(lib, []binding{
			{&miInit, "mi355x_init"},
			{&miLastError, "mi355x_last_error"},
			{&miSync, "mi355x_sync"},
			{&miQGemv, "mi355x_qgemv"},
			{&miQGemmBF16, "mi355x_qgemm_bf16"},
			{&miDequant, "mi355x_dequant"},
			{&miGatherRows, "mi355x_gather_rows"},
			{&miAttention, "mi355x_attention_d"},
			{&miStreamFree, "mi355x_stream_release"},
			{&miTune, "mi355x_tune"},
		}); libErr != nil {
			return
		}
		hip, err := dlopenFirst("MIMIR_HIP", "libamdhip64.so.7", "libamdhip64.so.6", "libamdhip64.so")
		if err != nil {
			libErr = err
			return
		}
		libErr = bindAll(hip, []binding{
			{&hipStreamBeginCapture, "hipStreamBeginCapture"},
			{&hipStreamEndCapture, "hipStreamEndCapture"},
			{&hipGraphInstantiate, "hipGraphInstantiateWithFlags"},
			{&hipGraphLaunch, "hipGraphLaunch"},
			{&hipGraphExecDestroy, "hipGraphExecDestroy"},
			{&hipGraphDestroy, "hipGraphDestroy"},
		})
	})
	return libErr
}

// lastError returns the calling thread's last message of the library.
func lastError() string {
	var buf [512]byte
	n := miLastError(&buf[0], uintptr(len(buf)))
	if n > uintptr(len(buf)) {
		n = uintptr(len(buf))
	}
	return strings.TrimRight(string(buf[:n]), "\x00")
}

// check turns a status into one of mimir's errors, as
// backend/rocm/rocm_linux.go:194-203 turns a hipError.
func check(s status, what string) error {
	switch s {
	case statusOK:
		return nil
	case statusOutOfMemory:
		return fmt.Errorf("mi355x: %s: %w", what, backend.ErrOutOfMemory)
	case statusShape:
		return fmt.Errorf("mi355x: %s: %s: %w", what, lastError(), backend.ErrShape)
	case statusDType:
		return fmt.Errorf("mi355x: %s: %s: %w", what, lastError(), backend.ErrDType)
	case statusIndex:
		return fmt.Errorf("mi355x: %s: %s: %w", what, lastError(), backend.ErrIndex)
	}
	return fmt.Errorf("mi355x: %s: %s (status %#x): %w", what, lastError(), uint32(s), backend.ErrInternal)
}

// checkHIP turns a hipError_t of the graph API into an error.
func checkHIP(r uint32, what string) error {
	if r == 0 {
		return nil
	}
	return fmt.Errorf("mi355x: %s: hip error %d: %w", what, r, backend.ErrInternal)
}

var _ = unsafe.Pointer(nil)
