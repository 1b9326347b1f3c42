//go:build linux

package mi355x

import (
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
	miAttention  func(q uint64, qStrides *int64, k uint64, kStrides *int64, v uint64, vStrides *int64, kvDType int32,
		mask uint64, maskStrides *int64, out uint64, outStrides *int64, lse uint64,
		b int64, h, hk int32, nq, nk int64, d, dv int32, scale float64, causal int32, causalOffset int64, stream uintptr) status
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

// symbol is a function pointer to bind and the name of its symbol.
type symbol struct {
	fptr any
	name string
}

// libraries returns the names to try for a library: the one the environment
// variable env names, if it is set, otherwise names.
func libraries(env string, names ...string) []string {
	if path := os.Getenv(env); path != "" {
		return []string{path}
	}
	return names
}

// open loads the first of names the dynamic loader finds.
func open(names []string) (uintptr, error) {
	var err error
	for _, name := range names {
		var lib uintptr
		if lib, err = purego.Dlopen(name, purego.RTLD_GLOBAL|purego.RTLD_NOW); err == nil {
			return lib, nil
		}
	}
	return 0, fmt.Errorf("none of %s loads: %w", strings.Join(names, ", "), err)
}

// register binds each function pointer to the symbol of lib it names, or
// reports the first that is missing.
func register(lib uintptr, fns []symbol) error {
	for _, f := range fns {
		sym, err := purego.Dlsym(lib, f.name)
		if err != nil {
			return err
		}
		purego.RegisterFunc(f.fptr, sym)
	}
	return nil
}

// load loads the library and the HIP graph API once.
func load() error {
	libOnce.Do(func() {
		lib, err := open(libraries("MIMIR_MI355X_LIB", "libmimir_mi355x.so"))
		if err != nil {
			libErr = err
			return
		}
		if libErr = register(lib, []symbol{
			{&miInit, "mi355x_init"},
			{&miLastError, "mi355x_last_error"},
			{&miSync, "mi355x_sync"},
			{&miQGemv, "mi355x_qgemv"},
			{&miQGemmBF16, "mi355x_qgemm_bf16"},
			{&miDequant, "mi355x_dequant"},
			{&miGatherRows, "mi355x_gather_rows"},
			{&miAttention, "mi355x_attention"},
			{&miTune, "mi355x_tune"},
		}); libErr != nil {
			return
		}
		hip, err := open(libraries("MIMIR_HIP", "libamdhip64.so.7", "libamdhip64.so.6", "libamdhip64.so"))
		if err != nil {
			libErr = err
			return
		}
		libErr = register(hip, []symbol{
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
