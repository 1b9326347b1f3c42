//go:build !linux

package mi355x

import (
	"fmt"

	"github.com/gsoultan/mimir/backend"
	"github.com/gsoultan/mimir/backend/rocm"
)

// Backend is unavailable off Linux, where neither ROCm nor the library exist.
type Backend struct{ *rocm.Backend }

// New reports that the backend needs Linux.
func New(dev int) (*Backend, error) {
	return nil, fmt.Errorf("mi355x: device %d: linux only: %w", dev, backend.ErrInternal)
}
