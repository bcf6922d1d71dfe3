//go:build linux && amd64

package cgo_bridge

// Linux / ROCm counterpart of build.go (cgo_bridge/build.go:3-6, which gets `//go:build darwin`): the C side of
// the optimizer and buffer wrappers in bridge.go is libgometal_hip.so instead of the Objective-C sources.
// The prototypes bridge.go's preamble declares for those wrappers are the ones gometal_hip.h declares, so
// bridge.go compiles unchanged against this library.
//
// Layout assumed below: third_party/gometal_hip/include/gometal_hip.h and
// third_party/gometal_hip/lib/libgometal_hip.so under the module root.

/*
#cgo CFLAGS: -I${SRCDIR}/../third_party/gometal_hip/include
#cgo LDFLAGS: -L${SRCDIR}/../third_party/gometal_hip/lib -lgometal_hip -Wl,-rpath,${SRCDIR}/../third_party/gometal_hip/lib -Wl,-rpath,/opt/rocm/lib
*/
import "C"
