// Package hipq is a GoMLX backend that runs FusedQuantizedDense and
// QuantizedEmbeddingLookup on an AMD MI355X through libgomlx_hipq.so and
// delegates every other op to the pure-Go backend.
package hipq

/*
#cgo CFLAGS: -I${SRCDIR}/../../third_party/gomlx_hipq/include
#cgo LDFLAGS: -L${SRCDIR}/../../third_party/gomlx_hipq/lib -lgomlx_hipq -Wl,-rpath,${SRCDIR}/../../third_party/gomlx_hipq/lib
#include <stdlib.h>
#include "gomlx_hipq.h"
*/
import "C"

import (
	"fmt"
	"runtime"
	"unsafe"

	"github.com/gomlx/compute"
	"github.com/gomlx/compute/dtypes"
	"github.com/gomlx/compute/shapes"
	"github.com/pkg/errors"
)

// status turns an ABI status into a Go error.  Status 2 wraps compute.ErrNotImplemented so
// that graph.InternalFusedOpCaller falls back to the decomposed graph
// (core/graph/fused_ops.go:357-363); everything else aborts graph building (:365).
// The goroutine must stay on its OS thread between the failing call and gq_last_error().
func status(rc C.int) error {
	if rc == C.GQ_OK {
		return nil
	}
	msg := C.GoString(C.gq_last_error())
	if rc == C.GQ_ERR_NOT_IMPLEMENTED {
		return errors.Wrapf(compute.ErrNotImplemented, "hipq: %s", msg)
	}
	return errors.Errorf("hipq: %s (status %d)", msg, int(rc))
}

func call(f func() C.int) error {
	runtime.LockOSThread()
	defer runtime.UnlockOSThread()
	return status(f())
}

// ---- Backend --------------------------------------------------------------------------------

type Backend struct {
	fallback compute.Backend // pure-Go backend for every op outside the hot path
}

func New(config string) (compute.Backend, error) {
	device := 0
	if config != "" {
		if _, err := fmt.Sscanf(config, "%d", &device); err != nil {
			return nil, errors.Errorf("hipq: bad device %q", config)
		}
	}
	if err := call(func() C.int { return C.gq_init(C.int(device)) }); err != nil {
		return nil, err
	}
	fb, err := compute.NewWithConfig("go")
	if err != nil {
		return nil, err
	}
	return &Backend{fallback: fb}, nil
}

func (b *Backend) Name() string          { return "hipq" }
func (b *Backend) NumDevices() int       { return 1 }
func (b *Backend) HasSharedBuffers() bool { return false } // weights live in HBM, not in host memory

// Buffer is a device allocation plus its shape.
type Buffer struct {
	backend *Backend
	shape   shapes.Shape
	dptr    unsafe.Pointer
}

func (b *Backend) BufferFromFlatData(dev compute.DeviceNum, flat any, shape shapes.Shape) (compute.Buffer, error) {
	ptr, nbytes := flatPointer(flat) // pointer to the first element of the Go slice, length in bytes
	buf := &Buffer{backend: b, shape: shape}
	if err := call(func() C.int { return C.gq_malloc(&buf.dptr, C.size_t(nbytes)) }); err != nil {
		return nil, err
	}
	// gq_h2d returns after the copy is done: no Go pointer is retained by C.
	if err := call(func() C.int { return C.gq_h2d(buf.dptr, ptr, C.size_t(nbytes), nil) }); err != nil {
		C.gq_free(buf.dptr)
		return nil, err
	}
	return buf, nil
}

func (buf *Buffer) ToFlatData(flat any) error {
	ptr, nbytes := flatPointer(flat)
	return call(func() C.int { return C.gq_d2h(ptr, buf.dptr, C.size_t(nbytes), nil) })
}

func (buf *Buffer) Finalize() error {
	if buf.dptr == nil {
		return nil
	}
	err := call(func() C.int { return C.gq_free(buf.dptr) })
	buf.dptr = nil
	return err
}

// ---- Function: the two fused ops ----------------------------------------------------------------

// node is what Execute later runs; every other op kind is forwarded to the fallback builder.
type node struct {
	kind       opKind
	shape      shapes.Shape
	inputs     []*node
	ggmlType   C.int
	act        C.int
	k          int64
}

// FusedQuantizedDense validates at graph-build time and records the node
// (core/graph/fused_ops.go:231-232).  It launches nothing.
func (f *Function) FusedQuantizedDense(x, weights, bias compute.Value, wq *compute.Quantization,
	activation compute.ActivationType) (compute.Value, error) {
	if wq == nil {
		return nil, errors.New("hipq: FusedQuantizedDense: wq must not be nil")
	}
	if wq.Scheme != compute.QuantGGML {
		return nil, errors.Wrap(compute.ErrNotImplemented, "hipq: only the GGML scheme runs on the GPU")
	}
	xn, wn := f.node(x), f.node(weights)
	if wn.shape.DType != dtypes.Uint8 || wn.shape.Rank() != 2 {
		return nil, errors.Errorf("hipq: GGML weights must be Uint8 [N, bytesPerRow], got %s", wn.shape)
	}
	xd, ok := map[dtypes.DType]C.int{dtypes.Float32: C.GQ_F32, dtypes.BFloat16: C.GQ_BF16}[xn.shape.DType]
	if !ok {
		return nil, errors.Wrapf(compute.ErrNotImplemented, "hipq: activations of dtype %s", xn.shape.DType)
	}
	kIn := int64(xn.shape.Dimensions[xn.shape.Rank()-1])
	m := int64(xn.shape.Size()) / max(kIn, 1)
	biasLen := int64(-1)
	if bias != nil {
		biasLen = int64(f.node(bias).shape.Size())
	}
	var k C.int64_t
	err := call(func() C.int {
		return C.gq_qdense_check(C.int(wq.GGMLType.TypeID()), xd, C.int64_t(m), C.int64_t(kIn),
			C.int64_t(wn.shape.Dimensions[0]), C.int64_t(wn.shape.Dimensions[1]), C.int64_t(biasLen),
			C.int(activation), &k)
	})
	if err != nil {
		return nil, err
	}
	outDims := append([]int(nil), xn.shape.Dimensions...)
	outDims[len(outDims)-1] = wn.shape.Dimensions[0]
	n := &node{kind: opFusedQuantizedDense, shape: shapes.Make(dtypes.Float32, outDims...),
		inputs: f.nodes(x, weights, bias), ggmlType: C.int(wq.GGMLType.TypeID()), act: C.int(activation), k: int64(k)}
	return f.register(n), nil
}

// QuantizedEmbeddingLookup validates at graph-build time and records the node
// (core/graph/fused_ops.go:295-296; shapes as in ml/ggml/gather.go:21-49: table Uint8 [vocab, bytesPerRow],
// indices an integer tensor whose last dimension is 1, output Float32 [batch..., K]).
func (f *Function) QuantizedEmbeddingLookup(table, indices compute.Value, tq *compute.Quantization) (compute.Value, error) {
	if tq == nil {
		return nil, errors.New("hipq: QuantizedEmbeddingLookup: tq must not be nil")
	}
	if tq.Scheme != compute.QuantGGML {
		return nil, errors.Wrap(compute.ErrNotImplemented, "hipq: only the GGML scheme runs on the GPU")
	}
	tn, in := f.node(table), f.node(indices)
	if tn.shape.DType != dtypes.Uint8 || tn.shape.Rank() != 2 {
		return nil, errors.Errorf("hipq: GGML table must be Uint8 [vocab, bytesPerRow], got %s", tn.shape)
	}
	if in.shape.DType != dtypes.Int32 { // other integer types are converted by a node in front (fallback backend)
		return nil, errors.Wrapf(compute.ErrNotImplemented, "hipq: indices of dtype %s", in.shape.DType)
	}
	if in.shape.Rank() < 1 || in.shape.Dimensions[in.shape.Rank()-1] != 1 {
		return nil, errors.Errorf("hipq: indices must end in a dimension of 1, got %s", in.shape)
	}
	typeID := C.int(tq.GGMLType.TypeID())
	bpb, vpb := int(C.gq_bytes_per_block(typeID)), int(C.gq_values_per_block(typeID))
	if bpb == 0 {
		return nil, errors.Wrapf(compute.ErrNotImplemented, "hipq: GGML type %d", int(typeID))
	}
	if tn.shape.Dimensions[1]%bpb != 0 {
		return nil, errors.Errorf("hipq: %d bytes per row is not a whole number of %d-byte blocks", tn.shape.Dimensions[1], bpb)
	}
	k := tn.shape.Dimensions[1] / bpb * vpb
	outDims := append([]int(nil), in.shape.Dimensions[:in.shape.Rank()-1]...)
	outDims = append(outDims, k)
	n := &node{kind: opQuantizedEmbeddingLookup, shape: shapes.Make(dtypes.Float32, outDims...),
		inputs: f.nodes(table, indices), ggmlType: typeID, k: int64(k)}
	return f.register(n), nil
}

// ---- Executable.Execute: one FusedQuantizedDense node ---------------------------------------------

func (e *Executable) runQuantizedDense(n *node, x, w, bias, y *Buffer, stream unsafe.Pointer) error {
	m := int64(x.shape.Size()) / n.k
	var b *C.float
	if bias != nil {
		b = (*C.float)(bias.dptr)
	}
	return call(func() C.int {
		if x.shape.DType == dtypes.BFloat16 {
			return C.gq_qdense_bf16(n.ggmlType, (*C.uint16_t)(x.dptr), C.int64_t(m), C.int64_t(n.k), w.dptr,
				C.int64_t(w.shape.Dimensions[0]), b, n.act, (*C.float)(y.dptr), stream)
		}
		return C.gq_qdense_f32(n.ggmlType, (*C.float)(x.dptr), C.int64_t(m), C.int64_t(n.k), w.dptr,
			C.int64_t(w.shape.Dimensions[0]), b, n.act, (*C.float)(y.dptr), stream)
	})
}

// runEmbeddingLookup gathers and dequantises rows.  errFlag is a device int32 the Executable clears before the
// call and reads back with the outputs: 1 means an index was outside [0, vocab) (its row is NaN), which Execute
// reports as an error like the reference's bounds check.
func (e *Executable) runEmbeddingLookup(n *node, table, indices, out, errFlag *Buffer, stream unsafe.Pointer) error {
	count := int64(indices.shape.Size())
	return call(func() C.int {
		return C.gq_embedding_lookup(n.ggmlType, table.dptr, C.int64_t(table.shape.Dimensions[0]), C.int64_t(n.k),
			(*C.int32_t)(indices.dptr), C.int64_t(count), (*C.float)(out.dptr), (*C.int32_t)(errFlag.dptr), stream)
	})
}

func init() {
	// The registration call lives in github.com/gomlx/compute (not visible from the gomlx tree;
	// every backend self-registers from init() when blank-imported, backends/default/default.go:12-14).
	compute.Register("hipq", New)
}
