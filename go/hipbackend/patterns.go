// Sub-graphs around a projection that the Executable replaces by one ABI call at Compile(): RMSNorm + projection,
// projection + residual, and the gated feed-forward product (ml/zoo/transformer/transformer.go:1099-1101, 1045, 1055,
// 1276-1294).  The reference has no fused op for these; they arrive as separate nodes and are matched by pattern.
package hipq

/*
#include "gomlx_hipq.h"
*/
import "C"

import "unsafe"

// pattern: Mul(act(FusedQuantizedDense(xn, Wg, bg)), FusedQuantizedDense(xn, Wu, bu)), xn = RMSNorm(x) or x
func (e *Executable) runGatedFeedForward(n *node, x, gain, wg, bg, wu, bu, y *Buffer, stream unsafe.Pointer) error {
	var norm *C.gq_rmsnorm
	if n.hasNorm {
		norm = &C.gq_rmsnorm{dGain: (*C.float)(ptrOrNil(gain)), eps: C.float(n.eps), gain_offset: C.float(n.scaleOffset)}
	}
	m := int64(x.shape.Size()) / n.k
	return call(func() C.int {
		return C.gq_qdense_gated_f32(n.ggmlType, (*C.float)(x.dptr), C.int64_t(m), C.int64_t(n.k), norm,
			wg.dptr, (*C.float)(ptrOrNil(bg)), wu.dptr, (*C.float)(ptrOrNil(bu)),
			C.int64_t(wg.shape.Dimensions[0]), n.act, (*C.float)(y.dptr), stream)
	})
}

// pattern: Add(residual, FusedQuantizedDense(RMSNorm(x) or x, W, b)); y may be the residual's buffer when it is donated
func (e *Executable) runDenseBlock(n *node, x, gain, w, b, residual, y *Buffer, stream unsafe.Pointer) error {
	var norm *C.gq_rmsnorm
	if n.hasNorm {
		norm = &C.gq_rmsnorm{dGain: (*C.float)(ptrOrNil(gain)), eps: C.float(n.eps), gain_offset: C.float(n.scaleOffset)}
	}
	m := int64(x.shape.Size()) / n.k
	return call(func() C.int {
		return C.gq_qdense_block_f32(n.ggmlType, (*C.float)(x.dptr), C.int64_t(m), C.int64_t(n.k), norm,
			w.dptr, C.int64_t(w.shape.Dimensions[0]), (*C.float)(ptrOrNil(b)), n.act,
			(*C.float)(ptrOrNil(residual)), (*C.float)(y.dptr), stream)
	})
}

// pattern: several FusedQuantizedDense nodes that read one RMSNorm(x) (the q / k / v projections of a layer): one submission
func (e *Executable) runNormBatch(n *node, x, gain *Buffer, ws, bs, ys []*Buffer, stream unsafe.Pointer) error {
	norm := C.gq_rmsnorm{dGain: (*C.float)(ptrOrNil(gain)), eps: C.float(n.eps), gain_offset: C.float(n.scaleOffset)}
	m := int64(x.shape.Size()) / n.k
	descs := make([]C.gq_dense_desc, len(ws))
	for i := range ws {
		descs[i] = C.gq_dense_desc{
			_type: n.ggmlType, act: C.GQ_ACT_NONE, dX: (*C.float)(x.dptr), M: C.int64_t(m), K: C.int64_t(n.k),
			dW: ws[i].dptr, N: C.int64_t(ws[i].shape.Dimensions[0]), dBias: (*C.float)(ptrOrNil(bs[i])), dY: (*C.float)(ys[i].dptr),
		}
	}
	return call(func() C.int {
		return C.gq_qdense_norm_f32_batch(C.int(len(descs)), &descs[0], &norm, stream)
	})
}

// ptrOrNil is the device pointer of an optional operand (bias, gain, residual).
func ptrOrNil(b *Buffer) unsafe.Pointer {
	if b == nil {
		return nil
	}
	return b.dptr
}
