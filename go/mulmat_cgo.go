//go:build ignore

// NOT COMPILED in this repository: the image holds no Go toolchain.  This file is the binding a maintainer of the
// reference would add to call libmi_qmm.so for the quantized Mulmat path -- the declarations and the few lines of glue
// per call, kept beside the C header so that the two can be read together.  Every function names the entry point of
// include/mi_qmm.h it binds and the line of the reference's interface it serves.
//
// Where it would live: a backend package registered under the name the product asks for
// (ml.RegisterBackend, /root/reference/ml/backend.go:78), implementing ml.Backend / ml.Context / ml.Tensor
// (/root/reference/ml/backend.go:16, :94, :130) for the operations of this path: Mulmat (:151), MulmatID (:153),
// RMSNorm (:159) and SILU (:180) in front of them, FromFloats / Floats / Compute for the data movement.
package mi355

/*
#cgo CFLAGS: -I${SRCDIR}/../include
#cgo LDFLAGS: -L${SRCDIR}/../ollama_amd -lmi_qmm
#include <stdlib.h>
#include "mi_qmm.h"
*/
import "C"

import (
	"fmt"
	"unsafe"
)

// Backend owns one device context (mi_qmm_init / mi_qmm_destroy) and the resident weights by tensor name.
type Backend struct {
	ctx     *C.mi_qmm_ctx
	tensors map[string]*Tensor
}

// Context collects the nodes of one forward pass; Compute runs them (ml.Context, backend.go:94-128).
type Context struct {
	b     *Backend
	nodes []*Tensor
}

// Tensor is a resident quantized weight (w != nil), an input or result in host memory (data), or a pending node.
type Tensor struct {
	b     *Backend
	shape []int            // ggml order: shape[0] is the contiguous dimension
	w     *C.mi_qmm_weight // a weight uploaded with mi_qmm_weight_upload / mi_qmm_gguf_upload
	data  []float32

	opW, opX, opIDs *Tensor // pending Mulmat / MulmatID
	prod            C.int    // MI_QMM_PRODUCE_RMSNORM / _SWIGLU for a producer node
	prodSrc, prodAux *Tensor
	eps             float32
}

// check turns an error code into the panic a tensor operation of the reference raises (they have no error return).
func check(rc C.int) {
	if rc != C.MI_QMM_OK {
		panic(fmt.Sprintf("mi_qmm: %d: %s", int(rc), C.GoString(C.mi_qmm_last_error())))
	}
}

// New binds mi_qmm_init (Backend construction, backend.go:78-92; device choice ml/device.go:688-735).
func New(device int) (*Backend, error) {
	b := &Backend{tensors: map[string]*Tensor{}}
	if rc := C.mi_qmm_init(C.int(device), &b.ctx); rc != C.MI_QMM_OK {
		return nil, fmt.Errorf("mi_qmm_init: %s", C.GoString(C.mi_qmm_last_error()))
	}
	return b, nil
}

// Close binds mi_qmm_destroy (Backend.Close, backend.go:18).
func (b *Backend) Close() { C.mi_qmm_destroy(b.ctx) }

// load binds mi_qmm_weight_upload (Backend.Load, backend.go:20): kind is the fs/ggml TensorType id (2, 8, 12, 14; 13, 39; 0, 1, 30),
// raw the tensor's GGUF bytes; the library copies them before it returns, so a Go slice may be passed.
func (b *Backend) load(name string, kind uint32, k, m int, raw []byte) {
	t := &Tensor{b: b, shape: []int{k, m}}
	check(C.mi_qmm_weight_upload(b.ctx, C.int(kind), unsafe.Pointer(&raw[0]), C.int64_t(k), C.int64_t(m), C.MI_QMM_HOST, &t.w))
	b.tensors[name] = t
}

// Get serves Backend.Get (backend.go:26).
func (b *Backend) Get(name string) *Tensor { return b.tensors[name] }

// Mulmat records the node (Tensor.Mulmat, backend.go:151); Compute multiplies.
func (t *Tensor) Mulmat(ctx *Context, x *Tensor) *Tensor {
	out := &Tensor{b: t.b, shape: append([]int{t.shape[1]}, x.shape[1:]...), opW: t, opX: x}
	ctx.nodes = append(ctx.nodes, out)
	return out
}

// MulmatID records the expert-indexed node (Tensor.MulmatID, backend.go:153): t.shape = [K, M, E],
// x.shape = [K, B, T], ids.shape = [n_used, T], result [M, n_used, T].
func (t *Tensor) MulmatID(ctx *Context, x, ids *Tensor) *Tensor {
	out := &Tensor{b: t.b, shape: []int{t.shape[1], ids.shape[0], ids.shape[1]}, opW: t, opX: x, opIDs: ids}
	ctx.nodes = append(ctx.nodes, out)
	return out
}

// RMSNorm records a producer node (Tensor.RMSNorm, backend.go:159); a Mulmat that reads it alone is computed by
// mi_qmm_mulmat_produced, otherwise mi_qmm_rms_norm materializes it.
func (t *Tensor) RMSNorm(ctx *Context, w *Tensor, eps float32) *Tensor {
	out := &Tensor{b: t.b, shape: t.shape, prod: C.MI_QMM_PRODUCE_RMSNORM, prodSrc: t, prodAux: w, eps: eps}
	ctx.nodes = append(ctx.nodes, out)
	return out
}

// Compute binds mi_qmm_mulmat (Context.Compute + Tensor.Floats, backend.go:110, :140) for plain Mulmat nodes on host
// memory.  A production binding keeps activations on the device (MI_QMM_DEVICE), issues the nodes that share an x
// together (mi_qmm_mulmat_multi at up to 8 rows; mi_qmm_act_quantize once and mi_qmm_mulmat_q8_multi beyond), and
// routes MulmatID and producer nodes to mi_qmm_mulmat_id, mi_qmm_mulmat_produced, mi_qmm_mulmat_id_produced and
// mi_qmm_mulmat_swiglu: the mirrors ollama_amd/ml.py and ollama_amd/host/ml_backend.hpp carry that bookkeeping.
func (c *Context) Compute(ts ...*Tensor) {
	for _, n := range c.nodes {
		if n.data != nil || n.opW == nil || n.opIDs != nil {
			continue
		}
		k := n.opX.shape[0]
		rows := len(n.opX.data) / k
		n.data = make([]float32, rows*n.opW.shape[1])
		check(C.mi_qmm_mulmat(c.b.ctx, n.opW.w, (*C.float)(unsafe.Pointer(&n.opX.data[0])), C.int64_t(rows),
			(*C.float)(unsafe.Pointer(&n.data[0])), C.MI_QMM_HOST))
	}
}

// quantizeTensor binds mi_qmm_quantize_weights: the per-tensor step of quantize(), which the reference hands to the
// external llama-quantize (server/quantization.go:125-181, called from server/create.go:931-944).
func (b *Backend) quantizeTensor(typ uint32, rows []float32, k, m int) []byte {
	out := make([]byte, int(C.mi_qmm_row_size(C.int(typ), C.int64_t(k)))*m)
	check(C.mi_qmm_quantize_weights(b.ctx, C.int(typ), (*C.float)(unsafe.Pointer(&rows[0])), C.int64_t(k), C.int64_t(m),
		unsafe.Pointer(&out[0]), C.MI_QMM_HOST))
	return out
}
