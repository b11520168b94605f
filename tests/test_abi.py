"""Host-side checks of the C-ABI library that need no GPU: it loads, exports every symbol that
include/mi_qmm.h declares, its size tables reproduce the reference's golden table
(/root/reference/fs/ggml/ggml_test.go:163-213), and bad arguments come back as error codes."""
import ctypes
import json
import os
import re

import pytest

from ollama_amd import qmm

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLD = json.load(open(os.path.join(ROOT, "tests", "golden", "tensor_types.json")))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "mi_qmm.h")).read()
    declared = set(re.findall(r"\b(mi_qmm_[a-z0-9_]+)\s*\(", header))
    assert declared == set(qmm.EXPORTS), declared ^ set(qmm.EXPORTS)
    L = qmm.lib()
    for name in declared:
        assert hasattr(L, name), name


def test_size_tables_match_reference_golden():
    for row in GOLD["sizes"]:
        assert qmm.block_size(row["kind"]) == row["block_size"], row
        assert qmm.type_size(row["kind"]) == row["type_size"], row
    bad = GOLD["row_not_multiple_of_block"]
    assert qmm.row_size(bad["kind"], bad["shape0"]) == -1
    assert qmm.row_size(qmm.Q4_K, 4096) == 2304 and qmm.row_size(qmm.Q6_K, 14336) == 11760
    assert qmm.row_size(qmm.Q8_K, 14336) == 16352 and qmm.row_size(qmm.Q8_0, 4096) == 4352
    assert qmm.row_size(999, 32) == -1 and qmm.block_size(999) == 0


def test_vec_dot_type():
    assert qmm.vec_dot_type(qmm.Q4_0) == qmm.Q8_0 and qmm.vec_dot_type(qmm.Q8_0) == qmm.Q8_0
    assert qmm.vec_dot_type(qmm.Q4_K) == qmm.Q8_K and qmm.vec_dot_type(qmm.Q6_K) == qmm.Q8_K
    # the unquantized weight types are multiplied in their own type
    assert [qmm.vec_dot_type(t) for t in (qmm.F32, qmm.F16, qmm.BF16)] == [qmm.F32, qmm.F16, qmm.BF16]
    assert qmm.vec_dot_type(qmm.Q5_K) == qmm.Q8_K
    assert qmm.vec_dot_type(10) == -1 and qmm.vec_dot_type(qmm.Q8_K) == -1


def test_argument_errors_without_a_device():
    L = qmm.lib()
    h = ctypes.c_void_p()
    # null handles and out-pointers are rejected before any HIP call
    assert L.mi_qmm_init(0, None) == qmm.ERR_INVALID
    assert L.mi_qmm_sync(None) == qmm.ERR_INVALID and "NULL" in qmm.last_error()
    assert L.mi_qmm_mulmat(None, None, None, 1, None, 0) == qmm.ERR_INVALID
    assert L.mi_qmm_mulmat_q8_multi(None, None, 1, None, None, 0) == qmm.ERR_INVALID and "ctx is NULL" in qmm.last_error()
    assert L.mi_qmm_mulmat_noalloc(None, None, None, 1, None) == qmm.ERR_INVALID
    assert L.mi_qmm_scratch_freeze(None, 1) == qmm.ERR_INVALID
    assert L.mi_qmm_weight_upload(None, 10, None, 256, 1, 0, ctypes.byref(h)) == qmm.ERR_UNSUPPORTED
    assert L.mi_qmm_weight_upload(None, qmm.Q4_K, None, 100, 1, 0, ctypes.byref(h)) == qmm.ERR_INVALID
    assert "multiple of the block size" in qmm.last_error()
    assert L.mi_qmm_weight_upload(None, qmm.Q4_K, None, 256, 0, 0, ctypes.byref(h)) == qmm.ERR_INVALID
    assert L.mi_qmm_quantize_act(None, 9, None, 32, 1, None, 0) == qmm.ERR_UNSUPPORTED
    assert L.mi_qmm_quantize_act(None, qmm.Q8_K, None, 100, 1, None, 0) == qmm.ERR_INVALID
    assert L.mi_qmm_quantize_weights(None, qmm.Q8_K, None, 256, 1, None, 0) == qmm.ERR_UNSUPPORTED
    assert L.mi_qmm_quantize_weights(None, qmm.Q6_K, None, 300, 1, None, 0) == qmm.ERR_INVALID
    assert L.mi_qmm_quantize_weights(None, qmm.Q4_0, None, 32, 1, None, 7) == qmm.ERR_INVALID
    L.mi_qmm_destroy(None)
    L.mi_qmm_weight_free(None)


@pytest.mark.skipif(os.path.exists("/dev/kfd"), reason="only meaningful where no GPU is present")
def test_init_fails_loudly_without_gpu():
    with pytest.raises(qmm.QmmError) as e:
        qmm.Context(0)
    assert e.value.code == qmm.ERR_NODEVICE and "no CPU path" in str(e.value)
