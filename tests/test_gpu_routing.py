"""Which kernel takes which product: the routing table of the C library, pinned for the benchmark shapes.

Results are checked elsewhere; a threshold that slips sends a shape to a slower kernel without changing a single number,
so these tests ask the library (MI_QMM_PATH_QUERY: nothing is launched) which kernel it would take.  The routes depend on
the weight's type and shape, the number of activation rows and the number of compute units (256 on MI355X) only.
"""
import numpy as np
import pytest

from npref import Q4_0, Q4_K, Q6_K, Q8_0, Q8_K
from oracle import Q5_K
from ollama_amd import qmm, synth

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = qmm.Context(0)
    yield c
    c.close()


def _upload_any(ctx, t, m, k):
    """the route depends on type and shape only: a weight of repeated rows is enough"""
    rows = min(m, 64)
    raw = synth.weights(t, rows, k, seed=3)
    return ctx.upload(t, np.tile(raw, ((m + rows - 1) // rows, 1))[:m], k, m)


# (weight type, rows, K) -> {activation rows: kernel}; the decode / prefill shapes of a Llama-3-8B layer and its head
TABLE = [
    ("q_proj", Q4_K, 4096, 4096, {1: "gemv_f32", 2: "gemv_f32", 3: "deep_f32", 4: "deep_f32", 8: "deep_f32",
                                  16: "skinny_staged", 32: "gemm_int8", 256: "gemm_int8", 512: "gemm_f16", 2048: "gemm_f16"}),
    ("k_proj", Q4_K, 1024, 4096, {1: "gemv_f32", 4: "deep_f32", 8: "deep_f32", 512: "gemm_int8"}),
    ("Q4_K 8192x4096", Q4_K, 8192, 4096, {1: "gemv_f32", 4: "deep_f32", 5: "deep_f32", 8: "deep_f32", 16: "skinny_staged"}),
    ("Q4_K 4096x8192", Q4_K, 4096, 8192, {3: "deep_f32", 5: "deep_f32", 8: "skinny_deep"}),
    ("Q4_K 20000x1024", Q4_K, 20000, 1024, {3: "deep_f32", 8: "deep_f32"}),
    ("Q4_K 40000x1024", Q4_K, 40000, 1024, {3: "skinny_direct", 8: "skinny_rows_q4k"}),
    ("ffn_gate", Q4_K, 14336, 4096, {1: "gemv_f32", 2: "deep_f32", 3: "deep_f32", 4: "deep_f32", 8: "deep_f32",
                                     16: "skinny_staged", 32: "gemm_int8", 512: "gemm_f16"}),
    ("ffn_down Q4_K", Q4_K, 4096, 14336, {1: "gemv_f32", 2: "gemv_f32", 3: "deep_f32", 4: "skinny_deep", 8: "skinny_deep",
                                          16: "skinny_staged", 512: "gemm_int8"}),
    ("ffn_down Q6_K", Q6_K, 4096, 14336, {1: "gemv_f32", 2: "gemv_f32", 3: "skinny_deep", 4: "skinny_deep", 8: "skinny_deep",
                                          16: "skinny_staged", 32: "gemm_int8", 512: "gemm_q6k"}),
    ("ffn_gate Q6_K", Q6_K, 14336, 4096, {1: "gemv_f32", 2: "gemv_f32", 3: "deep_f32", 8: "deep_f32", 16: "skinny_staged"}),
    ("v_proj Q6_K", Q6_K, 1024, 4096, {1: "gemv_f32", 2: "gemv_f32", 3: "deep_f32", 4: "deep_f32", 8: "deep_f32", 16: "skinny_staged"}),
    ("Q6_K 4096^2", Q6_K, 4096, 4096, {1: "gemv_f32", 2: "gemv_f32", 3: "deep_f32", 4: "deep_f32", 8: "deep_f32", 16: "skinny_staged"}),
    ("Q6_K 2048x8192", Q6_K, 2048, 8192, {3: "gemv", 4: "deep_f32", 5: "skinny_deep"}),
    ("Q6_K 6144x4096", Q6_K, 6144, 4096, {2: "gemv_f32", 3: "deep_f32", 4: "deep_f32", 5: "skinny_deep", 8: "deep_f32"}),
    ("70B ffn_down Q4_K", Q4_K, 8192, 28672, {1: "gemv_f32", 2: "skinny_deep", 3: "skinny_deep", 4: "skinny_deep", 5: "skinny_staged", 8: "skinny_staged"}),
    ("70B ffn_down Q6_K", Q6_K, 8192, 28672, {1: "gemv_f32", 2: "skinny_deep", 3: "skinny_deep", 4: "skinny_deep", 5: "skinny_staged"}),
    ("head", Q6_K, 128256, 4096, {1: "gemv", 2: "skinny_rows_q6k", 4: "skinny_rows_q6k", 8: "skinny_rows_q6k",
                                  16: "skinny_staged", 512: "gemm_q6k"}),
    ("Q4_0 4096^2", Q4_0, 4096, 4096, {1: "gemv_f32", 2: "gemv_f32", 4: "skinny32", 8: "skinny32", 512: "gemm_blk32"}),
    ("Q8_0 4096^2", Q8_0, 4096, 4096, {1: "gemv_f32", 2: "gemv_f32", 4: "skinny32", 8: "skinny32", 512: "gemm_blk32"}),
    ("Q8_0 long rows", Q8_0, 4096, 14336, {1: "gemv", 2: "skinny32", 3: "skinny32"}),
    # Q5_K: the blocks as they are on the streaming kernel up to six activation rows (eight on small tensors), beyond that the
    # Q4_K tensor of doubled rows that stands for it
    ("v_proj Q5_K", Q5_K, 1024, 4096, {1: "gemv_f32", 2: "gemv_f32", 3: "gemv", 4: "gemv", 8: "gemv"}),
    ("ffn_down Q5_K", Q5_K, 4096, 14336, {1: "gemv_f32", 2: "gemv_f32", 3: "gemv", 4: "gemv", 6: "gemv", 7: "skinny_staged",
                                          8: "skinny_staged"}),
    ("ffn_gate Q5_K", Q5_K, 14336, 4096, {1: "gemv_f32", 2: "gemv_f32", 4: "gemv", 6: "gemv", 7: "skinny_deep", 8: "skinny_deep"}),
]


@pytest.mark.parametrize("name,t,m,k,routes", TABLE, ids=[row[0] for row in TABLE])
def test_routes_of_the_benchmark_shapes(ctx, name, t, m, k, routes):
    if ctx.device_info()["compute_units"] != 256:
        pytest.skip("the table is the one of a 256-CU part")
    W = _upload_any(ctx, t, m, k)
    got = {n: ctx.route(W, n) for n in routes}
    W.free()
    assert got == routes, name


def test_routes_of_quantized_planes(ctx):
    """the two-phase form (quantize once, multiply several weights): the kernels on planes"""
    if ctx.device_info()["compute_units"] != 256:
        pytest.skip("the table is the one of a 256-CU part")
    W = _upload_any(ctx, Q4_K, 14336, 4096)
    for n, want in ((1, "gemv"), (2, "skinny_deep"), (3, "skinny_deep"), (8, "skinny_deep"), (16, "skinny_staged"), (512, "gemm_f16")):
        act = ctx.act_create(Q8_K, 4096, n)
        ctx.act_quantize(act, np.zeros((n, 4096), np.float32))
        assert ctx.route_q8(W, act) == want, n
        act.free()
    W.free()


def test_query_launches_nothing_and_rejects_nonsense(ctx):
    W = _upload_any(ctx, Q4_K, 64, 256)
    assert ctx.route(W, 1) == "gemv_f32"
    with pytest.raises(qmm.QmmError):
        ctx.route(W, 0)
    W.free()
