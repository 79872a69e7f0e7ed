"""bm_moe_decode_noalloc through the C ABI against bm_moe_decode on the same inputs, bit for bit: the quantized h
between the two launches sits in the library's static device array instead of caller-held scratch. Two calls in a row,
the second over a smaller input (fewer tokens, so the array still holds columns of the first call past the part the
second writes), for a down stack on Q8_2_X4 columns and for one on Q8_K columns (whose f32 rows of h use the array's
second part); then the limit's refusal by name. Collected last: a failure here hides no other test."""
import numpy as np
import pytest

import bloomery_amd as bm
from common import normal_f32
from test_gpu_decode import Layer, route

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("types,hidden,ff,n_experts,top_k", (
    ((bm.Q4_K, bm.Q4_K, bm.Q6_K), 2048, 768, 10, 8),
    ((bm.Q4_K, bm.Q4_K, bm.IQ4_XS), 512, 512, 4, 3),
))
def test_noalloc_matches_bm_moe_decode_on_two_calls_in_a_row(types, hidden, ff, n_experts, top_k):
    gpu = bm.Gpu(0)
    L = Layer(gpu, types, hidden, ff, n_experts, 4100 + hidden, cheap=True)
    rng = np.random.default_rng(4101)
    for m in (5, 2):   # the second call is the smaller one
        x, resid = normal_f32(rng, (m, hidden)), normal_f32(rng, (m, hidden))
        ids, wts = route(rng, m, n_experts, top_k)
        xd, sel, wd, rd = (gpu.upload(x, np.float32), gpu.upload(ids, np.uint32), gpu.upload(wts, np.float32),
                           gpu.upload(resid, np.float32))
        act_h = gpu.act(types[2], ff, m * top_k)
        h = gpu.buffer(np.float32, m * top_k * ff)
        y_ref = gpu.buffer(np.float32, m * hidden).fill_bytes(0xFF)
        y_new = gpu.buffer(np.float32, m * hidden).fill_bytes(0xFF)
        gpu.enqueue_moe_decode(L.dg, L.du, L.dd, xd, sel, wd, rd, top_k, m, act_h, y_ref, h=h)
        gpu.enqueue_moe_decode_noalloc(L.dg, L.du, L.dd, xd, sel, wd, rd, top_k, m, y_new)
        want, got = y_ref.download(), y_new.download()
        assert np.isfinite(want).all()
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), f"m = {m}: {np.count_nonzero(got != want)} values differ"
        assert gpu.fault() == (bm.FAULT_NONE, 0)
        for b in (xd, sel, wd, rd, act_h, h, y_ref, y_new):
            b.free()
    # under graph capture (where an allocation would fail the capture), replayed twice with other work between the replays
    m = 2
    x, resid = normal_f32(rng, (m, hidden)), normal_f32(rng, (m, hidden))
    ids, wts = route(rng, m, n_experts, top_k)
    xd, sel, wd, rd = (gpu.upload(x, np.float32), gpu.upload(ids, np.uint32), gpu.upload(wts, np.float32), gpu.upload(resid, np.float32))
    act_h, h = gpu.act(types[2], ff, m * top_k), gpu.buffer(np.float32, m * top_k * ff)
    y_ref, y_new = gpu.buffer(np.float32, m * hidden).fill_bytes(0xFF), gpu.buffer(np.float32, m * hidden)
    gpu.enqueue_moe_decode(L.dg, L.du, L.dd, xd, sel, wd, rd, top_k, m, act_h, y_ref, h=h)
    want = y_ref.download()
    gpu.capture_begin()
    gpu.enqueue_moe_decode_noalloc(L.dg, L.du, L.dd, xd, sel, wd, rd, top_k, m, y_new)
    graph = gpu.capture_end()
    for replay in range(2):
        y_new.fill_bytes(0xFF)
        gpu.graph_launch(graph)
        got = y_new.download()
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), f"replay {replay}"
        gpu.enqueue_moe_decode(L.dg, L.du, L.dd, xd, sel, wd, rd, top_k, m, act_h, y_ref, h=h)  # eager work between the replays
        gpu.sync()
    gpu.graph_destroy(graph)
    assert gpu.fault() == (bm.FAULT_NONE, 0)
    for b in (xd, sel, wd, rd, act_h, h, y_ref, y_new):
        b.free()
    # past the array's size: refused by name before any launch
    m = 65536 // (top_k * ff) + 1
    xd, sel, wd = gpu.upload(np.zeros((m, hidden), np.float32)), gpu.upload(np.zeros((m, top_k), np.uint32)), \
        gpu.upload(np.zeros((m, top_k), np.float32))
    y = gpu.buffer(np.float32, m * hidden)
    with pytest.raises(bm.GpuError) as e:
        gpu.enqueue_moe_decode_noalloc(L.dg, L.du, L.dd, xd, sel, wd, None, top_k, m, y)
    assert e.value.code == bm.ESHAPE and "static scratch" in str(e.value) and "bm_moe_decode_noalloc" in str(e.value)
    for b in (xd, sel, wd, y):
        b.free()
    L.free()
    gpu.close()
