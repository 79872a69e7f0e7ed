"""Two contexts on two streams, forked and joined through events (bm_event_record / bm_event_wait, the reference's
Stream::record / Stream::wait): a shared expert's launches on one stream beside the routed experts' on the other, as one
captured graph, give the bits of the same launches in one row on one stream - on every replay."""
import numpy as np
import pytest

import bloomery_amd as bm
from common import normal_f32
from test_gpu_decode import Layer, gpu, route, stack  # noqa: F401  (gpu: module fixture)

pytestmark = pytest.mark.gpu


def test_fork_and_join_of_two_contexts_under_capture(gpu):
    types, hidden, ff, n_experts, top_k, m = (bm.IQ2_XXS, bm.IQ2_XXS, bm.IQ2_XXS), 1024, 512, 12, 4, 4
    L = Layer(gpu, types, hidden, ff, n_experts, 8100)
    rng = np.random.default_rng(8101)
    sg, su, sd = stack(bm.Q6_K, ff, hidden, 8102), stack(bm.Q6_K, ff, hidden, 8103), stack(bm.Q6_K, hidden, ff, 8104)
    dsg, dsu, dsd = gpu.weights(bm.Q6_K, ff, hidden, sg), gpu.weights(bm.Q6_K, ff, hidden, su), gpu.weights(bm.Q6_K, hidden, ff, sd)
    sets = 3
    x = normal_f32(rng, (sets * m, hidden))
    ids, wts = route(rng, sets * m, n_experts, top_k)
    xd, sel, wd = gpu.upload(x, np.float32), gpu.upload(ids, np.uint32), gpu.upload(wts, np.float32)
    zeros, ones = gpu.upload(np.zeros(m, np.uint32)), gpu.upload(np.ones(m, np.float32))
    act6, act_sh = gpu.act(bm.Q6_K, hidden, m), gpu.act(bm.Q6_K, ff, m)
    shared, routed = gpu.buffer(np.float32, m * hidden), gpu.buffer(np.float32, m * hidden)
    y_row, y_fork = gpu.buffer(np.float32, sets * m * hidden), gpu.buffer(np.float32, sets * m * hidden)
    sc = gpu.scratch(types[0], types[2], hidden, ff, n_experts, top_k, 16)
    side = bm.Gpu(0)  # a context of its own: another stream, another fault word
    forked, joined = gpu.event(), gpu.event()

    def shared_expert(ctx, s):
        ctx.enqueue_quantize(xd.ptr + 4 * s * m * hidden, m, act6)
        ctx.enqueue_gate_up(dsg, dsu, act6, zeros, m, ff, 1, None, act_sh)
        ctx.enqueue_gemv_sel(dsd, act_sh, zeros, m, hidden, shared)

    def step_in_a_row(s):
        shared_expert(gpu, s)
        gpu.enqueue_moe_forward(sc, L.dg, L.du, L.dd, xd.ptr + 4 * s * m * hidden, sel.ptr + 4 * s * m * top_k, wd.ptr + 4 * s * m * top_k,
                                None, m, routed)
        gpu.enqueue_combine_tokens(routed, ones, shared, hidden, 1, m, y_row.ptr + 4 * s * m * hidden)

    def step_forked(s):
        gpu.event_record(forked)
        side.event_wait(forked)
        shared_expert(side, s)
        side.event_record(joined)
        gpu.enqueue_moe_forward(sc, L.dg, L.du, L.dd, xd.ptr + 4 * s * m * hidden, sel.ptr + 4 * s * m * top_k, wd.ptr + 4 * s * m * top_k,
                                None, m, routed)
        gpu.event_wait(joined)
        gpu.enqueue_combine_tokens(routed, ones, shared, hidden, 1, m, y_fork.ptr + 4 * s * m * hidden)

    try:
        for s in range(sets):
            step_in_a_row(s)
        gpu.sync()
        want = y_row.download()
        assert np.isfinite(want).all()
        gpu.capture_begin()
        for s in range(sets):
            step_forked(s)
        graph = gpu.capture_end()
        for replay in range(3):
            y_fork.fill_bytes(0xFF)
            gpu.graph_launch(graph)
            gpu.sync()
            assert np.array_equal(y_fork.download().view(np.uint32), want.view(np.uint32)), f"replay {replay}"
        gpu.graph_destroy(graph)
        assert gpu.fault() == (bm.FAULT_NONE, 0) and side.fault() == (bm.FAULT_NONE, 0)
    finally:
        gpu.event_destroy(forked)
        gpu.event_destroy(joined)
        side.close()
        sc.free()
        for b in (dsg, dsu, dsd, xd, sel, wd, zeros, ones, act6, act_sh, shared, routed, y_row, y_fork):
            b.free()
        L.free()
