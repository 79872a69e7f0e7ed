"""GPU parity tests of bm_moe_forward, the one entry for any number of tokens: each of its three paths (per slot, grouped
by expert, the grouped GEMM) gives the oracle's layer output bit for bit on the same seeded inputs, so the choice among
them by batch size changes no bit; the automatic choice follows the crossovers; ids that name no expert add nothing."""
import numpy as np
import pytest

import bloomery_amd as bm
import ora
from common import normal_f32
from test_gpu_decode import Layer, assert_f32, gpu, route  # noqa: F401  (gpu: module fixture)

pytestmark = pytest.mark.gpu

PATHS = ((bm.PATH_PER_SLOT, "per slot"), (bm.PATH_GROUPED, "grouped"), (bm.PATH_GEMM, "gemm"))


@pytest.mark.parametrize("types,hidden,ff,n_experts,top_k,m", (
    ((bm.Q4_K, bm.Q4_K, bm.Q6_K), 2048, 768, 12, 8, 19),     # the headline layer's rows
    ((bm.Q5_K, bm.Q5_K, bm.Q4_K), 512, 512, 5, 3, 40),
    ((bm.IQ2_XXS, bm.IQ2_XXS, bm.IQ2_XXS), 1024, 512, 6, 4, 9),  # Q8_K columns on both sides
    ((bm.Q4_K, bm.Q4_K, bm.IQ2_XXS), 512, 768, 4, 2, 33),    # the two column forms in one layer
    ((bm.IQ4_XS, bm.IQ4_XS, bm.Q3_K), 512, 512, 5, 3, 25),   # the added types through the GEMM path as well
    ((bm.IQ3_XXS, bm.IQ3_XXS, bm.Q6_K), 768, 256, 4, 2, 18),
    ((bm.IQ2_XXS, bm.IQ2_XXS, bm.IQ2_XXS), 512, 512, 40, 4, 6),  # no more slots than experts, Q8_K columns on both sides: the
    ((bm.IQ4_XS, bm.IQ4_XS, bm.Q3_K), 512, 256, 64, 3, 7),       # grouped path's per-slot gate . up launch and slot-ordered down tiles
))
def test_every_path_gives_the_oracles_bits(gpu, types, hidden, ff, n_experts, top_k, m):
    L = Layer(gpu, types, hidden, ff, n_experts, 5100 + hidden)
    rng = np.random.default_rng(5101)
    x, resid = normal_f32(rng, (m, hidden)), normal_f32(rng, (m, hidden))
    ids, wts = route(rng, m, n_experts, top_k)
    want_y, _ = L.oracle(x, ids, wts, top_k)
    want = (want_y.reshape(m, hidden) + resid).astype(np.float32).reshape(-1)
    xd, sel, wd, rd = gpu.upload(x, np.float32), gpu.upload(ids, np.uint32), gpu.upload(wts, np.float32), gpu.upload(resid, np.float32)
    y = gpu.buffer(np.float32, m * hidden)
    sc = gpu.scratch(types[0], types[2], hidden, ff, n_experts, top_k, 64)
    gpu.fault_clear()
    try:
        for path, name in PATHS:
            sc.set_path(path)
            assert sc.path_for(m) == path
            for rep in range(2):  # the scratch is reused as it stands
                y.fill_bytes(0xFF)
                gpu.enqueue_moe_forward(sc, L.dg, L.du, L.dd, xd, sel, wd, rd, m, y)
                assert_f32(y.download(), want, f"{name}, call {rep}")
            # fewer tokens after more, over the same scratch
            y.fill_bytes(0xFF)
            gpu.enqueue_moe_forward(sc, L.dg, L.du, L.dd, xd, sel, wd, rd, 3, y)
            assert_f32(y.download()[:3 * hidden], want[:3 * hidden], f"{name}, three tokens")
        assert gpu.fault() == (bm.FAULT_NONE, 0)
    finally:
        sc.free()
        for b in (xd, sel, wd, rd, y):
            b.free()
        L.free()


def test_the_automatic_choice_follows_the_crossovers(gpu):
    sc = gpu.scratch(bm.Q4_K, bm.Q6_K, 2048, 768, 128, 8, 4096)
    try:
        assert [sc.path_for(m) for m in (1, 21, 22, 447, 448, 4096)] == [bm.PATH_PER_SLOT, bm.PATH_PER_SLOT, bm.PATH_GROUPED,
                                                                       bm.PATH_GROUPED, bm.PATH_GEMM, bm.PATH_GEMM]
        gpu.set_gemm_mode(bm.GEMM_FAST)  # the tolerance mode's GEMM is faster: its cut comes earlier
        try:
            assert [sc.path_for(m) for m in (21, 22, 95, 96)] == [bm.PATH_PER_SLOT, bm.PATH_GROUPED, bm.PATH_GROUPED, bm.PATH_GEMM]
        finally:
            gpu.set_gemm_mode(bm.GEMM_EXACT)
        sc.set_path(bm.PATH_AUTO, 4, 2000)
        assert [sc.path_for(m) for m in (3, 4, 1999, 2000)] == [bm.PATH_PER_SLOT, bm.PATH_GROUPED, bm.PATH_GROUPED, bm.PATH_GEMM]
        sc.set_path(bm.PATH_PER_SLOT)
        assert sc.path_for(1024) == bm.PATH_PER_SLOT and sc.path_for(1025) == bm.PATH_GROUPED  # past the fused step's token limit
        assert sc.path_for(0) == bm.ESHAPE and sc.path_for(4097) == bm.ESHAPE
        with pytest.raises(bm.GpuError) as e:
            sc.set_path(7)
        assert "bm_scratch_set_path" in str(e.value)
    finally:
        sc.free()
    # a shape whose slot columns do not fit the per-slot step's LDS (64 slots of ff 2048) goes grouped from the first token
    sc = gpu.scratch(bm.Q4_K, bm.Q6_K, 512, 2048, 4, 64, 8)
    try:
        assert [sc.path_for(m) for m in (1, 8)] == [bm.PATH_GROUPED, bm.PATH_GROUPED]
        sc.set_path(bm.PATH_PER_SLOT)
        assert sc.path_for(1) == bm.PATH_GROUPED
    finally:
        sc.free()
    # every type has a grouped GEMM: the same cut for a layer of the added types
    sc = gpu.scratch(bm.IQ4_XS, bm.Q3_K, 512, 256, 4, 2, 512)
    try:
        # (a gate/up stack on Q8_K columns: the exact GEMM is ahead from 96 tokens)
        assert [sc.path_for(m) for m in (21, 95, 96, 500)] == [bm.PATH_PER_SLOT, bm.PATH_GROUPED, bm.PATH_GEMM, bm.PATH_GEMM]
        sc.set_path(bm.PATH_GEMM)
        assert sc.path_for(3) == bm.PATH_GEMM
    finally:
        sc.free()
    for call, word in ((lambda: gpu.scratch(bm.Q4_K, bm.Q6_K, 2048, 768, 128, 8, 5121), "40960"),
                       (lambda: gpu.scratch(bm.Q4_K, bm.Q6_K, 2000, 768, 128, 8, 16), "256"),
                       (lambda: gpu.scratch(bm.Q4_K, 99, 2048, 768, 128, 8, 16), "type")):
        with pytest.raises(bm.GpuError) as e:
            call()
        assert word in str(e.value) and "bm_scratch_create" in str(e.value)


def test_a_slot_without_an_expert_on_the_grouped_path_of_few_slots(gpu):
    """The grouped path with no more slots than experts and Q8_K columns on both sides (the per-slot gate . up launch, the
    slot-aware quantizer of h, the down tiles reading their columns in slot order): a host-served slot and an id past the stack
    add nothing, the sums over the live slots are the oracle's, only the id past the stack raises; the scratch is poisoned first so
    that a stale row of h would show."""
    hidden, ff, n_experts, top_k, m = 512, 256, 16, 3, 3
    L = Layer(gpu, (bm.IQ2_XXS, bm.IQ2_XXS, bm.IQ4_XS), hidden, ff, n_experts, 5300)
    rng = np.random.default_rng(5301)
    x = normal_f32(rng, (m, hidden))
    wts = np.array([[0.5, 0.3, 0.2], [0.2, 0.5, 0.3], [0.1, 0.6, 0.3]], np.float32)
    xd, wd = gpu.upload(x, np.float32), gpu.upload(wts, np.float32)
    y = gpu.buffer(np.float32, m * hidden)
    sc = gpu.scratch(bm.IQ2_XXS, bm.IQ4_XS, hidden, ff, n_experts, top_k, 4)
    sc.set_path(bm.PATH_GROUPED)
    try:
        for ids, live, raises in ((np.array([[1, bm.HOST_SLOT, 3], [bm.HOST_SLOT, 0, bm.HOST_SLOT], [0, 2, 15]], np.uint32),
                                   ([(1, 0.5), (3, 0.2)], [(0, 0.5)], [(0, 0.1), (2, 0.6), (15, 0.3)]), False),
                                  (np.array([[1, 99, 3], [2, 0, 1], [0, 16, 2]], np.uint32),
                                   ([(1, 0.5), (3, 0.2)], [(2, 0.2), (0, 0.5), (1, 0.3)], [(0, 0.1), (2, 0.3)]), True)):
            want = np.concatenate([L.oracle(x[t:t + 1], np.array([[e for e, _ in live[t]]], np.uint32),
                                            np.array([[w for _, w in live[t]]], np.float32), len(live[t]))[0] for t in range(m)])
            sel = gpu.upload(ids, np.uint32)
            gpu.fault_clear()
            for rep in range(2):
                y.fill_bytes(0xFF)
                gpu.enqueue_moe_forward(sc, L.dg, L.du, L.dd, xd, sel, wd, None, m, y)
                assert_f32(y.download(), want, f"call {rep}")
            if raises:
                assert gpu.fault()[1] & (1 << bm.SITE_EXPERT_ID)
            else:
                assert gpu.fault() == (bm.FAULT_NONE, 0)
            sel.free()
        gpu.fault_clear()
    finally:
        sc.free()
        for b in (xd, wd, y):
            b.free()
        L.free()


def test_a_slot_without_an_expert_adds_nothing_on_every_path(gpu):
    """A host-served slot and an id past the stack: the token's sum is the oracle's over its live slots on each path, and
    the id past the stack raises ExpertId. With host-served slots only, no path raises anything (the GEMM path's route table
    does not list them and its SwiGLU quantizer leaves their columns alone, crates/gpu/src/gemm/swiglu.rs:96-140)."""
    L = Layer(gpu, (bm.Q4_K, bm.Q4_K, bm.Q6_K), 512, 256, 4, 5200)
    rng = np.random.default_rng(5201)
    m, top_k = 3, 3
    x = normal_f32(rng, (m, 512))
    ids = np.array([[1, bm.HOST_SLOT, 3], [2, 0, 1], [0, 9, 2]], np.uint32)
    wts = np.array([[0.5, 0.3, 0.2], [0.2, 0.5, 0.3], [0.1, 0.6, 0.3]], np.float32)
    want = np.concatenate([L.oracle(x[:1], np.array([[1, 3]], np.uint32), np.array([[0.5, 0.2]], np.float32), 2)[0],
                           L.oracle(x[1:2], ids[1:2], wts[1:2], 3)[0],
                           L.oracle(x[2:], np.array([[0, 2]], np.uint32), np.array([[0.1, 0.3]], np.float32), 2)[0]])
    xd, sel, wd = gpu.upload(x, np.float32), gpu.upload(ids, np.uint32), gpu.upload(wts, np.float32)
    y = gpu.buffer(np.float32, m * 512)
    sc = gpu.scratch(bm.Q4_K, bm.Q6_K, 512, 256, 4, top_k, 8)
    try:
        for path, name in PATHS:
            sc.set_path(path)
            gpu.fault_clear()
            y.fill_bytes(0xFF)
            gpu.enqueue_moe_forward(sc, L.dg, L.du, L.dd, xd, sel, wd, None, m, y)
            assert_f32(y.download(), want, name)
            assert gpu.fault()[1] & (1 << bm.SITE_EXPERT_ID)  # (the refused slot's NaN rows may raise the quantizer's site too)
        gpu.fault_clear()
        # host-served slots only: the same sums over the live slots, and no fault on any path
        ids_h = np.array([[1, bm.HOST_SLOT, 3], [bm.HOST_SLOT, 0, bm.HOST_SLOT], [0, 2, 1]], np.uint32)
        want_h = np.concatenate([L.oracle(x[:1], np.array([[1, 3]], np.uint32), np.array([[0.5, 0.2]], np.float32), 2)[0],
                                 L.oracle(x[1:2], np.array([[0]], np.uint32), np.array([[0.5]], np.float32), 1)[0],
                                 L.oracle(x[2:], ids_h[2:], wts[2:], 3)[0]])
        sel_h = gpu.upload(ids_h, np.uint32)
        for path, name in PATHS:
            sc.set_path(path)
            y.fill_bytes(0xFF)
            gpu.enqueue_moe_forward(sc, L.dg, L.du, L.dd, xd, sel_h, wd, None, m, y)
            assert_f32(y.download(), want_h, name + ", host-served slots")
            assert gpu.fault() == (bm.FAULT_NONE, 0), name
        sel_h.free()
    finally:
        sc.free()
        for b in (xd, sel, wd, y):
            b.free()
        L.free()
