"""Layers of random shape through every path of the library against the CPU oracle, bit for bit: weight types drawn from
all that the path takes, hidden and ff any number of super-blocks, 1 .. 79 tokens, 1 .. 4 slots a token over 1 .. 8 experts
(so runs from a single slot to several GEMM tiles), in three cases of ten a few tokens over up to 40 experts. Each case runs the per-slot chain or its fused form, the fused
two-launch step, the grouped GEMM step in both f32 modes where the types have one, and bm_moe_forward on each of its
paths. The fixed-shape tests beside this one hold the named configurations; this one holds what lies between them."""
import numpy as np
import pytest

import bloomery_amd as bm
import ora  # noqa: F401
from common import normal_f32
from test_gpu_decode import Layer, gpu, route, run_chain, run_fused_step  # noqa: F401
from test_gpu_prefill import run_prefill

pytestmark = pytest.mark.gpu

ALL_TYPES = (bm.Q4_K, bm.Q5_K, bm.Q6_K, bm.IQ2_XXS, bm.Q3_K, bm.IQ3_XXS, bm.IQ4_XS)


def same_bits(got, want, what):
    got, want = np.asarray(got, np.float32).reshape(-1), np.asarray(want, np.float32).reshape(-1)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), f"{what}: {float(np.abs(got - want).max())}"


@pytest.mark.parametrize("seed", range(6))
def test_random_layers_every_path(gpu, seed):
    rng = np.random.default_rng(9000 + seed)
    for case in range(8):
        with_gemm = rng.random() < 0.6
        tg, td = ALL_TYPES[rng.integers(len(ALL_TYPES))], ALL_TYPES[rng.integers(len(ALL_TYPES))]
        hidden, ff = 256 * int(rng.integers(1, 9)), 256 * int(rng.integers(1, 5))
        n_experts, m = int(rng.integers(1, 9)), int(rng.integers(1, 80))
        if rng.random() < 0.3:  # more experts than slots: bm_moe_forward's grouped form of few slots an expert among the cases
            n_experts, m = int(rng.integers(9, 41)), int(rng.integers(1, 9))
        top_k = min(int(rng.integers(1, 5)), n_experts)
        tag = f"seed {seed} case {case}: types {tg}/{td}, hidden {hidden}, ff {ff}, {n_experts} experts, {m} tokens, top-{top_k}"
        L = Layer(gpu, (tg, tg, td), hidden, ff, n_experts, 9100 + 16 * seed + case, cheap=True)
        x = normal_f32(rng, (m, hidden)) * np.float32(0.05)
        ids, wts = route(rng, m, n_experts, top_k)
        want_y, want_h = L.oracle(x, ids, wts, top_k)
        gpu.fault_clear()
        if m <= 64:
            y, h, _ = run_chain(gpu, L, x, ids, wts, top_k, fused=bool(rng.integers(2)))
            same_bits(y, want_y, tag + ", chain y")
            same_bits(h, want_h, tag + ", chain h")
            same_bits(run_fused_step(gpu, L, x, ids, wts, top_k)[0], want_y, tag + ", fused step")
        if with_gemm:
            y, g = run_prefill(gpu, L, x, ids, wts, top_k)[:2]
            same_bits(y, want_y, tag + ", GEMM step")
            gpu.set_gemm_mode(bm.GEMM_FAST)
            try:
                g_fast = run_prefill(gpu, L, x, ids, wts, top_k)[1]
            finally:
                gpu.set_gemm_mode(bm.GEMM_EXACT)
            ge, gf = g.reshape(m * top_k, ff), g_fast.reshape(m * top_k, ff)
            err = float((np.abs(ge - gf).max(axis=1) / np.maximum(np.abs(ge).max(axis=1), 1e-30)).max())
            assert err <= 1e-4, f"{tag}, tolerance mode gate rows: {err}"
        sc = gpu.scratch(tg, td, hidden, ff, n_experts, top_k, m)
        xd, sel, wd = gpu.upload(x, np.float32), gpu.upload(ids, np.uint32), gpu.upload(wts, np.float32)
        yb = gpu.buffer(np.float32, m * hidden)
        for path in (bm.PATH_PER_SLOT, bm.PATH_GROUPED) + ((bm.PATH_GEMM,) if with_gemm else ()):
            sc.set_path(path)
            yb.fill_bytes(0xFF)
            gpu.enqueue_moe_forward(sc, L.dg, L.du, L.dd, xd, sel, wd, None, m, yb)
            same_bits(yb.download(), want_y, f"{tag}, bm_moe_forward path {path}")
        assert gpu.fault() == (bm.FAULT_NONE, 0), tag
        for b in (xd, sel, wd, yb, sc):
            b.free()
        L.free()
