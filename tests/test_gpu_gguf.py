"""A model file's expert stacks on the GPU: a GGUF file holding a small layer's three stacks (Q4_K gate / up, Q6_K down,
and an IQ2_XXS one) is opened with the library's reader, each stack goes to the device with bm_weights_from_gguf, and the
decode step over them equals the oracle's over the same bytes (crates/model/src/moe.rs:330 expert_view: expert e is the
e-th equal part of a {k, n, n_expert} tensor)."""
import os

import numpy as np
import pytest

import bloomery_amd as bm
import gguf_file as gf
import ora
from common import normal_f32
from test_gpu_decode import assert_f32, gpu, route, stack  # noqa: F401  (gpu is the module fixture)

pytestmark = pytest.mark.gpu


def test_a_layer_from_a_file(gpu, tmp_path):
    hidden, ff, ne, top_k, m = 512, 256, 8, 2, 3
    wg, wu = stack(bm.Q4_K, ne * ff, hidden, 31), stack(bm.Q4_K, ne * ff, hidden, 32)
    wd = stack(bm.Q6_K, ne * hidden, ff, 33)
    path = os.path.join(str(tmp_path), "layer.gguf")
    gf.write(path, [("general.architecture", gf.STR, "qwen3moe"), ("qwen3moe.expert_count", gf.U32, ne),
                    ("qwen3moe.expert_used_count", gf.U32, top_k)],
             [("blk.0.ffn_gate_exps.weight", [hidden, ff, ne], 12, wg), ("blk.0.ffn_up_exps.weight", [hidden, ff, ne], 12, wu),
              ("blk.0.ffn_down_exps.weight", [ff, hidden, ne], 14, wd), ("blk.0.ffn_norm.weight", [hidden], 0, np.zeros(4 * hidden, np.uint8))])
    g = bm.Gguf(path)
    assert g.get_u64("qwen3moe.expert_count") == ne and g.get_u64("qwen3moe.expert_used_count") == top_k
    (dg, rpe_g, ne_g), (du, _, _), (dd, rpe_d, ne_d) = (g.weights(gpu, f"blk.0.ffn_{n}_exps.weight") for n in ("gate", "up", "down"))
    assert (rpe_g, ne_g, rpe_d, ne_d) == (ff, ne, hidden, ne)
    assert (dg.wtype, dg.rows, dg.k, dd.wtype, dd.rows, dd.k) == (bm.Q4_K, ne * ff, hidden, bm.Q6_K, ne * hidden, ff)
    with pytest.raises(bm.GpuError) as e:
        g.weights(gpu, "blk.0.ffn_norm.weight")
    assert e.value.code == bm.ETYPE and "ggml type 0" in str(e.value)
    with pytest.raises(bm.GpuError) as e:
        g.weights(gpu, "blk.0.ffn_gate.weight")
    assert "no tensor named" in str(e.value)
    g.close()  # the device copies outlive the mapping
    rng = np.random.default_rng(34)
    x = normal_f32(rng, (m, hidden))
    ids, wts = route(rng, m, ne, top_k)
    xd, sel, wt = gpu.upload(x, np.float32), gpu.upload(ids, np.uint32), gpu.upload(wts, np.float32)
    act_h = gpu.act(bm.Q6_K, ff, m * top_k)
    y = gpu.buffer(np.float32, m * hidden).fill_bytes(0xFF)
    gpu.enqueue_moe_decode(dg, du, dd, xd, sel, wt, None, top_k, m, act_h, y)
    want = ora.moe_forward(hidden, ff, ne, (bm.Q4_K, bm.Q4_K, bm.Q6_K), wg, wu, wd, x, ids, wts, top_k, n_threads=4)
    assert_f32(y.download(), want, "y")
    for b in (dg, du, dd, xd, sel, wt, act_h, y):
        b.free()


def test_an_iq2_xxs_matrix_from_a_file(gpu, tmp_path):
    rows, k = 64, 512
    w = stack(bm.IQ2_XXS, rows, k, 41)
    path = os.path.join(str(tmp_path), "iq.gguf")
    gf.write(path, [], [("m.weight", [k, rows], 16, w)])
    g = bm.Gguf(path)
    dw, rpe, ne = g.weights(gpu, "m.weight")
    assert (rpe, ne, dw.rows, dw.k) == (rows, 1, rows, k)
    rng = np.random.default_rng(42)
    x = normal_f32(rng, (1, k))
    act = gpu.act(bm.IQ2_XXS, k, 1)
    xd, y = gpu.upload(x, np.float32), gpu.buffer(np.float32, rows)
    gpu.enqueue_quantize(xd, 1, act)
    gpu.enqueue_gemv(dw, act, 1, y)
    want = ora.gemv(bm.IQ2_XXS, w, rows, k, ora.quantize_col(bm.IQ2_XXS, x[0]))
    assert_f32(y.download(), want, "y")
    g.close()
    for b in (dw, act, xd, y):
        b.free()


def test_a_layer_from_a_split_set(gpu, tmp_path):
    """A layer whose three stacks lie in three shards of a split set (Q5_K gate / up, IQ4_XS down): the set opens by
    its first shard, each stack is found in its own shard, and the step over them is the oracle's."""
    hidden, ff, ne, top_k, m = 512, 256, 6, 2, 2
    wg, wu = stack(bm.Q5_K, ne * ff, hidden, 51), stack(bm.Q5_K, ne * ff, hidden, 52)
    wd = stack(bm.IQ4_XS, ne * hidden, ff, 53)
    parts = ([("blk.0.ffn_gate_exps.weight", [hidden, ff, ne], bm.Q5_K, wg)],
             [("blk.0.ffn_up_exps.weight", [hidden, ff, ne], bm.Q5_K, wu)],
             [("blk.0.ffn_down_exps.weight", [ff, hidden, ne], bm.IQ4_XS, wd)])
    for i, tensors in enumerate(parts):
        kvs = [("split.no", gf.U16, i), ("split.count", gf.U16, 3), ("split.tensors.count", gf.I32, 3)]
        if i == 0:
            kvs.insert(0, ("qwen3moe.expert_count", gf.U32, ne))
        gf.write(os.path.join(str(tmp_path), f"layer-{i + 1:05d}-of-00003.gguf"), kvs, tensors)
    g = bm.Gguf(os.path.join(str(tmp_path), "layer-00001-of-00003.gguf"), split=True)
    assert g.get_u64("qwen3moe.expert_count") == ne and len(g.tensors()) == 3
    (dg, _, _), (du, _, _), (dd, rpe_d, ne_d) = (g.weights(gpu, f"blk.0.ffn_{n}_exps.weight") for n in ("gate", "up", "down"))
    assert (dg.wtype, dd.wtype, rpe_d, ne_d) == (bm.Q5_K, bm.IQ4_XS, hidden, ne)
    g.close()
    rng = np.random.default_rng(54)
    x = normal_f32(rng, (m, hidden))
    ids, wts = route(rng, m, ne, top_k)
    xd, sel, wt = gpu.upload(x, np.float32), gpu.upload(ids, np.uint32), gpu.upload(wts, np.float32)
    act_h = gpu.act(bm.IQ4_XS, ff, m * top_k)
    h = gpu.buffer(np.float32, m * top_k * ff)
    y = gpu.buffer(np.float32, m * hidden).fill_bytes(0xFF)
    gpu.enqueue_moe_decode(dg, du, dd, xd, sel, wt, None, top_k, m, act_h, y, h=h)
    want = ora.moe_forward(hidden, ff, ne, (bm.Q5_K, bm.Q5_K, bm.IQ4_XS), wg, wu, wd, x, ids, wts, top_k, n_threads=4)
    assert_f32(y.download(), want, "y")
    for b in (dg, du, dd, xd, sel, wt, act_h, h, y):
        b.free()
