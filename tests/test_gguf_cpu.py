"""The GGUF reader's host side (bm_gguf_*), without a GPU: a file written by tests/gguf_file.py is read back name by
name, byte by byte; damaged files are refused with a message that names the damage. The clauses follow the reference
reader's own (crates/gguf/src/lib.rs:143-260 LoadError: bad magic, version, truncation, a tensor past the file, an
offset off the alignment, a duplicate name)."""
import os
import struct

import numpy as np
import pytest

import bloomery_amd as bm
import gguf_file as gf
import ora


def sample(tmp_path, alignment=32, version=3):
    rng = np.random.default_rng(7)
    k, ff, ne = 256, 32, 4
    stack = rng.integers(0, 256, ne * ff * ora.row_bytes(ora.Q4_K, k), dtype=np.uint8)
    down = rng.integers(0, 256, ne * k * ora.row_bytes(ora.Q6_K, 256), dtype=np.uint8)
    norm = rng.standard_normal(k).astype(np.float32)
    kvs = [("general.architecture", gf.STR, "qwen3moe"), ("general.alignment", gf.U32, alignment),
           ("qwen3moe.expert_count", gf.U32, ne), ("qwen3moe.expert_used_count", gf.I32, 2),
           ("qwen3moe.attention.layer_norm_rms_epsilon", gf.F32, 1e-6), ("general.big", gf.U64, 1 << 40),
           ("tokenizer.ggml.tokens", gf.ARR, (gf.STR, ["a", "bc", ""])), ("tokenizer.ggml.scores", gf.ARR, (gf.F32, [0.5, 1.5])),
           ("general.neg", gf.I32, -3), ("general.flag", gf.BOOL, 1)]
    tensors = [("blk.0.ffn_norm.weight", [k], 0, norm.view(np.uint8)),
               ("blk.0.ffn_gate_exps.weight", [k, ff, ne], 12, stack),
               ("blk.0.ffn_down_exps.weight", [256, k, ne], 14, down),
               ("blk.0.odd.weight", [64], 99, np.zeros(0, np.uint8))]
    path = os.path.join(tmp_path, "sample.gguf")
    offsets = gf.write(path, kvs, tensors, alignment, version)
    return path, tensors, offsets


@pytest.mark.parametrize("alignment,version", ((32, 3), (64, 3), (4096, 3), (32, 2)))
def test_a_written_file_reads_back(tmp_path, alignment, version):
    path, tensors, offsets = sample(str(tmp_path), alignment, version)
    g = bm.Gguf(path)
    assert g.version == version
    assert g.get_str("general.architecture") == "qwen3moe" and g.get_str("general.big") is None and g.get_str("nope") is None
    assert g.get_u64("qwen3moe.expert_count") == 4 and g.get_u64("qwen3moe.expert_used_count") == 2
    assert g.get_u64("general.big") == 1 << 40 and g.get_u64("general.flag") == 1
    assert g.get_f32("qwen3moe.attention.layer_norm_rms_epsilon") == np.float32(1e-6)
    listed = g.tensors()
    assert [t["name"] for t in listed] == [t[0] for t in tensors]
    for (name, dims, ttype, data), off, t in zip(tensors, offsets, listed):
        assert t == {**g.find(name), "data": t["data"]} and t["dims"] == dims and t["type"] == ttype and t["offset"] == off
        assert t["offset"] % alignment == 0
        if ttype == 99:  # a type the table does not hold is listed and never handed out
            assert t["nbytes"] == 0 and t["data"] is None
        else:
            assert t["nbytes"] == data.size and np.array_equal(g.data(name), data)
    g.close()


def test_lookups_refuse_by_name(tmp_path):
    path, _, _ = sample(str(tmp_path))
    g = bm.Gguf(path)
    for call, word in ((lambda: g.find("blk.9.ffn_gate_exps.weight"), "blk.9.ffn_gate_exps.weight"),
                       (lambda: g.get_u64("general.neg"), "general.neg"), (lambda: g.get_u64("general.architecture"), "not a count"),
                       (lambda: g.get_u64("absent.key"), "absent.key"), (lambda: g.get_f32("qwen3moe.expert_count"), "not an f32")):
        with pytest.raises(bm.GpuError) as e:
            call()
        assert word in str(e.value)
    g.close()


def damaged(path, edit):
    raw = bytearray(open(path, "rb").read())
    raw = edit(raw)
    out = path + ".bad"
    open(out, "wb").write(bytes(raw))
    return out


def test_damaged_files_are_refused_by_name(tmp_path):
    path, tensors, offsets = sample(str(tmp_path))
    raw = open(path, "rb").read()
    gate = raw.index(b"blk.0.ffn_gate_exps.weight")
    dims_at = gate + len(b"blk.0.ffn_gate_exps.weight") + 4  # after the name and n_dims
    off_at = dims_at + 3 * 8 + 4

    def put(at, fmt, v):
        def edit(b):
            b[at:at + struct.calcsize(fmt)] = struct.pack(fmt, v)
            return b
        return edit

    cases = [
        (put(0, "<I", 0x46554746), "GGUF"),
        (put(4, "<I", 7), "version 7"),
        (lambda b: b[:20], "shorter"),
        (lambda b: b[:gate + 10], "not readable"),
        (put(8, "<Q", 1 << 60), "tensors in"),
        (put(16, "<Q", 1 << 61), "key-values"),
        (lambda b: b[:len(b) - 4096], "runs past the file"),
        (put(off_at, "<Q", offsets[1] + 8), "alignment"),
        (put(off_at, "<Q", 1 << 62), "runs past the file"),
        (put(dims_at, "<Q", 100), "do not size"),           # ne0 not whole blocks
        (put(dims_at + 16, "<Q", 1 << 61), "do not size"),  # the byte count overflows
        (put(dims_at - 4, "<I", 9), "not readable"),        # n_dims
        (lambda b: b.replace(b"blk.0.ffn_down_exps.weight", b"blk.0.ffn_gate_exps.weight"), "two tensors"),
    ]
    for edit, word in cases:
        bad = damaged(path, edit)
        with pytest.raises(bm.GpuError) as e:
            bm.Gguf(bad)
        assert word in str(e.value), (word, str(e.value))
    with pytest.raises(bm.GpuError) as e:
        bm.Gguf(os.path.join(str(tmp_path), "absent.gguf"))
    assert "cannot open" in str(e.value)


def test_a_bad_alignment_is_refused(tmp_path):
    path, _, _ = sample(str(tmp_path))
    raw = open(path, "rb").read()
    at = raw.index(b"general.alignment") + len(b"general.alignment") + 4
    for v in (0, 48, 1 << 30):
        bad = damaged(path, lambda b, v=v: b[:at] + struct.pack("<I", v) + b[at + 4:])
        with pytest.raises(bm.GpuError) as e:
            bm.Gguf(bad)
        assert "general.alignment" in str(e.value)


# --- split sets (crates/gguf/src/lib.rs:835-875 Split::open_model; its own tests, :2290 on, write shards the same way)

def shard_name(prefix, i, count):
    return f"{prefix}-{i + 1:05d}-of-{count:05d}.gguf"


def split_set(tmp_path, count=3, per=(2, 1, 3), prefix="model", edit=None):
    """`count` shards with per[i] F32 tensors each; edit(i, kvs, tensors) may damage shard i's lists before writing.
    The model's keys are in the first shard alone, as the splitter leaves them."""
    rng = np.random.default_rng(11)
    total, made, n = sum(per), {}, 0
    for i in range(count):
        kvs = [("split.no", gf.U16, i), ("split.count", gf.U16, count), ("split.tensors.count", gf.I32, total)]
        if i == 0:
            kvs = [("general.architecture", gf.STR, "qwen3moe"), ("qwen3moe.expert_count", gf.U32, 8)] + kvs
        tensors = []
        for _ in range(per[i]):
            data = rng.standard_normal(32 * (n + 1)).astype(np.float32)
            tensors.append((f"blk.{n}.w", [data.size], 0, data.view(np.uint8)))
            n += 1
        if edit:
            edit(i, kvs, tensors)
        gf.write(os.path.join(tmp_path, shard_name(prefix, i, count)), kvs, tensors)
        made.update({t[0]: t[3] for t in tensors})
    return os.path.join(tmp_path, shard_name(prefix, 0, count)), made


def test_a_split_set_reads_as_one_model(tmp_path):
    first, made = split_set(str(tmp_path))
    g = bm.Gguf(first, split=True)
    assert g.get_str("general.architecture") == "qwen3moe" and g.get_u64("qwen3moe.expert_count") == 8
    assert [t["name"] for t in g.tensors()] == list(made)  # shard order, then each shard's own
    for name, data in made.items():
        assert np.array_equal(g.data(name), data) and g.find(name)["nbytes"] == data.size
    g.close()
    # one shard read alone is that file: its own tensors, no siblings
    alone = bm.Gguf(os.path.join(str(tmp_path), shard_name("model", 1, 3)))
    assert [t["name"] for t in alone.tensors()] == ["blk.2.w"] and alone.get_u64("split.no") == 1
    alone.close()


def test_a_file_without_split_keys_is_a_set_of_one(tmp_path):
    path, tensors, _ = sample(str(tmp_path))
    g = bm.Gguf(path, split=True)
    assert [t["name"] for t in g.tensors()] == [t[0] for t in tensors]
    g.close()
    first, made = split_set(str(tmp_path), count=1, per=(2,), prefix="anyname")
    g = bm.Gguf(first, split=True)  # split.count = 1: the name is free, the keys are still checked
    assert len(g.tensors()) == 2
    g.close()


def set_kv(kvs, key, vtype, v):
    at = [k for k, _, _ in kvs].index(key)
    if v is None:
        del kvs[at]
    else:
        kvs[at] = (key, vtype, v)


@pytest.mark.parametrize("case,words", (
    ("missing_shard", ("shard 3 of 3", "cannot open", "-00003-of-00003.gguf")),
    ("wrong_no", ("-00002-of-00003.gguf", "split.no is 2", "shard 1")),
    ("no_absent", ("-00003-of-00003.gguf", "split.no is absent")),
    ("first_not_first", ("split.no is 1", "shard 0")),
    ("count_differs", ("-00002-of-00003.gguf", "split.count is not the first shard's 3")),
    ("count_zero", ("split.count is not a count",)),
    ("count_a_string", ("split.count is not a count",)),
    ("tensors_count", ("split.tensors.count is 7", "3 shards hold 6")),
    ("tensors_absent", ("split.tensors.count is absent",)),
    ("tensors_negative", ("split.tensors.count is absent or not a count",)),
    ("duplicate", ("blk.0.w", "two shards")),
    ("damaged_shard", ("shard 2 of 3", "does not start with GGUF")),
))
def test_a_broken_split_set_is_refused_by_name(tmp_path, case, words):
    def edit(i, kvs, tensors):
        if case == "wrong_no" and i == 1:
            set_kv(kvs, "split.no", gf.U16, 2)
        if case == "no_absent" and i == 2:
            set_kv(kvs, "split.no", gf.U16, None)
        if case == "first_not_first" and i == 0:
            set_kv(kvs, "split.no", gf.U16, 1)
        if case == "count_differs" and i == 1:
            set_kv(kvs, "split.count", gf.U16, 4)
        if case == "count_zero" and i == 0:
            set_kv(kvs, "split.count", gf.U16, 0)
        if case == "count_a_string" and i == 0:
            set_kv(kvs, "split.count", gf.STR, "3")
        if case == "tensors_count" and i == 0:
            set_kv(kvs, "split.tensors.count", gf.I32, 7)
        if case == "tensors_absent" and i == 0:
            set_kv(kvs, "split.tensors.count", gf.I32, None)
        if case == "tensors_negative" and i == 0:
            set_kv(kvs, "split.tensors.count", gf.I32, -6)
        if case == "duplicate" and i == 2:
            tensors[0] = ("blk.0.w",) + tensors[0][1:]
    first, _ = split_set(str(tmp_path), edit=edit)
    if case == "missing_shard":
        os.remove(os.path.join(str(tmp_path), shard_name("model", 2, 3)))
    if case == "damaged_shard":
        with open(os.path.join(str(tmp_path), shard_name("model", 1, 3)), "r+b") as f:
            f.write(b"GGUX")
    with pytest.raises(bm.GpuError) as e:
        bm.Gguf(first, split=True)
    for w in words:
        assert w in str(e.value), str(e.value)


def test_a_split_sets_first_shard_must_carry_the_sets_name(tmp_path):
    first, _ = split_set(str(tmp_path))
    odd = os.path.join(str(tmp_path), "model.gguf")
    os.rename(first, odd)
    with pytest.raises(bm.GpuError) as e:
        bm.Gguf(odd, split=True)
    assert "does not end in -00001-of-00003.gguf" in str(e.value)


def test_a_set_of_a_dozen_shards(tmp_path):
    """Two-digit shard numbers: the siblings' names are zero-padded to five digits on both sides of "-of-"."""
    first, made = split_set(str(tmp_path), count=12, per=(1,) * 12, prefix="big.model-v2")
    assert first.endswith("big.model-v2-00001-of-00012.gguf") and os.path.exists(first.replace("-00001-", "-00012-"))
    g = bm.Gguf(first, split=True)
    assert [t["name"] for t in g.tensors()] == [f"blk.{i}.w" for i in range(12)]
    assert np.array_equal(g.data("blk.11.w"), made["blk.11.w"])
    g.close()
