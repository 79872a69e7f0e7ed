"""CPU-side checks of the C ABI: the built library loads, exports every symbol include/bm_moe.h declares, and its
host-only entry points answer without a GPU. No kernel is launched here."""
import ctypes
import os
import re

import pytest

import bloomery_amd as bm

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "bm_moe.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(bm_[a-z0-9_]+)\s*\(", text)))


def test_library_is_built_and_exports_every_declared_symbol():
    assert os.path.exists(bm.LIB_PATH), "run __graft_entry__.build() first"
    lib = ctypes.CDLL(bm.LIB_PATH)
    names = declared_symbols()
    assert len(names) >= 30
    for name in names:
        assert hasattr(lib, name), f"{name} is declared in include/bm_moe.h but not exported"
    assert sorted(bm.SYMBOLS) == names, "the Python binding lists exactly the header's entry points"


def test_size_rules_match_the_block_layouts():
    # crates/gguf/src/qtype.rs:94,98,105 and crates/qdot/src/lib.rs:381-422
    assert bm.row_bytes(bm.Q4_K, 2048) == 1152 and bm.row_bytes(bm.Q6_K, 768) == 630
    assert bm.row_bytes(bm.IQ2_XXS, 7168) == 1848 and bm.row_bytes(bm.IQ2_XXS, 2048) == 528
    assert bm.col_bytes(bm.Q4_K, 2048) == 2304 and bm.col_bytes(bm.Q6_K, 768) == 864
    assert bm.col_bytes(bm.IQ2_XXS, 7168) == 8288
    for k in (0, -256, 100, 257):
        assert bm.row_bytes(bm.Q4_K, k) == bm.ESHAPE and bm.col_bytes(bm.Q6_K, k) == bm.ESHAPE
    assert bm.row_bytes(bm.Q5_K, 2304) == 176 * 9 and bm.col_bytes(bm.Q5_K, 2304) == 144 * 18
    assert bm.row_bytes(3, 256) == bm.ETYPE and bm.col_bytes(10, 256) == bm.ETYPE
    assert bm.load_library().bm_version() >= 100


def test_oracle_and_library_agree_on_sizes():
    import ora
    for wtype in (bm.Q3_K, bm.Q4_K, bm.Q5_K, bm.Q6_K, bm.IQ2_XXS, bm.IQ3_XXS, bm.IQ4_XS):
        for k in (256, 768, 2048, 7168):
            assert bm.row_bytes(wtype, k) == ora.row_bytes(wtype, k)
            assert bm.col_bytes(wtype, k) == ora.col_bytes(wtype, k)


def test_no_gpu_is_a_named_driver_error_not_a_fallback():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    with pytest.raises(bm.GpuError) as e:
        bm.Gpu(0)
    assert e.value.code == bm.EDRIVER and "bm_ctx_create" in str(e.value)


def test_a_missing_library_raises():
    saved = bm._lib
    bm._lib = None
    try:
        with pytest.raises(bm.GpuError) as e:
            bm.load_library("/nonexistent/libbm_moe_hip.so")
        assert "not built" in str(e.value)
    finally:
        bm._lib = saved


def test_the_benchmark_refuses_more_than_one_gpu():
    """Nothing in this build shards: bench.py --gpus 2 ends with a message that says so, before it touches a device."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0 and "one GPU" in r.stderr and r.stdout.strip() == ""
