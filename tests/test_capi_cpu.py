"""CPU-side checks of the C ABI: the library loads, exports every declared entry point,
rejects bad arguments with the documented codes, and its host row gathers match the
oracle and the reference's own compiled extension."""
import ctypes
import importlib.util
import os

import pytest
import torch

from lrqk_amd import _lib, ops

HERE = os.path.dirname(os.path.abspath(__file__))
REF_SO = os.path.join(os.path.dirname(HERE), "oracle", "_ref", "take_along_dim_grouped.so")


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = _lib.declared_symbols()
    assert "lrqk_decode_step" in names and "lrqk_score_select" in names and len(names) >= 20
    for n in names:
        assert hasattr(lib, n), n
    assert lib.lrqk_version() >= 1


def test_every_declaration_cites_the_reference():
    text = open(_lib.HEADER_PATH).read()
    for marker in ("py:1235-1273", "py:1275-1315", "cpp:133-183", "cpp:13-124", "py:2326", "py:529-628", "py:319-423",
                   "py:1506-1613", "py:1192-1196"):
        assert marker in text


def test_argument_errors_do_not_touch_the_gpu():
    lib = _lib.load()
    assert lib.lrqk_proxy_scores(None, 0, None, 1, 1, 1, 0, 0, None, None) == -1
    assert b"null" in lib.lrqk_last_error()
    assert lib.lrqk_diff(None, 0, None, 0, 1, 1, None, None, None, None) == -1
    assert lib.lrqk_diff(1, 8, 1, 8, 1, 100000, None, None, None, None) == -3          # k beyond the limit
    assert lib.lrqk_attention(None, None, None, None, 1, 1, None, 1, 8, 0, None) == -1
    with pytest.raises(ValueError):
        _lib.check(-1)
    with pytest.raises(_lib.LrqkError):
        _lib.check(-3)
    t = torch.zeros(4)
    with pytest.raises(ValueError):
        ops.proxy_scores(t.view(1, 1, 2, 2), t.view(1, 1, 1, 4)[..., :2])                  # CPU tensor rejected


def test_d0_index_select_matches_oracle(oracle):
    g = torch.Generator().manual_seed(0)
    for dtype in (torch.float32, torch.bfloat16):
        src = torch.randn((6400, 200), generator=g).to(dtype)
        idx = torch.randint(0, 6400, (9000,), generator=g)
        assert torch.equal(ops.d0_index_select(src, idx), oracle.d0_index_select(src, idx))
    with pytest.raises(ValueError):
        ops.d0_index_select(src, torch.tensor([6400]))
    assert ops.d0_index_select(src, torch.zeros(0, dtype=torch.int64)).shape == (0, 200)


def test_take_along_dim_with_mask_matches_oracle_and_reference(oracle):
    g = torch.Generator().manual_seed(1)
    b, hkv, grp, seq, hd, k = 2, 8, 4, 32, 64, 8
    src = torch.randn((b, hkv, seq, hd), generator=g).to(torch.bfloat16)
    ind = torch.randint(0, seq, (b, hkv, grp, k), generator=g)
    mask = torch.rand((b, hkv, grp, k), generator=g) < 0.4
    out = ops.take_along_dim_with_mask(src, ind, mask)
    assert torch.equal(out, oracle.take_along_dim_with_mask(src, ind, mask))
    if os.path.exists(REF_SO):
        spec = importlib.util.spec_from_file_location("take_along_dim_grouped", REF_SO)
        ref = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(ref)
        assert torch.equal(out, ref.take_along_dim_with_mask(src, ind, mask))
    none = ops.take_along_dim_with_mask(src, ind, torch.zeros_like(mask))
    assert none.shape == (0, hd)


def test_take_along_dim_with_mask_rejects_like_the_reference():
    # cpp_kernel/take_along_dim_grouped.cpp:16-29
    src = torch.zeros((1, 1, 4, 8))
    ind = torch.zeros((1, 1, 1, 2), dtype=torch.int64)
    mask = torch.ones((1, 1, 1, 2), dtype=torch.bool)
    with pytest.raises(RuntimeError):
        ops.take_along_dim_with_mask(src, ind.int(), mask)
    with pytest.raises(RuntimeError):
        ops.take_along_dim_with_mask(src, ind, mask.int())
    with pytest.raises(RuntimeError):
        ops.take_along_dim_with_mask(src[0], ind, mask)
    with pytest.raises(RuntimeError):
        ops.take_along_dim_with_mask(src, ind, mask[..., :1])
    with pytest.raises(RuntimeError):
        ops.take_along_dim_with_mask(src.transpose(2, 3), ind, mask)
    with pytest.raises(ValueError):
        ops.take_along_dim_with_mask(src, ind + 4, mask)                                    # out of range


def test_bench_refuses_more_than_one_gpu():
    """The path is measured on one GPU: any other count exits non-zero with a message."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert p.returncode != 0
    assert "one GPU" in p.stderr
