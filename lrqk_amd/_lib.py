"""ctypes loader for liblrqk_hip.so.  There is no fallback: if the library is missing the
first call raises, it never silently runs anything else."""
from __future__ import annotations

import ctypes
import os
import re
import subprocess

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "liblrqk_hip.so")
HEADER_PATH = os.path.join(os.path.dirname(_PKG), "include", "lrqk_hip.h")
CSRC = os.path.join(_PKG, "csrc")

F32, BF16 = 0, 1

_lib = None


class LrqkError(RuntimeError):
    pass


def build(jobs: int = 8) -> str:
    """Compile the HIP sources for gfx950 into liblrqk_hip.so (cross-compiles without a GPU)."""
    subprocess.run(["make", "-C", CSRC, f"-j{jobs}", "-B"], check=True)
    return LIB_PATH


def declared_symbols():
    """Entry points declared in include/lrqk_hip.h."""
    with open(HEADER_PATH) as f:
        text = re.sub(r"/\*.*?\*/", "", f.read(), flags=re.S)
    return sorted(set(re.findall(r"\b(lrqk_[a-z0-9_]+)\s*\(", text)))


def _sig(lib):
    c = ctypes
    vp, i32, i64, f32 = c.c_void_p, c.c_int, c.c_int64, c.c_float
    sigs = {
        "lrqk_version": ([], i32),
        "lrqk_last_error": ([], c.c_char_p),
        "lrqk_ctx_create": ([c.POINTER(vp)], i32),
        "lrqk_ctx_destroy": ([vp], i32),
        "lrqk_ctx_reserve": ([vp, i32, i64, i32, i32, i32, i32], i32),
        "lrqk_proxy_scores": ([vp, i64, vp, i32, i64, i32, i32, i32, vp, vp], i32),
        "lrqk_score_select": ([vp, vp, i64, vp, i32, i64, i32, i32, i32, i32, vp, i64, vp], i32),
        "lrqk_score_select_diff": ([vp, vp, i64, vp, i32, i64, i32, i32, i32, i32, vp, vp, i64, vp, vp, vp, vp], i32),
        "lrqk_select_from_scores": ([vp, vp, i32, i64, i32, vp, i64, vp], i32),
        "lrqk_diff": ([vp, i64, vp, i64, i32, i32, vp, vp, vp, vp], i32),
        "lrqk_replace_all": ([vp, i64, vp, i64, i32, i32, vp, vp, vp, vp], i32),
        "lrqk_fetch_rows": ([vp, i64, vp, vp, i32, vp, i64, vp, vp, i32, i32, i32, i32, i32, i32, vp], i32),
        "lrqk_fetch_rows_staged": ([vp, vp, i64, vp, vp, i32, vp, i64, vp, vp, i32, i32, i32, i32, i32, i32, vp], i32),
        "lrqk_ctx_set_fetch_mode": ([vp, i32, i32], i32),
        "lrqk_ctx_score_index": ([vp, i32], i32),
        "lrqk_ctx_victim_cache": ([vp, i32], i32),
        "lrqk_victim_stats": ([vp, c.POINTER(c.c_int64), i32], i32),
        "lrqk_ctx_factor_state": ([vp, i32], i32),
        "lrqk_last_iterates": ([vp, vp, i64, c.POINTER(i32), c.POINTER(i32), c.POINTER(i32), c.POINTER(i64)], i32),
        "lrqk_gather_rows": ([vp, i64, vp, i64, i32, vp, i32, i32, i32, i32, i32, i32, vp], i32),
        "lrqk_append_token": ([vp, vp, vp, vp, i32, i32, vp, i64, i32, i32, i32, i32, i32, i32, vp], i32),
        "lrqk_flush_ring": ([vp, vp, i32, i32, i32, vp, i64, i64, i32, i32, i32, i32, i32, vp], i32),
        "lrqk_attention": ([vp, vp, vp, vp, i32, i32, vp, i32, i32, i32, vp], i32),
        "lrqk_attention_static": ([vp, vp, vp, i32, i32, vp, i32, i32, i32, vp], i32),
        "lrqk_als_decode": ([vp, vp, vp, vp, i64, vp, i64, vp, i32, i32, vp, vp, i32, i32, i32, i32, i32, i32, f32,
                             vp, vp, i64, i32, vp], i32),
        "lrqk_als_prefill": ([vp, vp, vp, vp, vp, vp, vp, i32, i32, i32, i64, i32, i32, i32, f32, i32, vp], i32),
        "lrqk_decode_step": ([vp, vp, vp, vp, i64, vp, vp, vp, vp, i64, vp, vp, vp, i32, i32, i32, i32, i32, i32, i32,
                              i32, i32, i64, i64, i32, f32, i32, i32, vp, vp, vp, vp, vp, i32, vp], i32),
        "lrqk_select_stats": ([vp, c.POINTER(i32), c.POINTER(i32), i32], i32),
        "lrqk_scan_stats": ([vp, c.POINTER(c.c_int64), c.POINTER(c.c_int64)], i32),
        "lrqk_select_stats_detail": ([vp, c.POINTER(i32), c.POINTER(i32)], i32),
        "lrqk_timing_enable": ([vp, i32], i32),
        "lrqk_timing_stride": ([vp, i32], i32),
        "lrqk_timing_read": ([vp, c.POINTER(c.c_double), c.POINTER(i32)], i32),
        "lrqk_probe_bandwidth": ([vp, vp, i64, i32, c.POINTER(c.c_double), c.POINTER(c.c_double), vp], i32),
        "lrqk_probe_event_pair": ([i32, i32, c.POINTER(c.c_double), vp], i32),
        "lrqk_probe_read_variant": ([vp, vp, i64, i64, i32, i32, i32, i32, c.POINTER(c.c_double), vp], i32),
        "lrqk_d0_indices_select": ([vp, vp, vp, i64, i64, i64, i32], i32),
        "lrqk_take_along_dim_with_mask": ([vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, i32], i64),
    }
    for name, (args, res) in sigs.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = res
    return sigs


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise LrqkError(
                f"{LIB_PATH} is missing: the HIP extension has not been built "
                f"(run `python -c 'import __graft_entry__ as g; g.build()'` or `make -C {CSRC}`)")
        lib = ctypes.CDLL(LIB_PATH)
        _sig(lib)
        _lib = lib
    return _lib


def check(rc: int) -> int:
    if rc < 0:
        msg = load().lrqk_last_error().decode(errors="replace")
        if rc == -1:
            raise ValueError(f"lrqk: {msg}")
        raise LrqkError(f"lrqk error {rc}: {msg}")
    return rc
