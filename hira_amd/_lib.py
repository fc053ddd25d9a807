"""ctypes binding of libhira_hip.so (include/hira_hip.h).

The library is the product: when it is missing or an entry point is absent this module
raises, it never falls back to a host implementation.
"""
from __future__ import annotations

import ctypes as C
import subprocess
from pathlib import Path

HERE = Path(__file__).resolve().parent
CSRC = HERE / "csrc"
LIB_PATH = CSRC / "libhira_hip.so"

HIRA_MAX_LEVELS = 8
HIRA_STATS_COLS = HIRA_MAX_LEVELS + 3  # counters per tree a search can fill in
HIRA_F32, HIRA_BF16 = 0, 1
HIRA_ROW_MAJOR, HIRA_TILE16, HIRA_TILE16_Q8 = 0, 1, 2
HIRA_ABI_VERSION = 7

_vp = C.c_void_p


class HiraTree(C.Structure):
    _fields_ = [
        ("num_trees", C.c_int32),
        ("num_levels", C.c_int32),
        ("bf", C.c_int32),
        ("dim", C.c_int32),
        ("vdim", C.c_int32),
        ("dtype", C.c_int32),
        ("layout", C.c_int32),
        ("reserved_", C.c_int32),
        ("size", C.c_int32 * HIRA_MAX_LEVELS),
        ("cap", C.c_int32 * HIRA_MAX_LEVELS),
        ("keys", _vp),
        ("values", _vp),
        ("perm", _vp),
        ("centers", _vp * HIRA_MAX_LEVELS),
        ("radii", _vp * HIRA_MAX_LEVELS),
        ("counts", _vp * HIRA_MAX_LEVELS),
        ("keys8", _vp),
        ("kscale", _vp),
        ("keps", _vp),
    ]


class HiraQuery(C.Structure):
    _fields_ = [
        ("num_q_heads", C.c_int32),
        ("q", _vp),
        ("tau", _vp),
        ("scaling", _vp),
        ("tree_q_off", _vp),
        ("tree_q_heads", _vp),
        ("max_group", C.c_int32),
        ("group_size", C.c_int32),
    ]


class HiraQueue(C.Structure):
    _fields_ = [("keys", _vp), ("values", _vp), ("len", C.c_int32), ("cap", C.c_int32)]


class HiraSearchOut(C.Structure):
    _fields_ = [
        ("dense", _vp),
        ("dense_stride", C.c_int64),
        ("dense_by_position", C.c_int32),
        ("dense_fill", C.c_int32),
        ("sel_index", _vp),
        ("sel_score", _vp),
        ("sel_count", _vp),
        ("sel_cap", C.c_int32),
        ("dense_fill_value", C.c_float),
        ("attn_out", _vp),
        ("stats", _vp),
    ]


class HiraLaunch(C.Structure):
    _fields_ = [
        ("block_threads", C.c_int32),
        ("nodes_per_wave", C.c_int32),
        ("kernel", C.c_int32),
        ("separate_merge", C.c_int32),
    ]


# every symbol include/hira_hip.h declares: (restype, argtypes)
SYMBOLS = {
    "hira_abi_version": (C.c_int, []),
    "hira_last_error": (C.c_char_p, []),
    "hira_search_workspace_bytes": (
        C.c_size_t,
        [C.POINTER(HiraTree), C.POINTER(HiraQuery), C.POINTER(HiraQueue), C.POINTER(HiraLaunch)],
    ),
    "hira_search": (
        C.c_int,
        [C.POINTER(HiraTree), C.POINTER(HiraQuery), C.POINTER(HiraQueue),
         C.POINTER(HiraSearchOut), C.POINTER(HiraLaunch), _vp, C.c_size_t, _vp],
    ),
    "hira_search_noalloc": (
        C.c_int,
        [C.POINTER(HiraTree), C.POINTER(HiraQuery), C.POINTER(HiraQueue),
         C.POINTER(HiraSearchOut), C.POINTER(HiraLaunch), _vp],
    ),
    "hira_build_workspace_bytes": (C.c_size_t, [C.POINTER(HiraTree), C.c_int32]),
    "hira_build": (
        C.c_int,
        [C.POINTER(HiraTree), _vp, _vp, C.c_int32, C.c_int32, C.c_int32, C.c_uint64, _vp,
         C.c_size_t, _vp],
    ),
    "hira_build_ragged": (
        C.c_int,
        [C.POINTER(HiraTree), _vp, _vp, C.c_int32, _vp, C.c_int32, C.c_int32, C.c_uint64, _vp,
         C.c_size_t, _vp],
    ),
    "hira_nearest_workspace_bytes": (C.c_size_t, [C.c_int32, C.c_int32, C.c_int32, C.c_int32]),
    "hira_nearest": (
        C.c_int,
        [_vp, C.c_int32, C.c_int32, C.c_int32, _vp, C.c_int32, C.c_int32, _vp, _vp, _vp, _vp,
         C.c_size_t, _vp],
    ),
    "hira_quantize": (C.c_int, [C.POINTER(HiraTree), C.c_int32, C.c_int32, C.c_int32, _vp]),
    "hira_update": (C.c_int, [C.POINTER(HiraTree), _vp, _vp, C.c_int32, _vp, _vp]),
    "hira_sparse_attention": (
        C.c_int,
        [C.POINTER(HiraTree), C.POINTER(HiraQuery), _vp, _vp, _vp, C.c_int32, _vp, _vp],
    ),
    "hira_update_threshold": (
        C.c_int,
        [C.POINTER(HiraTree), _vp, _vp, C.c_int32, _vp, _vp, C.c_int32, C.POINTER(HiraQuery),
         C.c_int32, C.c_int32, _vp, _vp],
    ),
    "hira_threshold": (
        C.c_int,
        [_vp, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.POINTER(HiraQuery), C.c_int32,
         C.c_int32, _vp, _vp],
    ),
}

_lib = None


def build_library(verbose: bool = False) -> None:
    """Compile libhira_hip.so for gfx950 (hipcc cross-compiles without a GPU)."""
    r = subprocess.run(["make", "-C", str(CSRC), "-B", "-j8"], capture_output=True, text=True)
    if verbose or r.returncode != 0:
        print(r.stdout[-4000:], r.stderr[-4000:])
    if r.returncode != 0:
        raise RuntimeError("building libhira_hip.so failed")


def use_library(path) -> None:
    """Load another build of the library than the default one (the build with time stamps that
    `make -C hira_amd/csrc timeline` makes, for looking at a decode step): call before anything
    else has used the library."""
    global LIB_PATH
    if _lib is not None:
        raise RuntimeError("the library is already loaded")
    LIB_PATH = Path(path).resolve()


def lib() -> C.CDLL:
    """The loaded library; raises when it has not been built."""
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `make -C {CSRC}` "
                "(or __graft_entry__.build()); there is no host fallback")
        l = C.CDLL(str(LIB_PATH))
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(l, name)  # AttributeError if the export is absent
            fn.restype = res
            fn.argtypes = args
        got = l.hira_abi_version()
        if got != HIRA_ABI_VERSION:
            raise RuntimeError(f"libhira_hip.so ABI {got}, expected {HIRA_ABI_VERSION}")
        _lib = l
    return _lib


def check(rc: int) -> None:
    """Map a return code to the exception the reference's wrappers raise
    (kernels/triton_search_wrappers.py:9-110: ValueError for bad shapes)."""
    if rc == 0:
        return
    msg = lib().hira_last_error().decode(errors="replace")
    if rc == -1:
        raise ValueError(msg)
    raise RuntimeError(f"hira error {rc}: {msg}")


def current_stream(device) -> int:
    """Handle of torch's current HIP stream on `device`, for the `stream` argument of the
    library's calls.  The raw getter costs a fraction of a microsecond where
    ``torch.cuda.current_stream(device).cuda_stream`` builds two Python objects (some 15 us, once
    per layer and decode step)."""
    import torch

    idx = device.index if isinstance(device, torch.device) else torch.device(device).index
    if idx is None:
        idx = torch.cuda.current_device()
    raw = getattr(torch._C, "_cuda_getCurrentRawStream", None)
    if raw is not None:
        return int(raw(idx))
    return torch.cuda.current_stream(idx).cuda_stream
