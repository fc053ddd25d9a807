"""The C-ABI library loads and exports every symbol include/hira_hip.h declares (no
compute calls: this runs without a GPU)."""
import ctypes
import re
from pathlib import Path

import pytest

from hira_amd import _lib

ROOT = Path(__file__).resolve().parents[1]


def _declared_symbols():
    text = (ROOT / "include" / "hira_hip.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hira_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = _declared_symbols()
    assert "hira_search" in names and "hira_build" in names
    lib = ctypes.CDLL(str(_lib.LIB_PATH))
    for n in names:
        assert hasattr(lib, n), f"{n} declared in hira_hip.h but not exported"
    assert set(names) == set(_lib.SYMBOLS), "binding table and header disagree"


def test_abi_version_and_error_text():
    lib = _lib.lib()
    assert lib.hira_abi_version() == _lib.HIRA_ABI_VERSION
    assert isinstance(lib.hira_last_error(), bytes)


def test_argument_validation_needs_no_gpu():
    """Bad descriptors are rejected before anything is launched."""
    lib = _lib.lib()
    t = _lib.HiraTree()
    t.num_trees, t.num_levels, t.bf, t.dim, t.dtype = 1, 2, 99, 64, _lib.HIRA_F32
    assert lib.hira_build_workspace_bytes(ctypes.byref(t), 100) == 0
    assert b"branching factor" in lib.hira_last_error()
    rc = lib.hira_build(ctypes.byref(t), None, None, 100, 1, 4, 0, None, 0, None)
    assert rc == -1
    with pytest.raises(ValueError):
        _lib.check(rc)
    t.bf, t.dim = 8, 6  # rows not a multiple of 16 bytes
    assert lib.hira_build_workspace_bytes(ctypes.byref(t), 100) == 0
    t.dim = 64
    t.size[0], t.size[1], t.cap[0], t.cap[1] = 104, 13, 104, 13
    assert lib.hira_build_workspace_bytes(ctypes.byref(t), 100) > 0
    t.size[1] = 12  # not the padded layout of 100 keys
    assert lib.hira_build_workspace_bytes(ctypes.byref(t), 100) == 0


def test_struct_layout_matches_header():
    """ctypes mirrors of the header structs: field order and sizes."""
    assert ctypes.sizeof(_lib.HiraTree) == 8 * 4 + 2 * 8 * 4 + 3 * 8 + 3 * 8 * 8 + 3 * 8
    assert ctypes.sizeof(_lib.HiraQueue) == 24
    assert ctypes.sizeof(_lib.HiraLaunch) == 16
    assert _lib.HiraQuery.max_group.offset == 48 and _lib.HiraQuery.group_size.offset == 52
    assert _lib.HiraSearchOut.attn_out.offset == 56
    # (the two fields of the fused fill sit in what used to be padding: older callers' structs,
    # zero there, keep their meaning)
    assert _lib.HiraSearchOut.dense_fill.offset == 20 and _lib.HiraSearchOut.dense_fill_value.offset == 52
    assert ctypes.sizeof(_lib.HiraSearchOut) == 72


def test_new_entry_points_validate_without_a_gpu():
    """hira_threshold and hira_sparse_attention reject bad arguments before any launch."""
    lib = _lib.lib()
    q = _lib.HiraQuery(4, 1, None, 1, None, None, 2, 2)
    one = ctypes.c_void_p(1)
    # too many samples, odd row width, k out of range, heads that do not fit the trees
    assert lib.hira_threshold(one, _lib.HIRA_F32, 2, 5000, 32, ctypes.byref(q), 0, 1, one, None) == -1
    assert b"samples" in lib.hira_last_error()
    assert lib.hira_threshold(one, _lib.HIRA_BF16, 2, 100, 20, ctypes.byref(q), 0, 1, one, None) == -1
    assert lib.hira_threshold(one, _lib.HIRA_F32, 2, 100, 32, ctypes.byref(q), 1, 101, one, None) == -1
    assert lib.hira_threshold(one, _lib.HIRA_F32, 3, 100, 32, ctypes.byref(q), 0, 1, one, None) == -1
    assert lib.hira_threshold(None, _lib.HIRA_F32, 2, 100, 32, ctypes.byref(q), 0, 1, one, None) == -1
    t = _lib.HiraTree()
    t.num_trees, t.num_levels, t.bf, t.dim, t.vdim, t.dtype = 2, 2, 8, 32, 0, _lib.HIRA_F32
    assert lib.hira_sparse_attention(ctypes.byref(t), ctypes.byref(q), one, one, one, 8, one, None) == -1
    assert b"no values" in lib.hira_last_error()
    t.values, t.vdim = 1, 1024   # rows of 4 KiB: too wide
    assert lib.hira_sparse_attention(ctypes.byref(t), ctypes.byref(q), one, one, one, 8, one, None) == -1
    t.vdim = 32
    assert lib.hira_sparse_attention(ctypes.byref(t), ctypes.byref(q), one, one, one, 0, one, None) == -1


def _partials_per_head(num_trees, keys_per_tree, heads_per_tree, dim=128, bf=32, levels=3):
    """Workgroups (= attention partials per head) the launch plan makes for a tiled bf16 index of
    this shape, read off hira_search_workspace_bytes (host arithmetic only; the pointers in the
    descriptors are never followed)."""
    lib = _lib.lib()
    t = _lib.HiraTree()
    t.num_trees, t.num_levels, t.bf, t.dim, t.vdim = num_trees, levels, bf, dim, dim
    t.dtype, t.layout = _lib.HIRA_BF16, _lib.HIRA_TILE16
    n = keys_per_tree
    sizes = [n]
    for _ in range(1, levels):
        sizes.append(-(-sizes[-1] // bf))
    for l in range(levels - 2, -1, -1):  # the padded layout: every node owns bf slots below it
        sizes[l] = sizes[l + 1] * bf
    for l in range(levels):
        t.size[l] = sizes[l]
        t.cap[l] = -(-sizes[l] // 16) * 16
    dummy = ctypes.c_void_p(4096)
    t.keys = t.values = t.perm = dummy
    for l in range(1, levels):
        t.centers[l] = t.radii[l] = t.counts[l] = dummy
    q = _lib.HiraQuery(num_trees * heads_per_tree, dummy, dummy, dummy, dummy, dummy,
                       heads_per_tree, heads_per_tree)
    need = lib.hira_search_workspace_bytes(ctypes.byref(t), ctypes.byref(q), None, None)
    assert need > 0, lib.hira_last_error()
    counters = -(-num_trees * 4 // 256) * 256
    per_part = num_trees * heads_per_tree * (dim + 2) * 4
    assert (need - counters) % per_part == 0
    return (need - counters) // per_part


def test_launch_plan_fills_the_compute_units():
    """What the plan of the matrix-core kernel promises (256 compute units assumed where no GPU
    is present): one workgroup per compute unit where the launch fits one round -- also when a
    tree's tiles do not divide evenly, as in an index that grew since its last rebuild --, at
    most 128 partials per head for a tree alone on the chip, workgroups of up to 16 tiles where
    the launch takes several rounds."""
    assert _partials_per_head(8, 32768, 4) == 32            # 64 tiles a tree, 8 trees
    assert _partials_per_head(8, 32768 + 32 * 32, 4) == 32  # 66 tiles: 2 or 3 a workgroup, not 22 x 3
    assert _partials_per_head(8, 131072, 8, levels=4) == 32
    assert _partials_per_head(1, 131072, 4) == 128          # 256 tiles, one tree
    assert _partials_per_head(1, 8192, 4) == 16             # fewer tiles than compute units
    assert _partials_per_head(128, 32768, 4) == 4           # several rounds: 16 tiles a workgroup
