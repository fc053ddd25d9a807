"""HIPIndexer: the ball-tree index on one MI355X.

Replaces the reference's GPU indexer (indexer/cuda.py:16-108, 544-701) behind the same
surface: ``HIPIndexer(num_levels, max_iterations, branching_factor, verbose, pad_value)``,
``build(keys (1,H,L,D), values)``, ``update(new_keys (1,H,m,D), new_values)``; the
attributes other code reads (``children``, ``values``, ``parents``, ``parent_radii``,
``grand_parents``, ``grand_parent_radii``, ``branching_factor``, ``depth``, ``pad_value``,
``dim``, ``num_heads``, ``_child_counts``, ``_parent_valid``, ``_gp_child_counts``) are
views of the level arrays.  Differences, all deliberate:

* any depth (the reference GPU indexer stops at three levels, indexer/cuda.py:18-21);
* keys stay in the model's dtype (bf16 or fp32; the reference up-casts to fp32,
  indexer/cuda.py:365-368);
* per-node child counts are authoritative (the reference infers validity from
  "row is all pad_value", indexer/cuda.py:137-144);
* ``perm`` maps a key slot to the position the key was inserted at, so results can be
  reported in the CPU searcher's index space as well;
* a leading batch dimension B > 1 builds B*H independent trees that one launch searches.
"""
from __future__ import annotations

import ctypes as C
from enum import Enum
from typing import List, Optional, Tuple

import torch

from .. import _lib
from .base import BaseIndexer

DEFAULT_PAD_VALUE = 0.0

_DTYPES = {torch.float32: _lib.HIRA_F32, torch.bfloat16: _lib.HIRA_BF16}


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else C.c_void_p(t.data_ptr())


def to_tiled(x: torch.Tensor) -> torch.Tensor:
    """(T, R, D) row-major -> the same shape holding the HIRA_TILE16 arrangement: the
    16-byte chunk with columns [32 s + 8 kb, +8) of row 16 t + i moves to chunk index
    (t*(D/32) + s)*64 + kb*16 + i.  R must be a multiple of 16, D of 32."""
    t, r, d = x.shape
    v = x.reshape(t, r // 16, 16, d // 32, 4, 8).permute(0, 1, 3, 4, 2, 5)
    return v.contiguous().reshape(t, r, d)


def from_tiled(x: torch.Tensor) -> torch.Tensor:
    """Inverse of to_tiled."""
    t, r, d = x.shape
    v = x.reshape(t, r // 16, d // 32, 4, 16, 8).permute(0, 1, 4, 2, 3, 5)
    return v.contiguous().reshape(t, r, d)


def level_sizes(n: int, bf: int, num_levels: int) -> List[int]:
    """Slots per level of the padded tree: K_1 = ceil(n/bf), K_l = ceil(K_{l-1}/bf); the
    root keeps K_root nodes and each lower level has bf slots per node of the level above
    (the reference's m = ceil(n/bf), g = ceil(m/bf), children (h, g*bf*bf, d):
    indexer/cuda.py:223-224, 439-446)."""
    if num_levels == 1:
        return [n]
    k = n
    for _ in range(1, num_levels):
        k = max(1, -(-k // bf))
    sizes = [0] * num_levels
    sizes[-1] = k
    for l in range(num_levels - 2, -1, -1):
        sizes[l] = sizes[l + 1] * bf
    return sizes


# layout="auto" adds the 8-bit shadow of the keys where the search measurably gains from it: long
# scans shared by many heads (131072 keys a tree and 8 query heads per KV head: a decode step of
# 64 heads takes 54.8 us against 63.9 us); shorter trees or fewer heads a tree lose to the extra
# dependent step of the exact test
Q8_AUTO_MIN_KEYS = 131072
Q8_AUTO_MIN_HEADS = 8


def choose_layout(request: str, dtype: torch.dtype, dim: int, vdim: int, num_levels: int, bf: int,
                  n: int, heads_per_tree: Optional[int] = None) -> Tuple[bool, bool]:
    """(tiled, q8) for a layout request: which arrangement an index of `n` keys a tree gets.
    Raises ValueError for an explicit request the keys cannot have."""
    tile_ok = dtype == torch.bfloat16 and dim % 32 == 0
    if request == "tiled" and not tile_ok:
        raise ValueError("the tiled layout needs bfloat16 keys with dim a multiple of 32")
    q8_ok = tile_ok and dim in (64, 128) and num_levels >= 2
    if request == "q8" and not q8_ok:
        raise ValueError("the q8 layout needs bfloat16 keys with dim 64 or 128 and at least two "
                         "levels")
    auto_tiled = (request == "auto" and tile_ok and num_levels >= 2 and bf % 16 == 0
                  and dim in (64, 128, 256) and vdim in (0, dim))
    q8 = request == "q8" or (
        auto_tiled and q8_ok and vdim == dim and heads_per_tree is not None
        and heads_per_tree >= Q8_AUTO_MIN_HEADS and n >= Q8_AUTO_MIN_KEYS)
    tiled = tile_ok and (request in ("tiled", "q8") or auto_tiled)
    return tiled, q8


class HIPIndexer(BaseIndexer):
    class DEPTH(Enum):
        TWO_LEVELS = 2
        THREE_LEVELS = 3

    def __init__(
        self,
        num_levels,
        max_iterations: int = 1,
        branching_factor: int = 32,
        verbose: bool = False,
        pad_value: float = DEFAULT_PAD_VALUE,
        *,
        seed: int = 1234,
        capacity: Optional[int] = None,
        pack_rounds: int = 8,
        layout: str = "auto",
        device: str = "cuda",
        graft_min: Optional[int] = None,
        heads_per_tree: Optional[int] = None,
    ):
        if isinstance(num_levels, HIPIndexer.DEPTH):
            num_levels = num_levels.value
        num_levels = int(num_levels)
        if not 1 <= num_levels <= _lib.HIRA_MAX_LEVELS:
            raise ValueError(f"num_levels must be in 1..{_lib.HIRA_MAX_LEVELS}, got {num_levels}")
        if not 1 <= int(branching_factor) <= 64:
            raise ValueError(f"branching_factor must be in 1..64, got {branching_factor}")
        self.num_levels = num_levels
        self.max_iterations = int(max_iterations)
        self.branching_factor = int(branching_factor)
        self.verbose = verbose
        self.pad_value = pad_value
        self.seed = int(seed)
        self.pack_rounds = int(pack_rounds)
        if layout not in ("auto", "row_major", "tiled", "q8"):
            raise ValueError("layout must be 'auto', 'row_major', 'tiled' or 'q8'")
        self.layout_request = layout
        # query heads per KV head the searches will come with, when the caller knows (the cache
        # layer does): layout="auto" takes it into account, see choose_layout
        self.heads_per_tree = None if heads_per_tree is None else int(heads_per_tree)
        self.tiled = False  # centers (and, unless q8, keys) stored in the MFMA tile arrangement
        # q8: tiled centers, row-major keys and beside them an 8-bit shadow copy of the keys
        # (keys8, one step per tree and channel in kscale, error bounds per level-1 node in
        # keps) that the search scans first; bf16 rows are then fetched only for the keys the
        # shadow cannot rule out
        self.q8 = False
        self.keys8: Optional[torch.Tensor] = None
        self.kscale: Optional[torch.Tensor] = None
        self.keps: Optional[torch.Tensor] = None
        self.capacity = capacity  # key slots to reserve per tree (room for appends)
        # update() calls with at least this many keys per tree build a sub-tree over the new
        # keys and graft it at the tail instead of placing the keys one by one
        # (default: half of what one root node holds, at least 256)
        self.graft_min = graft_min
        self.device = torch.device(device)

        self.dim = 0
        self.vdim = 0
        self.batch = 1
        self.num_heads = 0
        self.num_trees = 0
        self.num_keys = 0  # keys given to the index so far, per tree
        # appends whose level sizes have not been read back yet (update(sync=False)): then
        # self.size holds upper bounds and _exact_size the sizes as of the last read-back
        self._pending = 0
        self._exact_size: Optional[List[int]] = None
        self._unsynced_room = 0  # appends a stretch opened by begin_unsynced still has room for
        # whether a decode step has looked at its attention mask for this index (padding cannot be
        # honoured by the sparse step: the attention function checks once per built index)
        self._decode_mask_checked = False
        self.dtype: Optional[torch.dtype] = None
        self.size: List[int] = []
        self.cap: List[int] = []
        self.keys_buf: Optional[torch.Tensor] = None
        self.values_buf: Optional[torch.Tensor] = None
        self.perm: Optional[torch.Tensor] = None
        self.centers: List[Optional[torch.Tensor]] = []
        self.radii: List[Optional[torch.Tensor]] = []
        self.counts: List[Optional[torch.Tensor]] = []
        self._tree_struct = None
        self._state: Optional[torch.Tensor] = None  # device-side bookkeeping of update()

    # ------------------------------------------------------------------ reference views
    @property
    def depth(self):
        try:
            return HIPIndexer.DEPTH(self.num_levels)
        except ValueError:
            return self.num_levels

    def _head_view(self, t: torch.Tensor, n: int, rows: bool = False) -> torch.Tensor:
        """(T, cap, ...) -> (H, n, ...) for batch 1, (B, H, n, ...) otherwise.  `rows`: t is
        a key / centre matrix; it is returned row-major (a copy when the index is tiled)."""
        if rows and (self.keys_tiled if t is self.keys_buf else self.tiled):
            t = from_tiled(t)
        v = t[:, :n]
        return v if self.batch == 1 else v.reshape(self.batch, self.num_heads, *v.shape[1:])

    @property
    def keys_tiled(self) -> bool:
        return self.tiled and not self.q8

    @property
    def layout_name(self) -> str:
        return "q8" if self.q8 else ("tiled" if self.tiled else "row_major")

    @property
    def children(self):
        return None if self.keys_buf is None else self._head_view(self.keys_buf, self.size[0], True)

    def keys_rowmajor(self) -> torch.Tensor:
        """(T, N_pad, D) keys in slot order, row-major (a copy when the index is tiled)."""
        k = from_tiled(self.keys_buf) if self.keys_tiled else self.keys_buf
        return k[:, : self.size[0]]

    def centers_rowmajor(self, l: int) -> torch.Tensor:
        c = from_tiled(self.centers[l]) if self.tiled else self.centers[l]
        return c[:, : self.size[l]]

    @property
    def values(self):
        if self.values_buf is None:
            return None
        v = self._head_view(self.values_buf, self.size[0])
        return v.unsqueeze(0) if self.batch == 1 else v

    def _level(self, arr, l, rows: bool = False):
        if l >= self.num_levels or not arr or arr[l] is None:
            return None
        return self._head_view(arr[l], self.size[l], rows)

    @property
    def parents(self):
        return self._level(self.centers, 1, True)

    @property
    def parent_radii(self):
        return self._level(self.radii, 1)

    @property
    def grand_parents(self):
        return self._level(self.centers, 2, True)

    @property
    def grand_parent_radii(self):
        return self._level(self.radii, 2)

    @property
    def _child_counts(self):
        return self._level(self.counts, 1)

    @property
    def _parent_valid(self):
        c = self._level(self.counts, 1)
        return None if c is None else c > 0

    @property
    def _gp_child_counts(self):
        return self._level(self.counts, 2)

    # ------------------------------------------------------------------ device state
    def _allocate(self, batch: int, heads: int, n: int, dim: int, vdim: int,
                  dtype: torch.dtype) -> None:
        if dtype not in _DTYPES:
            raise ValueError(f"unsupported key dtype {dtype}: use float32 or bfloat16")
        esize = 4 if dtype == torch.float32 else 2
        if (dim * esize) % 16 or (vdim * esize) % 16:
            raise ValueError(f"dim {dim} / vdim {vdim}: rows must be a multiple of 16 bytes")
        self.batch, self.num_heads = batch, heads
        self.num_trees = batch * heads
        self.dim, self.vdim, self.dtype = dim, vdim, dtype
        self._decode_mask_checked = False  # a new index: maybe a new, padded batch
        self._pending, self._exact_size, self._unsynced_room = 0, None, 0
        bf, nl = self.branching_factor, self.num_levels
        self.size = level_sizes(n, bf, nl)
        want = max(n, int(self.capacity or 0))
        self.cap = level_sizes(want, bf, nl) if want > n else list(self.size)
        self.tiled, self.q8 = choose_layout(self.layout_request, dtype, dim, vdim, nl, bf, n,
                                            self.heads_per_tree)
        if self.tiled:
            self.cap = [-(-c // 16) * 16 for c in self.cap]
        dev, t = self.device, self.num_trees
        self.keys_buf = torch.zeros((t, self.cap[0], dim), dtype=dtype, device=dev)
        self.values_buf = (
            torch.zeros((t, self.cap[0], vdim), dtype=dtype, device=dev) if vdim else None)
        self.perm = torch.full((t, self.cap[0]), -1, dtype=torch.int32, device=dev)
        self.keys8 = self.kscale = self.keps = None
        if self.q8:
            self.keys8 = torch.zeros((t, self.cap[0], dim), dtype=torch.int8, device=dev)
            self.kscale = torch.ones((t, dim), dtype=torch.float32, device=dev)
            self.keps = torch.zeros((t, self.cap[1]), dtype=torch.float32, device=dev)
        self.centers, self.radii, self.counts = [None], [None], [None]
        for l in range(1, nl):
            self.centers.append(torch.zeros((t, self.cap[l], dim), dtype=dtype, device=dev))
            self.radii.append(
                torch.full((t, self.cap[l]), float("-inf"), dtype=torch.float32, device=dev))
            self.counts.append(torch.zeros((t, self.cap[l]), dtype=torch.int32, device=dev))
        self._tree_struct = None
        self._state = None

    def tree_struct(self) -> _lib.HiraTree:
        """The C view of the tree; valid while this indexer's tensors are alive."""
        if self.keys_buf is None:
            raise ValueError("Indexer is not built: missing children tensor.")
        if self._tree_struct is None:
            t = _lib.HiraTree()
            t.num_trees = self.num_trees
            t.num_levels = self.num_levels
            t.bf = self.branching_factor
            t.dim, t.vdim = self.dim, self.vdim
            t.dtype = _DTYPES[self.dtype]
            t.layout = (_lib.HIRA_TILE16_Q8 if self.q8 else
                        _lib.HIRA_TILE16 if self.tiled else _lib.HIRA_ROW_MAJOR)
            if self.q8:
                t.keys8, t.kscale = self.keys8.data_ptr(), self.kscale.data_ptr()
                t.keps = self.keps.data_ptr()
            for l in range(self.num_levels):
                t.size[l], t.cap[l] = self.size[l], self.cap[l]
            t.keys = self.keys_buf.data_ptr()
            t.values = None if self.values_buf is None else self.values_buf.data_ptr()
            t.perm = self.perm.data_ptr()
            for l in range(1, self.num_levels):
                t.centers[l] = self.centers[l].data_ptr()
                t.radii[l] = self.radii[l].data_ptr()
                t.counts[l] = self.counts[l].data_ptr()
            self._tree_struct = t
        return self._tree_struct

    # ------------------------------------------------------------------ layouts
    @classmethod
    def from_layout(cls, *, bf: int, keys, perm, centers, radii, counts, values=None,
                    dtype: torch.dtype = torch.float32, batch: int = 1, device: str = "cuda",
                    num_keys: Optional[int] = None, capacity: Optional[int] = None,
                    layout: str = "auto"):
        """Adopt a padded tree given as host arrays: keys (T, N_pad, D), perm (T, N_pad),
        and per level l >= 1 (index 0 is None) centers (T, K_l, D), radii (T, K_l), counts
        (T, K_l); values (T, N_pad, Dv) follow the key slots.  Used to restore a saved index
        and by tests that walk a tree built on the host."""
        nl = len(centers)
        self = cls(nl, 1, bf, device=device, capacity=capacity, layout=layout)
        keys = torch.as_tensor(keys)
        t, n_pad, d = keys.shape
        vdim = 0 if values is None else int(torch.as_tensor(values).shape[-1])
        self._allocate(batch, t // batch, n_pad, d, vdim, dtype)
        if self.size[0] != n_pad:
            raise ValueError(f"keys have {n_pad} slots, layout needs {self.size[0]}")
        self.keys_buf[:, :n_pad] = keys.to(device=self.device, dtype=dtype)
        if self.keys_tiled:
            self.keys_buf.copy_(to_tiled(self.keys_buf))
        if values is not None:
            self.values_buf[:, :n_pad] = torch.as_tensor(values).to(device=self.device,
                                                                    dtype=dtype)
        perm = torch.as_tensor(perm).to(torch.int32)
        self.perm[:, :n_pad] = perm.to(self.device)
        for l in range(1, nl):
            k = self.size[l]
            self.centers[l][:, :k] = torch.as_tensor(centers[l]).to(self.device, dtype)
            if self.tiled:
                self.centers[l].copy_(to_tiled(self.centers[l]))
            self.radii[l][:, :k] = torch.as_tensor(radii[l]).to(self.device, torch.float32)
            self.counts[l][:, :k] = torch.as_tensor(counts[l]).to(self.device, torch.int32)
        self.num_keys = int(num_keys if num_keys is not None else (perm[0] >= 0).sum().item())
        if self.q8:
            self.quantize(new_steps=True)
        return self

    def quantize(self, slot_first: int = 0, slot_count: Optional[int] = None,
                 new_steps: bool = False) -> "HIPIndexer":
        """(Re)make the 8-bit shadow of the keys in slots [slot_first, +slot_count) of every tree
        (whole level-1 nodes; default: all slots in use) from the bf16 keys as they stand;
        ``new_steps`` first derives the step of every channel from all keys (then the whole
        shadow must be remade).  A q8 index only; one or four small launches."""
        if not self.q8:
            return self
        bf = self.branching_factor
        if slot_count is None:
            slot_count = self.size[0] - slot_first
        slot_count = -(-slot_count // bf) * bf
        tree = self.tree_struct()
        stream = _lib.current_stream(self.device)
        _lib.check(_lib.lib().hira_quantize(C.byref(tree), int(slot_first), int(slot_count),
                                            1 if new_steps else 0, stream))
        return self

    # ------------------------------------------------------------------ persistence
    def save(self, path: str) -> None:
        """Write the index to one safetensors file: every level array as it is stored on the
        device (keys and centres in their storage layout, rows beyond the slots in use cut
        off), the update bookkeeping, and the constructor settings in the file's metadata.
        ``HIPIndexer.load`` restores it bit for bit.  (The reference has no persistence; its
        config loaders and example configs point at one: cache/hira_config.py:27-33.)"""
        import json

        from safetensors.torch import save_file

        if self.keys_buf is None:
            raise ValueError("Indexer is not built: nothing to save.")
        self.sync_sizes()
        rows = [(-(-s // 16) * 16 if self.tiled else s) for s in self.size]
        tensors = {"keys": self.keys_buf[:, : rows[0]], "perm": self.perm[:, : rows[0]]}
        if self.values_buf is not None:
            tensors["values"] = self.values_buf[:, : rows[0]]
        for l in range(1, self.num_levels):
            tensors[f"centers.{l}"] = self.centers[l][:, : rows[l]]
            tensors[f"radii.{l}"] = self.radii[l][:, : rows[l]]
            tensors[f"counts.{l}"] = self.counts[l][:, : rows[l]]
        if self._state is not None:
            tensors["update_state"] = self._state
        if self.q8:
            tensors["keys8"] = self.keys8[:, : rows[0]]
            tensors["kscale"] = self.kscale
            tensors["keps"] = self.keps[:, : rows[1]]
        meta = {
            "format": "hira_amd.index.v1", "num_levels": self.num_levels,
            "branching_factor": self.branching_factor, "max_iterations": self.max_iterations,
            "pack_rounds": self.pack_rounds, "seed": self.seed, "pad_value": self.pad_value,
            "layout_request": self.layout_request, "tiled": self.tiled, "q8": self.q8, "batch": self.batch,
            "num_heads": self.num_heads, "dim": self.dim, "vdim": self.vdim,
            "dtype": "bfloat16" if self.dtype == torch.bfloat16 else "float32",
            "size": list(self.size), "rows": rows, "num_keys": self.num_keys,
        }
        save_file({k: v.detach().cpu().contiguous() for k, v in tensors.items()}, path,
                  metadata={"hira": json.dumps(meta)})

    @classmethod
    def load(cls, path: str, device: str = "cuda", capacity: Optional[int] = None) -> "HIPIndexer":
        """Restore an index written by ``save`` (safetensors: nothing from the file is
        executed).  ``capacity`` reserves key slots per tree for later appends."""
        import json

        from safetensors import safe_open

        with safe_open(path, framework="pt", device="cpu") as f:
            raw = (f.metadata() or {}).get("hira")
            if raw is None:
                raise ValueError(f"{path}: not an index file (no 'hira' metadata)")
            meta = json.loads(raw)
            if meta.get("format") != "hira_amd.index.v1":
                raise ValueError(f"{path}: unknown index format {meta.get('format')!r}")
            tensors = {k: f.get_tensor(k) for k in f.keys()}
        self = cls(meta["num_levels"], meta["max_iterations"], meta["branching_factor"],
                   pad_value=meta["pad_value"], seed=meta["seed"], pack_rounds=meta["pack_rounds"],
                   layout="q8" if meta.get("q8") else ("tiled" if meta["tiled"] else "row_major"),
                   capacity=capacity, device=device)
        dtype = torch.bfloat16 if meta["dtype"] == "bfloat16" else torch.float32
        size, rows = list(meta["size"]), list(meta["rows"])
        # room for what the file holds (and for `capacity`), then the saved sizes
        self._allocate(meta["batch"], meta["num_heads"], max(rows[0], 1), meta["dim"],
                       meta["vdim"], dtype)
        if self.tiled != bool(meta["tiled"]) or self.q8 != bool(meta.get("q8", False)):
            raise ValueError(f"{path}: stored layout does not match what this build would choose")
        self.size = list(rows)
        self._grow(rows)
        self.size = size

        def put(dst, name):
            src = tensors[name]
            if tuple(src.shape[2:]) != tuple(dst.shape[2:]) or src.shape[0] != dst.shape[0] \
                    or src.shape[1] > dst.shape[1] or src.dtype != dst.dtype:
                raise ValueError(f"{path}: tensor {name} {tuple(src.shape)} {src.dtype} does not fit")
            dst[:, : src.shape[1]] = src.to(self.device)

        put(self.keys_buf, "keys")
        put(self.perm, "perm")
        if self.values_buf is not None:
            put(self.values_buf, "values")
        for l in range(1, self.num_levels):
            put(self.centers[l], f"centers.{l}")
            put(self.radii[l], f"radii.{l}")
            put(self.counts[l], f"counts.{l}")
        if "update_state" in tensors:
            self._state = tensors["update_state"].to(self.device)
            if self.num_levels >= 2:
                self._state[:, 0] = 0
        if self.q8:
            put(self.keys8, "keys8")
            self.kscale.copy_(tensors["kscale"].to(self.device))
            put(self.keps, "keps")
        self.num_keys = int(meta["num_keys"])
        self._tree_struct = None
        return self

    @staticmethod
    def storage_dtype(dtype: torch.dtype) -> torch.dtype:
        """The dtype an index over keys of `dtype` stores: bf16 and fp32 as they are; fp16
        becomes bf16 (same size, the kernels' 16-bit type; a warning says so, since bf16 has
        three bits less of mantissa); anything else is up-cast to fp32 as the reference does
        for every input (indexer/cuda.py:365-368)."""
        if dtype in _DTYPES:
            return dtype
        if dtype == torch.float16:
            import warnings

            warnings.warn("HIPIndexer stores float16 keys/values as bfloat16 (8 bits of mantissa "
                          "instead of 11); pass float32 tensors to keep every bit", stacklevel=3)
            return torch.bfloat16
        return torch.float32

    # ------------------------------------------------------------------ build / update
    @torch.no_grad()
    def build(self, keys: torch.Tensor, values: Optional[torch.Tensor] = None, *,
              key_counts: Optional[torch.Tensor] = None):
        """keys (1, H, L, D) (or (B, H, L, D): one tree per sequence and KV head), values
        (1, H, L, Dv) aligned with the keys or None.  Runs on the current stream and
        returns self without waiting (indexer/cuda.py:56-108).

        ``key_counts`` (B*H,) int32 on the device (two levels only): tree t holds only the first
        key_counts[t] of its L keys; every tree still gets the layout of L keys, with emptier
        nodes where keys are missing (``num_keys`` then says L: the bound)."""
        if keys.ndim != 4:
            raise ValueError(f"keys must be (B,H,L,D), got {tuple(keys.shape)}")
        if values is not None and values.shape[:3] != keys.shape[:3]:
            raise ValueError("values must be aligned with keys: (B,H,L,Dv)")
        b, h, n, d = keys.shape
        dtype = self.storage_dtype(keys.dtype)
        vdim = 0 if values is None else int(values.shape[-1])
        self._allocate(b, h, n, d, vdim, dtype)
        kin = keys.to(device=self.device, dtype=dtype).reshape(b * h, n, d).contiguous()
        vin = None
        if values is not None:
            vin = values.to(device=self.device, dtype=dtype).reshape(b * h, n, vdim).contiguous()
        lib = _lib.lib()
        tree = self.tree_struct()
        need = lib.hira_build_workspace_bytes(C.byref(tree), n)
        if need == 0:
            _lib.check(-1)
        ws = torch.empty(need, dtype=torch.uint8, device=self.device)
        stream = _lib.current_stream(self.device)
        if key_counts is not None:
            if key_counts.dtype != torch.int32 or tuple(key_counts.shape) != (b * h,) \
                    or key_counts.device.type != self.device.type or not key_counts.is_contiguous():
                raise ValueError(f"key_counts must be a contiguous int32 tensor of {b * h} counts on "
                                 f"{self.device}")
            rc = lib.hira_build_ragged(C.byref(tree), kin.data_ptr(),
                                       None if vin is None else vin.data_ptr(), n,
                                       key_counts.data_ptr(), self.max_iterations, self.pack_rounds,
                                       self.seed, ws.data_ptr(), need, stream)
        else:
            rc = lib.hira_build(C.byref(tree), kin.data_ptr(),
                                None if vin is None else vin.data_ptr(), n, self.max_iterations,
                                self.pack_rounds, self.seed, ws.data_ptr(), need, stream)
        _lib.check(rc)
        self.num_keys = n
        if self.verbose:
            print(f"built {self.num_trees} trees, level sizes {self.size}")
        return self

    def _needed_caps(self, m: int) -> List[int]:
        """Slots every level may need after m more keys: at most ceil(m/bf)+1 new level-1
        nodes, ceil(that/bf)+1 new level-2 nodes, ...; a new node's children sit at
        position node*bf, so a level below must reach (nodes above)*bf."""
        bf, nl = self.branching_factor, self.num_levels
        if nl == 1:
            return [self.num_keys + m]
        # (new nodes appear only once every node of a level is full, so the bound holds for
        # the total of several calls: count from the last sizes that were read back)
        # (while an unsynced stretch is open self.size holds bounds, not sizes)
        base = self._exact_size if self._exact_size is not None else self.size
        need = [0] * nl
        new = m + self._pending
        for l in range(1, nl):
            new = -(-new // bf) + 1
            need[l] = base[l] + new
        for l in range(nl - 2, -1, -1):
            need[l] = max(need[l], need[l + 1] * bf)
        return need

    def _grow(self, need: List[int]) -> None:
        """Re-allocate the level arrays with at least `need` slots (doubling), keeping the
        contents.  A tile of 16 rows is contiguous, so a tiled matrix grows by rows too."""
        caps = []
        for l, (c, n) in enumerate(zip(self.cap, need)):
            c2 = c if n <= c else max(n, 2 * c)
            caps.append(-(-c2 // 16) * 16 if self.tiled else c2)
        if caps == self.cap:
            return
        if self._unsynced_room > 0:
            # a launch captured by begin_unsynced holds the current pointers
            raise RuntimeError(
                "the index would have to re-allocate while a stretch of unsynced updates is open "
                "(a captured decode step holds its pointers): call sync_sizes() first, or "
                "reserve() more room before begin_unsynced()")

        def grown(old, cap, fill):
            new = torch.full((old.shape[0], cap) + tuple(old.shape[2:]), fill, dtype=old.dtype,
                             device=old.device)
            new[:, : old.shape[1]] = old
            return new

        self.keys_buf = grown(self.keys_buf, caps[0], 0)
        if self.values_buf is not None:
            self.values_buf = grown(self.values_buf, caps[0], 0)
        self.perm = grown(self.perm, caps[0], -1)
        if self.q8:
            self.keys8 = grown(self.keys8, caps[0], 0)
            self.keps = grown(self.keps, caps[1], 0)
        for l in range(1, self.num_levels):
            self.centers[l] = grown(self.centers[l], caps[l], 0)
            self.radii[l] = grown(self.radii[l], caps[l], float("-inf"))
            self.counts[l] = grown(self.counts[l], caps[l], 0)
        self.cap = caps
        self._tree_struct = None

    @torch.no_grad()
    def _room_under_a_root(self, new_keys, m: int):
        """Per tree, the root node nearest to the window's mean among those with free child
        slots for a sub-tree of one level less over m keys: (roots (T,), their child counts
        (T,)) on the host, or None when some tree has no such root (then the keys go one by
        one, or, if there are enough of them, under new roots)."""
        self.sync_sizes()
        bf, top = self.branching_factor, self.num_levels - 1
        nroot = self.size[top]
        if nroot <= 0:
            return None
        cnt = self.counts[top][:, :nroot]
        k = level_sizes(m, bf, top)[-1]  # nodes the sub-tree puts under the root
        ok = (cnt > 0) & (cnt + k <= bf)
        if not bool(ok.any(dim=1).all()):
            return None
        mean = new_keys.to(self.device).reshape(self.num_trees, m, self.dim).float().mean(dim=1)
        c = self.centers_rowmajor(top)[:, :nroot].float()
        dist = (c - mean[:, None]).norm(dim=-1).masked_fill(~ok, float("inf"))
        roots = dist.argmin(dim=1)
        have = cnt.gather(1, roots[:, None]).squeeze(1)
        return roots.cpu(), have.cpu()

    @torch.no_grad()
    def _graft(self, new_keys, new_values, m: int, sub_levels: int, under) -> "HIPIndexer":
        """A large window of new keys: cluster them among themselves (one ``hira_build`` over
        all trees) and graft the resulting sub-tree into the tail of the index.  With
        ``sub_levels == num_levels`` its roots become new root nodes after the existing ones;
        with one level less (``under = (roots, child counts)``, per tree) they become further
        children of an existing root, whose radius grows to cover them.  Either way the descendants sit in
        the slot ranges their parents own.  This is the shape of the reference's CPU update
        (indexer/cpu.py:124-190: an independent sub-tree over the new keys, concatenated level
        by level) in the fixed-fan-out layout; placing the keys one by one (the small-window
        path) costs a few microseconds per key and tree, serially."""
        self.sync_sizes()
        bf, nl = self.branching_factor, self.num_levels
        sub = HIPIndexer(sub_levels, self.max_iterations, bf, seed=self.seed + self.num_keys,
                         device=str(self.device), pack_rounds=self.pack_rounds,
                         layout=self.layout_name, graft_min=1 << 62)
        sub.build(new_keys.to(self.device, self.dtype),
                  None if new_values is None else new_values.to(self.device, self.dtype))
        if sub.tiled != self.tiled or sub.q8 != self.q8:
            raise RuntimeError("sub-tree layout differs from the index's")
        stop = sub_levels - 1  # the sub-tree's top level, as a level of the index
        r16 = (lambda n: -(-n // 16) * 16) if self.tiled else (lambda n: n)
        # where the sub-tree's top nodes go: after the existing roots (the same place in every
        # tree), or after the children the chosen root already has (tree by tree)
        if under is None:
            groups = [(slice(None), self.size[stop])]
        else:
            roots, have = under
            place = roots.long() * bf + have.long()  # (T,) first free child slot of the chosen root
            groups = [((place == v).nonzero().squeeze(1).to(self.device), int(v))
                      for v in torch.unique(place).tolist()]
        offs = []
        for _, top_off in groups:
            off = [0] * sub_levels
            off[stop] = top_off
            for l in range(stop - 1, -1, -1):
                off[l] = off[l + 1] * bf
            offs.append(off)
        need = list(self.size)
        for off in offs:
            for l in range(sub_levels):
                need[l] = max(need[l], off[l] + r16(sub.size[l]))
        self._grow(need)
        if self._state is None:
            self._init_state()
        n0 = sub.size[0]
        sp = sub.perm[:, :n0]
        sp = torch.where(sp >= 0, sp + self.num_keys, torch.full_like(sp, -1))
        quant = []  # key slot ranges whose 8-bit shadow has to be remade (q8)
        for (trees, _), off in zip(groups, offs):
            # level 0 and the inner levels start at multiples of bf (of 16 where tiled): whole
            # tiles copy as they are
            self.keys_buf[trees, off[0]:off[0] + r16(n0)] = sub.keys_buf[trees, : r16(n0)]
            quant.append((off[0], n0))
            if self.values_buf is not None:
                self.values_buf[trees, off[0]:off[0] + n0] = sub.values_buf[trees, :n0]
            self.perm[trees, off[0]:off[0] + n0] = sp[trees]
            for l in range(1, sub_levels):
                k = sub.size[l]
                self.radii[l][trees, off[l]:off[l] + k] = sub.radii[l][trees, :k]
                self.counts[l][trees, off[l]:off[l] + k] = sub.counts[l][trees, :k]
                if not self.tiled:
                    self.centers[l][trees, off[l]:off[l] + k] = sub.centers[l][trees, :k]
                elif off[l] % 16 == 0:
                    self.centers[l][trees, off[l]:off[l] + r16(k)] = sub.centers[l][trees, : r16(k)]
                else:  # the top level starts where the old nodes end: through row-major
                    lo, hi = off[l] // 16 * 16, r16(off[l] + k)
                    rows = from_tiled(self.centers[l][trees, lo:hi])
                    rows[:, off[l] - lo:off[l] - lo + k] = sub.centers_rowmajor(l)[trees, :k]
                    self.centers[l][trees, lo:hi] = to_tiled(rows)
        if under is not None:  # the roots take the sub-tree's top nodes as further children
            k = sub.size[stop]
            ar = torch.arange(self.num_trees, device=self.device)
            rt = under[0].to(self.device)
            c_root = self.centers_rowmajor(nl - 1)[ar, rt].float()
            c_new = sub.centers_rowmajor(stop)[:, :k].float()
            reach = ((c_new - c_root[:, None]).norm(dim=-1) + sub.radii[stop][:, :k]).max(dim=1).values
            self.radii[nl - 1][ar, rt] = torch.maximum(self.radii[nl - 1][ar, rt], reach * (1 + 1e-6))
            self.counts[nl - 1][ar, rt] += k
        size = list(self.size)
        for off in offs:
            for l in range(sub_levels):
                size[l] = max(size[l], off[l] + sub.size[l])
        self.size = size
        for l in range(1, nl):
            self._state[:, l] = torch.maximum(self._state[:, l], torch.tensor(
                [max(off[l] + sub.size[l] for off in offs) if l < sub_levels else 0],
                dtype=torch.int32, device=self.device))
        self._state[:, _lib.HIRA_MAX_LEVELS] += m
        self.num_keys += m
        self._tree_struct = None
        for first, count in quant:  # with the index's own steps (a sub-tree has others)
            self.quantize(first, count)
        return self

    def reserve(self, appends: int) -> "HIPIndexer":
        """Room for `appends` more keys per tree, so that updates up to that many do not
        re-allocate: device pointers (and with them captured graphs and plans) stay valid."""
        if self.keys_buf is None:
            raise ValueError("Indexer is not built: call build() first.")
        self._grow(self._needed_caps(int(appends)))
        return self

    def begin_unsynced(self, appends: int) -> None:
        """Prepare for `appends` updates whose sizes are not read back: room for all of them,
        and level sizes fixed at their bound for the whole stretch (a launch captured now
        stays right until ``sync_sizes``).  The caller reports what it appended through
        ``note_unsynced``."""
        if self.num_levels < 2:
            raise ValueError("needs a tree of at least two levels")
        self.sync_sizes()
        self._unsynced_room = 0  # (the stretch before this one is over: pointers may move now)
        need = self._needed_caps(int(appends))
        self._grow(need)
        if self._state is None:
            self._init_state()
        self._exact_size = list(self.size)
        self.size = [need[1] * self.branching_factor] + list(need[1:])
        self._unsynced_room = int(appends)
        self._tree_struct = None

    def note_unsynced(self, m: int) -> None:
        """`m` keys per tree were appended by a launch outside ``update`` (a graph replay)."""
        if m > self._unsynced_room:
            raise RuntimeError("more appends than begin_unsynced made room for")
        self._unsynced_room -= m
        self._pending += m
        self.num_keys += m

    def _init_state(self) -> None:
        st = torch.zeros((self.num_trees, _lib.HIRA_MAX_LEVELS + 2), dtype=torch.int32)
        for l in range(self.num_levels):
            st[:, l] = self.size[l]
        if self.num_levels >= 2:
            st[:, 0] = 0  # "every level-1 node below this index is full": nothing known yet
        st[:, _lib.HIRA_MAX_LEVELS] = self.num_keys
        self._state = st.to(self.device)

    def sync_sizes(self) -> "HIPIndexer":
        """Read the level sizes back after updates with ``sync=False`` (one small copy that
        waits for the stream) and check that no key was dropped."""
        if self._state is None or (self._pending == 0 and self._exact_size is None):
            return self
        self._adopt_state(self._state.cpu())
        self._unsynced_room = 0
        return self

    def _adopt_state(self, st: torch.Tensor) -> None:
        if int(st[:, _lib.HIRA_MAX_LEVELS + 1].max()) != 0:
            raise RuntimeError("index update ran out of capacity")
        if self.num_levels == 1:
            self.size = [self.num_keys]
        else:
            size = [0] * self.num_levels
            for l in range(1, self.num_levels):
                size[l] = int(st[:, l].max())
            size[0] = size[1] * self.branching_factor
            self.size = size
        self._pending, self._exact_size = 0, None
        self._tree_struct = None

    def update(self, new_keys: torch.Tensor, new_values: Optional[torch.Tensor] = None, *,
               sync: bool = True):
        """Append new_keys (1, H, m, D) (and new_values (1, H, m, Dv)) in order
        (indexer/cuda.py:544-701).  One launch; afterwards the level sizes are read back
        (one small device-to-host copy), as the next search needs them.

        ``sync=False`` skips the read-back: the host then carries upper bounds of the level
        sizes (slots past a tree's real size hold nodes without children, which every search
        prunes at once), nothing waits for the stream, and with ``reserve`` called beforehand
        the call is a single launch on fixed pointers, fit for a captured graph.
        ``sync_sizes`` (or the next update with ``sync=True``) brings the exact sizes back."""
        if self.keys_buf is None:
            raise ValueError("Indexer is not built: call build() first.")
        if new_keys.ndim != 4 or new_keys.shape[0] != self.batch or \
                new_keys.shape[1] != self.num_heads or new_keys.shape[3] != self.dim:
            raise ValueError(
                f"new_keys must be ({self.batch},{self.num_heads},m,{self.dim}), got "
                f"{tuple(new_keys.shape)}")
        if (new_values is None) != (self.values_buf is None):
            raise ValueError("values must be given exactly when the index was built with values")
        m = int(new_keys.shape[2])
        if new_values is not None and tuple(new_values.shape[:3]) != tuple(new_keys.shape[:3]):
            raise ValueError("new_values must be aligned with new_keys")
        if m == 0:
            return self
        if not sync and self.num_levels < 2:
            raise ValueError("sync=False needs a tree of at least two levels (a one-level index "
                             "has no node counts to tell empty key slots by)")
        if self.num_levels >= 2 and (not self.tiled or self.branching_factor % 16 == 0):
            bf, nl = self.branching_factor, self.num_levels
            full = self.graft_min if self.graft_min is not None else max(256, bf ** (nl - 1) // 2)
            part = self.graft_min if self.graft_min is not None else max(256, bf ** (nl - 2) // 2)
            if m >= full:
                return self._graft(new_keys, new_values, m, nl, None)
            if nl >= 3 and m >= part:
                # a mid-size window: further children of an existing root where every tree has
                # one with room, else a new root (whose free child slots take the next ones)
                where = self._room_under_a_root(new_keys, m)
                if where is not None:
                    return self._graft(new_keys, new_values, m, nl - 1, where)
                return self._graft(new_keys, new_values, m, nl, None)
        if not sync and 0 < self._unsynced_room < m:  # (checked before anything is launched)
            raise RuntimeError("more appends than begin_unsynced made room for")
        need = self._needed_caps(m)
        self._grow(need)
        t = self.num_trees
        if self._state is None:
            self._init_state()
        kin = new_keys.to(device=self.device, dtype=self.dtype).reshape(t, m, self.dim).contiguous()
        vin = None
        if new_values is not None:
            vin = new_values.to(device=self.device, dtype=self.dtype).reshape(
                t, m, self.vdim).contiguous()
        tree = self.tree_struct()
        stream = _lib.current_stream(self.device)
        rc = _lib.lib().hira_update(C.byref(tree), kin.data_ptr(),
                                    None if vin is None else vin.data_ptr(), m,
                                    self._state.data_ptr(), stream)
        _lib.check(rc)
        self.num_keys += m
        if sync:
            self._adopt_state(self._state.cpu())
            self._unsynced_room = 0
            return self
        if self._exact_size is None:  # (inside a stretch self.size already holds bounds)
            self._exact_size = list(self.size)
        if self._unsynced_room > 0:   # a stretch opened by begin_unsynced: its room is used up
            self._unsynced_room -= m
        self._pending += m
        bound = [need[1] * self.branching_factor] + list(need[1:])
        bound = [max(a, b) for a, b in zip(bound, self.size)]  # (bounds never shrink)
        if bound != self.size:
            self.size = bound
            self._tree_struct = None
        return self

    _warmed: set = set()

    @torch.no_grad()
    def warm_up(self) -> None:
        """The first append, window append and subtree rebuild of a process pay for code that is
        loaded on first use (this library's kernels, torch's sort / gather / reduction kernels,
        the allocator's first blocks): some 60 ms for the first append and 0.4-0.6 s for the first
        rebuild, in the middle of a decode.  This runs them once on a throw-away index of this
        one's kind (levels, fan-out, row widths, storage type, layout) with a few hundred keys,
        so that a serving process pays at set-up; once per kind and process.  The index itself
        is not touched."""
        if self.keys_buf is None:
            raise ValueError("Indexer is not built: call build() first.")
        kind = (self.num_levels, self.branching_factor, self.dim, self.vdim, self.dtype,
                self.layout_name, str(self.device), self.values_buf is not None)
        if kind in HIPIndexer._warmed:
            return
        HIPIndexer._warmed.add(kind)
        bf = self.branching_factor
        n = 2 * bf ** min(self.num_levels - 1, 2) + 3
        # the smallest window that update() builds as a subtree of its own and grafts in (its
        # own rule, below), where that is small enough for a toy
        big = 0
        if self.num_levels >= 2 and (not self.tiled or bf % 16 == 0):
            big = self.graft_min if self.graft_min is not None else \
                max(256, bf ** max(self.num_levels - 2, 1) // 2)
            big = big if big <= 1024 else 0
        g = torch.Generator().manual_seed(7)
        k = torch.randn((1, 2, n + 9 + big, self.dim), generator=g).to(self.dtype).to(self.device)
        v = None
        if self.values_buf is not None:
            v = torch.randn((1, 2, n + 9 + big, self.vdim), generator=g).to(self.dtype).to(self.device)
        toy = HIPIndexer(self.num_levels, self.max_iterations, bf, seed=self.seed,
                         pack_rounds=self.pack_rounds, layout=self.layout_name,
                         device=str(self.device), graft_min=self.graft_min)
        toy.build(k[:, :, :n], None if v is None else v[:, :, :n])
        if toy.layout_name != self.layout_name:
            return  # (a layout that a toy of this size cannot take: nothing more to run)

        def rows(x, a, b):
            return None if x is None else x[:, :, a:b]

        toy.update(k[:, :, n:n + 1], rows(v, n, n + 1))               # a key
        if self.num_levels >= 2:
            toy.update(k[:, :, n + 1:n + 9], rows(v, n + 1, n + 9), sync=False)  # a window
            if big:
                toy.update(k[:, :, n + 9:n + 9 + big], rows(v, n + 9, n + 9 + big))  # a grafted one
        if self.num_levels >= 3 and not (self.tiled and bf % 16):
            toy.rebuild_subtree(0)
        torch.cuda.synchronize(self.device)

    @torch.no_grad()
    def rebuild_subtree(self, node: int) -> "HIPIndexer":
        """Re-cluster everything under node `node` of level 2 (its bf level-1 nodes and their
        keys), in every tree: appends only ever grow radii around centres that never move
        (indexer/cuda.py:544-701), so a subtree that took many of them is rebuilt from its
        keys now and then.  The keys stay in the subtree's own slots [node*bf*bf,
        (node+1)*bf*bf); its level-1 nodes get new centres, radii and counts; the level-2
        node keeps its centre, gets the radius its new children need, and its ancestors are
        inflated where that radius grew.  One build over all trees (hira_build_ragged: the trees
        hold different numbers of keys there) and a few batched tensor operations; nothing is
        read back to the host."""
        if self.keys_buf is None:
            raise ValueError("Indexer is not built: call build() first.")
        if self.num_levels < 3:
            raise ValueError("rebuild_subtree needs at least three levels")
        bf = self.branching_factor
        if self.tiled and bf % 16:
            raise ValueError("rebuild_subtree on a tiled index needs a fan-out that is a multiple "
                             "of 16 (a subtree's slots must start on a tile)")
        self.sync_sizes()
        if not 0 <= node < self.size[2]:
            raise ValueError(f"level-2 node {node} not in 0..{self.size[2] - 1}")
        T, nsub = self.num_trees, bf * bf
        s0, n0 = node * nsub, node * bf
        if s0 + nsub > self.cap[0] or n0 + bf > self.cap[1]:
            raise ValueError("the subtree's slots lie beyond the capacity of the index")
        # the subtree's keys of every tree, those it holds first (in slot order); how many each
        # tree holds stays on the device: nothing here waits for the GPU
        perm_sub = self.perm[:, s0:s0 + nsub]
        live = perm_sub >= 0
        order = torch.sort((~live).to(torch.uint8), dim=1, stable=True).indices  # (T, nsub)
        counts = live.sum(dim=1, dtype=torch.int32).contiguous()
        rows = self.keys_buf[:, s0:s0 + nsub]
        rows = from_tiled(rows) if self.keys_tiled else rows
        rows = torch.gather(rows, 1, order[:, :, None].expand(-1, -1, self.dim))
        vals = None
        if self.values_buf is not None:
            vals = torch.gather(self.values_buf[:, s0:s0 + nsub], 1,
                                order[:, :, None].expand(-1, -1, self.vdim))
        pos = torch.gather(perm_sub, 1, order)  # insertion positions, the missing ones (-1) last
        # one build over all trees: two levels, bf nodes of bf slots, fewer keys in some trees
        sub = HIPIndexer(2, self.max_iterations, bf, seed=self.seed + node,
                         device=str(self.device), pack_rounds=self.pack_rounds,
                         layout=self.layout_name)
        sub.build(rows.reshape(self.batch, self.num_heads, nsub, self.dim),
                  None if vals is None else vals.reshape(self.batch, self.num_heads, nsub, self.vdim),
                  key_counts=counts)
        if sub.size[0] != nsub or sub.size[1] != bf or sub.tiled != self.tiled or sub.q8 != self.q8:
            raise RuntimeError("sub-tree layout differs from the index's")
        # a node's children fill its slots from the first one on (appends open the next child
        # behind them): the new level-1 nodes that hold keys go first, whole nodes moving with
        # their bf key slots (a node's rows are whole tiles, so tiled rows move as they are)
        cnt1 = sub.counts[1][:, :bf]
        nodes = torch.sort((cnt1 == 0).to(torch.uint8), dim=1, stable=True).indices  # (T, bf)

        def by_node(x, width):  # (T, bf * bf, width) in slot order -> nodes in the new order
            idx = nodes[:, :, None].expand(-1, -1, bf * width)
            return torch.gather(x.reshape(T, bf, bf * width), 1, idx).reshape(T, nsub, width)

        self.keys_buf[:, s0:s0 + nsub] = by_node(sub.keys_buf[:, :nsub], self.dim)
        if vals is not None:
            self.values_buf[:, s0:s0 + nsub] = by_node(sub.values_buf[:, :nsub], self.vdim)
        sp = by_node(sub.perm[:, :nsub, None], 1)[:, :, 0].long()
        self.perm[:, s0:s0 + nsub] = torch.where(
            sp >= 0, torch.gather(pos, 1, sp.clamp(min=0)), torch.full_like(pos, -1))
        c1 = torch.gather(sub.centers_rowmajor(1)[:, :bf], 1,
                          nodes[:, :, None].expand(-1, -1, self.dim))     # (T, bf, D), storage type
        r1 = torch.gather(sub.radii[1][:, :bf], 1, nodes)                  # (T, bf), -inf: empty
        cnt1 = torch.gather(cnt1, 1, nodes)
        self.centers[1][:, n0:n0 + bf] = to_tiled(c1) if self.tiled else c1
        self.radii[1][:, n0:n0 + bf] = r1
        self.counts[1][:, n0:n0 + bf] = cnt1
        # level 2: same centre, the radius its new children need; ancestors cover it where it grew
        c1 = c1.float()
        child, c_child, r_child = node, None, None
        for l in range(2, self.num_levels):
            tile0 = child // 16 * 16  # (de-tiling needs whole tiles)
            cl = self.centers[l][:, tile0:tile0 + 16]
            cl = (from_tiled(cl) if self.tiled else cl)[:, child - tile0].float()  # (T, D)
            if l == 2:
                r = ((c1 - cl[:, None]).norm(dim=2) + r1).amax(dim=1) * (1 + 1e-6)
                self.counts[2][:, child] = (cnt1 > 0).sum(dim=1, dtype=torch.int32)
            else:
                r = torch.maximum(self.radii[l][:, child],
                                  ((c_child - cl).norm(dim=1) + r_child) * (1 + 1e-6))
            self.radii[l][:, child] = r
            c_child, r_child, child = cl, r, child // bf
        if self._state is not None:
            self._state[:, 0] = 0  # the rebuilt nodes may have room again
        self._tree_struct = None
        self.quantize(s0, nsub)
        return self


# the class name the reference's indexer/cuda.py defines (PyTorch-ROCm calls the device "cuda")
CUDAIndexer = HIPIndexer
