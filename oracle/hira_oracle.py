"""ctypes front end of the CPU oracle (oracle/hira_oracle.c).  TEST INFRASTRUCTURE ONLY.

Only tests/, the smoke check and the benchmark's CPU-baseline leg may import this
module; nothing under hira_amd/ does.  All arrays are numpy, fp32/int64, C-contiguous.

Host-side helpers restate the reference's Python glue:
  build_cpu_tree       indexer/cpu.py:48-122 (bottom-up levels, level_size = prev // bf)
  csr_levels           searcher/cpu.py:280-363 (per-level CSR adjacency)
  search_v3            searcher/cpu.py:206-240 -> kernels/cpp/torch_ext_v3.cpp:149-244
  fixed_fanout_tree    indexer/cuda.py:200-336, 338-538 (padded child blocks of exactly bf
                       slots per parent), with Lloyd centroids instead of sampled points
  radii_from_layout    indexer/cuda.py:114-198
  sample_thresholds    cache/threshold_finder.py:1-14 (the two rules the reference names and
                       leaves unwritten), float64 numpy; pinned against torch's topk / max /
                       mean and the special cases k = 1 (the maximum) and k = all (the mean)

Centroid values of the k-means against faiss (indexer/cpu.py:239-250; faiss is not installed
and not vendored): parity unpinned; see the pinning table at the top of hira_oracle.c.
"""
from __future__ import annotations

import ctypes as C
import subprocess
from dataclasses import dataclass, field
from pathlib import Path
from typing import List, Optional

import numpy as np

HERE = Path(__file__).resolve().parent
_LIBS: dict = {}

_f32p = C.POINTER(C.c_float)
_i64p = C.POINTER(C.c_int64)
_f64p = C.POINTER(C.c_double)
_u8p = C.POINTER(C.c_uint8)


def build_library() -> None:
    """Compile both oracle libraries (strict checker + reference-flag timed build)."""
    subprocess.run(["make", "-C", str(HERE), "-B"], check=True, capture_output=True)


def load(fast: bool = False) -> C.CDLL:
    """Load the strict (default) or the reference-flag (`fast`) oracle library."""
    name = "libhira_oracle_fast.so" if fast else "libhira_oracle.so"
    if name not in _LIBS:
        path = HERE / name
        if not path.exists():
            build_library()
        lib = C.CDLL(str(path))
        lib.hira_oracle_abi_version.restype = C.c_int
        _LIBS[name] = lib
    return _LIBS[name]


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _i64(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.int64)


def _p(a: np.ndarray, t):
    return a.ctypes.data_as(t)


def default_q2kv(h_q: int, h_kv: int) -> np.ndarray:
    """searcher/cpu.py:103-109."""
    if h_q == h_kv:
        return np.arange(h_q, dtype=np.int64)
    assert h_q % h_kv == 0
    return np.arange(h_q, dtype=np.int64) // (h_q // h_kv)


def scores(keys, query, q2kv=None, fast: bool = False) -> np.ndarray:
    keys, query = _f32(keys), _f32(query)
    h_kv, n, d = keys.shape
    h_q = query.shape[0]
    q2kv = _i64(default_q2kv(h_q, h_kv) if q2kv is None else q2kv)
    out = np.empty((h_q, n), dtype=np.float32)
    load(fast).hira_oracle_scores(
        _p(keys, _f32p), C.c_int64(h_kv), C.c_int64(n), C.c_int64(d), _p(query, _f32p),
        C.c_int64(h_q), _p(q2kv, _i64p), _p(out, _f32p))
    return out


def sample_thresholds(samples, query, method: str, k: int = 1, q2kv=None) -> np.ndarray:
    """The two threshold rules the reference names and leaves unwritten
    (cache/threshold_finder.py:1-14; settings in cache/hira_config.py:20-22): per query head,
    the largest score q.x over its tree's samples ("sample_max") or the mean of the k largest
    ("sample_mean_topk").  Scores and the mean in float64."""
    x, q = np.asarray(samples, np.float64), np.asarray(query, np.float64)
    h_q = q.shape[0]
    q2kv = default_q2kv(h_q, x.shape[0]) if q2kv is None else np.asarray(q2kv)
    s = np.einsum("hsd,hd->hs", x[q2kv], q)
    if method == "sample_max":
        return s.max(1).astype(np.float32)
    assert method == "sample_mean_topk" and 1 <= k <= s.shape[1]
    return (-np.sort(-s, axis=1))[:, :k].mean(1).astype(np.float32)


def brute_force(keys, query, th, sc=None, q2kv=None) -> np.ndarray:
    keys, query, th = _f32(keys), _f32(query), _f32(th)
    h_kv, n, d = keys.shape
    h_q = query.shape[0]
    sc = np.ones(h_q, np.float32) if sc is None else _f32(sc)
    q2kv = _i64(default_q2kv(h_q, h_kv) if q2kv is None else q2kv)
    out = np.zeros((h_q, n), dtype=np.float32)
    load().hira_oracle_brute_force(
        _p(keys, _f32p), C.c_int64(h_kv), C.c_int64(n), C.c_int64(d), _p(query, _f32p),
        C.c_int64(h_q), _p(th, _f32p), _p(sc, _f32p), _p(q2kv, _i64p), _p(out, _f32p))
    return out


@dataclass
class Level:
    """indexer/cpu.py:12-21."""
    level_idx: int
    ball_centers: np.ndarray  # (H, K, D) fp32
    ball_radii: np.ndarray  # (H, K) fp32
    size: int
    child2parent: Optional[np.ndarray] = None  # (H, K) int64 -> node at level_idx+1


@dataclass
class CPUTree:
    levels: List[Level] = field(default_factory=list)

    @property
    def keys(self) -> np.ndarray:
        return self.levels[0].ball_centers


def kmeans(x, k: int, niter: int, seed: int):
    """One head.  Returns (centroids (K, D), assign (n,), inertia trace (niter+1,))."""
    x = _f32(x)
    n, d = x.shape
    assert 1 <= k <= n
    cent = np.empty((k, d), np.float32)
    assign = np.empty(n, np.int64)
    trace = np.empty(niter + 1, np.float64)
    load().hira_oracle_kmeans(
        _p(x, _f32p), C.c_int64(n), C.c_int64(d), C.c_int64(k), C.c_int64(niter),
        C.c_uint64(seed), _p(cent, _f32p), _p(assign, _i64p), _p(trace, _f64p))
    return cent, assign, trace


def refine_radii(child_centers, child_radii, assign, parent_centers) -> np.ndarray:
    """One head; indexer/cpu.py:263-311."""
    cc, cr, pc = _f32(child_centers), _f32(child_radii), _f32(parent_centers)
    assign = _i64(assign)
    out = np.empty(pc.shape[0], np.float32)
    load().hira_oracle_refine_radii(
        _p(cc, _f32p), _p(cr, _f32p), _p(assign, _i64p), C.c_int64(cc.shape[0]),
        C.c_int64(cc.shape[1]), _p(pc, _f32p), C.c_int64(pc.shape[0]), _p(out, _f32p))
    return out


def build_cpu_tree(keys, num_levels: int, branching_factor: int, max_iterations: int = 1,
                   seed: int = 12345) -> CPUTree:
    """keys (H, N, D).  Level sizes N, N//bf, ... truncated at num_levels (indexer/cpu.py:78-83);
    per-head k-means seed = seed + 9973*h (indexer/cpu.py:237-238)."""
    keys = _f32(keys)
    h, n, d = keys.shape
    tree = CPUTree()
    tree.levels.append(Level(0, keys, np.zeros((h, n), np.float32), n, None))
    level_size, level_idx, centers = n, 0, keys
    niter = max(int(max_iterations), 1)
    while True:
        level_size //= branching_factor
        if level_size < 1 or level_idx + 1 >= num_levels:
            break
        child = tree.levels[level_idx]
        new_c = np.empty((h, level_size, d), np.float32)
        new_r = np.empty((h, level_size), np.float32)
        assign = np.empty((h, centers.shape[1]), np.int64)
        for hh in range(h):
            new_c[hh], assign[hh], _ = kmeans(centers[hh], level_size, niter, seed + 9973 * hh)
            new_r[hh] = refine_radii(child.ball_centers[hh], child.ball_radii[hh], assign[hh],
                                     new_c[hh])
        child.child2parent = assign
        tree.levels.append(Level(level_idx + 1, new_c, new_r, level_size, None))
        centers = new_c
        level_idx += 1
    return tree


def build_csr(c2p, num_parents: int):
    """(H, C) child->parent ids -> offsets (H, P+1), children (H, C)."""
    c2p = _i64(c2p)
    h, c = c2p.shape
    off = np.empty((h, num_parents + 1), np.int64)
    ch = np.empty((h, c), np.int64)
    lib = load()
    for hh in range(h):
        lib.hira_oracle_build_csr(_p(c2p[hh], _i64p), C.c_int64(c), C.c_int64(num_parents),
                                  _p(off[hh], _i64p), _p(ch[hh], _i64p))
    return off, ch


def csr_levels(tree: CPUTree):
    offs, chs = [], []
    for l, lev in enumerate(tree.levels):
        if lev.child2parent is None:
            offs.append(np.empty(0, np.int64))
            chs.append(np.empty(0, np.int64))
        else:
            o, c = build_csr(lev.child2parent, tree.levels[l + 1].size)
            offs.append(o)
            chs.append(c)
    return offs, chs


def _level_args(tree: CPUTree, offs, chs):
    nl = len(tree.levels)
    cen = [_f32(l.ball_centers) for l in tree.levels]
    rad = [_f32(l.ball_radii) for l in tree.levels]
    offs = [_i64(o) for o in offs]
    chs = [_i64(c) for c in chs]
    sizes = _i64([l.size for l in tree.levels])
    cen_p = (_f32p * nl)(*[_p(a, _f32p) for a in cen])
    rad_p = (_f32p * nl)(*[_p(a, _f32p) for a in rad])
    off_p = (_i64p * nl)(*[_p(a, _i64p) for a in offs])
    ch_p = (_i64p * nl)(*[_p(a, _i64p) for a in chs])
    keep = (cen, rad, offs, chs, sizes)
    return nl, cen_p, rad_p, sizes, off_p, ch_p, keep


def search_v3(tree: CPUTree, query, th, sc=None, rscale=None, q2kv=None, want_stats=False,
              fast: bool = False, num_threads: int = 0, csr=None):
    """query (H_q, D).  Returns out (H_q, N) [, stats (H_q, L+1)]."""
    keys = _f32(tree.keys)
    query, th = _f32(query), _f32(th)
    h_kv, n, d = keys.shape
    h_q = query.shape[0]
    sc = np.ones(h_q, np.float32) if sc is None else _f32(sc)
    rscale = np.ones(h_q, np.float32) if rscale is None else _f32(rscale)
    q2kv = _i64(default_q2kv(h_q, h_kv) if q2kv is None else q2kv)
    offs, chs = csr_levels(tree) if csr is None else csr
    nl, cen_p, rad_p, sizes, off_p, ch_p, keep = _level_args(tree, offs, chs)
    out = np.zeros((h_q, n), np.float32)
    stats = np.zeros((h_q, nl + 1), np.int64)
    load(fast).hira_oracle_search_v3(
        _p(keys, _f32p), C.c_int64(h_kv), C.c_int64(n), C.c_int64(d), _p(query, _f32p),
        C.c_int64(h_q), _p(th, _f32p), _p(sc, _f32p), _p(rscale, _f32p), _p(q2kv, _i64p),
        C.c_int64(nl), cen_p, rad_p, _p(sizes, _i64p), off_p, ch_p, _p(out, _f32p),
        _p(stats, _i64p) if want_stats else None, C.c_int(num_threads))
    del keep
    return (out, stats) if want_stats else out


def group_traffic(tree: CPUTree, query, th, rscale=None, q2kv=None, csr=None) -> np.ndarray:
    """(H_kv, L+1): per KV head, nodes evaluated per level by any head of its group
    (column 0 = candidate keys), last column = keys selected by any head of the group."""
    keys = _f32(tree.keys)
    query, th = _f32(query), _f32(th)
    h_kv, n, d = keys.shape
    h_q = query.shape[0]
    rscale = np.ones(h_q, np.float32) if rscale is None else _f32(rscale)
    q2kv = _i64(default_q2kv(h_q, h_kv) if q2kv is None else q2kv)
    offs, chs = csr_levels(tree) if csr is None else csr
    nl, cen_p, rad_p, sizes, off_p, ch_p, keep = _level_args(tree, offs, chs)
    out = np.zeros((h_kv, nl + 1), np.int64)
    load().hira_oracle_group_traffic(
        _p(keys, _f32p), C.c_int64(h_kv), C.c_int64(n), C.c_int64(d), _p(query, _f32p),
        C.c_int64(h_q), _p(th, _f32p), _p(rscale, _f32p), _p(q2kv, _i64p), C.c_int64(nl),
        cen_p, rad_p, _p(sizes, _i64p), off_p, ch_p, _p(out, _i64p))
    del keep
    return out


def attention(keys, values, query, sc, mask, q2kv=None) -> np.ndarray:
    """fp64 softmax(sc * q.K_S^T) V_S over mask (H_q, N) != 0.  Returns (H_q, Dv) fp64."""
    keys, values, query, sc = _f32(keys), _f32(values), _f32(query), _f32(sc)
    h_kv, n, d = keys.shape
    dv = values.shape[-1]
    h_q = query.shape[0]
    q2kv = _i64(default_q2kv(h_q, h_kv) if q2kv is None else q2kv)
    mask = np.ascontiguousarray(mask, dtype=np.uint8)
    out = np.empty((h_q, dv), np.float64)
    load().hira_oracle_attention(
        _p(keys, _f32p), _p(values, _f32p), C.c_int64(h_kv), C.c_int64(n), C.c_int64(d),
        C.c_int64(dv), _p(query, _f32p), C.c_int64(h_q), _p(sc, _f32p), _p(q2kv, _i64p),
        _p(mask, _u8p), _p(out, _f64p))
    return out


# ----------------------------------------------------------------------------------
# Fixed-fan-out (padded) layout: the shape of tree the device kernels walk.
# ----------------------------------------------------------------------------------
@dataclass
class FixedFanoutTree:
    """Level l has K_l = ceil(K_{l-1} / bf) nodes; children of node p of level l+1 occupy
    slots [p*bf, (p+1)*bf) of level l, filled from slot 0 (`counts`), the rest padded."""
    bf: int
    keys: np.ndarray  # (H, K_1*bf, D) slot order, pad rows = 0
    perm: np.ndarray  # (H, K_1*bf) slot -> original key index, -1 for pad
    centers: List[np.ndarray]  # [l] (H, K_l, D), l >= 1 (index 0 unused -> None)
    radii: List[np.ndarray]  # [l] (H, K_l) fp32, -inf for a node without children
    counts: List[np.ndarray]  # [l] (H, K_l) int32 children in use, l >= 1
    sizes: List[int]  # padded node count per level; sizes[0] = K_1*bf

    @property
    def num_levels(self) -> int:
        return len(self.sizes)


def _pack_level(x: np.ndarray, bf: int, niter: int, seed: int):
    """Cluster the rows of x (n, D) into K = ceil(n/bf) groups of at most bf.
    Returns (centroids (K, D), slots (K, bf) row ids or -1).  Closest-first per centroid
    (indexer/cuda.py:247-307); a row that finds its centroid full goes to the nearest
    centroid that still has room; the centroid of a block is then the mean of its rows."""
    n = x.shape[0]
    k = max(1, -(-n // bf))
    cent, assign, _ = kmeans(x, k, niter, seed)
    own = ((x - cent[assign]) ** 2).sum(-1)
    order = np.lexsort((np.arange(n), own, assign))
    slots = -np.ones((k, bf), np.int64)
    fill = np.zeros(k, np.int64)
    left = []
    for i in order:
        c = assign[i]
        if fill[c] < bf:
            slots[c, fill[c]] = i
            fill[c] += 1
        else:
            left.append(i)
    for i in left:
        free = np.nonzero(fill < bf)[0]
        dd = ((cent[free] - x[i]) ** 2).sum(-1)
        c = free[int(np.argmin(dd))]
        slots[c, fill[c]] = i
        fill[c] += 1
    for c in range(k):
        m = slots[c][slots[c] >= 0]
        if m.size:
            cent[c] = x[m].astype(np.float64).mean(0).astype(np.float32)
    return cent, slots


def radii_from_layout(child_centers, child_radii, child_valid, parent_centers, bf: int):
    """r_p = max over valid children (||c - p|| + r_c); -inf when no valid child.
    Closed form of indexer/cuda.py:114-198 with explicit validity instead of pad detection."""
    k = parent_centers.shape[0]
    cc = child_centers.reshape(k, bf, -1).astype(np.float32)
    diff = cc - parent_centers[:, None, :].astype(np.float32)
    dist = np.sqrt((diff * diff).sum(-1, dtype=np.float32)).astype(np.float32)
    tot = dist + child_radii.reshape(k, bf).astype(np.float32)
    tot = np.where(child_valid.reshape(k, bf), tot, -np.inf).astype(np.float32)
    return tot.max(1)


def fixed_fanout_sizes(n: int, bf: int, num_levels: int) -> List[int]:
    """Padded node count per level: K_1 = ceil(n/bf), K_l = ceil(K_{l-1}/bf); the root keeps
    K_root nodes and every lower level holds bf slots per node of the level above."""
    if num_levels == 1:
        return [n]
    k = n
    for _ in range(1, num_levels):
        k = max(1, -(-k // bf))
    sizes = [0] * num_levels
    sizes[num_levels - 1] = k
    for l in range(num_levels - 2, -1, -1):
        sizes[l] = sizes[l + 1] * bf
    return sizes


def fixed_fanout_tree(keys, bf: int, num_levels: int, niter: int = 1, seed: int = 12345,
                      round_fn=None) -> FixedFanoutTree:
    """keys (H, N, D) -> padded tree with `num_levels` levels (level 0 = keys).
    round_fn (optional) rounds centroids to the storage dtype before radii are taken."""
    keys = _f32(keys)
    h, n, d = keys.shape
    sizes = fixed_fanout_sizes(n, bf, num_levels)
    if num_levels == 1:
        return FixedFanoutTree(bf, keys.copy(), np.tile(np.arange(n), (h, 1)), [None], [None],
                               [None], sizes)
    out_keys = np.zeros((h, sizes[0], d), np.float32)
    perm = -np.ones((h, sizes[0]), np.int64)
    centers = [None] + [np.zeros((h, sizes[l], d), np.float32) for l in range(1, num_levels)]
    radii = [None] + [np.full((h, sizes[l]), -np.inf, np.float32) for l in range(1, num_levels)]
    counts = [None] + [np.zeros((h, sizes[l]), np.int32) for l in range(1, num_levels)]
    top = num_levels - 1
    for hh in range(h):
        x = keys[hh]
        slots_l, cents_l = [None], [None]
        for l in range(1, num_levels):
            cent, slots = _pack_level(x, bf, niter, seed + 9973 * hh + 31 * l)
            if round_fn is not None:
                cent = round_fn(cent)
            slots_l.append(slots)
            cents_l.append(cent)
            x = cent
        # order[l][s] = id (in clustering order) of the level-l node stored at slot s, or -1
        order = {top: -np.ones(sizes[top], np.int64)}
        order[top][: cents_l[top].shape[0]] = np.arange(cents_l[top].shape[0])
        for l in range(top, 0, -1):
            nxt = -np.ones(sizes[l - 1], np.int64)
            for s, node in enumerate(order[l]):
                if node >= 0:
                    nxt[s * bf:(s + 1) * bf] = slots_l[l][node]
            order[l - 1] = nxt
        for l in range(1, num_levels):
            ok = order[l] >= 0
            centers[l][hh][ok] = cents_l[l][order[l][ok]]
        ok0 = order[0] >= 0
        out_keys[hh][ok0] = keys[hh][order[0][ok0]]
        perm[hh] = order[0]
        child_c, child_r, child_ok = out_keys[hh], np.zeros(sizes[0], np.float32), ok0
        for l in range(1, num_levels):
            radii[l][hh] = radii_from_layout(child_c, child_r, child_ok, centers[l][hh], bf)
            blk = child_ok.reshape(sizes[l], bf)
            counts[l][hh] = blk.sum(1).astype(np.int32)
            assert np.all(blk[:, :-1] >= blk[:, 1:])  # children packed from slot 0
            child_c, child_r, child_ok = centers[l][hh], radii[l][hh], counts[l][hh] > 0
    return FixedFanoutTree(bf, out_keys, perm, centers, radii, counts, sizes)


def fixed_fanout_as_cpu_tree(t: FixedFanoutTree):
    """View a padded tree as the reference's level list plus CSR adjacency that lists only
    the children in use (slots [p*bf, p*bf+count[p])), so the v3 walk and the compiled
    reference kernels can run on the very same tree.  Returns (CPUTree, (offsets, children));
    indices are slot indices."""
    h = t.keys.shape[0]
    nl = t.num_levels
    tree = CPUTree()
    offs, chs = [], []
    for l in range(nl):
        if l == 0:
            c, r = t.keys, np.zeros(t.keys.shape[:2], np.float32)
        else:
            c, r = t.centers[l], t.radii[l]
        c2p = None
        if l + 1 < nl:
            c2p = np.tile(np.arange(t.sizes[l], dtype=np.int64) // t.bf, (h, 1))
            cnt = t.counts[l + 1].astype(np.int64)  # (H, K_{l+1})
            off = np.zeros((h, t.sizes[l + 1] + 1), np.int64)
            off[:, 1:] = np.cumsum(cnt, 1)
            ch = np.zeros((h, t.sizes[l]), np.int64)
            for hh in range(h):
                base = np.repeat(np.arange(t.sizes[l + 1], dtype=np.int64) * t.bf, cnt[hh])
                within = np.arange(base.size, dtype=np.int64) - np.repeat(off[hh, :-1], cnt[hh])
                ch[hh, : base.size] = base + within
            offs.append(off)
            chs.append(ch)
        else:
            offs.append(np.empty(0, np.int64))
            chs.append(np.empty(0, np.int64))
        tree.levels.append(Level(l, c, r, t.sizes[l], c2p))
    return tree, (offs, chs)
