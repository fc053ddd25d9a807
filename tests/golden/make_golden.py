"""Write the golden fixtures under tests/golden/ from the reference's own C++ kernels.

Run once in a container that has the reference tree (the compiled kernels live in
oracle/_ref/, built by oracle/build_ref.py from the reference sources in place):

    python tests/golden/make_golden.py

Each case regenerates the seeded inputs of one of the reference's known-answer tests
(tests/test_cpp_kernels.py:226-565: L2-normalised keys/queries from
torch.Generator().manual_seed, 4-level bf=8 tree over 192 keys, per-head quantile
threshold), builds the tree with the oracle's Lloyd restatement (faiss, which the
reference uses for the centroids, is not installed), runs the compiled reference kernels
v1..v4 on that tree and stores inputs, tree and outputs.  The fixtures are data only.
"""
from __future__ import annotations

import sys
from pathlib import Path

import numpy as np
import torch

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))

from oracle import hira_oracle as ho  # noqa: E402
from oracle.build_ref import load_ref  # noqa: E402

OUT = Path(__file__).resolve().parent


def normalized_keys(h, n, d, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((1, h, n, d), generator=g, dtype=torch.float32)
    return (x / x.norm(dim=-1, keepdim=True).clamp_min(1e-12))[0]


def random_query(h, d, seed):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn((h, d), generator=g, dtype=torch.float32)
    return q / q.norm(dim=-1, keepdim=True).clamp_min(1e-12)


# name, h_kv, h_q, n, d, num_levels, bf, key seed, query seed, quantile, q2kv, scaling
CASES = [
    ("kat_h2_d64", 2, 2, 192, 64, 4, 8, 31, 32, 0.75, None, None),
    ("kat_h2_d128", 2, 2, 192, 128, 4, 8, 41, 42, 0.75, None, None),
    ("kat_scaling_d64", 2, 2, 192, 64, 4, 8, 51, 52, 0.8, None, [0.5, 2.0]),
    ("kat_gqa_d64", 2, 6, 192, 64, 4, 8, 301, 302, 0.75, [0, 0, 0, 1, 1, 1], None),
    ("kat_gqa_d128", 2, 6, 192, 128, 4, 8, 301, 302, 0.75, [0, 0, 0, 1, 1, 1], None),
    ("kat_map_1010_d64", 2, 4, 192, 64, 4, 8, 311, 312, 0.8, [1, 0, 1, 0], None),
    ("kat_3level_n769_d32", 3, 3, 769, 32, 3, 4, 61, 62, 0.9, None, None),
]


def run_case(refs, name, h_kv, h_q, n, d, nl, bf, kseed, qseed, quant, q2kv, scaling):
    keys = normalized_keys(h_kv, n, d, kseed)
    query = random_query(h_q, d, qseed)
    q2kv_t = torch.tensor(ho.default_q2kv(h_q, h_kv) if q2kv is None else q2kv, dtype=torch.long)
    sc = torch.ones(h_q) if scaling is None else torch.tensor(scaling, dtype=torch.float32)
    tree = ho.build_cpu_tree(keys.numpy(), nl, bf, max_iterations=2)
    offs, chs = ho.csr_levels(tree)
    gt = torch.einsum("hnd,hd->hn", keys.index_select(0, q2kv_t), query)
    th = torch.quantile(gt, quant, dim=-1)

    T = torch.from_numpy
    centers = [T(l.ball_centers) for l in tree.levels]
    radii = [T(l.ball_radii) for l in tree.levels]
    c2p = [T(l.child2parent) if l.child2parent is not None else torch.empty(0, dtype=torch.long)
           for l in tree.levels]
    sizes = [l.size for l in tree.levels]
    outs = {}
    base = (keys.contiguous(), query, th, centers, radii, c2p, sizes)
    outs["v1"] = refs["v1"].fused_tree_search(*base, q2kv_t, sc).numpy()
    outs["v2"] = refs["v2"].fused_tree_search_v2(*base, q2kv_t, sc).numpy()
    adj = ([T(o) for o in offs], [T(c) for c in chs])
    outs["v3"] = refs["v3"].fused_tree_search_v3(*base, *adj, q2kv_t, sc).numpy()
    if d == 128:
        outs["v4"] = refs["v4"].fused_tree_search_v4(*base, *adj, q2kv_t, sc).numpy()
    sel = {k: (v != 0) for k, v in outs.items()}
    for k in sel:
        assert np.array_equal(sel[k], sel["v3"]), (name, k)
    arrays = dict(keys=keys.numpy(), query=query.numpy(), threshold=th.numpy(),
                  scaling=sc.numpy(), q2kv=q2kv_t.numpy(), num_levels=np.int64(len(tree.levels)),
                  bf=np.int64(bf), out_v3=outs["v3"])
    for k, v in outs.items():
        arrays[f"sel_{k}"] = np.packbits(v != 0, axis=1)
    for l, lev in enumerate(tree.levels):
        if l > 0:
            arrays[f"centers_{l}"] = lev.ball_centers
            arrays[f"radii_{l}"] = lev.ball_radii
        if lev.child2parent is not None:
            arrays[f"c2p_{l}"] = lev.child2parent.astype(np.int32)
    np.savez_compressed(OUT / f"{name}.npz", **arrays)
    print(name, "levels", sizes, "selected", int((outs["v3"] != 0).sum()))


def main():
    refs = {v: load_ref(f"hira_ref_{v}") for v in ("v1", "v2", "v3", "v4")}
    missing = [k for k, m in refs.items() if m is None]
    if missing:
        raise SystemExit(f"reference kernels not built: {missing}; run oracle/build_ref.py")
    for case in CASES:
        run_case(refs, *case)


if __name__ == "__main__":
    main()
