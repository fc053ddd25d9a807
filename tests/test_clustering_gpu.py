"""What the build and the append CHOOSE, checked against brute force: a wrong nearest-centre
choice still yields a valid tree (every other test would pass) and only loosens the balls.

* hira_nearest (the assignment kernels of every Lloyd and packing round of hira_build, the
  reference's nearest_l2_triton_batched, kernels/triton_update_kernels.py:6-123, 329-418, and
  the cdist + argmin of indexer/cuda.py:244-264) against a float64 argmin;
* planted clusters: K well-separated centres with exactly bf points each must come back as
  the K level-1 blocks;
* an appended key must land in the nearest level-1 node that still has a free slot, and open
  a node of its own once none has (indexer/cuda.py:544-701)."""
import ctypes as C

import numpy as np
import pytest
import torch

from helpers import bf16_round

pytestmark = pytest.mark.gpu


def _nearest(x: torch.Tensor, centers: torch.Tensor, valid=None):
    from hira_amd import _lib

    lib = _lib.lib()
    t, n, d = x.shape
    m = centers.shape[1]
    dt = _lib.HIRA_BF16 if x.dtype == torch.bfloat16 else _lib.HIRA_F32
    need = lib.hira_nearest_workspace_bytes(dt, t, m, d)
    assert need > 0
    ws = torch.empty(need, dtype=torch.uint8, device=x.device)
    idx = torch.empty((t, n), dtype=torch.int32, device=x.device)
    d2 = torch.empty((t, n), dtype=torch.float32, device=x.device)
    v = None if valid is None else valid.to(torch.int32).contiguous()
    _lib.check(lib.hira_nearest(x.data_ptr(), dt, t, n, centers.data_ptr(), m, d,
                                None if v is None else v.data_ptr(), idx.data_ptr(),
                                d2.data_ptr(), ws.data_ptr(), need,
                                torch.cuda.current_stream().cuda_stream))
    return idx, d2


def _dist64(x, c):
    """Squared distances (t, n, m) in float64 (expanded form: float64 has the digits for it)."""
    return ((x ** 2).sum(-1)[:, :, None] + (c ** 2).sum(-1)[:, None, :]
            - 2.0 * np.einsum("tnd,tmd->tnm", x, c))


NEAREST_CASES = [
    # trees, n rows, m centres, d, dtype, masked
    (2, 3000, 100, 128, torch.bfloat16, False),   # matrix cores
    (1, 1000, 1024, 128, torch.bfloat16, True),
    (3, 777, 37, 64, torch.bfloat16, True),       # ragged tiles of rows and of centres
    (1, 2000, 300, 256, torch.bfloat16, False),
    (2, 1500, 90, 128, torch.float32, True),      # vector ALUs
    (2, 500, 33, 48, torch.bfloat16, False),      # bf16 rows of a width the matrix-core kernel does not take
]


@pytest.mark.parametrize("case", NEAREST_CASES, ids=[f"t{c[0]}_n{c[1]}_m{c[2]}_d{c[3]}_"
                                                       f"{'bf16' if c[4] == torch.bfloat16 else 'f32'}"
                                                       f"{'_masked' if c[5] else ''}" for c in NEAREST_CASES])
def test_nearest_centre_matches_float64_argmin(case, gpu_device):
    """Centres are fp32 numbers with all 24 bits in use (means of many rows), offset from the
    origin so that ||c||^2 dwarfs the differences between neighbours: rounding the centres to
    bf16 (using only one half of the split) would pick another centre for a good share of the
    rows; the split must not."""
    t, n, m, d, dtype, masked = case
    print(f"case {case}", flush=True)
    g = torch.Generator().manual_seed(1000 + n + m)
    off = 4.0 * torch.randn((t, 1, d), generator=g)
    cen = (off + torch.randn((t, m, d), generator=g)).float()
    x = (off + 1.2 * torch.randn((t, n, d), generator=g)).to(dtype)
    valid = (torch.rand((t, m), generator=g) < 0.6) if masked else None
    if masked:
        valid[:, 0] = True
    idx, d2 = _nearest(x.cuda(), cen.cuda(), None if valid is None else valid.cuda())
    idx, d2 = idx.cpu().numpy(), d2.cpu().numpy().astype(np.float64)
    xd, cd = x.double().numpy(), cen.double().numpy()
    dist = _dist64(xd, cd)                                               # (t, n, m) float64
    if masked:
        dist = np.where(valid.numpy()[:, None, :], dist, np.inf)
    best = dist.argmin(-1)
    dbest = np.take_along_axis(dist, best[..., None], -1)[..., 0]
    dgot = np.take_along_axis(dist, idx[..., None].astype(np.int64), -1)[..., 0]
    assert (idx >= 0).all() and (idx < m).all()
    assert np.isfinite(dgot).all(), "a masked centre was chosen"
    # the chosen centre is the nearest one up to fp32 rounding of the products
    scale = (xd ** 2).sum(-1) + (cd ** 2).sum(-1).max(-1)[:, None]
    tol = 2e-5 * scale
    assert ((dgot - dbest) <= tol).all(), float(((dgot - dbest) / scale).max())
    assert (idx == best).mean() > 0.98
    np.testing.assert_allclose(d2, dgot, rtol=1e-4, atol=float(tol.max()))
    # control: with centres rounded to bf16 (one half of the split only) the same check fails,
    # so it does tell the split from a plain bf16 product
    if dtype == torch.bfloat16 and d in (64, 128, 256):
        cr = cen.to(torch.bfloat16).double().numpy()
        dr = _dist64(xd, cr)
        if masked:
            dr = np.where(valid.numpy()[:, None, :], dr, np.inf)
        d_ctl = np.take_along_axis(dist, dr.argmin(-1)[..., None], -1)[..., 0]
        assert ((d_ctl - dbest) > tol).any()


def test_nearest_centre_no_valid_centre(gpu_device):
    x = torch.randn((1, 40, 64)).to(torch.bfloat16).cuda()
    cen = torch.randn((1, 20, 64)).cuda()
    idx, d2 = _nearest(x, cen, torch.zeros((1, 20), dtype=torch.bool).cuda())
    assert bool((idx == -1).all()) and bool(torch.isinf(d2).all())


def _planted(t, k, bf, d, seed, spread=0.05):
    """k centres at pairwise distance ~ sqrt(2), bf points each within ~spread of their centre;
    the points of a cluster are consecutive (the build draws one initial centroid from every
    stretch of n/K consecutive rows), their order inside the cluster is shuffled."""
    g = torch.Generator().manual_seed(seed)
    cen = torch.randn((t, k, d), generator=g)
    cen = cen / cen.norm(dim=-1, keepdim=True)
    pts = cen[:, :, None, :] + spread * torch.randn((t, k, bf, d), generator=g) / d ** 0.5
    return cen, pts.reshape(t, k * bf, d)


@pytest.mark.parametrize("d,dtype,bf,k", [(128, torch.bfloat16, 32, 96), (64, torch.bfloat16, 16, 200),
                                          (256, torch.bfloat16, 16, 64), (128, torch.float32, 32, 64),
                                          (64, torch.float32, 8, 100)],
                         ids=["d128_bf16", "d64_bf16", "d256_bf16", "d128_f32", "d64_f32"])
def test_planted_clusters_come_back_as_blocks(d, dtype, bf, k, gpu_device):
    from hira_amd.indexer.hip import HIPIndexer

    t = 2
    cen, pts = _planted(t, k, bf, d, seed=d + bf + k)
    keys = pts.to(dtype)
    idx = HIPIndexer(2, 3, bf).build(keys[None].cuda())
    torch.cuda.synchronize()
    assert idx.size == [k * bf, k]
    perm = idx.perm[:, : k * bf].cpu().numpy()
    assert (perm >= 0).all()
    blocks = (perm // bf).reshape(t, k, bf)             # planted cluster of every slot
    assert (blocks == blocks[:, :, :1]).all(), "a level-1 block mixes planted clusters"
    assert all(len(set(blocks[h, :, 0].tolist())) == k for h in range(t))
    # the balls are as tight as the planted spread allows
    kf = keys.float()
    spread = (kf.reshape(t, k, bf, d) - kf.reshape(t, k, bf, d).mean(2, keepdim=True)).norm(dim=-1).amax(-1)
    rad = idx.radii[1][:, :k].cpu()
    which = torch.from_numpy(blocks[:, :, 0])
    want = torch.gather(spread, 1, which)
    assert bool((rad <= want * 1.02 + 4e-3).all()), float((rad - want).max())
    assert bool((idx.counts[1][:, :k] == bf).all())


def _host_nearest_with_room(key, centers, counts, bf):
    """Distances in float64 from the stored centres; nodes in use (count > 0) with a free slot."""
    ok = (counts > 0) & (counts < bf)
    if not ok.any():
        return -1, None
    dist = ((centers.astype(np.float64) - key.astype(np.float64)[None]) ** 2).sum(-1)
    dist = np.where(ok, dist, np.inf)
    return int(dist.argmin()), dist


@pytest.mark.parametrize("dtype,d,bf,nl,n0", [(torch.bfloat16, 128, 32, 3, 2000), (torch.float32, 64, 8, 3, 500),
                                              (torch.bfloat16, 64, 16, 2, 1000)],
                         ids=["bf16_tiled", "f32", "bf16_two_levels"])
def test_append_lands_in_the_nearest_node_with_room(dtype, d, bf, nl, n0, gpu_device):
    """Key by key: the host predicts the node from the index as it stands (nearest level-1
    centre among the nodes in use with a free slot; none: a new node after the last one in use,
    centred on the key) and the device must agree."""
    from hira_amd.indexer.hip import HIPIndexer

    rnd = bf16_round if dtype == torch.bfloat16 else (lambda a: a)
    rng = np.random.default_rng(n0)
    keys = rnd(rng.normal(size=(2, n0, d)).astype(np.float32))
    idx = HIPIndexer(nl, 1, bf, graft_min=1 << 30).build(torch.from_numpy(keys)[None].to(dtype).cuda())
    c0 = idx.counts[1][:, : idx.size[1]]
    room = ((bf - c0) * (c0 > 0)).sum(dim=1)     # free slots in the nodes in use, per tree
    assert int(room.min()) > 0, "the case needs nodes with room"
    steps = int(room.max()) + 3                  # fill every free slot, then three more
    new = rnd(rng.normal(size=(2, steps, d)).astype(np.float32))
    opened = 0
    for i in range(steps):
        k1 = idx.size[1]
        cen = idx.centers_rowmajor(1)[:, :k1].float().cpu().numpy()
        cnt = idx.counts[1][:, :k1].cpu().numpy()
        idx.update(torch.from_numpy(new[:, i:i + 1])[None].to(dtype).cuda())
        perm = idx.perm[:, : idx.size[0]].cpu().numpy()
        for h in range(2):
            slot = int(np.nonzero(perm[h] == n0 + i)[0][0])
            node = slot // bf
            want, dist = _host_nearest_with_room(new[h, i], cen[h], cnt[h], bf)
            if want >= 0:
                assert dist[node] <= dist[want] * (1 + 1e-5) + 1e-6, (i, h, node, want)
                assert slot == node * bf + cnt[h][node]
            else:
                # a node that was not in use: past the level's size, or a free child slot of
                # the level above
                assert (node >= k1 or cnt[h][node] == 0) and slot == node * bf, (i, h, node, k1)
                c_new = idx.centers_rowmajor(1)[h, node].float().cpu().numpy()
                assert np.array_equal(c_new, new[h, i])
                assert int(idx.counts[1][h, node]) == 1
                opened += 1
    assert opened >= 2, "the case never ran out of room"
