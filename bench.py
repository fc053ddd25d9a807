#!/usr/bin/env python3
"""Decode benchmark: one "step" = index search + sparse attention for one fresh query of every
head of one layer (32 query / 8 KV heads, d = 128, bf16) over a 32k-token context; keys,
values, index, queries and thresholds are resident in HBM before the timed region starts.

    python bench.py [--gpus 1] [--steps 256] [--warmup 16] [--config 2]

Prints ONE JSON line.  `value` = microseconds per step (whole layer, all heads) with the K
steps replayed back to back from one HIP graph; `roofline` prices the search kernel against
HBM bandwidth using the ALGORITHMIC bytes of the walk (nodes evaluated x (d*e + 4) +
candidate keys x d*e + selected values x d*e + queries + output; counted by the kernel's
own counters, which the tests tie to the CPU oracle); `cpu_baseline` times the reference's
own C++ search kernel (compiled into oracle/_ref) -- or, if that is absent, the C
restatement in oracle/ -- plus a host softmax-V, on a bounded sample of the same steps, and
the CPU index build (the oracle's restatement of the reference's CPU indexer) of one tree.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def algorithmic_bytes(stats, w, num_levels, steps, shadow=False):
    """Mean algorithmic bytes per step from the device counters summed over `steps` steps.
    stats: (T, HIRA_STATS_COLS) int64.  Scan of the bf16 keys: every candidate key costs its row
    (d*e bytes).  Scan of the 8-bit shadow (`shadow`): a candidate costs d bytes, and the rows
    that the shadow cannot rule out (counted by the kernel) cost their bf16 row on top; a node
    costs four more bytes (its error bound).  Returns (bytes of the path that ran, bytes by the
    bf16-scan formula for the same walk, counts)."""
    import numpy as np
    from hira_amd import _lib

    e = 2 if str(w.dtype).endswith("bfloat16") else 4
    s = stats.astype(np.float64).sum(0) / steps
    nodes = sum(s[l] for l in range(1, num_levels))
    cand = s[0]
    sel_any = s[_lib.HIRA_MAX_LEVELS]
    fetched = s[_lib.HIRA_MAX_LEVELS + 2]
    h_q = w.h_q * w.batch
    b_attn = sel_any * w.d * e + h_q * w.d * 4 + h_q * w.d * e
    b_bf16 = nodes * (w.d * e + 4) + cand * w.d * e + b_attn
    b_ran = b_bf16
    if shadow:
        b_ran = nodes * (w.d * e + 8) + cand * w.d + fetched * w.d * e + b_attn
    return b_ran, b_bf16, dict(nodes_per_step=nodes, candidates_per_step=cand,
                               selected_union_per_step=sel_any,
                               selected_pairs_per_step=s[_lib.HIRA_MAX_LEVELS + 1],
                               exact_rows_per_step=fetched)


def measured_traffic(workload_name):
    """HBM bytes per launch of the search kernel from the committed rocprofv3 --pmc summary
    (FETCH_SIZE + WRITE_SIZE, each scaled by what the same counter reads for a kernel of
    known traffic), or None when no summary for this workload is committed."""
    f = ROOT / "profiles" / f"search_traffic_{workload_name}.txt"
    if not f.exists():
        return None
    try:
        return json.loads(f.read_text())["hbm_bytes_per_launch"]
    except Exception:  # noqa: BLE001
        return None


def cpu_index_build(w, keys_slots, perm):
    """The reference's CPU indexer (indexer/cpu.py:48-122: bottom-up k-means levels, radii from
    the assignment) on ONE tree of the workload -- a bounded sample: the trees are independent
    and alike -- restated in oracle/ with a plain Lloyd k-means where the reference calls faiss
    (not installed here): kind "port", one thread."""
    import numpy as np
    from oracle import hira_oracle as ho

    live = perm[0] >= 0
    keys = np.ascontiguousarray(keys_slots[0][live][np.argsort(perm[0][live])])[None]  # insertion order
    n_all = keys.shape[1]
    keys = keys[:, :32768]  # (bounded: k-means over n keys and n / bf centroids grows with n^2)
    t0 = time.perf_counter()
    tree = ho.build_cpu_tree(keys, w.num_levels, w.bf, max_iterations=w.kmeans_iters)
    dt = time.perf_counter() - t0
    trees = w.batch * w.h_kv
    return {"build_ms_one_tree": round(dt * 1e3, 1), "trees": trees, "kind": "port", "cores": 1,
            "build_ms_all_trees_one_core": round(dt * 1e3 * trees, 1),
            "levels": [int(l.size) for l in tree.levels], "kmeans_iters": w.kmeans_iters,
            "keys_built": int(keys.shape[1]), "keys_in_tree": int(n_all),
            "sample": "tree 0 of the workload (keys of KV head 0 of sequence 0; its first 32768 keys "
                      "where it holds more), built once"}


def host_cpu():
    """The host this process runs on: model name, logical CPUs of the machine, physical cores,
    and the logical CPUs this process may use (the box's share of a shared machine)."""
    model, cores = "unknown", set()
    try:
        phys = core = None
        for line in open("/proc/cpuinfo", encoding="utf-8", errors="replace"):
            key, _, val = line.partition(":")
            key, val = key.strip(), val.strip()
            if key == "model name" and model == "unknown":
                model = val
            elif key == "physical id":
                phys = val
            elif key == "core id":
                core = val
            elif not key and phys is not None and core is not None:
                cores.add((phys, core))
                phys = core = None
    except OSError:
        pass
    try:
        usable = len(os.sched_getaffinity(0))
    except AttributeError:
        usable = os.cpu_count() or 1
    return {"cpu_model": model, "nproc": os.cpu_count() or 1, "physical_cores": len(cores) or None,
            "usable_cpus": usable}


def cpu_baseline(w, index, queries, taus, scale, budget_s=20.0, gpu_out=None, gpu_sel=None):
    """Reference CPU search (+ host softmax-V) on the same trees, first steps of the same
    queries, for about `budget_s` seconds of CPU work; one sequence after the other when the
    workload holds several.  With the GPU's results for the same steps (`gpu_out` (steps,
    B*H_q, Dv) attention outputs, `gpu_sel(i)` -> (B*H_q, N_slots) bool selection of step i) the
    two are compared on the way: selected sets outside a 1e-5 |tau| band, attention outputs."""
    import numpy as np
    import torch
    from oracle import hira_oracle as ho
    from oracle.build_ref import load_ref

    # threads: the host cores this process may use (the box's share of a shared machine is what
    # OMP_NUM_THREADS says), at most one per query head -- the reference kernel's parallel loop
    # is over the heads (kernels/cpp/torch_ext_v3.cpp:149)
    try:
        usable = len(os.sched_getaffinity(0))
    except AttributeError:
        usable = os.cpu_count() or 1
    threads = max(1, min(usable, int(os.environ.get("OMP_NUM_THREADS", "16")), w.h_q))
    torch.set_num_threads(threads)
    n0 = index.size[0]
    keys_all = index.keys_rowmajor().float().cpu().numpy()
    perm_all = index.perm[:, :n0].cpu().numpy().astype(np.int64)
    cen_all = [None] + [index.centers_rowmajor(l).float().cpu().numpy() for l in range(1, index.num_levels)]
    rad_all = [None] + [index.radii[l][:, : index.size[l]].cpu().numpy() for l in range(1, index.num_levels)]
    cnt_all = [None] + [index.counts[l][:, : index.size[l]].cpu().numpy() for l in range(1, index.num_levels)]
    vals_all = index.values_buf[:, :n0].float().cpu().numpy()
    ref = None
    try:
        ref = load_ref("hira_ref_v3")
    except Exception as ex:  # noqa: BLE001
        log(f"[cpu_baseline] compiled reference not loadable ({ex}); timing the C port")
    q2kv = ho.default_q2kv(w.h_q, w.h_kv)
    T = torch.from_numpy
    seqs = []
    for b in range(w.batch):
        hs = slice(b * w.h_kv, (b + 1) * w.h_kv)
        pick = lambda arr: [None] + [a[hs] for a in arr[1:]]  # noqa: E731
        ff = ho.FixedFanoutTree(bf=index.branching_factor, keys=keys_all[hs], perm=perm_all[hs],
                                centers=pick(cen_all), radii=pick(rad_all), counts=pick(cnt_all),
                                sizes=list(index.size))
        tree, csr = ho.fixed_fanout_as_cpu_tree(ff)
        args_tree = None
        if ref is not None:
            args_tree = ([T(l.ball_centers) for l in tree.levels], [T(l.ball_radii) for l in tree.levels],
                         [T(l.child2parent) if l.child2parent is not None
                          else torch.empty(0, dtype=torch.long) for l in tree.levels],
                         [l.size for l in tree.levels], [T(o) for o in csr[0]], [T(c) for c in csr[1]])
        seqs.append((ff, tree, csr, args_tree, T(ff.keys), vals_all[hs]))

    def one_step(i, nthreads):
        if ref is not None:
            os.environ["OMP_NUM_THREADS"] = str(nthreads)
            torch.set_num_threads(nthreads)
        qa = queries[i].float().cpu().numpy().reshape(w.batch, w.h_q, w.d)
        tha = taus[i].cpu().numpy().reshape(w.batch, w.h_q)
        sc = np.full(w.h_q, scale, np.float32)
        outs, os_ = [], []
        t0 = time.perf_counter()
        for b, (ff, tree, csr, args_tree, keys_t, vals) in enumerate(seqs):
            q, th = qa[b], tha[b]
            qn = np.linalg.norm(q, axis=1).astype(np.float32)
            if ref is not None:
                # unit-norm query, threshold and scaling rescaled: the same set, the bound the
                # reference assumes (searcher/cpu.py:61-63)
                out = ref.fused_tree_search_v3(keys_t, T(q / qn[:, None]), T(th / qn), *args_tree,
                                               T(q2kv), T(sc * qn)).numpy()
            else:
                out = ho.search_v3(tree, q, th, sc, rscale=qn, q2kv=q2kv, csr=csr, fast=True,
                                   num_threads=nthreads)
            # host attention over the selected keys, fp32
            o = np.zeros((w.h_q, w.d), np.float32)
            for h in range(w.h_q):
                idx = np.nonzero(out[h])[0]
                if idx.size:
                    z = out[h, idx]
                    p = np.exp(z - z.max())
                    o[h] = (p[:, None] * vals[q2kv[h], idx]).sum(0) / p.sum()
            outs.append(out)
            os_.append(o)
        return time.perf_counter() - t0, np.concatenate(outs), np.concatenate(os_)

    one_step(0, threads)  # warm-up
    times, times1 = [], []
    attn_err, set_diff, band_flips, compared = 0.0, 0, 0, 0
    t_start = time.perf_counter()
    i = 0
    while i < len(queries) and (time.perf_counter() - t_start) < budget_s * 0.75:
        dt, out, o = one_step(i, threads)
        times.append(dt)
        if gpu_out is not None:
            # the sets first: only scores within rounding of tau may be decided differently;
            # the heads where that happened are left out of the comparison of the outputs
            same_set = np.ones(w.batch * w.h_q, bool)
            if gpu_sel is not None:
                tha = taus[i].cpu().numpy().reshape(-1)
                qa = queries[i].float().cpu().numpy().reshape(-1, w.d)
                kv = np.repeat(np.arange(w.batch * w.h_kv), w.h_q // w.h_kv)
                diff = (out != 0) != gpu_sel(i)
                for h, j in zip(*np.nonzero(diff)):
                    same_set[h] = False
                    sco = float(keys_all[kv[h], j] @ qa[h])
                    if abs(sco - tha[h]) > 1e-5 * abs(tha[h]):
                        set_diff += 1
                    else:
                        band_flips += 1
            g = gpu_out[i].float().cpu().numpy()
            den = np.abs(o).max(axis=1, keepdims=True) + 1e-30
            err = (np.abs(g - o) / den).max(axis=1)
            if same_set.any():
                attn_err = max(attn_err, float(err[same_set].max()))
            compared += 1
        i += 1
    t_start = time.perf_counter()
    j = 0
    while j < len(queries) and (time.perf_counter() - t_start) < budget_s * 0.25:
        dt, _, _ = one_step(j, 1)
        times1.append(dt)
        j += 1
    times, times1 = np.array(times), np.array(times1)
    res = dict(value=float(np.median(times) * 1e6), unit="us/layer", cores=threads,
               kind="reference" if ref is not None else "port",
               sample=f"first {len(times)} of the timed decode steps (same trees, queries, "
                      f"thresholds); median; p99 {float(np.percentile(times, 99) * 1e6):.0f} us; "
                      f"search = reference v3 C++ kernel, attention = numpy fp32",
               one_thread_us=float(np.median(times1) * 1e6), one_thread_steps=len(times1))
    res.update(host_cpu())  # (`cores` above: the threads the timed kernel used)
    res["index_build"] = cpu_index_build(w, keys_all, perm_all)
    if gpu_out is not None:
        res["gpu_vs_cpu"] = {"steps_compared": compared, "attn_max_rel_err": attn_err,
                             "selected_set_mismatches": set_diff if gpu_sel is not None else None,
                             "decided_differently_within_1e-5_of_tau": band_flips}
    return res


def streaming(a, w, index, plan, q_d, taus, out, dev):
    """Decode with a growing index: per step one key/value per tree is appended (one update
    launch), then one search + attention over the index as it stands; every
    a.rebuild_every steps one level-2 subtree is re-clustered (round-robin).  Times are GPU
    times between events.  The appends do not read the level sizes back (update(sync=False)
    after reserve(): the host carries bounds); the sizes are re-read before every rebuild."""
    import torch

    from hira_amd import synth

    S = a.stream
    sk, sv = synth.make_stream(w, S)
    # one contiguous (B, H, 1, D) tensor per token, as a model's decode step hands them over
    sk = sk.to(dev).permute(2, 0, 1, 3).contiguous()[:, :, :, None, :]
    sv = sv.to(dev).permute(2, 0, 1, 3).contiguous()[:, :, :, None, :]
    index.reserve(S)  # room for all appends: no re-allocation while timed
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(S)]
    rb = []
    nq = q_d.shape[0]
    torch.cuda.synchronize()
    t_host_upd = 0.0
    for t in range(S):
        ev[t][0].record()
        h0 = time.perf_counter()
        index.update(sk[t], sv[t], sync=False)
        t_host_upd += time.perf_counter() - h0
        ev[t][1].record()
        plan.run(q_d[t % nq], taus[t % nq], out)
        ev[t][2].record()
        if a.rebuild_every > 0 and (t + 1) % a.rebuild_every == 0 and index.num_levels >= 3:
            r0, r1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            r0.record()
            index.rebuild_subtree(((t + 1) // a.rebuild_every - 1) % index.size[2])
            r1.record()
            rb.append((r0, r1))
    torch.cuda.synchronize()
    upd = [e[0].elapsed_time(e[1]) * 1e3 for e in ev]
    sea = [e[1].elapsed_time(e[2]) * 1e3 for e in ev]
    upd.sort()
    sea.sort()
    res = {"steps": S, "keys_after": index.num_keys, "level_sizes": index.size,
           "update_us_per_step": {"mean": round(sum(upd) / S, 2), "median": round(upd[S // 2], 2),
                                  "p99": round(upd[min(S - 1, int(S * 0.99))], 2)},
           "update_host_us_per_step": round(t_host_upd * 1e6 / S, 2),
           "search_attn_us_per_step": {"mean": round(sum(sea) / S, 2),
                                       "median": round(sea[S // 2], 2),
                                       "p99": round(sea[min(S - 1, int(S * 0.99))], 2)},
           "subtree_rebuilds": len(rb),
           "rebuild_ms_each": [round(x.elapsed_time(y), 2) for x, y in rb]}
    # the same step (append, search + attention) captured as one graph and replayed per token:
    # no read-back, no host work between the launches; sizes re-read every 512 tokens
    from hira_amd.searcher import StreamingStep

    sk2, sv2 = synth.make_stream(w, S)  # (same drift again: only the timing matters here)
    sk2, sv2 = sk2.to(dev), sv2.to(dev)
    step = StreamingStep(plan.searcher, index, q_d.shape[1], plan.scaling, horizon=512)
    for t in range(8):
        step.step(sk2[:, :, t], sv2[:, :, t], q_d[t % nq], taus[t % nq])
    torch.cuda.synchronize()
    g0, g1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    h0 = time.perf_counter()
    g0.record()
    for t in range(8, S):
        step.step(sk2[:, :, t], sv2[:, :, t], q_d[t % nq], taus[t % nq])
    g1.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - h0) * 1e6 / (S - 8)
    res["graph_step"] = {"steps": S - 8, "us_per_step_wall": round(wall, 2),
                         "us_per_step_events": round(g0.elapsed_time(g1) * 1e3 / (S - 8), 2),
                         "keys_after": index.num_keys}
    # the graph alone, for callers whose own kernels write the step's buffers (no copies in)
    n2 = 256
    step.replay()  # (may be the one that re-captures)
    torch.cuda.synchronize()
    h0 = time.perf_counter()
    for _ in range(n2):
        step.replay()
    torch.cuda.synchronize()
    res["graph_step"]["us_per_step_replay_only"] = round((time.perf_counter() - h0) * 1e6 / max(n2, 1), 2)
    # the same with the thresholds taken from a key sample inside the step (512 keys a tree, mean
    # of the 8 best): the append and the thresholds share a launch (hira_update_threshold)
    index.sync_sizes()
    rows = index.keys_rowmajor()
    pick = torch.linspace(0, w.n - 1, 512, device=rows.device).long()
    live = index.perm[:, : index.size[0]] >= 0
    samples = torch.stack([rows[t][live[t]][pick] for t in range(index.num_trees)]).contiguous()
    step2 = StreamingStep(plan.searcher, index, q_d.shape[1], plan.scaling, horizon=512, samples=samples,
                          method="sample_mean_topk", k=8)
    step2.step(sk2[:, :, 0], sv2[:, :, 0], q_d[0])
    for _ in range(8):
        step2.replay()
    torch.cuda.synchronize()
    h0 = time.perf_counter()
    for _ in range(n2):
        step2.replay()
    torch.cuda.synchronize()
    res["graph_step_sampled_thresholds"] = {
        "samples_per_tree": 512, "rule": "mean of the 8 best",
        "us_per_step_replay_only": round((time.perf_counter() - h0) * 1e6 / n2, 2)}
    log(f"[bench] streaming: {res}")
    return res


# columns of a workgroup's row of time stamps (hira_amd/csrc/search_mfma_timeline.h)
TL_STAMPS = ["start", "arguments in registers", "gate operands asked for", "wave 0 gated",
             "barrier behind the gates", "first key tiles asked for", "wave 0: first products done",
             "wave 0: first round listed", "wave 0: first round gathered", "wave 0 at the merge",
             "all waves at the merge", "partial on its way", "partial arrived", "ticket drawn",
             "fold: partials listed", "fold: output written"]
TL_ROWS, TL_ROUNDS, TL_ALIVE = 16, 17, 18
TL_WAVE_END, TL_WAVE_ROWS, TL_WAVE_SCANNED, TL_WAVE_ISSUED, TL_WAVE_CONSUMED, TL_COLS = 24, 32, 40, 48, 56, 64


def timeline_report(a, w, index, searcher, q_d, taus, outs, W, total, scale):
    """Steps on the library built with time stamps: per phase, when the workgroups of a step
    reach it (microseconds after the step's first workgroup started; mean over the steps of the
    minimum / mean / maximum over the workgroups), and the differences between consecutive
    phases on the path of the workgroup that finishes last (the one that folds last)."""
    import numpy as np
    import torch

    dev = q_d.device
    h_all = w.batch * w.h_q
    # a row per workgroup: a tree is walked by at most 128 workgroups plus one for a queue, per
    # pass of 16 heads
    passes = (-(-h_all // index.num_trees) + 15) // 16
    nwg = index.num_trees * 129 * max(passes, 1)
    tl = torch.zeros((nwg, TL_COLS), dtype=torch.int64, device=dev)
    plan = searcher.plan_attention(index, h_all, scaling=torch.full((h_all,), scale), stats=tl)
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
    per_step, lens, wave_rows, wave_end, crit = [], [], [], [], []
    for i in range(W, total):
        tl.zero_()
        torch.cuda.synchronize()
        ev[0].record()
        plan.run(q_d[i], taus[i], outs[i])
        ev[1].record()
        torch.cuda.synchronize()
        t = tl.cpu().numpy()
        t = t[t[:, 0] != 0]
        t0 = t[:, 0].min()
        r = (t[:, :16] - t0) / 100.0  # the clock runs at 100 MHz
        r[t[:, :16] == 0] = np.nan
        per_step.append(np.stack([np.nanmin(r, 0), np.nanmean(r, 0), np.nanmax(r, 0)]))
        lens.append(ev[0].elapsed_time(ev[1]) * 1e3)
        we = (t[:, TL_WAVE_END:TL_WAVE_END + 8] - t0) / 100.0
        ok = t[:, TL_WAVE_END:TL_WAVE_END + 8] != 0
        wave_end.append(we[ok])
        wave_rows.append(t[:, TL_WAVE_ROWS:TL_WAVE_ROWS + 8][ok])
        # the workgroup whose fold ends last: its own stamps, phase by phase
        last = np.nanargmax(np.where(np.isnan(r[:, 15]), -1.0, r[:, 15]))
        crit.append(r[last])
    m = np.nanmean(np.stack(per_step), 0)
    c = np.nanmean(np.stack(crit), 0)
    print(f"# where a decode step goes: {w.name}, {total - W} steps, library with time stamps")
    print(f"# step between HIP events (eager launch, stamps on): mean {np.mean(lens):.2f} us")
    print("# microseconds after the first workgroup's start; min / mean / max over the "
          "workgroups, mean over the steps; last column: the workgroup that folds last")
    print(f"{'phase':34s} {'min':>7s} {'mean':>7s} {'max':>7s} {'last folder':>12s} {'its step':>9s}")
    prev = 0.0
    for k, name in enumerate(TL_STAMPS):
        step = c[k] - prev if not np.isnan(c[k]) else float('nan')
        print(f"{name:34s} {m[0, k]:7.2f} {m[1, k]:7.2f} {m[2, k]:7.2f} {c[k]:12.2f} {step:9.2f}")
        if not np.isnan(c[k]):
            prev = c[k]
    print("# workgroups of the last step by when all their waves are at the merge: nodes that "
          "survived the gates, rows listed, the waves' arrival times")
    merged = np.where(np.isnan(r[:, 10]), -1.0, r[:, 10])
    alive_n = t[:, TL_ALIVE].astype(float)
    rows_wg = t[:, TL_WAVE_ROWS:TL_WAVE_ROWS + 8].sum(1).astype(float)
    for k in np.argsort(-merged)[:8]:
        ends = (t[k, TL_WAVE_END:TL_WAVE_END + 8] - t0) / 100.0
        print(f"  merged {merged[k]:6.2f}  tiles asked {r[k, 5]:5.2f}  alive {int(alive_n[k]):3d}  rows {int(rows_wg[k]):4d}  "
              f"waves {' '.join(f'{x:5.1f}' for x in ends)}  rows/wave {t[k, TL_WAVE_ROWS:TL_WAVE_ROWS + 8].tolist()}")
    okm = merged > 0
    print(f"# correlation of a workgroup's merge time with its surviving nodes "
          f"{np.corrcoef(merged[okm], alive_n[okm])[0, 1]:.2f}, with its rows "
          f"{np.corrcoef(merged[okm], rows_wg[okm])[0, 1]:.2f}; surviving nodes mean "
          f"{alive_n[okm].mean():.1f} max {alive_n[okm].max():.0f}; rows mean {rows_wg[okm].mean():.1f} "
          f"max {rows_wg[okm].max():.0f}")
    for lo, hi in ((0, 9), (9, 17), (17, 25), (25, 33), (33, 1 << 30)):
        sel = okm & (alive_n >= lo) & (alive_n < hi)
        if sel.any():
            print(f"  workgroups with {lo:2d}..{min(hi - 1, 999):3d} surviving nodes: {int(sel.sum()):4d}  merged at mean "
                  f"{merged[sel].mean():6.2f} max {merged[sel].max():6.2f}  rows mean {rows_wg[sel].mean():6.1f}")
    # (last step) per wave with rows: when its scan ended, its first batch of value rows was asked
    # for and was in the sums
    wsc = (t[:, TL_WAVE_SCANNED:TL_WAVE_SCANNED + 8] - t0) / 100.0
    wis = (t[:, TL_WAVE_ISSUED:TL_WAVE_ISSUED + 8] - t0) / 100.0
    wco = (t[:, TL_WAVE_CONSUMED:TL_WAVE_CONSUMED + 8] - t0) / 100.0
    wrl = t[:, TL_WAVE_ROWS:TL_WAVE_ROWS + 8]
    has = (t[:, TL_WAVE_ISSUED:TL_WAVE_ISSUED + 8] != 0) & (wrl > 0)
    print("# waves of the last step with rows, by when their scan ended: scan end -> first batch asked "
          "for -> in the sums (mean microseconds), rows")
    for lo, hi in ((0, 6), (6, 8), (8, 10), (10, 12), (12, 99)):
        sel = has & (wsc >= lo) & (wsc < hi)
        if sel.any():
            print(f"  scan ended {lo:2d}..{hi:2d}: {int(sel.sum()):4d} waves  scanned {wsc[sel].mean():6.2f}  asked "
                  f"{wis[sel].mean():6.2f}  in the sums {wco[sel].mean():6.2f}  (trip + sums "
                  f"{(wco[sel] - wis[sel]).mean():5.2f})  rows {wrl[sel].mean():5.1f}")
    we, wr = np.concatenate(wave_end), np.concatenate(wave_rows)
    print("# waves by the rows they listed: count per step, when they arrive at the merge (mean, max)")
    for lo, hi in ((0, 1), (1, 9), (9, 17), (17, 33), (33, 65), (65, 1 << 30)):
        sel = (wr >= lo) & (wr < hi)
        if sel.any():
            print(f"rows {lo:3d}..{min(hi - 1, 9999):4d}: {sel.sum() / len(lens):8.1f} waves  "
                  f"mean {we[sel].mean():6.2f}  max {we[sel].max():6.2f}")


# Search alone at the shapes the reference publishes (single head, d = 128, fp32, one unit-norm random
# query, a threshold that keeps 10 keys; its figures are from an unnamed NVIDIA GPU on real Llama-3
# keys that are not shipped): (N, fan-out, levels, published us, where)
PUBLISHED_SEARCH = [
    (10000, 4, 3, 8.16, "benchmark_area/cuda_bench/reports/three_level_filter_real.csv:2"),
    (40000, 4, 3, 11.11, "benchmark_area/cuda_bench/reports/three_level_filter_real.csv:4"),
    (90000, 4, 3, 14.43, "benchmark_area/cuda_bench/reports/three_level_filter_real.csv:7"),
    (40000, 8, 2, 13.54, "benchmark_area/cuda_bench/reports/three_level_filter_real.csv:4"),
    (90000, 8, 2, 20.65, "benchmark_area/cuda_bench/reports/three_level_filter_real.csv:7"),
    (40000, 16, 3, 20.43, "benchmark_area/cuda_bench/reports/triton_benchmarking.csv:4"),
    (40000, 32, 3, 34.74, "benchmark_area/cuda_bench/reports/triton_benchmarking.csv:4"),
    (40000, 64, 3, 626.2, "benchmark_area/cuda_bench/reports/triton_benchmarking.csv:4"),
    (90000, 32, 3, 45.97, "benchmark_area/cuda_bench/reports/triton_benchmarking.csv:7"),
]


# (window, published ms per call with two / three levels: the "v2" columns, its current code)
PUBLISHED_UPDATE = [
    (64, 1.02, 2.25, "benchmark_area/updating_index/cuda/cuda_updating_results.csv:2"),
    (1024, 1.45, 3.58, "benchmark_area/updating_index/cuda/cuda_updating_results.csv:22"),
    (4096, 2.59, 6.73, "benchmark_area/updating_index/cuda/cuda_updating_results.csv:32"),
]


def published_shapes(spreads=(0.5, 0.15)):
    """`HIPSearcher.search` (dense output, as the reference's searcher returns it) at the shapes of
    PUBLISHED_SEARCH, on synthetic keys: 256 Gaussian clusters of a given spread around unit-scale
    centres, normalised.  The published figures are on real keys, whose balls prune (the
    reference's own study counts 2512 leaf products for 10 000 keys at fan-out 4,
    benchmark_area/pruning/notebooks/ball_pruning_power_results.csv:2); a spread of 0.5 gives keys
    whose balls prune almost nothing, 0.15 keys that prune about as the real ones do, and the share
    of the keys a query's walk reads is reported with every figure.  One JSON line."""
    import torch

    from hira_amd import _lib
    from hira_amd.cache.threshold_finder import exact_topk
    from hira_amd.indexer import HIPIndexer
    from hira_amd.searcher import HIPSearcher

    def replayed_us(f, n=100):
        for _ in range(5):
            f()
        torch.cuda.synchronize()
        st = torch.cuda.Stream()
        st.wait_stream(torch.cuda.current_stream())
        g = torch.cuda.CUDAGraph()
        with torch.cuda.stream(st):
            with torch.cuda.graph(g, stream=st):
                for _ in range(n):
                    f()
            g.replay()
            st.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(st)
            g.replay()
            e1.record(st)
            st.synchronize()
        return e0.elapsed_time(e1) / n * 1e3

    rows = []
    for spread in spreads:
        gen = torch.Generator().manual_seed(0)
        for n, bf, levels, pub, where in PUBLISHED_SEARCH:
            c = torch.randn(256, 128, generator=gen)
            keys = torch.nn.functional.normalize(
                c[torch.randint(0, 256, (n,), generator=gen)] + spread * torch.randn(n, 128, generator=gen), dim=-1)
            q = torch.nn.functional.normalize(torch.randn(1, 128, generator=gen), dim=-1).cuda()
            kd = keys[None, None].cuda()
            idx = HIPIndexer(levels, 1, bf).build(kd)
            th = exact_topk(kd[0], q, 10)
            se = HIPSearcher()
            stats = torch.zeros(1, _lib.HIRA_STATS_COLS, dtype=torch.int64, device="cuda")
            out = se.search(q, th, idx, stats=stats)
            assert int((out != 0).sum()) == 10
            us = replayed_us(lambda: se.search(q, th, idx))
            kq = kd[0, 0].float()
            qt = q.float().T.contiguous()
            dense = replayed_us(lambda: kq @ qt)
            rows.append({"n": n, "fanout": bf, "levels": levels, "cluster_spread": spread,
                         "us": round(us, 2), "published_us": pub, "published_at": where,
                         "keys_read_share": round(float(stats[0, 0]) / n, 3), "torch_k_at_q_us": round(dense, 2)})
            log(f"[bench] published shape N={n} fan-out {bf} levels {levels} spread {spread}: "
                f"{us:.2f} us (published {pub}), keys read {rows[-1]['keys_read_share']:.2f} of N")
            del idx, kd
    # ---- the reference's update benchmark (benchmark_area/updating_index/cuda/cuda_updating_bench.ipynb:
    # one head, d = 128, fp32, fan-out 8, an index of 10 000 keys grown to 90 000 in windows; mean
    # time per update call, host clock, synchronised before AND after the call here)
    upd = []
    gen = torch.Generator().manual_seed(42)
    c = torch.randn(256, 128, generator=gen)
    allk = torch.nn.functional.normalize(
        c[torch.randint(0, 256, (90000,), generator=gen)] + 0.15 * torch.randn(90000, 128, generator=gen),
        dim=-1)[None, None].cuda()
    for window, pub2, pub3, where in PUBLISHED_UPDATE:
        for levels, pub in ((2, pub2), (3, pub3)):
            idx = HIPIndexer(levels, 1, 8).build(allk[:, :, :10000])
            torch.cuda.synchronize()
            times = []
            for at in range(10000, 90000 - window + 1, window):
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                idx.update(allk[:, :, at:at + window])
                torch.cuda.synchronize()
                times.append(time.perf_counter() - t0)
            assert idx.num_keys == 10000 + len(times) * window
            times = times[2:]  # (the first calls load code objects)
            upd.append({"window": window, "levels": levels, "ms_per_call": round(1e3 * sum(times) / len(times), 4),
                        "calls": len(times), "published_ms": pub, "published_at": where})
            log(f"[bench] published update: window {window}, {levels} levels: "
                f"{upd[-1]['ms_per_call']:.3f} ms per call (published {pub})")
            del idx
    print(json.dumps({"mode": "published_shapes", "dtype": "f32", "data": "synthetic", "rows": rows,
                      "updates": upd}), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--config", type=int, default=2)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-budget", type=float, default=20.0)
    ap.add_argument("--block-threads", type=int, default=0)
    ap.add_argument("--nodes-per-wave", type=int, default=0)
    ap.add_argument("--kernel", type=int, default=0)
    ap.add_argument("--kmeans-iters", type=int, default=-1)
    ap.add_argument("--layout", default="auto", choices=["auto", "tiled", "q8", "row_major"],
                    help="index layout (q8: an 8-bit shadow of the keys is scanned first)")
    ap.add_argument("--separate-merge", action="store_true",
                    help="fold the attention partials in a second launch")
    ap.add_argument("--profile", action="store_true",
                    help="only the warm-up and the timed steps (no counter pass, no dense or "
                         "CPU comparators): every launch a profiler sees is the measured one")
    ap.add_argument("--stream", type=int, default=0,
                    help="after the timed steps: append this many keys one per step, a search "
                         "after each, one level-2 subtree rebuilt every --rebuild-every steps")
    ap.add_argument("--rebuild-every", type=int, default=512)
    ap.add_argument("--layers", type=int, default=-1,
                    help="also time the steps over this many copies of the index in turn "
                         "(each with its own memory, like the layers of a model); default: 8 "
                         "where one index fits the Infinity Cache, else none")
    ap.add_argument("--published", action="store_true",
                    help="search alone at the single-head shapes the reference publishes figures for")
    ap.add_argument("--context", type=int, default=0,
                    help="keys per KV head instead of the configuration's (a sweep point, not a "
                         "benchmark configuration)")
    ap.add_argument("--npz", default=None,
                    help="keys and queries captured from a model (the reference sampler's .npz: "
                         "keys (N,D), queries (N,D)) instead of the synthetic ones")
    ap.add_argument("--taus", default=None,
                    help="file that keeps the steps' thresholds: written when absent, read when "
                         "present (so that a run under a profiler's counters need not launch "
                         "the sort kernels that find them)")
    ap.add_argument("--lib", default=None,
                    help="another build of libhira_hip.so to load instead of the one in hira_amd/csrc "
                         "(to compare two builds on one machine)")
    ap.add_argument("--timeline", action="store_true",
                    help="run the steps on the library built with time stamps "
                         "(`make -C hira_amd/csrc timeline`) and print where a step's time goes")
    ap.add_argument("--counters", action="store_true",
                    help="run the steps once, untimed, plus a kernel of known traffic "
                         "(for rocprofv3 --pmc runs)")
    a = ap.parse_args()
    if a.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        log("bench.py: this path is built and measured on ONE GPU (each KV head owns an "
            "independent tree, so more GPUs would shard by head without any exchange); "
            "run with --gpus 1")
        sys.exit(2)

    import numpy as np
    import torch

    from hira_amd import _lib, synth
    from hira_amd.cache.threshold_finder import exact_topk
    from hira_amd.indexer import HIPIndexer
    from hira_amd.searcher import HIPSearcher

    assert torch.cuda.is_available(), "bench.py needs the GPU"
    dev = torch.device("cuda:0")
    if a.published:
        if a.lib:
            _lib.use_library(a.lib)
        published_shapes()
        return
    if a.timeline:
        _lib.use_library(_lib.CSRC / "libhira_hip_timeline.so")
    elif a.lib:
        _lib.use_library(a.lib)
    w = synth.WORKLOADS[a.config]
    if a.context > 0:
        import dataclasses

        w = dataclasses.replace(w, n=a.context, name=f"{w.name}@ctx{a.context}")
    K, W = a.steps, a.warmup
    total = K + W
    log(f"[bench] workload {w.name}: generating keys/values/queries on the host")
    if a.npz:
        w, keys, values, queries = synth.load_capture(a.npz, w, total)
    else:
        keys, values = synth.make_kv(w)
        queries = synth.make_queries(w, keys, total)  # (total, B, H_q, D)
    keys_d, values_d = keys.to(dev), values.to(dev)
    niter = w.kmeans_iters if a.kmeans_iters < 0 else a.kmeans_iters
    t0 = time.perf_counter()
    index = HIPIndexer(w.num_levels, niter, w.bf, device="cuda:0", layout=a.layout,
                       heads_per_tree=w.group).build(keys_d, values_d)
    torch.cuda.synchronize()
    build_ms = (time.perf_counter() - t0) * 1e3
    # (the first build of a process also loads the library and its code objects)
    t0 = time.perf_counter()
    again = HIPIndexer(w.num_levels, niter, w.bf, device="cuda:0", layout=a.layout,
                       heads_per_tree=w.group).build(keys_d, values_d)
    torch.cuda.synchronize()
    build_again_ms = (time.perf_counter() - t0) * 1e3
    del again
    log(f"[bench] index built in {build_ms:.1f} ms (again: {build_again_ms:.1f} ms), level sizes {index.size}")

    # thresholds: exactly ceil(p*N) keys per head (midpoint between neighbouring scores)
    fr = synth.select_fractions(w)
    q_d = queries.to(dev).reshape(total, w.batch * w.h_q, w.d).contiguous()
    taus = torch.empty((total, w.batch * w.h_q), dtype=torch.float32, device=dev)
    ksel = [int(np.ceil(float(fr[b]) * w.n)) for b in range(w.batch)]
    if a.taus and os.path.exists(a.taus):
        kept = torch.load(a.taus, weights_only=True)
        if tuple(kept.shape) != tuple(taus.shape):
            raise SystemExit(f"{a.taus} holds thresholds of shape {tuple(kept.shape)}, this run "
                             f"needs {tuple(taus.shape)}: made with other --steps/--warmup/--config?")
        taus.copy_(kept)
        log(f"[bench] thresholds read from {a.taus}")
    else:
        for b in range(w.batch):
            hs = slice(b * w.h_q, (b + 1) * w.h_q)
            for i in range(total):
                taus[i, hs] = exact_topk(keys_d[b], q_d[i, hs], ksel[b])
        if a.taus:
            torch.save(taus.cpu(), a.taus)
            log(f"[bench] thresholds written to {a.taus}")
    scale = w.d ** -0.5
    searcher = HIPSearcher(block_threads=a.block_threads, nodes_per_wave=a.nodes_per_wave,
                           kernel=a.kernel, separate_merge=a.separate_merge)
    h_all = w.batch * w.h_q
    plan = searcher.plan_attention(index, h_all, scaling=torch.full((h_all,), scale))
    outs = torch.empty((total, h_all, w.d), dtype=torch.float32, device=dev)

    # ---- warm-up (eager) -----------------------------------------------------------
    for i in range(W):
        plan.run(q_d[i], taus[i], outs[i])
    torch.cuda.synchronize()

    if a.timeline:
        timeline_report(a, w, index, searcher, q_d, taus, outs, W, total, scale)
        return

    if a.counters:
        # For `rocprofv3 --pmc FETCH_SIZE` / `--pmc WRITE_SIZE`: K plain launches of the
        # search kernel and one elementwise kernel of known traffic (reads 256 MiB, writes
        # 256 MiB in a single dispatch) that scales the counters; nothing is timed.
        src = torch.ones(64 * 1024 * 1024, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        torch.add(src, 1.0, out=dst)
        torch.cuda.synchronize()
        for i in range(W, total):
            plan.run(q_d[i], taus[i], outs[i])
        torch.cuda.synchronize()
        print(json.dumps({"mode": "counters", "steps": K,
                          "calibration_kernel_bytes_read": src.numel() * 4,
                          "calibration_kernel_bytes_written": dst.numel() * 4}), flush=True)
        return

    # ---- counters: algorithmic bytes of the K timed steps ---------------------------
    stats = torch.zeros((index.num_trees, _lib.HIRA_STATS_COLS), dtype=torch.int64, device=dev)
    splan = searcher.plan_attention(index, h_all, scaling=torch.full((h_all,), scale), stats=stats)
    scratch = torch.empty((h_all, w.d), dtype=torch.float32, device=dev)
    if not a.profile:
        for i in range(W, total):
            splan.run(q_d[i], taus[i], scratch)
        torch.cuda.synchronize()
    alg_bytes, alg_bytes_bf16, counts = algorithmic_bytes(stats.cpu().numpy(), w, index.num_levels, K,
                                                          shadow=index.q8)
    want_pairs = sum(ksel[b] * w.h_q for b in range(w.batch))
    if abs(counts["selected_pairs_per_step"] - want_pairs) > 1e-6 * want_pairs:
        log(f"[bench] WARNING: selected {counts['selected_pairs_per_step']} pairs/step, "
            f"expected {want_pairs}")

    # ---- timed: K steps captured in one HIP graph, replayed once --------------------
    stream = torch.cuda.Stream(device=dev)
    stream.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            for i in range(W, total):
                plan.run(q_d[i], taus[i], outs[i])
        graph.replay()  # untimed: first replay uploads the graph
        stream.synchronize()
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        ev0.record(stream)
        graph.replay()
        ev1.record(stream)
        # (the host polls for the end instead of sleeping until it is woken: a blocking wait's
        # wake-up is tens of microseconds, which a run of few steps would carry in its figure)
        while not ev1.query():
            pass
        torch.cuda.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3
        graph_ms = ev0.elapsed_time(ev1)

        # eager loop (one library call per step from Python), for comparison
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for i in range(W, total):
            plan.run(q_d[i], taus[i], outs[i], stream=stream.cuda_stream)
        e1.record(stream)
        stream.synchronize()
        eager_ms = e0.elapsed_time(e1)

        # the same loop with an event after every step: the spread of single steps
        # (event to event, so a step's figure includes its launch gap and the marker)
        evs = [torch.cuda.Event(enable_timing=True) for _ in range(K + 1)]
        evs[0].record(stream)
        for i in range(W, total):
            plan.run(q_d[i], taus[i], outs[i], stream=stream.cuda_stream)
            evs[i - W + 1].record(stream)
        stream.synchronize()
        per_step = np.array([evs[i].elapsed_time(evs[i + 1]) * 1e3 for i in range(K)])

        # what a plain streaming kernel reaches on this GPU: torch's elementwise add over
        # 1 GiB in, 1 GiB out
        src = torch.empty(256 * 1024 * 1024, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(2):
            torch.add(src, 1.0, out=dst)
        b0, b1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        b0.record(stream)
        for _ in range(8):
            torch.add(src, 1.0, out=dst)
        b1.record(stream)
        stream.synchronize()
        stream_gbs = 8 * 2.0 * src.numel() * 4 / (b0.elapsed_time(b1) * 1e-3) / 1e9
        del src, dst
    us_per_step = wall_ms * 1e3 / K
    kernel_us = graph_ms * 1e3 / K

    # ---- the same steps over several copies of the index in turn (a model's layers each have
    # their own): what one index alone leaves in the 256 MB Infinity Cache between steps is
    # gone by the time its turn comes again
    rot = None
    if a.layers < 0:
        one_index = 2 * keys_d.numel() * keys_d.element_size()
        a.layers = 8 if one_index <= 256 * 1024 * 1024 else 0
    if a.layers > 1 and not a.profile:
        copies = [index] + [HIPIndexer(w.num_levels, niter, w.bf, device="cuda:0", layout=a.layout,
                       heads_per_tree=w.group).build(keys_d, values_d)
                            for _ in range(a.layers - 1)]
        plans = [plan] + [searcher.plan_attention(c, h_all, scaling=torch.full((h_all,), scale))
                          for c in copies[1:]]
        outs2 = torch.empty_like(outs)
        g3 = torch.cuda.CUDAGraph()
        with torch.cuda.stream(stream):
            with torch.cuda.graph(g3, stream=stream):
                for i in range(W, total):
                    plans[i % a.layers].run(q_d[i], taus[i], outs2[i])
            g3.replay()
            stream.synchronize()
            r0, r1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            r0.record(stream)
            g3.replay()
            r1.record(stream)
            stream.synchronize()
        same = bool(torch.equal(outs2[W:], outs[W:]))
        rot = {"indexes": a.layers, "us_per_step": round(r0.elapsed_time(r1) * 1e3 / K, 3),
               "bytes_of_all_indexes": int(a.layers * (2 * keys_d.numel() * keys_d.element_size()
                                                        + (keys_d.numel() if index.q8 else 0))),
               "same_outputs": same}
        del copies, plans, g3

    # ---- the same steps over an index in the other layout: with an 8-bit shadow of its keys
    # (layout q8: the scan reads the shadow, the exact test only the rows the shadow cannot rule
    # out) when the index above has none, without one when it has (layout="auto" adds the shadow
    # to long trees with many heads)
    q8_leg = None
    other_layout = "tiled" if index.q8 else "q8"
    if not a.profile and w.dtype == torch.bfloat16 and w.d in (64, 128) \
            and index.num_levels >= 2 and a.kernel != 1:
        try:
            qindex = HIPIndexer(w.num_levels, niter, w.bf, device="cuda:0", layout=other_layout).build(keys_d, values_d)
            qstats = torch.zeros_like(stats)
            qsplan = searcher.plan_attention(qindex, h_all, scaling=torch.full((h_all,), scale), stats=qstats)
            qouts = torch.empty_like(outs)
            for i in range(W, total):
                qsplan.run(q_d[i], taus[i], qouts[i])
            torch.cuda.synchronize()
            qb, qb16, qcounts = algorithmic_bytes(qstats.cpu().numpy(), w, qindex.num_levels, K,
                                                  shadow=qindex.q8)
            qplan = searcher.plan_attention(qindex, h_all, scaling=torch.full((h_all,), scale))
            gq = torch.cuda.CUDAGraph()
            with torch.cuda.stream(stream):
                with torch.cuda.graph(gq, stream=stream):
                    for i in range(W, total):
                        qplan.run(q_d[i], taus[i], qouts[i])
                gq.replay()
                stream.synchronize()
                q0, q1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                q0.record(stream)
                gq.replay()
                q1.record(stream)
                stream.synchronize()
            q_us = q0.elapsed_time(q1) * 1e3 / K
            q8_leg = {"layout": qindex.layout_name, "us_per_step": round(q_us, 3), "algorithmic_bytes_per_step": round(qb),
                      "achieved_GBps": round(qb / (q_us * 1e-6) / 1e9, 1),
                      "frac_of_hbm_peak": round(qb / (q_us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
                      "exact_rows_per_step": round(qcounts["exact_rows_per_step"], 1),
                      "same_selection_counts": bool(
                          qcounts["selected_pairs_per_step"] == counts["selected_pairs_per_step"]
                          and qcounts["candidates_per_step"] == counts["candidates_per_step"]),
                      "max_abs_diff_of_outputs": float((qouts[W:] - outs[W:]).abs().max())}
            del qindex, qsplan, qplan, gq
        except Exception as ex:  # noqa: BLE001
            log(f"[bench] leg in the {other_layout} layout failed: {ex!r}")

    # ---- dense comparators ------------------------------------------------------------
    dense_us = {}
    if a.profile:
        print(json.dumps({"mode": "profile", "steps": K, "us_per_step_wall": round(us_per_step, 3),
                          "us_per_step_events": round(kernel_us, 3),
                          "eager_us_per_step": round(eager_ms * 1e3 / K, 3)}), flush=True)
        return
    try:
        qd = q_d[W:].reshape(K, w.batch, w.h_q, 1, w.d)
        kk = keys_d[:, :, None].expand(w.batch, w.h_kv, w.group, w.n, w.d).reshape(
            w.batch, w.h_q, w.n, w.d)
        vv = values_d[:, :, None].expand(w.batch, w.h_kv, w.group, w.n, w.d).reshape(
            w.batch, w.h_q, w.n, w.d)
        reps = min(K, 32)
        for name, kw in (("sdpa_gqa", dict(enable_gqa=True)), ("sdpa_expanded", {})):
            kx, vx = (keys_d, values_d) if kw else (kk, vv)
            for _ in range(3):
                torch.nn.functional.scaled_dot_product_attention(qd[0], kx, vx, scale=scale, **kw)
            torch.cuda.synchronize()
            d0, d1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            d0.record()
            for i in range(reps):
                torch.nn.functional.scaled_dot_product_attention(qd[i], kx, vx, scale=scale, **kw)
            d1.record()
            torch.cuda.synchronize()
            dense_us[name] = d0.elapsed_time(d1) * 1e3 / reps
    except Exception as ex:  # noqa: BLE001
        log(f"[bench] dense SDPA comparator failed: {ex}")
    # our kernel with every key selected (threshold -inf): a dense decode attention
    # (always over bf16 keys in the tiled layout: with every key selected an 8-bit scan ahead of
    # the exact test would only add work, and the comparator should be the best dense path)
    ninf = torch.full((h_all,), -3.0e38, dtype=torch.float32, device=dev)
    dplan = plan
    if index.q8:
        dindex = HIPIndexer(w.num_levels, niter, w.bf, device="cuda:0").build(keys_d, values_d)
        dplan = searcher.plan_attention(dindex, h_all, scaling=torch.full((h_all,), scale))
    for _ in range(3):
        dplan.run(q_d[0], ninf, scratch)
    torch.cuda.synchronize()
    d0, d1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    d0.record()
    for i in range(16):
        dplan.run(q_d[W + i % K], ninf, scratch)
    d1.record()
    torch.cuda.synchronize()
    dense_us["ours_all_selected"] = d0.elapsed_time(d1) * 1e3 / 16
    if index.q8:
        del dplan, dindex

    # thresholds from a key sample (1000 keys per tree, mean of the 10 best): the launch a
    # deployment puts ahead of every search; K of them in one graph
    from hira_amd.cache.threshold_finder import device_thresholds
    pick = torch.randperm(w.n, generator=torch.Generator().manual_seed(12345))[:1000].to(dev)
    samples = keys_d[:, :, pick].reshape(w.batch * w.h_kv, 1000, w.d).contiguous()
    tau_s = torch.empty((h_all,), dtype=torch.float32, device=dev)
    device_thresholds(samples, q_d[0], "sample_mean_topk", 10, out=tau_s)
    g2 = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(g2, stream=stream):
            for i in range(W, total):
                device_thresholds(samples, q_d[i], "sample_mean_topk", 10, out=tau_s,
                                  stream=stream.cuda_stream)
        g2.replay()
        stream.synchronize()
        t0e, t1e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0e.record(stream)
        g2.replay()
        t1e.record(stream)
        stream.synchronize()
    thr_us = t0e.elapsed_time(t1e) * 1e3 / K
    # and the whole step a deployment without given thresholds runs: thresholds from the sample,
    # then search + attention with them (two launches per step, K steps in one graph)
    g4 = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(g4, stream=stream):
            for i in range(W, total):
                plan.run_sampled(q_d[i], samples, "sample_mean_topk", 10, scratch,
                                 stream=stream.cuda_stream)
        g4.replay()
        stream.synchronize()
        t0e.record(stream)
        g4.replay()
        t1e.record(stream)
        stream.synchronize()
    step_thr_us = t0e.elapsed_time(t1e) * 1e3 / K
    del g4
    dense_best = min(dense_us.values())

    e = 2 if w.dtype == torch.bfloat16 else 4
    dense_bytes = 2.0 * w.batch * w.h_kv * w.n * w.d * e
    achieved = alg_bytes / (kernel_us * 1e-6) / 1e9
    result = {
        "metric": "decode search+sparse-attn us/layer at 32k ctx; achieved HBM GB/s vs 8 TB/s",
        "value": round(us_per_step, 3),
        "unit": "us/layer",
        "n_gpus": 1,
        "steps": K,
        "warmup": W,
        "ms_per_step": round(us_per_step / 1e3, 6),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if w.dtype == torch.bfloat16 else "f32",
        "data": "captured keys/queries, synthetic values" if a.npz else "synthetic",
        "config": {"workload": w.name, "h_q": w.h_q, "h_kv": w.h_kv, "context": w.n,
                   "head_dim": w.d, "batch": w.batch, "levels": w.num_levels, "bf": w.bf,
                   "select_per_head": ksel, "kmeans_iters": niter, "layout": index.layout_name},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": measured_traffic(w.name + ("_q8" if index.q8 else ""))},
        "algorithmic_bytes_per_step": round(alg_bytes),
        "algorithmic_bytes_per_step_bf16_scan": round(alg_bytes_bf16),
        "gpu_us_per_step_events": round(kernel_us, 3),
        "eager_us_per_step": round(eager_ms * 1e3 / K, 3),
        "eager_step_us": {"mean": round(float(per_step.mean()), 2),
                          "median": round(float(np.median(per_step)), 2),
                          "p99": round(float(np.percentile(per_step, 99)), 2)},
        "streaming_add_GBps": round(stream_gbs, 1),
        "rotating_indexes": rot,
        ("bf16_scan_layout" if index.q8 else "q8_shadow_layout"): q8_leg,
        "sample_threshold_us": round(thr_us, 2),
        "step_with_sample_threshold_us": round(step_thr_us, 2),
        "dense_attention_us": {k: round(v, 2) for k, v in dense_us.items()},
        "dense_attention_bytes": dense_bytes,
        "frac_of_dense_time": round(kernel_us / dense_best, 4),
        "counters": {k: round(v, 1) for k, v in counts.items()},
        "index_build_ms": round(build_ms, 1),
        "index_build_again_ms": round(build_again_ms, 2),
    }
    if a.stream > 0:
        result["streaming"] = streaming(a, w, index, plan, q_d, taus, scratch, dev)
    if not a.no_cpu:
        try:
            if a.stream > 0:  # the index has grown since the timed steps: timing only
                result["cpu_baseline"] = cpu_baseline(w, index, q_d[W:], taus[W:], scale, a.cpu_budget)
            else:
                dense_searcher = HIPSearcher()
                result["cpu_baseline"] = cpu_baseline(
                    w, index, q_d[W:], taus[W:], scale, a.cpu_budget, gpu_out=outs[W:],
                    gpu_sel=lambda i: (dense_searcher.search(q_d[W + i], taus[W + i], index) != 0).cpu().numpy())
        except Exception as ex:  # noqa: BLE001
            log(f"[bench] cpu baseline failed: {ex!r}")
            result["cpu_baseline"] = None
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
