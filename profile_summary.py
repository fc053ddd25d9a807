"""Turn rocprofv3 CSV output into the short text summaries kept under profiles/.

    python profile_summary.py kernels <kernel_trace.csv>      # per-kernel time
    python profile_summary.py counters <fetch.csv> <write.csv> \
        --calib-read BYTES --calib-write BYTES [--json OUT.json]
    python profile_summary.py build <kernel_trace.csv> [--which N]   # one index build
    python profile_summary.py pmc <counter_collection.csv> --kernel NAME   # counters per dispatch

`counters` scales FETCH_SIZE / WRITE_SIZE of the search kernel by what the same counters
read for the calibration kernel of known traffic that `bench.py --counters` launches (a
torch elementwise add: one dispatch reading and writing a known number of bytes).
"""
from __future__ import annotations

import argparse
import collections
import csv
import json


def kernel_table(path: str):
    rows = list(csv.DictReader(open(path)))
    agg = collections.defaultdict(list)
    for r in rows:
        agg[r["Kernel_Name"]].append((int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3)
    total = sum(sum(v) for v in agg.values())
    out = ["| kernel | calls | total us | avg us | min us | max us | % |", "|---|---|---|---|---|---|---|"]
    for k, v in sorted(agg.items(), key=lambda kv: -sum(kv[1])):
        out.append(f"| `{k[:90]}` | {len(v)} | {sum(v):.1f} | {sum(v) / len(v):.2f} | {min(v):.2f} | "
                   f"{max(v):.2f} | {100 * sum(v) / total:.1f} |")
    return "\n".join(out)


def counter_means(path: str, counter: str):
    agg = collections.defaultdict(list)
    for r in csv.DictReader(open(path)):
        if r["Counter_Name"] == counter:
            agg[r["Kernel_Name"]].append(float(r["Counter_Value"]))
    return {k: (sum(v) / len(v), len(v)) for k, v in agg.items()}


def build_table(path: str, which: int):
    """One index build of the trace: from a `k_level_init` whose grid is the trace's largest to
    the last `k_radii` behind it; launches, the span from the first kernel's start to the last
    one's end, the kernels' own time, and the table per kernel."""
    rows = [r for r in csv.DictReader(open(path)) if "hira::" in r["Kernel_Name"]]
    rows.sort(key=lambda r: int(r["Start_Timestamp"]))
    inits = [i for i, r in enumerate(rows) if "k_level_init" in r["Kernel_Name"]]
    top = max(int(rows[i]["Grid_Size_X"]) for i in inits)
    starts = [i for i in inits if int(rows[i]["Grid_Size_X"]) == top]
    i0 = starts[min(which, len(starts) - 1)]
    i1 = i0
    while i1 + 1 < len(rows) and not ("k_radii" in rows[i1]["Kernel_Name"]
                                      and "k_radii" not in rows[i1 + 1]["Kernel_Name"]):
        i1 += 1
    one = rows[i0:i1 + 1]
    dur = lambda r: (int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3  # noqa: E731
    span = (int(one[-1]["End_Timestamp"]) - int(one[0]["Start_Timestamp"])) / 1e3
    agg = collections.defaultdict(list)
    for r in one:
        agg[r["Kernel_Name"].split("(")[0]].append(dur(r))
    out = [f"builds in the trace: {len(starts)}; build {min(which, len(starts) - 1)}: {len(one)} launches, "
           f"{span:.1f} us from the first kernel's start to the last one's end, "
           f"{sum(map(dur, one)):.1f} us inside kernels", "",
           "| kernel | calls | total us | avg us | min us | max us |", "|---|---|---|---|---|---|"]
    for k, v in sorted(agg.items(), key=lambda kv: -sum(kv[1])):
        out.append(f"| `{k[:70]}` | {len(v)} | {sum(v):.1f} | {sum(v) / len(v):.2f} | {min(v):.2f} | {max(v):.2f} |")
    asg = [f"{dur(r):.0f}" for r in one if "k_assign_mfma" in r["Kernel_Name"]]
    out += ["", "assignment launches in order (us): " + " ".join(asg)]
    return "\n".join(out)


def pmc_table(path: str, kernel: str, top: int = 3):
    """Counters of the `top` dispatches of `kernel` with the largest grids, one line each."""
    by = collections.defaultdict(dict)
    for r in csv.DictReader(open(path)):
        if kernel in r["Kernel_Name"]:
            by[(int(r["Dispatch_Id"]), int(r["Grid_Size"]))][r["Counter_Name"]] = float(r["Counter_Value"])
    items = sorted(by.items(), key=lambda kv: (-kv[0][1], kv[0][0]))[:top]
    out = []
    for (d, g), v in sorted(items):
        out.append(f"dispatch {d}, grid {g}: " + ", ".join(f"{k} {int(x)}" for k, x in sorted(v.items())))
        if "SQ_VALU_MFMA_BUSY_CYCLES" in v and "GRBM_GUI_ACTIVE" in v:
            out.append(f"  MFMA utilisation = SQ_VALU_MFMA_BUSY_CYCLES / (GRBM_GUI_ACTIVE / 8 x 256 CUs x 4 SIMDs) = "
                       f"{100 * v['SQ_VALU_MFMA_BUSY_CYCLES'] / (v['GRBM_GUI_ACTIVE'] / 8 * 256 * 4):.1f} %")
    return "\n".join(out)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("what", choices=["kernels", "counters", "build", "pmc"])
    ap.add_argument("--which", type=int, default=1)
    ap.add_argument("files", nargs="+")
    ap.add_argument("--calib-read", type=float, default=0)
    ap.add_argument("--calib-write", type=float, default=0)
    ap.add_argument("--calib-kernel", default="vectorized_elementwise_kernel")
    ap.add_argument("--kernel", default="search_")
    ap.add_argument("--json", default=None)
    a = ap.parse_args()
    if a.what == "kernels":
        print(kernel_table(a.files[0]))
        return
    if a.what == "build":
        print(build_table(a.files[0], a.which))
        return
    if a.what == "pmc":
        print(pmc_table(a.files[0], a.kernel))
        return
    fetch = counter_means(a.files[0], "FETCH_SIZE")
    write = counter_means(a.files[1], "WRITE_SIZE")

    def pick(d, key, biggest=False):
        c = {k: v for k, v in d.items() if key in k}
        if not c:
            raise SystemExit(f"no kernel matching {key!r}")
        k = max(c, key=lambda x: c[x][0]) if biggest else next(iter(c))
        return k, c[k]

    ck_f, (cf, _) = pick(fetch, a.calib_kernel, biggest=True)
    ck_w, (cw, _) = pick(write, a.calib_kernel, biggest=True)
    fscale = a.calib_read / cf  # bytes per counter unit
    wscale = a.calib_write / cw
    k_f, (sf, nf) = pick(fetch, a.kernel, biggest=True)
    k_w, (sw, nw) = pick(write, a.kernel, biggest=True)
    res = dict(kernel=k_f, launches=nf, fetch_counter_per_launch=sf, write_counter_per_launch=sw,
               fetch_bytes_per_unit=fscale, write_bytes_per_unit=wscale,
               fetch_bytes_per_launch=sf * fscale, write_bytes_per_launch=sw * wscale,
               hbm_bytes_per_launch=sf * fscale + sw * wscale,
               calibration=dict(kernel=ck_f, fetch_counter=cf, write_counter=cw,
                                bytes_read=a.calib_read, bytes_written=a.calib_write))
    print(json.dumps(res, indent=1))
    if a.json:
        with open(a.json, "w") as f:
            json.dump(res, f, indent=1)


if __name__ == "__main__":
    main()
