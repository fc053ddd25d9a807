"""Turn rocprofv3 CSV output into the short text summaries kept under profiles/.

    python profile_summary.py kernels <kernel_trace.csv>      # per-kernel time
    python profile_summary.py counters <fetch.csv> <write.csv> \
        --calib-read BYTES --calib-write BYTES [--json OUT.json]

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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("what", choices=["kernels", "counters"])
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
