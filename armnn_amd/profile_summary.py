"""Turns raw rocprofv3 output into the short text summaries kept under profiles/.

  python -m armnn_amd.profile_summary traffic FETCH_DIR WRITE_DIR ORDER_JSON
      HBM bytes per launch of every layer of a network.  FETCH_DIR / WRITE_DIR hold the pmc_counter_collection.csv of
      two runs of `rocprofv3 --pmc FETCH_SIZE` / `--pmc WRITE_SIZE` over `python3 bench.py --profile-pass --no-graph`;
      ORDER_JSON is the line that command printed (dispatch order, kernel names, algorithmic bytes).  Each counter is
      scaled by what it reads for the 64 MiB calibration copy that the pass launches first.  Prints the markdown table
      bench.py reads back (profiles/<workload>_hbm_traffic.md).
  python -m armnn_amd.profile_summary stats KERNEL_STATS_CSV
      The per-kernel table of `rocprofv3 --kernel-trace --stats` as markdown.
  python -m armnn_amd.profile_summary pmc PMC_DIR [KERNEL_SUBSTRING]
      Counter values of the last dispatch of every kernel (all pass directories under PMC_DIR merged), as text.
"""
from __future__ import annotations

import collections
import csv
import glob
import json
import os
import sys


def short_name(kernel: str) -> str:
    """'void mi355x::Foo<1, 2>(mi355x::Args)' -> 'Foo<1, 2>'"""
    k = kernel.replace("void ", "").replace("mi355x::", "").replace("(anonymous namespace)::", "")
    depth, out = 0, []
    for ch in k:
        if ch == "<":
            depth += 1
        elif ch == ">":
            depth -= 1
        elif ch == "(" and depth == 0:
            break
        out.append(ch)
    return "".join(out).strip()


def _counter_csv(d):
    hits = glob.glob(os.path.join(d, "**", "*counter_collection.csv"), recursive=True)
    if not hits:
        raise SystemExit(f"no *counter_collection.csv under {d}")
    return hits[0]


def _per_dispatch(path, counter):
    disp = collections.OrderedDict()
    for r in csv.DictReader(open(path)):
        if r["Counter_Name"] != counter:
            continue
        k = int(r["Dispatch_Id"])
        e = disp.setdefault(k, {"kernel": r["Kernel_Name"], "value": 0.0})
        e["value"] += float(r["Counter_Value"])
    return [disp[k] for k in sorted(disp)]


def traffic(fetch_dir, write_dir, order_json):
    order = json.loads(open(order_json).read().strip().splitlines()[-1])
    names, kernels, alg = order["dispatch_order"], order["kernels"], order["algorithmic_bytes"]
    f = _per_dispatch(_counter_csv(fetch_dir), "FETCH_SIZE")[-len(names):]
    w = _per_dispatch(_counter_csv(write_dir), "WRITE_SIZE")[-len(names):]
    if len(f) != len(names) or len(w) != len(names):
        raise SystemExit(f"{len(f)} / {len(w)} dispatches in the counter files, {len(names)} in the dispatch order")
    n = alg[1] // 2
    kf, kw = n / (f[1]["value"] * 1024.0), n / (w[1]["value"] * 1024.0)
    print(f"Calibration ({kernels[1]} over {n} B read, {n} B written): FETCH_SIZE read {f[1]['value']:.1f} -> factor {kf:.3f}; "
          f"WRITE_SIZE read {w[1]['value']:.1f} -> factor {kw:.3f}.  Every value below is the counter x 1024 x that factor.\n")
    print("| layer | kernel | read MB | written MB | total MB | algorithmic MB | total / algorithmic |")
    print("|---|---|---:|---:|---:|---:|---:|")
    for i in range(2, len(names)):
        if short_name(f[i]["kernel"]) != kernels[i]:
            raise SystemExit(f"dispatch {i} ({names[i]}): the profile saw {short_name(f[i]['kernel'])!r}, the library reported {kernels[i]!r}")
        rd, wr = f[i]["value"] * 1024.0 * kf, w[i]["value"] * 1024.0 * kw
        print(f"| {names[i]} | `{kernels[i]}` | {rd / 1e6:.2f} | {wr / 1e6:.2f} | {(rd + wr) / 1e6:.2f} | {alg[i] / 1e6:.2f} | {(rd + wr) / alg[i]:.2f} |")


def stats(path):
    print("| kernel | calls | average us | total ms | share % |")
    print("|---|---:|---:|---:|---:|")
    for r in csv.DictReader(open(path)):
        print(f"| `{short_name(r['Name'])}` | {r['Calls']} | {float(r['AverageNs']) / 1e3:.2f} | {float(r['TotalDurationNs']) / 1e6:.3f} | {float(r['Percentage']):.2f} |")


def pmc(d, substring=""):
    tab = collections.OrderedDict()
    for path in sorted(glob.glob(os.path.join(d, "**", "*counter_collection.csv"), recursive=True)):
        rows = list(csv.DictReader(open(path)))
        last = {}
        for r in rows:
            last[r["Kernel_Name"]] = max(last.get(r["Kernel_Name"], 0), int(r["Dispatch_Id"]))
        for r in rows:
            if int(r["Dispatch_Id"]) == last[r["Kernel_Name"]]:
                e = tab.setdefault(short_name(r["Kernel_Name"]), collections.OrderedDict())
                e[r["Counter_Name"]] = e.get(r["Counter_Name"], 0.0) + float(r["Counter_Value"])
    for k, v in tab.items():
        if substring and substring not in k:
            continue
        print(f"== {k}")
        for name, x in v.items():
            print(f"   {name:42s} {x:18.0f}")


def main(argv):
    if len(argv) >= 4 and argv[0] == "traffic":
        traffic(argv[1], argv[2], argv[3])
    elif len(argv) >= 2 and argv[0] == "stats":
        stats(argv[1])
    elif len(argv) >= 2 and argv[0] == "pmc":
        pmc(argv[1], argv[2] if len(argv) > 2 else "")
    else:
        print(__doc__, file=sys.stderr)
        return 2
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
