"""Turns rocprofv3 CSV output into the figures quoted for the kernels.

    python -m intra_amd.rocprof_summary kernels  <dir>            # per-kernel calls / avg / min / max ns
    python -m intra_amd.rocprof_summary counters <dir> [<dir>..]  # per-kernel average of every counter
    python -m intra_amd.rocprof_summary traffic --fetch <dir> --write <dir> --seqlen S --out profiles/hbm_traffic.json

`<dir>` is what `rocprofv3 -d <dir> --output-format csv` wrote (searched recursively for
*_kernel_stats.csv / *_kernel_trace.csv / *_counter_collection.csv).

`traffic` converts FETCH_SIZE and WRITE_SIZE (KiB per dispatch, one counter run each) of the forward
kernel into HBM bytes per launch.  The raw readings are scaled by what the same counter shows for
a plain device-to-device copy of known size in the same run (`bench.py --copy-calib` issues three
1 GiB copies), and the result is stored together with a hash of the kernel sources, so that
bench.py reports it only for the kernel it was measured on.
"""
import argparse
import collections
import csv
import glob
import hashlib
import json
import os

HERE = os.path.dirname(os.path.abspath(__file__))
KERNEL_SOURCES = [os.path.join(HERE, "csrc", n) for n in ("intra_kernel.hip.h", "intra_maps.h", "intra_api.hip")]
COPY_BYTES = 1 << 30


def source_hash():
    h = hashlib.sha256()
    for path in KERNEL_SOURCES:
        h.update(open(path, "rb").read())
    return h.hexdigest()[:16]


def _find(directory, suffix):
    hits = sorted(glob.glob(os.path.join(directory, "**", "*" + suffix), recursive=True))
    if not hits:
        raise SystemExit(f"no *{suffix} under {directory}")
    return hits[0]


def short(name):
    name = name.replace("void ", "")
    return name if len(name) <= 90 else name[:87] + "..."


def kernels(directory):
    rows = collections.defaultdict(list)
    for r in csv.DictReader(open(_find(directory, "_kernel_trace.csv"))):
        rows[r["Kernel_Name"]].append(int(r["End_Timestamp"]) - int(r["Start_Timestamp"]))
    total = sum(sum(v) for v in rows.values())
    print("| kernel | calls | avg ns | min ns | max ns | share |\n|---|---|---|---|---|---|")
    for name, v in sorted(rows.items(), key=lambda kv: -sum(kv[1])):
        print(f"| `{short(name)}` | {len(v)} | {sum(v) / len(v):.0f} | {min(v)} | {max(v)} | {100 * sum(v) / total:.1f} % |")


def counter_values(directory):
    """{kernel name: {counter: [value per dispatch]}}"""
    acc = collections.defaultdict(lambda: collections.defaultdict(list))
    for r in csv.DictReader(open(_find(directory, "_counter_collection.csv"))):
        acc[r["Kernel_Name"]][r["Counter_Name"]].append(float(r["Counter_Value"]))
    return acc


def counter_means(directory):
    """{kernel name: {counter: (dispatches, mean value)}}"""
    return {k: {c: (len(v), sum(v) / len(v)) for c, v in cs.items()} for k, cs in counter_values(directory).items()}


def counters(directories, only):
    for d in directories:
        for name, cs in counter_means(d).items():
            if only and only not in name:
                continue
            for c, (n, mean) in sorted(cs.items()):
                print(f"{os.path.basename(os.path.normpath(d)):10s} {short(name)[:60]:60s} {c:34s} n={n:<4d} {mean:.6g}")


def _reading(directory, counter, kernel_part, largest=False):
    """Mean over the dispatches of the first kernel whose name contains kernel_part; largest=True
    takes its largest dispatch instead (the 1 GiB calibration copies among smaller copies)."""
    hits = [cs[counter] for name, cs in counter_values(directory).items() if kernel_part in name and counter in cs]
    if not hits:
        raise SystemExit(f"{counter} of a kernel matching {kernel_part!r} not found under {directory}")
    return max(hits[0]) if largest else sum(hits[0]) / len(hits[0])


def traffic(args):
    out = {"kernel": args.kernel, "seqlen": args.seqlen, "source_sha256_16": source_hash(),
           "copy_calibration_bytes": COPY_BYTES}
    total = 0.0
    for counter, directory in (("FETCH_SIZE", args.fetch), ("WRITE_SIZE", args.write)):
        raw = _reading(directory, counter, args.kernel)            # KiB per dispatch as the counter reports it
        copy = _reading(directory, counter, args.copy_kernel, largest=True)  # the same counter for a 1 GiB copy
        scale = (COPY_BYTES / 1024) / copy
        out[counter.lower()] = {"raw_kib": round(raw, 1), "copy_raw_kib": round(copy, 1), "scale": round(scale, 4),
                                "bytes": round(raw * scale * 1024)}
        total += raw * scale * 1024
    out["hbm_bytes_per_launch"] = round(total)
    with open(args.out, "w") as f:
        json.dump(out, f, indent=1)
        f.write("\n")
    print(json.dumps(out))


def main():
    ap = argparse.ArgumentParser()
    sub = ap.add_subparsers(dest="cmd", required=True)
    k = sub.add_parser("kernels")
    k.add_argument("dir")
    c = sub.add_parser("counters")
    c.add_argument("dirs", nargs="+")
    c.add_argument("--kernel", default="intra_", help="only kernels whose name contains this")
    t = sub.add_parser("traffic")
    t.add_argument("--fetch", required=True)
    t.add_argument("--write", required=True)
    t.add_argument("--kernel", default="intra_fwd_kernel")
    t.add_argument("--copy-kernel", default="copyBuffer", help="name part of the calibration copy's kernel")
    t.add_argument("--seqlen", type=int, default=32768)
    t.add_argument("--out", required=True)
    args = ap.parse_args()
    if args.cmd == "kernels":
        kernels(args.dir)
    elif args.cmd == "counters":
        counters(args.dirs, args.kernel)
    else:
        traffic(args)


if __name__ == "__main__":
    main()
