"""HBM traffic per kernel launch from two hardware-counter runs, and the file bench.py reads it from.

    python -m tfjs_amd.traffic FETCH.csv WRITE.csv [--json profiles/traffic.json] [--md SUMMARY.md]
                               [--command "the profiled command"] [--title "..."]

FETCH.csv and WRITE.csv are the `*_counter_collection.csv` files of two `rocprofv3 --pmc` runs of the
same command, one collecting FETCH_SIZE, the other WRITE_SIZE (one counter per run). The command must
also launch the plain copy kernel `copy_f4` on a buffer of known size (`bench.py --copy-yardstick MIB`):
what the counters read for it fixes the unit of every other reading. The JSON holds bytes per launch by
kernel symbol, spelled as tfhip_last_kernel spells it, with the commit and a hash of the kernel sources
the figures belong to; `load()` compares that hash with the sources as they are now.
"""
import argparse
import csv
import hashlib
import json
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "tfjs_amd", "csrc")


def source_hash():
    """sha256 over the kernel sources (names and contents, in name order)."""
    h = hashlib.sha256()
    for name in sorted(os.listdir(CSRC)):
        if name.endswith((".hip", ".h", ".cc")):
            h.update(name.encode())
            with open(os.path.join(CSRC, name), "rb") as f:
                h.update(f.read())
    return h.hexdigest()


def symbol(kernel_name):
    """'void tfhip::(anonymous namespace)::gemm_kernel<32, 32>(float const*, ...)' -> 'gemm_kernel<32, 32>'"""
    text = kernel_name.strip()
    if text.startswith("void "):
        text = text[5:]
    depth = 0
    for i, ch in enumerate(text):
        if ch == "<":
            depth += 1
        elif ch == ">":
            depth -= 1
        elif ch == "(" and depth == 0 and not text.startswith("(anonymous namespace)", i):
            text = text[:i]
            break
    # namespaces in front of the name (not those inside template arguments)
    head = text.split("<", 1)[0]
    tail = text[len(head):]
    return head.split("::")[-1] + tail.replace("tfhip::", "").replace("(anonymous namespace)::", "")


def read_counter(path, counter, by_grid=False, copy_bytes=None):
    """{symbol: [value per dispatch]} for one counter; the values of one dispatch (one row per
    XCD or shader engine in some rocprofv3 versions) are summed. by_grid: a symbol's launches are
    told apart by their grid size (one template serves several shapes). copy_bytes: only the
    copy_f4 launches of that size (one float4 per lane) keep the plain name `copy_f4`, the unit
    of the scaling; other copies (a benchmark row of their own) are named with their grid."""
    per_dispatch = {}
    with open(path, newline="") as f:
        for row in csv.DictReader(f):
            if row["Counter_Name"] != counter:
                continue
            name = symbol(row["Kernel_Name"])
            if name == "copy_f4":
                if copy_bytes is not None and int(row["Grid_Size"]) != copy_bytes // 16:
                    name += " grid " + row["Grid_Size"]
            elif by_grid:
                name += " grid " + row["Grid_Size"]
            key = (row["Dispatch_Id"], name)
            per_dispatch[key] = per_dispatch.get(key, 0.0) + float(row["Counter_Value"])
    out = {}
    for (_, name), value in per_dispatch.items():
        out.setdefault(name, []).append(value)
    return out


def summarise(fetch_csv, write_csv, copy_bytes, by_grid=False):
    fetch = read_counter(fetch_csv, "FETCH_SIZE", by_grid, copy_bytes)
    write = read_counter(write_csv, "WRITE_SIZE", by_grid, copy_bytes)
    if "copy_f4" not in fetch or "copy_f4" not in write:
        raise SystemExit("the profiled command launched no copy_f4 kernel: nothing to scale the counters by")
    mean = lambda v: sum(v) / len(v)
    copy_kib = copy_bytes / 1024.0
    fetch_scale, write_scale = copy_kib / mean(fetch["copy_f4"]), copy_kib / mean(write["copy_f4"])
    rows = []
    for name in fetch:
        f, w = mean(fetch[name]), mean(write.get(name, [0.0]))
        rows.append(dict(kernel=name, dispatches=len(fetch[name]), fetch_avg=f, write_avg=w,
                         read_kib=f * fetch_scale, write_kib=w * write_scale,
                         bytes_per_launch=int(round((f * fetch_scale + w * write_scale) * 1024))))
    rows.sort(key=lambda r: -r["bytes_per_launch"] * r["dispatches"])
    return rows, fetch_scale, write_scale, mean(fetch["copy_f4"]), mean(write["copy_f4"])


def git_head():
    try:
        return subprocess.run(["git", "-C", ROOT, "rev-parse", "HEAD"], stdout=subprocess.PIPE, stderr=subprocess.DEVNULL,
                              text=True, timeout=10).stdout.strip() or None
    except (OSError, subprocess.SubprocessError):
        return None


def load(path):
    """(bytes per launch by symbol, stale): stale when the file is missing or the kernel sources
    have changed since it was written."""
    try:
        with open(path) as f:
            data = json.load(f)
    except (OSError, ValueError):
        return {}, True
    return data.get("bytes_per_launch", {}), data.get("source_hash") != source_hash()


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("fetch_csv")
    ap.add_argument("write_csv")
    ap.add_argument("--copy-mib", type=int, default=256, help="size of the copy_f4 launches of the profiled command")
    ap.add_argument("--json", help="write the bytes-per-launch table here (bench.py reads profiles/traffic.json)")
    ap.add_argument("--md", help="write a readable summary here")
    ap.add_argument("--command", default="", help="the profiled command, quoted into the summary")
    ap.add_argument("--by-grid", action="store_true", help="one row per symbol and grid size")
    ap.add_argument("--title", default="HBM traffic per launch (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE)")
    args = ap.parse_args()
    rows, fs, ws, fcopy, wcopy = summarise(args.fetch_csv, args.write_csv, args.copy_mib << 20, args.by_grid)
    head, digest = git_head(), source_hash()
    if args.json:
        with open(args.json, "w") as f:
            json.dump(dict(git_head=head, source_hash=digest, command=args.command,
                           scale=dict(fetch=round(fs, 4), write=round(ws, 4), copy_mib=args.copy_mib),
                           bytes_per_launch={r["kernel"]: r["bytes_per_launch"] for r in rows}), f, indent=1)
            f.write("\n")
    if args.md:
        with open(args.md, "w") as f:
            f.write("# %s\n\nTwo runs, one counter each (FETCH_SIZE, then WRITE_SIZE):\n\n```\n%s\n```\n\n" % (args.title, args.command))
            f.write("Kernel sources: commit %s, source hash %s.\n\n" % (head, digest[:16]))
            f.write("Scaling: the command's `copy_f4` launches read %d MiB and write %d MiB each; the counters read "
                    "FETCH_SIZE = %.1f and WRITE_SIZE = %.1f for them, so readings are multiplied by %.3f (reads) and "
                    "%.3f (writes) to give KiB. Averages are over all dispatches of a symbol in the run.\n\n"
                    % (args.copy_mib, args.copy_mib, fcopy, wcopy, fs, ws))
            f.write("| kernel | dispatches | FETCH_SIZE avg | WRITE_SIZE avg | read KiB | write KiB | traffic bytes / launch |\n")
            f.write("|---|---:|---:|---:|---:|---:|---:|\n")
            for r in rows:
                f.write("| `%s` | %d | %.1f | %.1f | %.0f | %.0f | %d |\n" % (
                    r["kernel"], r["dispatches"], r["fetch_avg"], r["write_avg"], r["read_kib"], r["write_kib"],
                    r["bytes_per_launch"]))
    if not args.json and not args.md:
        for r in rows:
            print("%-60s %6d %14d" % (r["kernel"], r["dispatches"], r["bytes_per_launch"]))


if __name__ == "__main__":
    main()
