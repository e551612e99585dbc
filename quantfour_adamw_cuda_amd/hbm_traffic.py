"""HBM traffic of the step's kernels as hardware counters saw it, kept in
profiles/hbm_traffic.json and read by bench.py for its `roofline.traffic` field.

An entry is valid for the kernel sources it was measured on: every entry carries the hash of
csrc/q4adamw*.hip and csrc/q4adamw_*.h at that time, and `lookup` returns None for an entry
whose hash differs from the sources in the tree, so a number never outlives the kernel it
describes.  The exceptions are spelled out in the entry itself: when a WRITE_SIZE session could
not be taken on the present sources, `--write-from-record` takes the written bytes from an
earlier record file, and `--restamp-from-record` carries whole entries over a change of the
sources; such an entry names the sources each of its sessions ran on (`fetch_source_hash`,
`write_source_hash`) and why they still describe the present kernels (`write_note`, `note`).

One profiler session per job on the GPU machine, `python3 -u`, `--progress` and a hard
`timeout -s KILL`: counter sessions of this command have stopped responding now and then, and
that way a stalled one ends with a non-zero status and shows the phase it stopped in.

Recording (rocprofv3 cannot split counters over passes, so one run per counter; on the GPU
machine, from the repository root, after `cd /tmp && export TMPDIR=/tmp && cd -`):

    rocprofv3 --pmc FETCH_SIZE --output-format csv -d out/pmc_fetch -o fetch -- \\
        python3 -u bench.py --steps 3 --warmup 1 --configs none --no-ceiling --no-cpu-baseline --calibrate-copy --progress
    rocprofv3 --pmc WRITE_SIZE --output-format csv -d out/pmc_write -o write -- \\
        python3 -u bench.py --steps 3 --warmup 1 --configs none --no-ceiling --no-cpu-baseline --calibrate-copy --progress
    python3 -m quantfour_adamw_cuda_amd.hbm_traffic --workload llama3-8b --steps 4 \\
        --fetch-csv 'out/pmc_fetch/**/*counter_collection.csv' \\
        --write-csv 'out/pmc_write/**/*counter_collection.csv' \\
        --out profiles/hbm_traffic.json

(add the bench's --workload / --variance-scale / --round-type options to all three; --progress
names the bench's phases on stderr, so that a profiler run that stops shows where).  Both
counters are in KiB per dispatch; each is scaled by what the same counter reads for the
probe library's plain copy of 4 GiB (--calibrate-copy), whose traffic is known.
"""
import argparse
import csv
import glob
import hashlib
import json
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(_HERE)
DEFAULT_PATH = os.path.join(ROOT, "profiles", "hbm_traffic.json")
COPY_KERNEL = "probe_move_kernel<0>"
COPY_BYTES = 4 << 30
STEP_KERNELS = ("fused_4bit_kernel", "fused_4bit_rank1", "rank1_stats_kernel", "rank1_stats_any_kernel", "rank1_commit_kernel",
                "rank1_fold_kernel", "single_tensor_kernel")


def source_hash():
    """sha256 over the sources libq4adamw.so is built from (names and contents)."""
    h = hashlib.sha256()
    csrc = os.path.join(_HERE, "csrc")
    for name in sorted(os.listdir(csrc)):
        if name.startswith("q4adamw") and name.endswith((".hip", ".h")):
            h.update(name.encode())
            with open(os.path.join(csrc, name), "rb") as f:
                h.update(f.read())
    return h.hexdigest()[:16]


def key(workload, variance_scale="group", round_type="real-nearest", param_update="auto"):
    """param_update: the optimizer's option; anything but "auto" (the library's own choice of
    the parameter update's form) gets an entry of its own"""
    return f"{workload}|{variance_scale}|{round_type}" + ("" if param_update == "auto" else f"|{param_update}")


def lookup(workload, variance_scale="group", round_type="real-nearest", param_update="auto", path=DEFAULT_PATH):
    """The recorded entry (a dict with bytes_per_step ...) if one exists for these kernel
    sources, else None."""
    try:
        with open(path) as f:
            entries = json.load(f)["entries"]
    except (OSError, ValueError, KeyError):
        return None
    e = entries.get(key(workload, variance_scale, round_type, param_update))
    if not e or e.get("source_hash") != source_hash():
        return None
    return e


def _sum_counter(csv_paths, counter):
    """{kernel name: [sum of the counter over its dispatches, dispatches]} of one run"""
    out = {}
    for pattern in csv_paths:
        for path in glob.glob(pattern, recursive=True):
            with open(path, newline="") as f:
                for row in csv.DictReader(f):
                    if row["Counter_Name"] != counter:
                        continue
                    k = out.setdefault(row["Kernel_Name"], [0.0, 0])
                    k[0] += float(row["Counter_Value"])
                    k[1] += 1
    return out


def _store(out_path, entry_key, entry):
    """adds or replaces one entry of the record file"""
    try:
        with open(out_path) as f:
            doc = json.load(f)
    except (OSError, ValueError):
        doc = {"entries": {}}
    doc.setdefault("entries", {})[entry_key] = entry
    doc["unit"] = "bytes of HBM traffic per optimizer step (FETCH_SIZE + WRITE_SIZE, scaled by a copy of known size)"
    with open(out_path, "w") as f:
        json.dump(doc, f, indent=1, sort_keys=True)
        f.write("\n")
    return entry


def record(workload, variance_scale, round_type, fetch_csv, write_csv, steps, out_path, profile=None,
           param_update="auto", write_from_record=None, write_note=None):
    """write_from_record: instead of a WRITE_SIZE session (write_csv is then ignored), take the
    written bytes from the same key of an earlier record file -- for a session that could not
    be taken on the present sources.  The entry then names the sources that half was measured on
    (`write_source_hash`) and must say why it still describes the present kernels (`write_note`);
    bench.py repeats both beside the number."""
    if write_from_record:
        if not write_note:
            raise SystemExit("--write-from-record needs --write-note: why the earlier session still describes these kernels")
        return _record_with_earlier_write(workload, variance_scale, round_type, fetch_csv, steps, out_path, profile,
                                          param_update, write_from_record, write_note)
    fetch, write = _sum_counter(fetch_csv, "FETCH_SIZE"), _sum_counter(write_csv, "WRITE_SIZE")

    def pick(table, names):
        return {k: v for k, v in table.items() if any(n in k for n in names)}

    scales = {}
    for what, table in (("fetch", fetch), ("write", write)):
        copies = pick(table, (COPY_KERNEL,))
        if not copies:
            raise SystemExit(f"no {COPY_KERNEL} dispatch in the {what} run: profile bench.py with --calibrate-copy")
        kib, n = map(sum, zip(*copies.values()))
        scales[what] = (COPY_BYTES / 1024.0) / (kib / n)
    fetch_b = sum(v[0] for v in pick(fetch, STEP_KERNELS).values()) * 1024.0 * scales["fetch"] / steps
    write_b = sum(v[0] for v in pick(write, STEP_KERNELS).values()) * 1024.0 * scales["write"] / steps
    dispatches = sum(v[1] for v in pick(fetch, STEP_KERNELS).values()) / steps
    entry = {
        "source_hash": source_hash(),
        "bytes_per_step": fetch_b + write_b,
        "fetch_bytes_per_step": fetch_b,
        "write_bytes_per_step": write_b,
        "fetch_scale": scales["fetch"],
        "write_scale": scales["write"],
        "dispatches_per_step": dispatches,
        "steps_profiled": steps,
        "kernels": sorted(pick(fetch, STEP_KERNELS)),
    }
    if profile:
        entry["profile"] = profile
    return _store(out_path, key(workload, variance_scale, round_type, param_update), entry)


def _record_with_earlier_write(workload, variance_scale, round_type, fetch_csv, steps, out_path, profile,
                               param_update, earlier_path, note):
    fetch = _sum_counter(fetch_csv, "FETCH_SIZE")
    copies = {k: v for k, v in fetch.items() if COPY_KERNEL in k}
    if not copies:
        raise SystemExit(f"no {COPY_KERNEL} dispatch in the fetch run: profile bench.py with --calibrate-copy")
    kib, n = map(sum, zip(*copies.values()))
    fetch_scale = (COPY_BYTES / 1024.0) / (kib / n)
    step_kernels = {k: v for k, v in fetch.items() if any(name in k for name in STEP_KERNELS)}
    fetch_b = sum(v[0] for v in step_kernels.values()) * 1024.0 * fetch_scale / steps
    k = key(workload, variance_scale, round_type, param_update)
    with open(earlier_path) as f:
        earlier = json.load(f)["entries"].get(k)
    if not earlier:
        raise SystemExit(f"{earlier_path} holds no entry {k}")
    entry = {
        "source_hash": source_hash(),
        "bytes_per_step": fetch_b + earlier["write_bytes_per_step"],
        "fetch_bytes_per_step": fetch_b,
        "write_bytes_per_step": earlier["write_bytes_per_step"],
        "fetch_scale": fetch_scale,
        "write_scale": earlier["write_scale"],
        "write_source_hash": earlier["source_hash"],
        "write_note": note,
        "dispatches_per_step": sum(v[1] for v in step_kernels.values()) / steps,
        "steps_profiled": steps,
        "kernels": sorted(step_kernels),
    }
    if profile:
        entry["profile"] = profile
    return _store(out_path, k, entry)


def restamp(from_path, out_path, note, keys=None):
    """Carries entries of an earlier record over to the present sources: for a change of the
    sources after which the sessions could not be taken again.  Every carried entry keeps the
    hashes of the sources its two sessions ran on (`fetch_source_hash`, `write_source_hash`)
    and says why they still describe the present kernels (`note`); `source_hash` becomes the
    present one, which is what `lookup` compares."""
    if not note:
        raise SystemExit("a carried entry needs a note: why the earlier sessions still describe these kernels")
    with open(from_path) as f:
        earlier = json.load(f)["entries"]
    out = []
    for k in (keys or sorted(earlier)):
        if k not in earlier:
            raise SystemExit(f"{from_path} holds no entry {k}")
        e = dict(earlier[k])
        e["fetch_source_hash"] = e.get("fetch_source_hash", e["source_hash"])
        e["write_source_hash"] = e.get("write_source_hash", e["source_hash"])
        e["source_hash"] = source_hash()
        e["note"] = note
        out.append(_store(out_path, k, e))
    return out


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--workload", default=None)
    ap.add_argument("--variance-scale", default="group")
    ap.add_argument("--round-type", default="real-nearest")
    ap.add_argument("--param-update", default="auto")
    ap.add_argument("--fetch-csv", nargs="+", default=[])
    ap.add_argument("--write-csv", nargs="+", default=[])
    ap.add_argument("--write-from-record", default=None,
                    help="take the written bytes from this earlier record file instead of a WRITE_SIZE session")
    ap.add_argument("--write-note", default=None,
                    help="with --write-from-record: why that session still describes the present kernels")
    ap.add_argument("--steps", type=int, default=None, help="optimizer steps the profiled command ran (warm-up included)")
    ap.add_argument("--out", default=DEFAULT_PATH)
    ap.add_argument("--profile", default=None, help="the profiles/ summary that documents the run")
    ap.add_argument("--restamp-from-record", default=None,
                    help="carry every entry of this earlier record file over to the present sources (needs --note)")
    ap.add_argument("--note", default=None, help="with --restamp-from-record: why the earlier sessions still hold")
    a = ap.parse_args()
    if a.restamp_from_record:
        print(json.dumps(restamp(a.restamp_from_record, a.out, a.note), indent=1))
        return
    if not a.workload or not a.fetch_csv or a.steps is None:
        ap.error("give --workload, --fetch-csv and --steps (or --restamp-from-record)")
    if not a.write_csv and not a.write_from_record:
        ap.error("give --write-csv or --write-from-record")
    print(json.dumps(record(a.workload, a.variance_scale, a.round_type, a.fetch_csv, a.write_csv, a.steps,
                            a.out, a.profile, a.param_update, a.write_from_record, a.write_note), indent=1))


if __name__ == "__main__":
    main()
