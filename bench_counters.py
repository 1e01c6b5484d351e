"""Turns the two rocprofv3 counter runs of the headline benchmark into the small summary
that bench.py reads for `roofline.traffic`:

    cd /tmp && export TMPDIR=/tmp
    B="python3 /root/repo/bench.py --steps 3 --warmup 1 --no-cpu --no-extra --copy-probe"
    rocprofv3 --pmc FETCH_SIZE --output-format csv -d OUT/fetch -o fetch -- $B
    rocprofv3 --pmc WRITE_SIZE --output-format csv -d OUT/write -o write -- $B
    python3 /root/repo/bench_counters.py OUT/fetch/fetch_counter_collection.csv \
            OUT/write/write_counter_collection.csv

FETCH_SIZE and WRITE_SIZE count KiB per dispatch in units that depend on the chip; the
copy probe of bench.py (relu_fwd_kernel with alpha = 1 over 64 Mi floats: 256 MiB read and
256 MiB written per launch) says what one count is worth, and every kernel's counts are
scaled by that.  Written: profiles/conv_f32_resnet3x3_256x56x56x64.counters.json, stamped with the date and a
digest of the kernel sources the counters were taken on (bench.py reports a summary from other sources as stale).
"""
import collections
import csv
import json
import os
import sys

ROOT = os.path.dirname(os.path.abspath(__file__))
OUT = os.path.join(ROOT, "profiles", "conv_f32_resnet3x3_256x56x56x64.counters.json")
PROBE = "relu_fwd_kernel"
PROBE_KIB = 64 * 1024 * 1024 * 4 / 1024.0          # read and written per probe launch


def short(name):
    name = name.replace("void ", "").replace("aeth::", "")
    return name.split("(")[0].split("<")[0]


def averages(path, counter):
    per = collections.defaultdict(list)
    # one row per dispatch and counter (several rows per dispatch when the counter is split by instance)
    by_dispatch = collections.defaultdict(float)
    names = {}
    for r in csv.DictReader(open(path)):
        if r["Counter_Name"] != counter:
            continue
        key = r.get("Dispatch_Id") or r.get("Correlation_Id")
        by_dispatch[key] += float(r["Counter_Value"])
        names[key] = short(r["Kernel_Name"])
    for key, v in by_dispatch.items():
        per[names[key]].append(v)
    return {k: (sum(v) / len(v), len(v)) for k, v in per.items()}


def main(fetch_csv, write_csv):
    fetch = averages(fetch_csv, "FETCH_SIZE")
    write = averages(write_csv, "WRITE_SIZE")
    if PROBE not in fetch or PROBE not in write:
        raise SystemExit("the copy probe is missing: run bench.py with --copy-probe")
    f_scale = PROBE_KIB / fetch[PROBE][0]
    w_scale = PROBE_KIB / write[PROBE][0]
    kernels = {}
    for k in sorted(set(fetch) & set(write)):
        if k == PROBE:
            continue
        rd = fetch[k][0] * f_scale * 1024.0
        wr = write[k][0] * w_scale * 1024.0
        kernels[k] = {"fetch_size_raw": round(fetch[k][0], 1), "write_size_raw": round(write[k][0], 1),
                      "launches": fetch[k][1], "read_bytes": round(rd), "written_bytes": round(wr),
                      "traffic_bytes": round(rd + wr)}
    import datetime
    import bench
    out = {"measured": {"date": datetime.date.today().isoformat(), "sources_digest": bench.sources_digest(),
                        "note": "SHA-256 (16 hex digits) over aether-ml_amd/csrc/*.h, *.hip as bench.sources_digest() forms it"},
           "workload": "fp32 conv fprop + wgrad + dgrad, input NHWC [256,56,56,64], 64 filters 3x3 s1 same",
           "command": "rocprofv3 --pmc FETCH_SIZE (then WRITE_SIZE) --output-format csv -- python3 bench.py "
                      "--steps 3 --warmup 1 --no-cpu --no-extra --copy-probe",
           "copy_probe": {"kernel": PROBE, "kib_read_and_written": PROBE_KIB,
                          "fetch_size_raw": round(fetch[PROBE][0], 1), "write_size_raw": round(write[PROBE][0], 1),
                          "fetch_scale": round(f_scale, 4), "write_scale": round(w_scale, 4)},
           "kernels": kernels}
    with open(OUT, "w") as f:
        json.dump(out, f, indent=1)
    print(json.dumps(out, indent=1))


if __name__ == "__main__":
    main(sys.argv[1], sys.argv[2])
