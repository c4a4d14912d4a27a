"""HBM <-> L2 traffic of one kernel family of `bench.py`, from two rocprofv3 counter runs.

    cd /tmp && export TMPDIR=/tmp && cd <repo>
    rocprofv3 --pmc FETCH_SIZE --output-format csv -d prof_out/pmc_fetch -o b -- python3 bench.py --only-label 'gemm_w8a8[256]' --steps 3 --warmup 1 --calib-copy --calls-json prof_out/pmc_calls.json
    rocprofv3 --pmc WRITE_SIZE --output-format csv -d prof_out/pmc_write -o b -- python3 bench.py --only-label 'gemm_w8a8[256]' --steps 3 --warmup 1 --calib-copy
    python3 -m kairos_amd.traffic --label 'gemm_w8a8[256]' --kernel gemm_direct_kernel --fetch prof_out/pmc_fetch/b_counter_collection.csv \
        --write prof_out/pmc_write/b_counter_collection.csv --calls-json prof_out/pmc_calls.json --out profiles/bench_llama3_8b_traffic.json

`bench.py --only-label L` runs only the calls of the step that the benchmark books under label L, so every dispatch of
the kernel family in the counter files belongs to L (a call may be two dispatches: head and tail launch).  `--calib-copy`
adds one 1 GiB device-to-device copy, whose known size gives the factor each counter has to be scaled with (KiB as
reported -> bytes moved).  The result carries a hash of the kernel sources; `bench.py` reports the traffic figure only
while that hash still matches the sources it runs.
"""
import argparse
import csv
import hashlib
import json
import os

HERE = os.path.dirname(os.path.abspath(__file__))
HASHED_SOURCES = ["csrc/gemm_mfma.hip", "csrc/gemm_parts.h", "csrc/kmi_common.h"]
COPY_BYTES = 1 << 30


def source_hash():
    h = hashlib.sha256()
    for rel in HASHED_SOURCES:
        with open(os.path.join(HERE, rel), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def _sum_counter(path, counter, kernel_substr):
    total, n = 0.0, 0
    with open(path) as f:
        for r in csv.DictReader(f):
            if r["Counter_Name"] == counter and kernel_substr in r["Kernel_Name"]:
                total += float(r["Counter_Value"])
                n += 1
    return total, n


def _copy_factor(path, counter):
    """bytes per reported KiB for this counter, from the 1 GiB calibration copy (the largest copy dispatch)."""
    best = 0.0
    with open(path) as f:
        for r in csv.DictReader(f):
            if r["Counter_Name"] == counter and "copyBuffer" in r["Kernel_Name"]:
                best = max(best, float(r["Counter_Value"]))
    if best <= 0:
        raise SystemExit(f"{path}: no calibration copy found (run bench.py with --calib-copy)")
    return COPY_BYTES / best


def load(label, path):
    """-> (traffic bytes per call or None, note).  None when there is no measurement for `label` or it is stale."""
    if not os.path.exists(path):
        return None, "no counter measurement committed"
    with open(path) as f:
        rec = json.load(f)
    if rec.get("label") != label:
        return None, f"counter measurement is for {rec.get('label')}, the dominant kernel is {label}"
    if rec.get("source_hash") != source_hash():
        return None, "counter measurement predates the current kernel sources"
    return int(rec["traffic_bytes_per_call"]), f"rocprofv3 FETCH_SIZE / WRITE_SIZE, {os.path.relpath(path, os.path.dirname(HERE))}"


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--label", required=True)
    ap.add_argument("--kernel", required=True, help="substring of the mangled kernel name of the label's family")
    ap.add_argument("--fetch", required=True)
    ap.add_argument("--write", required=True)
    ap.add_argument("--calls-json", required=True, help="written by bench.py --only-label: calls made, algorithmic bytes")
    ap.add_argument("--out", required=True)
    a = ap.parse_args(argv)
    with open(a.calls_json) as f:
        calls = json.load(f)
    if calls["label"] != a.label:
        raise SystemExit(f"{a.calls_json} belongs to {calls['label']}")
    fetch, nf = _sum_counter(a.fetch, "FETCH_SIZE", a.kernel)
    write, nw = _sum_counter(a.write, "WRITE_SIZE", a.kernel)
    if nf == 0 or nf != nw:
        raise SystemExit(f"dispatch counts differ or are zero: {nf} (fetch run) vs {nw} (write run)")
    ff, wf = _copy_factor(a.fetch, "FETCH_SIZE"), _copy_factor(a.write, "WRITE_SIZE")
    n = calls["calls"]
    rec = {"label": a.label, "kernel": a.kernel, "calls": n, "dispatches": nf,
           "fetch_kib_per_call": round(fetch / n, 1), "write_kib_per_call": round(write / n, 1),
           "bytes_per_reported_kib": {"FETCH_SIZE": round(ff, 2), "WRITE_SIZE": round(wf, 2)},
           "traffic_bytes_per_call": int((fetch * ff + write * wf) / n),
           "algorithmic_bytes_per_call": calls["algorithmic_bytes_per_call"],
           "source_hash": source_hash(), "hashed_sources": HASHED_SOURCES}
    rec["traffic_over_algorithmic"] = round(rec["traffic_bytes_per_call"] / rec["algorithmic_bytes_per_call"], 3)
    with open(a.out, "w") as f:
        json.dump(rec, f, indent=1)
        f.write("\n")
    print(json.dumps(rec))


if __name__ == "__main__":
    main()
