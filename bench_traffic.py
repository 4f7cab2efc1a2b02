"""HBM bytes per launch of the six GEMM launches of a bench.py step, from two rocprofv3 counter runs.

  cd /tmp; export TMPDIR=/tmp; cd <repository>
  rocprofv3 --pmc FETCH_SIZE --output-format csv -d prof_out/fetch -- python3 bench.py --steps 3 --warmup 1 \
      --no-cpu-baseline --no-graph --copy-calibration
  rocprofv3 --pmc WRITE_SIZE --output-format csv -d prof_out/write -- python3 bench.py --steps 3 --warmup 1 \
      --no-cpu-baseline --no-graph --copy-calibration
  python3 bench_traffic.py prof_out/fetch prof_out/write --config c3

writes profiles/bench_<config>_hbm_traffic.json (read by bench.py for roofline.traffic) and prints the table kept
next to it as text.  Both counters are in KiB per dispatch; each is scaled by what it reads for the one 256 MiB
device-to-device copy that --copy-calibration issues first.  The JSON carries a digest of the kernel sources: bench.py
reports no traffic figure when the sources have changed since the counters were read.
"""
import argparse
import csv
import glob
import hashlib
import json
import os
import sys

ROOT = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(ROOT, "analog_moe_amd", "csrc")
COPY_BYTES = 256 << 20
ROLES = {"fwd": ("fwd_up", "fwd_down"), "xgrad": ("xgrad_down", "xgrad_up"), "wgrad": ("wgrad_down", "wgrad_up")}


def source_digest() -> str:
    """sha256 over the kernel sources (names and contents), the same for the profiling run and for bench.py"""
    h = hashlib.sha256()
    for dirpath, _, files in sorted(os.walk(CSRC)):
        for f in sorted(files):
            if f.endswith((".h", ".hip")):
                h.update(f.encode())
                with open(os.path.join(dirpath, f), "rb") as fh:
                    h.update(fh.read())
    return h.hexdigest()


def traffic_file(config: str) -> str:
    return os.path.join(ROOT, "profiles", f"bench_{config}_hbm_traffic.json")


def load_traffic(config: str):
    """(bytes per launch by role, note): the figures, or None and the reason there are none."""
    path = traffic_file(config)
    if not os.path.exists(path):
        return None, "no counter run recorded for this workload"
    with open(path) as fh:
        rec = json.load(fh)
    if rec.get("source_digest") != source_digest():
        return None, "the kernel sources changed after the recorded counter run"
    out = {role: v["total_bytes"] for role, v in rec["launches"].items()}
    out["step_total"] = rec.get("step_total_bytes")
    return out, None


def family(kernel: str):
    """Which of the three GEMM families a kernel name belongs to (None: a companion)."""
    if "ws256_kernel<" in kernel:                # <T, weights-K-contiguous, ...>: the input gradient reads W that way
        args = kernel.split("ws256_kernel<", 1)[1].split(">", 1)[0].split(",")
        return "xgrad" if args[1].strip() == "true" else "fwd"
    if "fwd256_kernel" in kernel:
        return "fwd"
    if "bwdx256_kernel" in kernel:
        return "xgrad"
    if "gemm_wgrad_kernel" in kernel or "wgrad256_kernel" in kernel:
        return "wgrad"
    if "gemm_rows_kernel<" in kernel:            # <T, W_KC, MODE, FAST>: mode 2 is the input gradient
        args = kernel.split("gemm_rows_kernel<", 1)[1].split(">", 1)[0].split(",")
        return "xgrad" if args[2].strip() == "2" else "fwd"
    return None


def read_counter(directory: str, counter: str, others: dict):
    """Per role: list of counter readings (one per step); and the copy's reading.  others: filled with the summed
    readings of the launches that are not one of the six (by kernel name)."""
    files = glob.glob(os.path.join(directory, "**", "*counter_collection.csv"), recursive=True)
    if not files:
        sys.exit(f"no *counter_collection.csv under {directory}")
    files.sort(key=os.path.getmtime)
    if len(files) > 1:
        print(f"{len(files)} counter files under {directory}: reading the newest, {files[-1]}", file=sys.stderr)
    with open(files[-1]) as fh:
        rows = [r for r in csv.DictReader(fh) if r["Counter_Name"] == counter]
    rows.sort(key=lambda r: int(r.get("Dispatch_Id", 0)))
    seen = {"fwd": 0, "xgrad": 0, "wgrad": 0}
    out, copy, kernels = {}, None, {}
    for r in rows:
        name, val = r["Kernel_Name"], float(r["Counter_Value"])
        if "copyBuffer" in name:
            copy = val if copy is None else max(copy, val)
            continue
        fam = family(name)
        if fam is None:                            # a companion launch: summed per kernel over the whole run
            if "amoe::" in name:
                short = name.split("(")[0].replace("void ", "").replace("amoe::", "")
                others[short] = others.get(short, 0.0) + val
            continue
        role = ROLES[fam][seen[fam] % 2]
        seen[fam] += 1
        out.setdefault(role, []).append(val)
        kernels[role] = name.split("(")[0].replace("void ", "")
    if copy is None:
        sys.exit(f"no device copy in {directory}: run bench.py with --copy-calibration")
    return out, copy, kernels


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("fetch_dir")
    ap.add_argument("write_dir")
    ap.add_argument("--config", default="c3")
    ap.add_argument("--skip-first", type=int, default=1, help="steps at the start (warm-up) left out of the average")
    args = ap.parse_args()
    ofetch, owrite = {}, {}
    fetch, fcopy, kernels = read_counter(args.fetch_dir, "FETCH_SIZE", ofetch)
    write, wcopy, _ = read_counter(args.write_dir, "WRITE_SIZE", owrite)
    fscale, wscale = COPY_BYTES / (fcopy * 1024.0), COPY_BYTES / (wcopy * 1024.0)
    launches = {}
    print(f"copy of {COPY_BYTES >> 20} MiB reads FETCH_SIZE {fcopy:.0f}, WRITE_SIZE {wcopy:.0f} (KiB): "
          f"scale factors fetch x{fscale:.3f}, write x{wscale:.3f}")
    print(f"{'launch':12s} {'FETCH_SIZE':>11s} {'WRITE_SIZE':>11s} {'read MB':>9s} {'write MB':>9s} {'total MB':>9s}  kernel")
    for fam in ("fwd", "xgrad", "wgrad"):
        for role in ROLES[fam]:
            f = fetch[role][args.skip_first:] or fetch[role]
            w = write[role][args.skip_first:] or write[role]
            fk, wk = sum(f) / len(f), sum(w) / len(w)
            rb, wb = fk * 1024.0 * fscale, wk * 1024.0 * wscale
            launches[role] = {"fetch_size_kib": fk, "write_size_kib": wk, "read_bytes": rb, "write_bytes": wb,
                              "total_bytes": rb + wb, "kernel": kernels[role]}
            print(f"{role:12s} {fk:11.0f} {wk:11.0f} {rb / 1e6:9.1f} {wb / 1e6:9.1f} {(rb + wb) / 1e6:9.1f}  {kernels[role]}")
    # the other launches of a step, per step (all traced steps: they have no warm-up effects worth a separate average)
    n_steps = len(fetch["fwd_up"])
    companions = {}
    for name in sorted(ofetch, key=lambda n: -(ofetch[n] * fscale + owrite.get(n, 0.0) * wscale)):
        rb, wb = ofetch[name] * 1024.0 * fscale / n_steps, owrite.get(name, 0.0) * 1024.0 * wscale / n_steps
        if rb + wb < 1e6:
            continue
        companions[name] = {"read_bytes": rb, "write_bytes": wb, "total_bytes": rb + wb}
        print(f"{name[:40]:40s} {'':>11s} {'':>11s} {rb / 1e6:9.1f} {wb / 1e6:9.1f} {(rb + wb) / 1e6:9.1f}  (per step)")
    step_total = sum(v["total_bytes"] for v in launches.values()) + sum(v["total_bytes"] for v in companions.values())
    print(f"all launches of one step: {step_total / 1e6:.0f} MB")
    rec = {"workload": args.config, "source_digest": source_digest(), "companions": companions,
           "step_total_bytes": step_total,
           "copy_calibration": {"bytes": COPY_BYTES, "fetch_size_kib": fcopy, "write_size_kib": wcopy,
                                "fetch_scale": fscale, "write_scale": wscale},
           "launches": launches}
    with open(traffic_file(args.config), "w") as fh:
        json.dump(rec, fh, indent=1, sort_keys=True)
        fh.write("\n")
    print("wrote", os.path.relpath(traffic_file(args.config), ROOT))


if __name__ == "__main__":
    main()
