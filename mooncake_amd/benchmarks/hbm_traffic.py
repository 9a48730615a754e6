#!/usr/bin/env python3
"""Turns two `rocprofv3 --pmc` runs of bench.py (one with FETCH_SIZE, one with
WRITE_SIZE; the hardware cannot hold both) into the HBM traffic per launch of
every kernel of the library, scaled by what the same counter reads for the
library's plain copy kernel over a known size (`bench.py --copy-calibration`).

    rocprofv3 --pmc FETCH_SIZE --output-format csv -d OUT/fetch -o p -- python3 bench.py \\
        --no-cpu-baseline --no-flushed --no-buffer-api --steps 3 --warmup 1 --kernel-iters 2 --copy-calibration 1024
    rocprofv3 --pmc WRITE_SIZE --output-format csv -d OUT/write -o p -- python3 bench.py  (same arguments)
    python -m mooncake_amd.benchmarks.hbm_traffic OUT/fetch OUT/write --workload dsv3_decode \\
        --copy-mib 1024 --commit $(git rev-parse --short HEAD) > profiles/dsv3_decode_hbm_traffic.txt

The output is a text summary; its `traffic_bytes <kernel> <bytes>` lines are
what bench.py reports as `roofline.traffic` for that kernel.
"""
from __future__ import annotations

import argparse
import collections
import csv
import glob
import os
import sys
from typing import Dict, List

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
KERNEL_SOURCES = ("mooncake_amd/csrc/ep_kernels.hip", "mooncake_amd/csrc/ep_kernels.h",
                  "mooncake_amd/csrc/ep_runtime.hip")


def kernel_sources_sha256(root: str = ROOT) -> str:
    """One hash over the sources the library's kernels and their launch code are built from: a traffic
    summary records it, and bench.py reports the summary's figures only while the sources still hash to it."""
    import hashlib
    h = hashlib.sha256()
    for rel in KERNEL_SOURCES:
        with open(os.path.join(root, rel), "rb") as f:
            h.update(f.read())
    return h.hexdigest()


# kernel-name fragments -> the short names bench.py uses
KERNELS = [("copy_kernel", "copy"), ("count_kernel", "count"), ("prefix_kernel", "prefix"), ("pack_fp8_kernel", "pack"),
           ("pack_bf16_kernel", "pack"), ("scale_transpose_kernel", "scales"), ("resolve_kernel", "resolve"),
           ("reduce_packed_kernel", "reduce_packed"), ("reduce_kernel", "reduce"), ("cast_chunks_kernel", "cast_chunks"),
           ("cast_back_kernel", "cast_back"), ("dispatch_small_kernel", "dispatch_small")]


def per_kernel_kib(directory: str) -> Dict[str, List[float]]:
    files = glob.glob(os.path.join(directory, "**", "*counter_collection.csv"), recursive=True)
    if not files:
        raise SystemExit(f"no *counter_collection.csv under {directory}")
    acc: Dict[str, List[float]] = collections.defaultdict(list)
    for row in csv.DictReader(open(files[0])):
        name = row["Kernel_Name"]
        if "mcep" not in name:
            continue
        for fragment, short in KERNELS:
            if fragment in name:
                acc[short].append(float(row["Counter_Value"]))
                break
    return acc


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("fetch_dir")
    ap.add_argument("write_dir")
    ap.add_argument("--workload", required=True)
    ap.add_argument("--copy-mib", type=int, required=True, help="size the copy kernel was run over")
    ap.add_argument("--commit", default="unknown", help="commit of the library the counters were collected on")
    args = ap.parse_args(argv)
    fetch, write = per_kernel_kib(args.fetch_dir), per_kernel_kib(args.write_dir)
    mean = lambda v: sum(v) / len(v)
    if "copy" not in fetch or "copy" not in write:
        raise SystemExit("the runs hold no copy kernel: pass --copy-calibration to bench.py")
    known_kib = args.copy_mib * 1024.0
    f_scale, w_scale = known_kib / mean(fetch["copy"]), known_kib / mean(write["copy"])
    print(f"rocprofv3 counters: HBM traffic per launch, workload {args.workload}")
    print(f"measured_at_commit {args.commit}")
    print(f"kernel_sources_sha256 {kernel_sources_sha256()}")
    print(f"scale factors from the copy kernel over {args.copy_mib} MiB: FETCH_SIZE x {f_scale:.4f}, "
          f"WRITE_SIZE x {w_scale:.4f}")
    print()
    print(f"{'kernel':<16}{'launches':>9}{'FETCH_SIZE KiB':>16}{'WRITE_SIZE KiB':>16}{'read MB':>10}{'written MB':>12}"
          f"{'total MB':>10}")
    totals = {}
    for short in dict.fromkeys(s for _, s in KERNELS):
        if short not in fetch or short not in write or short == "copy":
            continue
        f_kib, w_kib = mean(fetch[short]), mean(write[short])
        rd, wr = f_kib * f_scale * 1024, w_kib * w_scale * 1024
        totals[short] = int(rd + wr)
        print(f"{short:<16}{len(fetch[short]):>9}{f_kib:>16.1f}{w_kib:>16.1f}{rd / 1e6:>10.1f}{wr / 1e6:>12.1f}"
              f"{(rd + wr) / 1e6:>10.1f}")
    print()
    for short, total in totals.items():
        print(f"traffic_bytes {short} {total}")
    print()
    alg = algorithmic(args.workload)
    if alg:
        print("measured / algorithmic bytes per launch (a ratio well above 1 means re-read or partly used sectors):")
        for short, (nbytes, formula) in alg.items():
            if short in totals:
                print(f"  {short:<14}{totals[short] / 1e6:>8.1f} /{nbytes / 1e6:>8.1f} MB = {totals[short] / nbytes:5.3f}   {formula}")
        print()
    bench_args = (f"--config {args.workload} --no-cpu-baseline --no-flushed --no-buffer-api --no-small-world --steps 3 "
                  f"--warmup 1 --kernel-iters 2 --copy-calibration {args.copy_mib}")
    print("Commands (on the GPU box, from the repository root; cd /tmp && export TMPDIR=/tmp first):")
    print(f"  rocprofv3 --pmc FETCH_SIZE --output-format csv -d {args.fetch_dir} -o p -- python3 bench.py {bench_args}")
    print(f"  rocprofv3 --pmc WRITE_SIZE --output-format csv -d {args.write_dir} -o p -- python3 bench.py {bench_args}")
    print(f"  python3 -m mooncake_amd.benchmarks.hbm_traffic {args.fetch_dir} {args.write_dir} --workload {args.workload} "
          f"--copy-mib {args.copy_mib} --commit {args.commit}")
    print("FETCH_SIZE and WRITE_SIZE are in KiB per dispatch; each is scaled by what it reads for the library's plain")
    print(f"copy kernel over {args.copy_mib} MiB in the same run.  bench.py reports the traffic_bytes line of its dominant")
    print("kernel as roofline.traffic while the kernel sources still hash to kernel_sources_sha256.")
    return 0


def algorithmic(workload: str):
    """Algorithmic bytes per launch of the data kernels of a named workload (seed 0), with their formulas:
    N tokens, S valid selections, H hidden, K top-k, E experts, R ranks."""
    try:
        from mooncake_amd.workloads import CONFIGS, algorithmic_bytes, generate
    except ImportError:
        return {}
    cfg = CONFIGS.get(workload)
    if cfg is None:
        return {}
    S = int((generate(cfg, seed=0)["topk_idx"] >= 0).sum())
    N, H = cfg.total_tokens, cfg.hidden
    alg = algorithmic_bytes(cfg, S)
    P = H + H // 128 * 4 if cfg.use_fp8 else 2 * H
    out = {
        "pack": (alg["dispatch"], "N*H*2 + N*K*8 read; S*(P+4) + E*4 + E*R*8 written (P = H + H/128*4 fp8, 2H bf16; "
                                  "fp8 scales leave through the scales kernel)"),
        "reduce": (alg["combine"], "S*H*2 + N*K*12 + S*4 read; N*H*2 written"),
        "reduce_packed": (S * P + alg["combine"] - S * 2 * H, "S*P + N*K*12 + S*4 read; N*H*2 written"),
        "cast_back": (S * P + S * 2 * H, "S*P read; S*H*2 written"),
    }
    return out


if __name__ == "__main__":
    sys.exit(main())
