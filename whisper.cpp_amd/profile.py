#!/usr/bin/env python3
"""rocprofv3 passes over the harness commands that bench.py times; run on a box with an MI355X:

    python whisper.cpp_amd/profile.py [--out DIR]

Writes, under --out: `kernel_stats_encoder.csv`, `kernel_stats_decoder.csv` (rocprofv3 --kernel-trace --stats), `decode_positions.txt`
(a decode step's launches one by one, from a kernel trace), `counters.json`
(per-kernel averages of the --pmc passes) and `traffic.json` — HBM bytes per launch for the kernels bench.py reports, FETCH_SIZE
and WRITE_SIZE per dispatch scaled by what the same counters read for a 256 MiB device copy.  `traffic.json` is what
bench.py reads as `roofline.traffic` once it is copied to profiles/traffic.json; the tables under profiles/ are written from
the other files.  Every pass is a run of its own (counters are not split over passes), each with the harness binary directly
behind `--`.
"""
from __future__ import annotations

import argparse
import collections
import csv
import glob
import json
import os
import shutil
import subprocess
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent
HARNESS = ROOT / "whisper.cpp_amd" / "lib" / "mi355x-harness"
ENC_MODEL = "/tmp/mi355x-synth-large-v3-q5_0.bin"
DEC_MODEL = "/tmp/mi355x-synth-large-v3-turbo-q8_0.bin"

ENC_CMD = [str(HARNESS), "bench", "--model", ENC_MODEL, "--what", "encoder", "--backend", "gpu"]
DEC_CMD = [str(HARNESS), "bench", "--model", DEC_MODEL, "--what", "decoder", "--backend", "gpu", "--batch", "5", "--kv-stride", "2"]

# kernel symbol (prefix) -> the name the backend's statistics and bench.py use, and the run it is taken from (the decoder
# command encodes a window first, with the turbo model's four decoder layers in the cross-attention launch)
BENCH_NAMES = [
    ("k_fattn_pk_tile", "flash_attn.seq_tile_pk", "encoder"), ("k_fattn_seq_tile", "flash_attn.seq_tile", "encoder"),
    ("void k_gemm_f16_dl_group", "mul_mat.gemm_group", "encoder"), ("void k_gemm_f16_dl<", "mul_mat.gemm_q5_0", "encoder"),
    ("void k_gemm_f16_rs<", "mul_mat.gemm_q5_0", "encoder"), ("void k_norm<5, 1", "norm_affine_emit", "encoder"), ("_Z6k_normILi5ELi1E", "norm_affine_emit", "encoder"),
    ("k_fattn_pk_row", "flash_attn.seq_row_pk", "decoder"), ("k_fattn_seq_row", "flash_attn.seq_row", "decoder"), ("void k_gemv_q8_0_tiles<20", "mul_mat.gemv_q8_0.vocab", "decoder"),
    ("void k_gemv_q8_0_tiles_norm<20", "norm_mul_mat.gemv_q8_0.vocab", "decoder"),
]

SQ_PASSES = [
    "SQ_WAVES SQ_WAVE_CYCLES SQ_BUSY_CYCLES SQ_ACTIVE_INST_VALU SQ_INSTS_VALU SQ_WAIT_INST_LDS SQ_WAIT_ANY SQ_ACTIVE_INST_LDS",
    "SQ_WAIT_INST_ANY SQ_ACTIVE_INST_ANY SQ_INSTS_LDS SQ_LDS_BANK_CONFLICT SQ_INSTS_SALU SQ_ACTIVE_INST_SCA SQ_VALU_MFMA_BUSY_CYCLES SQ_INSTS_VALU_MFMA_MOPS_F16",
    "SQ_INST_CYCLES_VMEM SQ_INSTS_VMEM SQ_LDS_IDX_ACTIVE SQ_LDS_ADDR_CONFLICT SQ_CYCLES SQ_INSTS_SMEM",
]


def run(cmd, log: Path, limit: int) -> None:
    print("+", " ".join(cmd), flush=True)
    with open(log, "w") as f:
        res = subprocess.run(["timeout", "-s", "KILL", str(limit), *cmd], stdout=f, stderr=subprocess.STDOUT)
    if res.returncode != 0:
        sys.stderr.write(log.read_text()[-2000:])
        raise SystemExit(f"failed ({res.returncode}): {' '.join(cmd)}")


def per_kernel(directory: Path) -> dict:
    """{kernel: {counter: (dispatches, sum)}} from a --pmc pass"""
    agg: dict = collections.defaultdict(lambda: collections.defaultdict(lambda: [0, 0.0]))
    for f in glob.glob(str(directory / "**" / "*counter_collection.csv"), recursive=True):
        for row in csv.DictReader(open(f)):
            a = agg[row["Kernel_Name"]][row["Counter_Name"]]
            a[0] += 1
            a[1] += float(row["Counter_Value"])
    return agg


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--out", default=str(ROOT / "gpurun_out" / "prof"))
    ap.add_argument("--skip-sq", action="store_true", help="only the kernel traces and the traffic counters")
    ap.add_argument("--head", default="", help="the commit of the tree being profiled (the GPU box's copy has no .git)")
    a = ap.parse_args()
    out = Path(a.out)
    out.mkdir(parents=True, exist_ok=True)
    os.environ.setdefault("TMPDIR", "/tmp")
    for model, arch, ftype in ((ENC_MODEL, "large-v3", "q5_0"), (DEC_MODEL, "large-v3-turbo", "q8_0")):
        if not Path(model).exists():
            run([str(HARNESS), "gen", "--arch", arch, "--ftype", ftype, "--out", model, "--seed", "1234"], out / "gen.log", 300)

    # ---- kernel traces
    for name, cmd in (("encoder", ENC_CMD + ["--reps", "10", "--warmup", "3"]), ("decoder", DEC_CMD + ["--reps", "3", "--warmup", "2", "--steps", "224"])):
        d = out / f"trace_{name}"
        run(["rocprofv3", "--kernel-trace", "--stats", "--output-format", "csv", "-d", str(d), "--", *cmd], out / f"trace_{name}.log", 170)
        for f in glob.glob(str(d / "**" / "*kernel_stats.csv"), recursive=True):
            shutil.copy(f, out / f"kernel_stats_{name}.csv")
        shutil.rmtree(d, ignore_errors=True)

    # ---- a decode step launch by launch: durations by position in the step (the steps begin where the token rows are
    # gathered: the instance of k_gemv_qr_norm_group whose last template argument is true, else k_get_rows_add)
    d = out / "trace_positions"
    run(["rocprofv3", "--kernel-trace", "--output-format", "csv", "-d", str(d), "--", *DEC_CMD, "--reps", "1", "--warmup", "1", "--steps", "224"], out / "trace_positions.log", 170)
    rows = []
    for f in glob.glob(str(d / "**" / "*kernel_trace.csv"), recursive=True):
        for r in csv.DictReader(open(f)):
            rows.append((int(r["Start_Timestamp"]), int(r["End_Timestamp"]), r["Kernel_Name"]))
    shutil.rmtree(d, ignore_errors=True)
    rows.sort()
    steps, cur = [], None
    for st, en, name in rows:
        if "k_get_rows_add" in name or ("k_gemv_qr_norm_group" in name and (", true>" in name or "ELb1EE" in name)):
            if cur: steps.append(cur)
            cur = []
        if cur is not None: cur.append((st, en, name))
    if cur: steps.append(cur)
    lengths = collections.Counter(len(x) for x in steps)
    n_launch = lengths.most_common(1)[0][0] if lengths else 0
    steps = [x for x in steps if len(x) == n_launch]
    with open(out / "decode_positions.txt", "w") as f:
        f.write(f"{len(steps)} steps of {n_launch} launches; microseconds; 'gap' is the idle time in front of the launch (under the profiler the host preparing it)\n")
        kernel_us = gap_us = 0.0
        for pos in range(n_launch):
            dur = sorted((x[pos][1] - x[pos][0]) / 1e3 for x in steps)
            gap = [(x[pos][0] - x[pos - 1][1]) / 1e3 for x in steps] if pos else [0.0]
            name = steps[0][pos][2].split("(")[0][:46]
            kernel_us += sum(dur) / len(dur); gap_us += sum(gap) / len(gap)
            f.write(f"{pos:2d} {name:46s} avg {sum(dur) / len(dur):6.2f} min {dur[0]:6.2f} med {dur[len(dur) // 2]:6.2f} max {dur[-1]:6.2f}  gap avg {sum(gap) / len(gap):5.2f}\n")
        f.write(f"kernel us per step {kernel_us:.1f}, gaps per step {gap_us:.1f}\n")

    # ---- HBM traffic: FETCH_SIZE and WRITE_SIZE, each a pass of its own, over encoder, decoder and a 256 MiB copy
    counters: dict = {}
    copy_cmd = [str(HARNESS), "copy", "--mib", "256", "--reps", "3"]
    for c in ("FETCH_SIZE", "WRITE_SIZE"):
        for name, cmd in (("encoder", ENC_CMD + ["--reps", "1", "--warmup", "0"]), ("decoder", DEC_CMD + ["--reps", "1", "--warmup", "0", "--steps", "16"]), ("copy", copy_cmd)):
            d = out / f"pmc_{name}_{c}"
            run(["rocprofv3", "--pmc", c, "--output-format", "csv", "-d", str(d), "--", *cmd], out / f"pmc_{name}_{c}.log", 120)
            for k, v in per_kernel(d).items():
                counters.setdefault(name, {}).setdefault(k, {})[c] = {"dispatches": v[c][0], "per_dispatch": v[c][1] / v[c][0]}
            shutil.rmtree(d, ignore_errors=True)
    copy_kernel = next(k for k in counters["copy"] if k.startswith("k_cpy"))
    copy_bytes = 256.0 * (1 << 20)
    scale = {c: copy_bytes / counters["copy"][copy_kernel][c]["per_dispatch"] for c in ("FETCH_SIZE", "WRITE_SIZE")}   # bytes per count

    traffic: dict = collections.defaultdict(lambda: [0.0, 0])
    detail = {}
    for name in ("encoder", "decoder"):
        for k, v in counters[name].items():
            bench = next((b for p, b, r in BENCH_NAMES if k.startswith(p) and r == name), None)
            if not bench or "FETCH_SIZE" not in v or "WRITE_SIZE" not in v:
                continue
            n = v["FETCH_SIZE"]["dispatches"]
            fetched, written = v["FETCH_SIZE"]["per_dispatch"] * scale["FETCH_SIZE"], v["WRITE_SIZE"]["per_dispatch"] * scale["WRITE_SIZE"]
            traffic[bench][0] += (fetched + written) * n
            traffic[bench][1] += n
            detail[k[:80]] = {"bench_name": bench, "dispatches": n, "fetched_bytes": round(fetched), "written_bytes": round(written)}
    head = a.head or subprocess.run(["git", "-C", str(ROOT), "rev-parse", "--short", "HEAD"], stdout=subprocess.PIPE, stderr=subprocess.DEVNULL, text=True).stdout.strip() or "unknown"
    doc = {"taken_at_commit": head,
           "how": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE per dispatch (a pass each) over the harness commands of bench.py, scaled by the same "
                  "counters over a 256 MiB device copy; a bench name that covers several kernels averages them by launch count",
           "bytes_per_count": {c: round(scale[c], 2) for c in scale},
           "bytes_per_launch": {b: round(s / n) for b, (s, n) in traffic.items()},
           "kernels": detail}
    (out / "traffic.json").write_text(json.dumps(doc, indent=1) + "\n")

    # ---- SQ counters of the encoder's kernels (three passes of at most eight counters)
    sq: dict = collections.defaultdict(dict)
    if not a.skip_sq:
        for i, ctrs in enumerate(SQ_PASSES):
            d = out / f"sq_{i}"
            run(["rocprofv3", "--pmc", *ctrs.split(), "--output-format", "csv", "-d", str(d), "--", *ENC_CMD, "--reps", "1", "--warmup", "0"], out / f"sq_{i}.log", 120)
            for k, v in per_kernel(d).items():
                if k.startswith(("k_fattn", "void k_gemm_f16", "void k_norm<5, 1", "_Z6k_normILi5ELi1E")):
                    for c, (n, s) in v.items():
                        sq[k[:80]][c] = round(s / n)
            shutil.rmtree(d, ignore_errors=True)
    (out / "counters.json").write_text(json.dumps({"taken_at_commit": head, "traffic_counters": counters, "sq_per_dispatch": sq}, indent=1) + "\n")
    print(json.dumps(doc["bytes_per_launch"], indent=1))
    return 0


if __name__ == "__main__":
    sys.exit(main())
