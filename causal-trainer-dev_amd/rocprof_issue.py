"""Turns ``rocprofv3 --pmc`` runs of bench.py with SQ counters into issue-slot shares per kernel.

Usage (each counter pass is a run of its own; at most 8 SQ counters fit one pass)::

    rocprofv3 --pmc SQ_WAVE_CYCLES SQ_BUSY_CYCLES SQ_VALU_MFMA_BUSY_CYCLES SQ_ACTIVE_INST_VALU \\
        SQ_ACTIVE_INST_LDS SQ_WAIT_INST_ANY SQ_WAIT_INST_LDS SQ_ACTIVE_INST_ANY \\
        --output-format csv -d DIR_A -o p -- python3 bench.py --steps 3 --warmup 1 --no-cutce \\
        --no-layer-ops --no-cpu-baseline
    rocprofv3 --pmc SQ_INSTS_VALU SQ_INSTS_MFMA SQ_INSTS_LDS SQ_INSTS_SALU SQ_WAVES \\
        SQ_LDS_BANK_CONFLICT SQ_LDS_IDX_ACTIVE SQ_INSTS_SMEM --output-format csv -d DIR_B -o p -- (same)
    python -m causal_trainer_dev_amd.rocprof_issue DIR_A DIR_B [--out FILE] [--command TEXT]

SQ_WAVE_CYCLES and the SQ_ACTIVE_INST_* / SQ_WAIT_* counters count in units of 4 cycles summed over
wavefronts; SQ_VALU_MFMA_BUSY_CYCLES counts cycles of the matrix pipe summed over SIMDs (32 per
v_mfma_f32_32x32x16_bf16). With W wavefronts resident per SIMD, SIMD time = 4 * SQ_WAVE_CYCLES / W;
the shares below are fractions of that time.
"""

from __future__ import annotations

import argparse
import collections
import csv
import glob
import os

from .rocprof_traffic import _short

# resident wavefronts per SIMD of the kernels reported (launch bounds and register use fix them)
WAVES_PER_SIMD = {"attn_fwd_kernel": 2, "attn_dq_kernel": 2, "attn_dkv_kernel": 2, "attn_dkv_wide_kernel": 1,
                  "attn_dq_blocks_kernel": 4, "cutce_stats_kernel": 1, "cutce_dlogits_kernel": 1,
                  "cutce_grads_kernel": 1, "cutce_dhidden_kernel": 1, "cutce_dhead_kernel": 1}


def read_counters(folders) -> dict[str, dict[str, float]]:
    """kernel -> counter -> mean value per dispatch (summed over the counter's instances)."""

    sums = collections.defaultdict(lambda: collections.defaultdict(float))
    dispatches = collections.defaultdict(lambda: collections.defaultdict(set))
    for folder in folders:
        for path in sorted(glob.glob(os.path.join(folder, "**", "*counter_collection.csv"), recursive=True)):
            with open(path, newline="") as handle:
                for row in csv.DictReader(handle):
                    kernel = _short(row["Kernel_Name"])
                    sums[kernel][row["Counter_Name"]] += float(row["Counter_Value"])
                    dispatches[kernel][row["Counter_Name"]].add(row.get("Dispatch_Id", ""))
    return {kernel: {name: value / max(len(dispatches[kernel][name]), 1) for name, value in counters.items()}
            for kernel, counters in sums.items()}


XCDS = 8  # GRBM_GUI_ACTIVE is reported as the sum over the accelerator dies


def shader_clocks(folders) -> dict[str, tuple[float, float, float, int]]:
    """kernel -> (mean, lowest, highest shader clock in GHz, dispatches) from a pass that collected
    GRBM_GUI_ACTIVE (busy cycles of the graphics engine, summed over the dies) together with each
    dispatch's start / end timestamps (ns). The counter window is wider than the kernel by a fixed
    amount; the smallest value any dispatch of the pass reads (a microsecond-scale kernel) is taken
    as that amount and subtracted, which leaves a few per cent of error on kernels under a millisecond
    and none that matters above."""

    samples = []
    for folder in folders:
        for path in sorted(glob.glob(os.path.join(folder, "**", "*counter_collection.csv"), recursive=True)):
            with open(path, newline="") as handle:
                for row in csv.DictReader(handle):
                    if row["Counter_Name"] != "GRBM_GUI_ACTIVE":
                        continue
                    span = float(row["End_Timestamp"]) - float(row["Start_Timestamp"])
                    if span > 0.0:
                        samples.append((_short(row["Kernel_Name"]), float(row["Counter_Value"]), span))
    if not samples:
        return {}
    window = min(cycles for _, cycles, _ in samples)
    per_kernel = collections.defaultdict(list)
    for kernel, cycles, span in samples:
        per_kernel[kernel].append((cycles - window) / XCDS / span)
    return {kernel: (sum(v) / len(v), min(v), max(v), len(v)) for kernel, v in per_kernel.items()}


def summarize(counters: dict[str, dict[str, float]]) -> list[str]:
    lines = ["%-22s %9s %9s %9s %9s %9s | %s" % ("kernel", "MFMA", "VALU", "LDS", "wait any", "wait LDS",
                                                  "instructions per MFMA: VALU (other than MFMA), LDS, SALU")]
    for kernel, waves in WAVES_PER_SIMD.items():
        c = counters.get(kernel)
        if not c or "SQ_WAVE_CYCLES" not in c:
            continue
        simd_cycles = 4.0 * c["SQ_WAVE_CYCLES"] / waves
        mfma = c.get("SQ_INSTS_MFMA", 0.0)
        valu_time = 4.0 * c.get("SQ_ACTIVE_INST_VALU", 0.0)
        if mfma and c.get("SQ_INSTS_VALU"):
            # the VALU counter includes the MFMA instructions' own issue; report the rest
            valu_time *= (c["SQ_INSTS_VALU"] - mfma) / c["SQ_INSTS_VALU"]
        per = lambda name: (c.get(name, 0.0) - (mfma if name == "SQ_INSTS_VALU" else 0.0)) / mfma if mfma else float("nan")
        lines.append("%-22s %8.1f%% %8.1f%% %8.1f%% %8.1f%% %8.1f%% | %.1f, %.1f, %.1f" % (
            kernel, 100 * c.get("SQ_VALU_MFMA_BUSY_CYCLES", 0.0) / simd_cycles, 100 * valu_time / simd_cycles,
            100 * 4.0 * c.get("SQ_ACTIVE_INST_LDS", 0.0) / simd_cycles,
            100 * 4.0 * c.get("SQ_WAIT_INST_ANY", 0.0) / waves / simd_cycles,
            100 * 4.0 * c.get("SQ_WAIT_INST_LDS", 0.0) / waves / simd_cycles,
            per("SQ_INSTS_VALU"), per("SQ_INSTS_LDS"), per("SQ_INSTS_SALU")))
    return lines


def main() -> None:
    parser = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    parser.add_argument("folders", nargs="+")
    parser.add_argument("--out", default=None)
    parser.add_argument("--command", default="")
    args = parser.parse_args()
    lines = ["Issue-slot shares of the MFMA kernels (fractions of SIMD time; MFMA = matrix pipe busy, VALU = vector",
             "ALU instructions other than MFMA executing, LDS = LDS instructions executing, wait = a wavefront waits",
             "for an instruction to issue; shares of different classes can overlap in time)"]
    if args.command:
        lines.append("command: " + args.command)
    lines.append("")
    lines += summarize(read_counters(args.folders))
    clocks = shader_clocks(args.folders)
    if clocks:
        lines += ["", "shader clock during the kernel (GRBM_GUI_ACTIVE / dies / dispatch duration; the part's peak",
                  "figures are quoted at 2.4 GHz): mean [lowest .. highest] GHz over the dispatches"]
        for kernel in WAVES_PER_SIMD:
            if kernel in clocks:
                mean, low, high, count = clocks[kernel]
                lines.append("%-22s %.2f [%.2f .. %.2f] over %d" % (kernel, mean, low, high, count))
    text = "\n".join(lines) + "\n"
    if args.out:
        with open(args.out, "w") as handle:
            handle.write(text)
    print(text, end="")


if __name__ == "__main__":
    main()
