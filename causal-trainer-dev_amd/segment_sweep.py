"""Times the attention kernels against segment length and fits ``time = fixed + slope * pairs``.

The benchmark shape (batch, sequence, heads of ``--shape``) is packed with segments of one fixed
length per run (64 ... the whole row), so the number of allowed (query, key) pairs changes while
the number of query tiles, key tiles and launches stays the same. Every kernel's time is then
close to a straight line in the pairs: the slope is its steady-state rate, the intercept what a
launch costs before any pair is worked: the prologue and epilogue of every query / key tile and
the one masked (diagonal) key tile that every row block has at any segment length. The last
lines apply the fit to the shape's own packing.

Usage::

    python -m causal_trainer_dev_amd.segment_sweep [--shape llama3_8b] [--steps 10] [--out FILE]
"""

from __future__ import annotations

import argparse
import dataclasses

import numpy as np
import torch

KERNELS = ("attn_fwd_kernel", "attn_dq_kernel", "attn_dkv_kernel", "attn_dkv_reduce_kernel")


def kernel_times(ct, config, steps):
    from . import profiling

    W = ct.workloads
    inputs = W.make_attention_inputs(config, "cuda")
    pairs = W.count_allowed_pairs(inputs["segment_ids"], inputs["attention_end"])
    profile = ct.resolve_attention_profile(inputs["q"].shape, inputs["k"].shape, None,
                                           has_attention_end=inputs["attention_end"] is not None)
    metadata = ct.prepare_attention_metadata(inputs["segment_ids"], mesh=None, profile=profile,
                                             attention_end=inputs["attention_end"])
    q, k, v, dout = inputs["q"], inputs["k"], inputs["v"], inputs["dout"]
    workspace = ct.BackwardWorkspace()

    def step():
        out, lse = ct.attention_forward_with_lse(q, k, v, metadata, scale=config.scale)
        ct.attention_backward(q, k, v, metadata, out, lse, dout, scale=config.scale, workspace=workspace,
                              dkv_kernel="narrow", dq_form="recompute")

    for _ in range(max(3, steps // 2)):
        step()
    with profiling.KernelTimer() as timer:
        for _ in range(steps):
            step()
    durations = timer.durations_ms()
    return pairs, {name: float(np.mean(durations[name])) for name in KERNELS if name in durations}


def main() -> None:
    import causal_trainer_dev_amd as ct

    parser = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    parser.add_argument("--shape", default="llama3_8b")
    parser.add_argument("--steps", type=int, default=10)
    parser.add_argument("--out", default=None)
    args = parser.parse_args()
    base = ct.workloads.ATTENTION_CONFIGS[args.shape]
    lengths = [n for n in (64, 128, 256, 512, 1024, 2048, 4096, 8192, 16384, 32768) if n <= base.seq]
    # warm the clocks on the shape's own packing first
    own_pairs, own = kernel_times(ct, base, max(args.steps, 50))
    rows = []
    for length in lengths:
        config = dataclasses.replace(base, layout="uniform", min_len=length, max_len=length)
        pairs, times = kernel_times(ct, config, args.steps)
        rows.append((length, pairs, times))
    lines = ["Attention kernel time against segment length: %s shape (B=%d, S=%d, %d/%d heads, D=%d), segments of one"
             % (base.name, base.batch, base.seq, base.q_heads, base.kv_heads, base.head_dim),
             "fixed length per run; narrow dK/dV kernel, recompute form; mean over %d steps; ms" % args.steps,
             "command: python -m causal_trainer_dev_amd.segment_sweep --shape %s --steps %d" % (args.shape, args.steps),
             "",
             "%8s %14s " % ("length", "pairs") + " ".join("%12s" % name.replace("attn_", "").replace("_kernel", "")
                                                         for name in KERNELS)]
    for length, pairs, times in rows:
        lines.append("%8d %14d " % (length, pairs) + " ".join("%12.4f" % times.get(name, float("nan")) for name in KERNELS))
    lines += ["", "least-squares fit time = fixed + slope * pairs over the runs above, and what it says about the shape's",
              "own packing (%d pairs): measured time, fixed share, the rate the slope corresponds to" % own_pairs]
    unit = base.head_dim * base.q_heads
    executed = {"attn_fwd_kernel": 4, "attn_dq_kernel": 6, "attn_dkv_kernel": 8}
    for name in KERNELS[:3]:
        x = np.array([pairs for _, pairs, _ in rows], dtype=np.float64)
        y = np.array([times[name] for _, _, times in rows], dtype=np.float64)
        slope, fixed = np.polyfit(x, y, 1)
        worst = float(np.max(np.abs(fixed + slope * x - y) / y))
        rate = executed[name] * unit / (slope * 1e-3) / 1e12
        lines.append("%-18s fixed %.4f ms  slope %.4f ms per 1e9 pairs (%.0f TFLOP/s executed, %d D per pair)  worst "
                     "residual %.1f %%  |  own packing: %.4f ms, fixed share %.0f %%"
                     % (name, fixed, slope * 1e9, rate, executed[name], 100 * worst, own[name], 100 * fixed / own[name]))
    text = "\n".join(lines) + "\n"
    if args.out:
        with open(args.out, "w") as handle:
            handle.write(text)
    print(text, end="")


if __name__ == "__main__":
    main()
