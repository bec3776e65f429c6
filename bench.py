#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload doc32k]

A step is one forward + backward pass of document-mask attention over one batch of seeded
synthetic tensors that already live in HBM, through the C ABI (kvax_fa_fwd, kvax_fa_bwd).  The
block masks are built once before the loop, as a training step would build them once per batch
and reuse them across layers; their build time is reported separately (``mask_build_ms``).
Prints ONE JSON line.  ``value`` counts only unmasked FLOPs: 4*D per attendable (q, kv) pair
and query head in the forward, 2.5x that in the backward.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np
import torch

MFMA_BF16_DENSE_PEAK_TFLOPS = 2516.6  # MI355X datasheet: 256 CU x 2.4 GHz x 4096 FLOP/clk/CU
HBM_PEAK_GBPS = 8000.0                # MI355X datasheet: HBM3E
CALIBRATION_BYTES = 1 << 30            # bytes read (and bytes written) by the --pmc-calibration kernel
ROOT = os.path.dirname(os.path.abspath(__file__))


def recorded_traffic(kernel: str, workload_name: str):
    """HBM bytes per launch of `kernel`, as measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE and
    written down in profiles/<kernel>_<workload>_pmc.md (line ``traffic_bytes_per_launch: N``).
    Hardware counters cannot be read from inside this process; None when no such record exists."""
    path = os.path.join(ROOT, "profiles", f"{kernel}_{workload_name}_pmc.md")
    try:
        with open(path) as f:
            for line in f:
                if line.startswith("traffic_bytes_per_launch:"):
                    return float(line.split(":", 1)[1])
    except OSError:
        pass
    return None

WORKLOAD_TEXT = {
    "dense_causal": "dense_causal: B1 S8192 Hq32/Hkv8 D128 bf16, one causal document, block 128, forward only",
    "doc32k": "doc32k: B1 S32768 Hq32/Hkv8 D128 bf16, causal document mask, lognormal document "
              "lengths (median 2048, sigma 1, clip [128,16384]), ~5% trailing padding, positions "
              "restart per document, dO~N(0,1), block 128, forward+backward",
    "cp_shard": "cp_shard: Sq16384 (chunks r,15-r of 16, r=3) x Sk131072, Hq32/Hkv8 D128 bf16, causal "
                "document mask (lognormal median 4096), forward+backward, one CP=8 shard",
    "block_skip": "block_skip: B4 S16384 Hq64/Hkv8 D128 bf16, bidirectional document mask, exponential "
                  "document lengths (mean 512, min 32), 20-30% padding per row, forward+backward",
    "decode32k": "decode32k: B8, one query per row against a 32768-slot key cache filled to 16384..32764 "
                 "keys (the rest padding), Hq32/Hkv8 D128 bf16, forward only (split mode)",
}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="doc32k", choices=sorted(WORKLOAD_TEXT))
    ap.add_argument("--block", type=int, default=128)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--pmc-calibration", action="store_true",
                    help="also run a plain streaming kernel of known size (reads and writes "
                         f"{CALIBRATION_BYTES >> 20} MiB) so that a rocprofv3 --pmc run of this command "
                         "shows what FETCH_SIZE / WRITE_SIZE read for a known amount of HBM traffic")
    ap.add_argument("--global-positions", action="store_true",
                    help="positions = token index instead of restarting per document")
    return ap.parse_args()


def cpu_baseline(w, seed, seconds_hint=20.0):
    """Dense masked attention (forward + backward) on the host cores for ONE query head of the
    workload, numpy float32, row-blocked; returns the JSON object.  The oracle is the thing
    timed here and nothing else uses it."""
    from oracle import attention_oracle as ao

    q, k, v, dout = w.draw_tensors(seed, "cpu", with_dout=True)
    b, head = 0, 0
    kvh = 0
    qs = q[b:b + 1, :, head:head + 1].float().numpy()
    ks = k[b:b + 1, :, kvh:kvh + 1].float().numpy()
    vs = v[b:b + 1, :, kvh:kvh + 1].float().numpy()
    ds = dout[b:b + 1, :, head:head + 1].float().numpy()
    ids = (w.q_pos[b:b + 1], w.q_seg[b:b + 1], w.kv_pos[b:b + 1], w.kv_seg[b:b + 1])
    t0 = time.perf_counter()
    ao.attention_forward(qs, ks, vs, *ids, w.scale, dtype=np.float32, row_block=2048)
    t1 = time.perf_counter()
    if w.backward:
        ao.attention_backward(qs, ks, vs, *ids, w.scale, ds, dtype=np.float32, row_block=2048)
    t2 = time.perf_counter()
    from kvax_amd.utils.benchmarking import count_unmasked_pairs
    pairs = count_unmasked_pairs(*ids)
    flops = 4.0 * w.head_dim * pairs * (3.5 if w.backward else 1.0)
    threads = int(os.environ.get("OMP_NUM_THREADS", 0)) or len(os.sched_getaffinity(0))
    return {
        "value": flops / (t2 - t0) / 1e12,
        "unit": "TFLOP/s",
        "cores": min(threads, len(os.sched_getaffinity(0))),
        "kind": "port",
        "sample": f"1 of {w.num_heads} query heads of batch row 0 (all {w.q_len} queries x {w.kv_len} "
                  f"keys, dense row-blocked numpy float32 softmax(mask(QK^T))V and its VJP; "
                  f"jax is not installed so the dense math runs in numpy); "
                  f"fwd {t1 - t0:.2f} s, bwd {t2 - t1:.2f} s; unmasked FLOPs of that head / time",
    }


def main():
    args = parse()
    if args.gpus != 1:
        print(f"bench.py: this build runs on one GPU only (got --gpus {args.gpus}); the path has no "
              "collectives.  Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    from kvax_amd import FlashAttentionParamsConfig, _native, attention_specs, create_attention_mask
    from kvax_amd.ops.flash_attention import (backward_workspace_bytes, flash_attention_backward,
                                              flash_attention_forward)
    from kvax_amd.utils.benchmarking import workload

    dev = torch.device("cuda:0")
    w = workload(args.workload, seed=args.seed, restart_positions=not args.global_positions,
                 block=args.block)
    tensors = w.draw_tensors(args.seed, dev, with_dout=True)
    q, k, v, dout = tensors
    decode = w.q_len == 1
    ids = w.ids(dev)
    fp, bp = FlashAttentionParamsConfig(*w.fwd_blocks), FlashAttentionParamsConfig(*w.bwd_blocks)
    specs = (("data", None, "model", None), ("data", None, "model", None))
    pairs = w.unmasked_pairs()
    f_fwd = 4.0 * w.head_dim * pairs * w.num_heads
    backward = w.backward

    def ev():
        return torch.cuda.Event(enable_timing=True)

    # ---- masks: built once, timed on their own -------------------------------------------------
    with attention_specs(*specs):
        for _ in range(3):
            masks = create_attention_mask(*ids, fwd_params=fp, bwd_params=bp, calc_bwd_mask=True)
        torch.cuda.synchronize()
        m0, m1 = ev(), ev()
        reps = 20
        m0.record()
        for _ in range(reps):
            masks = create_attention_mask(*ids, fwd_params=fp, bwd_params=bp, calc_bwd_mask=True)
        m1.record()
        torch.cuda.synchronize()
        mask_ms = m0.elapsed_time(m1) / reps

    # ---- reusable outputs / workspace ----------------------------------------------------------
    out = torch.empty_like(q)
    lse = torch.empty((w.batch, w.num_heads, w.q_len), dtype=torch.float32, device=dev)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    ws = torch.empty(backward_workspace_bytes(q, k) + 16, dtype=torch.uint8, device=dev)
    SD, SQ, SK = _native.KVAX_FA_SKIP_DELTA, _native.KVAX_FA_SKIP_DQ, _native.KVAX_FA_SKIP_DKDV

    def fwd():
        flash_attention_forward(q, k, v, *ids, masks[0], w.scale, fp, bp, buffers=(out, lse))

    def bwd(flags):
        flash_attention_backward(q, k, v, *ids, masks[1], masks[2], out, lse, dout, w.scale, fp, bp,
                                 flags=flags, buffers=(dq, dk, dv, ws))

    phases = [("fa_fwd_kernel", fwd)]
    if backward:
        # the dQ kernel also produces delta = rowsum(O * dO), which the dK/dV kernel reads
        phases += [("fa_bwd_dq_kernel", lambda: bwd(SK)),
                   ("fa_bwd_dkdv_kernel", lambda: bwd(SQ))]

    def step(events=None):
        for i, (_, fn) in enumerate(phases):
            if events is not None:
                events[i][0].record()
            fn()
            if events is not None:
                events[i][1].record()

    if args.pmc_calibration:
        src = torch.ones(CALIBRATION_BYTES // 4, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(2):
            torch.mul(src, 1.0, out=dst)  # elementwise kernel: reads and writes CALIBRATION_BYTES
        torch.cuda.synchronize()
        del src, dst

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    all_events = [[(ev(), ev()) for _ in phases] for _ in range(args.steps)]
    t0 = time.perf_counter()
    for s in range(args.steps):
        step(all_events[s])
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    kernel_ms = {name: float(np.mean([all_events[s][i][0].elapsed_time(all_events[s][i][1])
                                      for s in range(args.steps)]))
                 for i, (name, _) in enumerate(phases)}

    f_step = f_fwd * (3.5 if backward else 1.0)
    value = f_step / (ms_per_step * 1e-3) / 1e12
    # algorithmic FLOPs per launch of each kernel: 2*D per pair and head for every contraction the
    # kernel exists to produce or must recompute (forward: QK^T, PV; dQ: QK^T, dO V^T, dS K;
    # dK/dV: QK^T, dO V^T, P^T dO, dS^T Q)
    kernel_flops = {"fa_fwd_kernel": f_fwd, "fa_bwd_dq_kernel": 1.5 * f_fwd, "fa_bwd_dkdv_kernel": 2.0 * f_fwd}
    dominant = max(kernel_ms, key=kernel_ms.get)
    achieved = kernel_flops[dominant] / (kernel_ms[dominant] * 1e-3) / 1e12
    if decode:
        # one query per row: the kernel has to read every attendable key and value once (all query
        # heads of a group share them) plus Q, and write O and lse; HBM is the roof
        alg_bytes = (2 * pairs * w.num_kv_heads * w.head_dim * 2
                     + 2 * w.batch * w.num_heads * w.head_dim * 2 + w.batch * w.num_heads * 4)
        gbps = alg_bytes / (kernel_ms["fa_fwd_kernel"] * 1e-3) / 1e9
        roofline = {"bound": "hbm", "kernel": "fa_fwd_kernel (split mode) + fa_fwd_combine_kernel",
                    "achieved": gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": gbps / HBM_PEAK_GBPS,
                    "traffic": recorded_traffic("fa_fwd_kernel", args.workload),
                    "algorithmic_bytes": alg_bytes}
    else:
        roofline = {"bound": "mfma", "kernel": dominant, "achieved": achieved,
                    "peak": MFMA_BF16_DENSE_PEAK_TFLOPS, "unit": "TFLOP/s",
                    "frac": achieved / MFMA_BF16_DENSE_PEAK_TFLOPS,
                    "traffic": recorded_traffic(dominant, args.workload)}
    result = {
        # the headline metric's own wording for the configuration it is quoted on; `value` is its
        # forward+backward figure, the forward one and the mask build time follow as fwd_tflops and
        # mask_build_ms
        "metric": "doc-mask attn TFLOP/s fwd & fwd+bwd @32k bf16 (unmasked FLOPs); mask build ms"
                  if args.workload == "doc32k" else
                  ("doc-mask attention TFLOP/s, forward+backward, bf16, unmasked FLOPs" if backward
                   else "doc-mask attention TFLOP/s, forward, bf16, unmasked FLOPs"),
        "value_is": "forward+backward TFLOP/s" if backward else "forward TFLOP/s",
        "value": value,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": WORKLOAD_TEXT[args.workload],
            "seed": args.seed,
            "mask_block": args.block,
            "positions": "global" if args.global_positions else "restart per document",
            "unmasked_pairs": pairs,
            "flops_per_step": f_step,
            "num_documents": len(w.meta.get("doc_lengths", [])) or None,
            "padding_tokens": w.meta.get("pad"),
        },
        "roofline": roofline,
        "step_frac_of_mfma_peak": value / MFMA_BF16_DENSE_PEAK_TFLOPS,
        "fwd_tflops": f_fwd / (kernel_ms["fa_fwd_kernel"] * 1e-3) / 1e12,
        "mask_build_ms": mask_ms,
        "kernel_ms": kernel_ms,
        "kernel_tflops": {n: (kernel_flops[n] / (ms * 1e-3) / 1e12 if ms > 0 else 0.0)
                          for n, ms in kernel_ms.items()},
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(w, args.seed)
    print(json.dumps(result))


if __name__ == "__main__":
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    main()
