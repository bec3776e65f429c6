#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload doc32k]

A step is one forward + backward pass of document-mask attention over one batch of seeded
synthetic tensors that already live in HBM, through the C ABI (one kvax_fa_fwd and one kvax_fa_bwd
call, as a training step issues them).  The per-kernel times come from a second, untimed pass that
runs the backward's two kernels in separate calls with HIP events around each.  The
block masks are built once before the loop, as a training step would build them once per batch
and reuse them across layers; their build time is reported separately (``mask_build_ms``).
After the headline workload (doc32k) the other configurations of the baseline - dense causal forward,
the context-parallel shard, the block-skipping case at mask blocks 128 and 64, and a decoding step -
are timed for a few steps each and reported under ``other_workloads`` of the same line.
A library bf16 GEMM is timed in the same run (``mfma_reference``): what this machine's matrix
pipeline sustains for plain GEMMs, with the shader clock read while it runs.
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
    "dense64k": "dense64k: B1 S65536 Hq4/Hkv1 D128 bf16, one causal document, block 128, forward only",
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
    ap.add_argument("--no-clock-sample", action="store_true",
                    help="skip the extra steps enqueued after the timed region to read the shader clock under "
                         "load (keeps the launch counts of a profiler run at warmup + steps)")
    ap.add_argument("--block", type=int, default=128)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-secondary", action="store_true",
                    help="skip the brief timing of the other configurations (other_workloads)")
    ap.add_argument("--secondary-steps", type=int, default=10)
    ap.add_argument("--pmc-calibration", action="store_true",
                    help="also run a plain streaming kernel of known size (reads and writes "
                         f"{CALIBRATION_BYTES >> 20} MiB) so that a rocprofv3 --pmc run of this command "
                         "shows what FETCH_SIZE / WRITE_SIZE read for a known amount of HBM traffic")
    ap.add_argument("--fwd-wide", action="store_true",
                    help="run the forward with KVAX_FA_FWD_WIDE (64 query rows per wavefront, one wavefront "
                         "per SIMD): a variant kept to measure what halving the LDS traffic buys")
    ap.add_argument("--no-mfma-reference", action="store_true",
                    help="skip the library GEMM timed for the mfma_reference object")
    ap.add_argument("--global-positions", action="store_true",
                    help="positions = token index instead of restarting per document")
    return ap.parse_args()


def read_sclk_mhz():
    """Current shader clock in MHz as the amdgpu driver reports it for the first card
    (the starred line of pp_dpm_sclk), or None where the file is not there."""
    import glob
    import re
    for path in sorted(glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk")):
        try:
            for line in open(path):
                if line.rstrip().endswith("*"):
                    m = re.search(r"(\d+)\s*[Mm][Hh]z", line)
                    if m:
                        return float(m.group(1))
        except OSError:
            pass
    return None


def sample_sclk(step, ms_per_step, seconds=0.4, samples=8):
    """Shader clock while the timed work runs: enqueues about `seconds` of steps without waiting and
    reads the driver's clock from the host in the meantime.  Returns (mean MHz, samples) or None."""
    if read_sclk_mhz() is None:
        return None
    n = max(8, int(seconds * 1e3 / max(ms_per_step, 1e-3)))
    n = min(n, 2000)
    # enqueueing is much faster than the kernels run: the queue holds the work while the host samples
    for _ in range(n):
        step()
    got = []
    for i in range(samples):
        time.sleep(seconds * 0.8 / samples)
        v = read_sclk_mhz()
        if v is not None and i >= 1:  # the first interval lets the clock settle
            got.append(v)
    torch.cuda.synchronize()
    return (float(np.mean(got)), len(got)) if got else None


def mfma_reference(n=8192, iters=20):
    """What the matrix pipeline of this machine sustains for a plain library GEMM: torch.matmul of two
    n x n bf16 matrices (hipBLASLt), `iters` calls timed with HIP events after a warm-up, and the shader
    clock the driver reports while the same GEMMs run again.  The attention kernels cannot be faster
    per MFMA than this: they do their element-wise work on top."""
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(0)
    a = torch.randn((n, n), generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
    b = torch.randn((n, n), generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
    c = torch.empty((n, n), device=dev, dtype=torch.bfloat16)
    for _ in range(5):
        torch.matmul(a, b, out=c)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        torch.matmul(a, b, out=c)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / iters
    tflops = 2.0 * n ** 3 / (ms * 1e-3) / 1e12
    sclk = sample_sclk(lambda: torch.matmul(a, b, out=c), ms)
    return {"what": f"torch.matmul, bf16, {n} x {n} x {n}, {iters} calls", "value": tflops, "unit": "TFLOP/s",
            "ms": ms, "frac_of_datasheet_peak": tflops / MFMA_BF16_DENSE_PEAK_TFLOPS,
            "clock_under_load_mhz": sclk[0] if sclk else None}


def cpu_baseline(w, seed, seconds_hint=20.0):
    """Dense masked attention (forward + backward) on the host cores for TWO query heads (one kv
    head) of the workload, numpy float32, row-blocked, 10-20 s; returns the JSON object.  The oracle is the thing
    timed here and nothing else uses it."""
    from oracle import attention_oracle as ao

    q, k, v, dout = w.draw_tensors(seed, "cpu", with_dout=True)
    b, head, nh = 0, 0, min(2, w.num_heads // w.num_kv_heads)
    kvh = 0
    qs = q[b:b + 1, :, head:head + nh].float().numpy()
    ks = k[b:b + 1, :, kvh:kvh + 1].float().numpy()
    vs = v[b:b + 1, :, kvh:kvh + 1].float().numpy()
    ds = dout[b:b + 1, :, head:head + nh].float().numpy()
    ids = (w.q_pos[b:b + 1], w.q_seg[b:b + 1], w.kv_pos[b:b + 1], w.kv_seg[b:b + 1])
    t0 = time.perf_counter()
    ao.attention_forward(qs, ks, vs, *ids, w.scale, dtype=np.float32, row_block=2048)
    t1 = time.perf_counter()
    if w.backward:
        ao.attention_backward(qs, ks, vs, *ids, w.scale, ds, dtype=np.float32, row_block=2048)
    t2 = time.perf_counter()
    from kvax_amd.utils.benchmarking import count_unmasked_pairs
    pairs = count_unmasked_pairs(*ids)
    flops = 4.0 * w.head_dim * pairs * nh * (3.5 if w.backward else 1.0)
    threads = int(os.environ.get("OMP_NUM_THREADS", 0)) or len(os.sched_getaffinity(0))
    return {
        "value": flops / (t2 - t0) / 1e12,
        "unit": "TFLOP/s",
        "cores": min(threads, len(os.sched_getaffinity(0))),
        "kind": "port",
        "sample": f"{nh} of {w.num_heads} query heads of batch row 0 (all {w.q_len} queries x {w.kv_len} "
                  f"keys, dense row-blocked numpy float32 softmax(mask(QK^T))V and its VJP; "
                  f"jax is not installed so the dense math runs in numpy); "
                  f"fwd {t1 - t0:.2f} s, bwd {t2 - t1:.2f} s; unmasked FLOPs of these heads / time",
    }


def measure(args, name, block, steps, warmup, device_tensors=False):
    """Times `steps` forward(+backward) passes of one workload; returns (workload, dict of figures).
    device_tensors: draw Q/K/V/dO on the GPU (seeded) instead of on the host - same distribution,
    much faster for the large secondary workloads, whose values do not matter for timing."""
    from kvax_amd import FlashAttentionParamsConfig, _native, attention_specs, create_attention_mask
    from kvax_amd.ops.flash_attention import (backward_workspace_bytes, flash_attention_backward,
                                              flash_attention_forward)
    from kvax_amd.utils.benchmarking import workload

    dev = torch.device("cuda:0")
    w = workload(name, seed=args.seed, restart_positions=not args.global_positions, block=block)
    if device_tensors:
        g = torch.Generator(device=dev).manual_seed(args.seed)
        shape_q = (w.batch, w.q_len, w.num_heads, w.head_dim)
        shape_k = (w.batch, w.kv_len, w.num_kv_heads, w.head_dim)
        q, k, v, dout = (torch.randn(sh, generator=g, device=dev, dtype=torch.float32).to(w.dtype)
                         for sh in (shape_q, shape_k, shape_k, shape_q))
    else:
        q, k, v, dout = w.draw_tensors(args.seed, dev, with_dout=True)
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
        # the same calls without the host in the way: `reps` of them captured in one HIP graph (kernels
        # only, no memset nodes) and replayed, which leaves the device time of a call's two kernels
        mask_gpu_ms = None
        try:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                for _ in range(reps):
                    create_attention_mask(*ids, fwd_params=fp, bwd_params=bp, calc_bwd_mask=True)
            graph.replay()
            torch.cuda.synchronize()
            m0.record()
            graph.replay()
            m1.record()
            torch.cuda.synchronize()
            mask_gpu_ms = m0.elapsed_time(m1) / reps
            del graph
        except RuntimeError:
            mask_gpu_ms = None

    # ---- reusable outputs / workspace ----------------------------------------------------------
    out = torch.empty_like(q)
    lse = torch.empty((w.batch, w.num_heads, w.q_len), dtype=torch.float32, device=dev)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    ws = torch.empty(backward_workspace_bytes(q, k) + 16, dtype=torch.uint8, device=dev)
    SQ, SK = _native.KVAX_FA_SKIP_DQ, _native.KVAX_FA_SKIP_DKDV

    fwd_flags = _native.KVAX_FA_FWD_WIDE if args.fwd_wide else 0

    def fwd():
        flash_attention_forward(q, k, v, *ids, masks[0], w.scale, fp, bp, buffers=(out, lse), flags=fwd_flags)

    def bwd(flags):
        flash_attention_backward(q, k, v, *ids, masks[1], masks[2], out, lse, dout, w.scale, fp, bp,
                                 flags=flags, buffers=(dq, dk, dv, ws))

    # the timed step: one forward call and one backward call
    def step():
        fwd()
        if backward:
            bwd(0)

    # per-kernel pass (untimed for `value`): the backward's kernels in separate calls
    phases = [("fa_fwd_kernel", fwd)]
    if backward:
        # the dQ kernel also produces delta = rowsum(O * dO), which the dK/dV kernel reads
        phases += [("fa_bwd_dq_kernel", lambda: bwd(SK)),
                   ("fa_bwd_dkdv_kernel", lambda: bwd(SQ))]

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for s_ in range(steps):
        step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / steps

    all_events = [[(ev(), ev()) for _ in phases] for _ in range(steps)]
    for s_ in range(steps):
        for i, (_, fn) in enumerate(phases):
            all_events[s_][i][0].record()
            fn()
            all_events[s_][i][1].record()
    torch.cuda.synchronize()
    kernel_ms = {name_: float(np.mean([all_events[s_][i][0].elapsed_time(all_events[s_][i][1])
                                       for s_ in range(steps)]))
                 for i, (name_, _) in enumerate(phases)}

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
                    "traffic": recorded_traffic("fa_fwd_kernel", name),
                    "algorithmic_bytes": alg_bytes}
    else:
        roofline = {"bound": "mfma", "kernel": dominant, "achieved": achieved,
                    "peak": MFMA_BF16_DENSE_PEAK_TFLOPS, "unit": "TFLOP/s",
                    "frac": achieved / MFMA_BF16_DENSE_PEAK_TFLOPS,
                    "traffic": recorded_traffic(dominant, name)}
    sclk = sample_sclk(step, ms_per_step) if args.workload == name and not args.no_clock_sample else None
    figures = {
        "sclk": sclk,
        "value": value, "ms_per_step": ms_per_step, "pairs": pairs, "f_step": f_step, "f_fwd": f_fwd,
        "roofline": roofline, "mask_build_ms": mask_ms, "mask_build_gpu_ms": mask_gpu_ms, "kernel_ms": kernel_ms,
        "kernel_tflops": {n: (kernel_flops[n] / (ms * 1e-3) / 1e12 if ms > 0 else 0.0)
                          for n, ms in kernel_ms.items()},
    }
    return w, figures


# The other configurations of the baseline, timed briefly after the headline one so that every
# configuration has a figure in the same JSON line: (workload, mask block size)
SECONDARY = [("dense_causal", 128), ("cp_shard", 128), ("block_skip", 128), ("block_skip", 64),
             ("decode32k", 128)]


def main():
    args = parse()
    if args.gpus != 1:
        print(f"bench.py: this build runs on one GPU only (got --gpus {args.gpus}); the path has no "
              "collectives.  Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")

    if args.pmc_calibration:
        src = torch.ones(CALIBRATION_BYTES // 4, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(2):
            torch.mul(src, 1.0, out=dst)  # elementwise kernel: reads and writes CALIBRATION_BYTES
        torch.cuda.synchronize()
        del src, dst

    w, m = measure(args, args.workload, args.block, args.steps, args.warmup)
    backward = w.backward
    result = {
        # the headline metric's own wording for the configuration it is quoted on; `value` is its
        # forward+backward figure, the forward one and the mask build time follow as fwd_tflops and
        # mask_build_ms
        "metric": "doc-mask attn TFLOP/s fwd & fwd+bwd @32k bf16 (unmasked FLOPs); mask build ms"
                  if args.workload == "doc32k" else
                  ("doc-mask attention TFLOP/s, forward+backward, bf16, unmasked FLOPs" if backward
                   else "doc-mask attention TFLOP/s, forward, bf16, unmasked FLOPs"),
        "value_is": "forward+backward TFLOP/s" if backward else "forward TFLOP/s",
        "value": m["value"],
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": m["ms_per_step"],
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
            "unmasked_pairs": m["pairs"],
            "flops_per_step": m["f_step"],
            "num_documents": len(w.meta.get("doc_lengths", [])) or None,
            "padding_tokens": w.meta.get("pad"),
            "forward_kernel": "wide (KVAX_FA_FWD_WIDE)" if args.fwd_wide else "default",
        },
        "roofline": m["roofline"],
        "step_frac_of_mfma_peak": m["value"] / MFMA_BF16_DENSE_PEAK_TFLOPS,
        "fwd_tflops": m["f_fwd"] / (m["kernel_ms"]["fa_fwd_kernel"] * 1e-3) / 1e12,
        # create_attention_mask(calc_bwd_mask=True): per call as the host sees it (20 calls back to
        # back), and the device time per call (the 20 calls replayed from one HIP graph)
        "mask_build_ms": m["mask_build_ms"],
        "mask_build_gpu_ms": m["mask_build_gpu_ms"],
        # per-kernel times: a separate pass with the backward's two kernels in separate calls
        "kernel_ms": m["kernel_ms"],
        "kernel_tflops": m["kernel_tflops"],
        # the peak above assumes the datasheet's 2.4 GHz; this is the shader clock the driver reported
        # (pp_dpm_sclk) while the same steps ran again after the timed region
        "clock": {"assumed_by_peak_mhz": 2400.0,
                  "under_load_mhz": m["sclk"][0] if m["sclk"] else None,
                  "samples": m["sclk"][1] if m["sclk"] else 0},
    }
    if not args.no_secondary and args.workload == "doc32k":
        others = {}
        for name, block in SECONDARY:
            torch.cuda.empty_cache()
            w2, m2 = measure(args, name, block, args.secondary_steps, 3, device_tensors=True)
            others[f"{name}@block{block}"] = {
                "workload": WORKLOAD_TEXT[name], "mask_block": block, "steps": args.secondary_steps,
                "value": m2["value"], "unit": "TFLOP/s",
                "value_is": "forward+backward TFLOP/s" if w2.backward else "forward TFLOP/s",
                "ms_per_step": m2["ms_per_step"], "unmasked_pairs": m2["pairs"],
                "roofline": m2["roofline"], "mask_build_ms": m2["mask_build_ms"],
                "mask_build_gpu_ms": m2["mask_build_gpu_ms"],
                "kernel_ms": m2["kernel_ms"], "kernel_tflops": m2["kernel_tflops"],
            }
            del w2, m2
        result["other_workloads"] = others
    if not args.no_mfma_reference:
        torch.cuda.empty_cache()
        ref = mfma_reference()
        result["mfma_reference"] = ref
        if result["roofline"]["bound"] == "mfma":
            result["roofline"]["frac_of_reference"] = result["roofline"]["achieved"] / ref["value"]
            result["step_frac_of_mfma_reference"] = result["value"] / ref["value"]
    if not args.no_cpu_baseline:
        from kvax_amd.utils.benchmarking import workload
        result["cpu_baseline"] = cpu_baseline(workload(args.workload, seed=args.seed,
                                                       restart_positions=not args.global_positions,
                                                       block=args.block), args.seed)
    print(json.dumps(result))


if __name__ == "__main__":
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    main()
