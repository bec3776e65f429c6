"""Command-line benchmarks of the attention path: ``python -m kvax_amd.benchmarks <command>``.

The four commands and their options carry the names of the reference's benchmark script
(benchmarks.py:34-411): ``mha`` / ``mha_bwd`` time the forward pass / forward+backward of one
device's work and check it against a library attention (there cuDNN, here PyTorch's
``scaled_dot_product_attention``); ``mha_cp`` / ``mha_cp_bwd`` compare a context-parallel run
(query shards, optionally load-balanced by the chunk-pair permutation) with the unsharded one.
This build drives one GPU, so the query shards of a context-parallel run are evaluated one
after another and ``--context-parallel-degree`` stands for the reference's device count.

Throughput is printed twice: on the reference's figure (dense FLOPs x block-mask density,
kvax/utils/benchmarking.py:423-430) and on the FLOPs of the element pairs that are really
attendable.
"""
from __future__ import annotations

import logging

import click
import torch

from kvax_amd.ops.flash_attention import flash_attention
from kvax_amd.ops.mask_creator import calculate_mask_sparsity, create_attention_mask, print_mask
from kvax_amd.utils.benchmarking import (
    check_outputs_bwd,
    check_outputs_fwd,
    count_unmasked_pairs,
    generate_random_segments_lengths,
    make_random_attention_inputs,
)
from kvax_amd.utils.common import PADDING_SEGMENT_ID, get_default_flash_attention_params
from kvax_amd.utils.math import attention_tflops_from_pairs, get_multi_head_attention_tflops
from kvax_amd.utils.permutation import (
    permute_tokens_context_parallelism,
    unpermute_tokens_context_parallelism,
)
from kvax_amd.utils.sharding import Mesh
from kvax_amd.utils.specs import attention_specs

logger = logging.getLogger("kvax_amd.benchmarks")

TP_SPECS = (("data", None, "model", None), ("data", None, "model", None))
CP_SPECS = (("data", "context", None, None), ("data", None, None, None))

# Largest sequence the library comparison materialises a dense boolean mask for.
MAX_DENSE_MASK_LEN = 16384


def format_duration(seconds: float) -> str:
    for unit, factor in (("s", 1.0), ("ms", 1e3), ("us", 1e6)):
        if seconds * factor >= 1.0 or unit == "us":
            return f"{seconds * factor:.3f} {unit}"
    return f"{seconds:.3e} s"


def time_on_device(fn, num_iters: int, device) -> float:
    """Mean seconds per call over ``num_iters`` calls after two untimed ones."""
    for _ in range(2):
        fn()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize(device)
    start.record()
    for _ in range(num_iters):
        fn()
    stop.record()
    torch.cuda.synchronize(device)
    return start.elapsed_time(stop) / 1e3 / num_iters


def report(name: str, seconds: float, tflops_reference_model: float, tflops_unmasked: float) -> None:
    logger.info(
        "%s: %s per iteration; %.1f TFLOP/s on dense FLOPs x block density, "
        "%.1f TFLOP/s on unmasked element pairs",
        name, format_duration(seconds), tflops_reference_model / seconds, tflops_unmasked / seconds,
    )


def make_inputs(batch_size, query_seq_len, kv_seq_len, num_heads, num_kv_heads, qk_head_dim,
                value_head_dim, num_segments, num_pad_tokens, device):
    return make_random_attention_inputs(
        batch_size=batch_size, query_seq_len=query_seq_len, kv_seq_len=kv_seq_len,
        num_query_heads=num_heads, num_kv_heads=num_kv_heads, qk_head_dim=qk_head_dim,
        value_head_dim=value_head_dim, num_pad_tokens=num_pad_tokens,
        list_of_segment_lengths=generate_random_segments_lengths(query_seq_len, num_segments),
        device=device,
    )


def zero_padding_rows(x: torch.Tensor, segment_ids: torch.Tensor) -> torch.Tensor:
    return torch.where((segment_ids == PADDING_SEGMENT_ID)[:, :, None, None], 0, x)


def library_attention(data, scale, dout=None):
    """PyTorch's fused attention on the same inputs (the role cuDNN plays in the reference,
    kvax/utils/benchmarking.py:331-370): output, and with ``dout`` also (dq, dk, dv)."""
    query, key, value, q_pos, q_seg, kv_pos, kv_seg = data
    need_grad = dout is not None
    q, k, v = (t.detach().transpose(1, 2).requires_grad_(need_grad) for t in (query, key, value))
    allowed = (q_seg[:, :, None] == kv_seg[:, None, :]) & (q_pos[:, :, None] >= kv_pos[:, None, :])
    allowed &= (q_seg != PADDING_SEGMENT_ID)[:, :, None]
    # A row with no attendable key would turn into NaN inside softmax; it is zeroed afterwards.
    allowed |= ~allowed.any(dim=-1, keepdim=True)
    out = torch.nn.functional.scaled_dot_product_attention(
        q, k, v, attn_mask=allowed[:, None], scale=scale, enable_gqa=q.shape[1] != k.shape[1])
    out = zero_padding_rows(out.transpose(1, 2), q_seg)
    if not need_grad:
        return out.detach(), None
    out.backward(zero_padding_rows(dout, q_seg))
    return out.detach(), tuple(t.grad.transpose(1, 2) for t in (q, k, v))


def run_kvax(data, scale, specs, mesh, *, backward, assume_sequential_positions, permute,
             show_attention_mask, num_iters, name, dout=None):
    """Build the masks, time ``flash_attention`` (and its backward), return outputs in the
    original token order plus the two TFLOP figures per iteration."""
    query, key, value, q_pos, q_seg, kv_pos, kv_seg = data
    batch, q_len, heads, dim = query.shape
    kv_len, dim_v = key.shape[1], value.shape[3]
    fwd_params = get_default_flash_attention_params(backward=False)
    bwd_params = get_default_flash_attention_params(backward=True)
    device = query.device
    with attention_specs(*specs):
        if permute:
            query, key, value, q_pos, q_seg = permute_tokens_context_parallelism(
                (query, key, value, q_pos, q_seg), mesh=mesh)
            if dout is not None:
                dout = permute_tokens_context_parallelism(dout, mesh=mesh)

        def build():
            return create_attention_mask(q_pos, q_seg, kv_pos, kv_seg, fwd_params=fwd_params,
                                         bwd_params=bwd_params, calc_bwd_mask=backward, mesh=mesh)

        mask = build()
        logger.info("%s: mask build %s", name, format_duration(time_on_device(build, num_iters, device)))
        if show_attention_mask:
            print_mask(mask[0], kv_len // fwd_params.kv_block_size)
            if backward:
                print_mask(mask[1], kv_len // bwd_params.query_block_size)
                print_mask(mask[2], q_len // bwd_params.query_block_size)

        leaves = [t.detach().requires_grad_(backward) for t in (query, key, value)]

        def forward():
            return flash_attention(
                *leaves, q_pos, q_seg, kv_pos, kv_seg, mask, scale=scale, fwd_params=fwd_params,
                bwd_params=bwd_params, assume_sequential_positions=assume_sequential_positions,
                permute_tokens_for_load_balance=permute, mesh=mesh)

        def step():
            out = forward()
            if backward:
                for t in leaves:
                    t.grad = None
                out.backward(dout)
            return out

        seconds = time_on_device(step, num_iters, device)
        out = step().detach()
        grads = tuple(t.grad for t in leaves) if backward else None
        if permute:
            out = unpermute_tokens_context_parallelism(out, mesh=mesh)
            if backward:
                grads = unpermute_tokens_context_parallelism(grads, mesh=mesh)

    density = calculate_mask_sparsity(mask[0], fwd_params.query_block_size,
                                      fwd_params.kv_block_size, q_len, kv_len)
    dense = get_multi_head_attention_tflops(batch, q_len, kv_len, heads, dim, dim_v, causal=False,
                                            forward_pass=True, backward_pass=backward)
    pairs = count_unmasked_pairs(*(t.cpu().numpy() for t in data[3:]))
    exact = attention_tflops_from_pairs(pairs, heads, dim, dim_v, True, backward)
    report(name, seconds, dense * density, exact)
    return zero_padding_rows(out, data[4]), grads


def common_options(cp: bool):
    options = [
        click.option("--num-iters", type=int, default=10),
        click.option("--batch-size", type=int, default=4),
        click.option("--query-seq-len", type=int, default=32768 if cp else 8192),
        click.option("--kv-seq-len", type=int, default=32768 if cp else 8192),
        click.option("--num-heads", type=int, default=32 if cp else 16),
        click.option("--num-kv-heads", type=int, default=8 if cp else 16),
        click.option("--qk-head-dim", type=int, default=128),
        click.option("--value-head-dim", type=int, default=128),
        click.option("--assume-sequential-positions", type=bool, default=True),
        click.option("--num-segments", type=int, default=1),
        click.option("--show-attention-mask", is_flag=True),
    ]
    if cp:
        options += [
            click.option("--permute-tokens-for-load-balance", type=bool, default=True),
            click.option("--context-parallel-degree", type=int, default=8,
                         help="query shards (the reference uses its device count)"),
        ]
    else:
        options.append(click.option("--num-pad-tokens", type=int, default=0))

    def decorate(fn):
        for option in reversed(options):
            fn = option(fn)
        return fn

    return decorate


def device_or_fail() -> torch.device:
    if not torch.cuda.is_available():
        raise click.ClickException("no GPU: the attention kernels only run on the device")
    return torch.device("cuda", torch.cuda.current_device())


def single_device_benchmark(backward: bool, *, num_iters, batch_size, query_seq_len, kv_seq_len,
                            num_heads, num_kv_heads, qk_head_dim, value_head_dim,
                            assume_sequential_positions, num_segments, num_pad_tokens,
                            show_attention_mask):
    device = device_or_fail()
    data, scale = make_inputs(batch_size, query_seq_len, kv_seq_len, num_heads, num_kv_heads,
                              qk_head_dim, value_head_dim, num_segments, num_pad_tokens, device)
    dout = torch.randn(data[0].shape[:3] + data[2].shape[3:], dtype=data[0].dtype, device=device) \
        if backward else None
    out, grads = run_kvax(
        data, scale, TP_SPECS, Mesh({"data": 1, "model": 1}), backward=backward,
        assume_sequential_positions=assume_sequential_positions, permute=False,
        show_attention_mask=show_attention_mask, num_iters=num_iters, name="flash_attention_kvax",
        dout=dout)
    if max(query_seq_len, kv_seq_len) > MAX_DENSE_MASK_LEN:
        logger.info("library comparison skipped: sequences above %d tokens", MAX_DENSE_MASK_LEN)
        return
    seconds = time_on_device(lambda: library_attention(data, scale, dout), num_iters, device)
    logger.info("library attention (dense boolean mask): %s per iteration", format_duration(seconds))
    ref_out, ref_grads = library_attention(data, scale, dout)
    check_outputs_fwd(ref_out, out)
    if backward:
        check_outputs_bwd(ref_grads, grads)
    logger.info("outputs agree with the library attention")


def context_parallel_benchmark(backward: bool, *, num_iters, batch_size, query_seq_len, kv_seq_len,
                               num_heads, num_kv_heads, qk_head_dim, value_head_dim,
                               assume_sequential_positions, num_segments,
                               permute_tokens_for_load_balance, context_parallel_degree,
                               show_attention_mask):
    device = device_or_fail()
    data, scale = make_inputs(batch_size, query_seq_len, kv_seq_len, num_heads, num_kv_heads,
                              qk_head_dim, value_head_dim, num_segments, 0, device)
    dout = torch.randn(data[0].shape[:3] + data[2].shape[3:], dtype=data[0].dtype, device=device) \
        if backward else None
    shared = dict(backward=backward, assume_sequential_positions=assume_sequential_positions,
                  show_attention_mask=show_attention_mask, num_iters=num_iters, dout=dout)
    cp = run_kvax(data, scale, CP_SPECS, Mesh({"data": 1, "context": context_parallel_degree}),
                  permute=permute_tokens_for_load_balance, name="flash_attention_kvax_cp", **shared)
    tp = run_kvax(data, scale, TP_SPECS, Mesh({"data": 1, "model": 1}), permute=False,
                  name="flash_attention_kvax_tp", **shared)
    check_outputs_fwd(tp[0], cp[0])
    if backward:
        check_outputs_bwd(tp[1], cp[1])
    logger.info("context-parallel and unsharded outputs agree")


@click.group()
def cli():
    logging.basicConfig(level=logging.INFO)


@cli.command("mha")
@common_options(cp=False)
def mha_benchmark(**options):
    single_device_benchmark(False, **options)


@cli.command("mha_bwd")
@common_options(cp=False)
def mha_benchmark_bwd(**options):
    single_device_benchmark(True, **options)


@cli.command("mha_cp")
@common_options(cp=True)
def mha_cp_fwd_benchmark(**options):
    context_parallel_benchmark(False, **options)


@cli.command("mha_cp_bwd")
@common_options(cp=True)
def mha_cp_bwd_benchmark(**options):
    context_parallel_benchmark(True, **options)


if __name__ == "__main__":
    cli()
