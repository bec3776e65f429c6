"""FLOP accounting for attention (model of kvax/utils/math.py:18-26)."""
from __future__ import annotations


def get_multi_head_attention_tflops(
    batch_size: int,
    query_seq_len: int,
    kv_seq_len: int,
    num_heads: int,
    qk_head_dim: int,
    value_head_dim: int,
    causal: bool,
    num_gpus: int = 1,
    forward_pass: bool = True,
    backward_pass: bool = False,
) -> float:
    """Dense-shape TFLOP count: 2*(dqk+dv) per (q, kv) pair, halved if causal, x2.5 for the
    backward pass and x3.5 for forward+backward."""
    if not forward_pass and not backward_pass:
        raise ValueError("At least one of the forward_pass or backward_pass should be True")
    pairs = float(query_seq_len) * float(kv_seq_len) * batch_size
    if causal:
        pairs *= 0.5
    return attention_tflops_from_pairs(
        pairs, num_heads, qk_head_dim, value_head_dim, forward_pass, backward_pass
    ) / num_gpus


def attention_tflops_from_pairs(
    unmasked_pairs: float,
    num_heads: int,
    qk_head_dim: int,
    value_head_dim: int,
    forward_pass: bool = True,
    backward_pass: bool = False,
) -> float:
    """TFLOPs when exactly ``unmasked_pairs`` (batch, q, kv) element pairs are attendable.

    Same per-pair cost as above; this is the figure throughput is quoted on (element-level
    unmasked FLOPs, not block-level density as in kvax/utils/benchmarking.py:423-430).
    """
    flops = 2.0 * (qk_head_dim + value_head_dim) * unmasked_pairs * num_heads
    if forward_pass and backward_pass:
        flops *= 3.5
    elif backward_pass:
        flops *= 2.5
    return flops / 1e12
