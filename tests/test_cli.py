"""The benchmark command line: every command runs end to end at a small size and its built-in
comparison (library attention, or context-parallel against unsharded) passes."""
import logging

import pytest
from click.testing import CliRunner

from kvax_amd.benchmarks import cli

SMALL = ["--num-iters", "2", "--batch-size", "2", "--num-heads", "4", "--num-kv-heads", "2",
         "--query-seq-len", "2048", "--kv-seq-len", "2048", "--num-segments", "3"]


def _invoke(args, caplog):
    with caplog.at_level(logging.INFO, logger="kvax_amd"):
        result = CliRunner().invoke(cli, args, catch_exceptions=False)
    assert result.exit_code == 0, result.output
    return caplog.text


@pytest.mark.gpu
@pytest.mark.parametrize("command", ["mha", "mha_bwd"])
@pytest.mark.parametrize("sequential", ["True", "False"])
def test_single_device_commands(device, caplog, command, sequential):
    text = _invoke([command, *SMALL, "--num-pad-tokens", "256", "--show-attention-mask",
                    "--assume-sequential-positions", sequential], caplog)
    assert "outputs agree with the library attention" in text
    assert "Attention masks:" in text and "TFLOP/s" in text


@pytest.mark.gpu
def test_head_dims_of_the_reference_tests(device, caplog):
    text = _invoke(["mha_bwd", *SMALL, "--qk-head-dim", "16", "--value-head-dim", "32"], caplog)
    assert "outputs agree with the library attention" in text


@pytest.mark.gpu
@pytest.mark.parametrize("command", ["mha_cp", "mha_cp_bwd"])
@pytest.mark.parametrize("permute", ["True", "False"])
def test_context_parallel_commands(device, caplog, command, permute):
    text = _invoke([command, *SMALL, "--context-parallel-degree", "4",
                    "--permute-tokens-for-load-balance", permute], caplog)
    assert "context-parallel and unsharded outputs agree" in text


def test_commands_and_option_names_follow_the_reference_script():
    # Option names of benchmarks.py:34-46 and :208-220 of the reference.
    shared = {"num_iters", "batch_size", "query_seq_len", "kv_seq_len", "num_heads", "num_kv_heads",
              "qk_head_dim", "value_head_dim", "assume_sequential_positions", "num_segments",
              "show_attention_mask"}
    assert set(cli.commands) == {"mha", "mha_bwd", "mha_cp", "mha_cp_bwd"}
    for name, command in cli.commands.items():
        names = {p.name for p in command.params}
        extra = ({"permute_tokens_for_load_balance", "context_parallel_degree"} if "cp" in name
                 else {"num_pad_tokens"})
        assert names == shared | extra, name
    defaults = {p.name: p.default for p in cli.commands["mha_cp"].params}
    assert (defaults["query_seq_len"], defaults["num_heads"], defaults["num_kv_heads"]) == (32768, 32, 8)
    defaults = {p.name: p.default for p in cli.commands["mha"].params}
    assert (defaults["query_seq_len"], defaults["num_heads"], defaults["batch_size"]) == (8192, 16, 4)
    import torch

    if not torch.cuda.is_available():  # the product path refuses to run without the device
        result = CliRunner().invoke(cli, ["mha", "--num-iters", "1"])
        assert result.exit_code != 0 and "no GPU" in result.output
