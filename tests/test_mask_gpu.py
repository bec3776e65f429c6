"""Bit-exact parity of the HIP block-mask builder (through the C ABI) with the CPU oracle."""
import numpy as np
import pytest
import torch

from kvax_amd.ops.mask_creator import build_masks, create_attention_mask
from kvax_amd.utils import FlashAttentionParamsConfig, Mesh, attention_specs
from kvax_amd.utils.benchmarking import workload
from oracle import mask_oracle as mo
from tests.test_oracle_mask import (REFERENCE_MASK_CASES, STYLE_SEEDS, _random_ids,
                                     hand_worked_mask_cases, reference_mask_case)

pytestmark = pytest.mark.gpu

TP_SPECS = (("data", None, "model", None), ("data", None, "model", None))
CP_SPECS = (("data", "context", None, None), ("data", None, None, None))


def _dev(device, *arrays):
    return [torch.from_numpy(np.ascontiguousarray(a)).to(device) for a in arrays]


def _assert_masks_equal(got, want):
    assert len(got) == len(want)
    for g, w in zip(got, want):
        for name, x, y in zip(("lower", "upper", "lower_full", "upper_full"), g.flatten(), w):
            assert x.dtype == torch.int32 and tuple(x.shape) == y.shape, (name, x.shape, y.shape)
            np.testing.assert_array_equal(x.cpu().numpy(), y, err_msg=name)


@pytest.mark.parametrize("style", ["restart", "global", "unsorted", "shuffled_pos"])
@pytest.mark.parametrize("skip_pad", [True, False])
def test_random_ragged_inputs(device, style, skip_pad):
    rng = np.random.default_rng([STYLE_SEEDS[style], int(skip_pad), 7])
    for trial in range(10):
        batch = int(rng.integers(1, 4))
        sq = int(rng.integers(1, 700))
        sk = sq if trial % 2 == 0 else int(rng.integers(1, 700))
        qbs, kbs = int(rng.choice([16, 64, 128, 256])), int(rng.choice([16, 64, 128]))
        q_pos, q_seg = _random_ids(rng, batch, sq, style)
        kv_pos, kv_seg = (q_pos.copy(), q_seg.copy()) if sk == sq else _random_ids(rng, batch, sk, style)
        got = build_masks(*_dev(device, q_pos, q_seg, kv_pos, kv_seg),
                          [(qbs, kbs, False), (kbs, qbs, False), (qbs, kbs, True)], skip_pad)
        want = [mo.block_mask_c(q_pos, q_seg, kv_pos, kv_seg, qbs, kbs, skip_pad, False),
                mo.block_mask_c(q_pos, q_seg, kv_pos, kv_seg, kbs, qbs, skip_pad, False),
                mo.block_mask_c(q_pos, q_seg, kv_pos, kv_seg, qbs, kbs, skip_pad, True)]
        _assert_masks_equal(got, want)


@pytest.mark.parametrize("ids, m", hand_worked_mask_cases())
def test_hand_worked_vectors(device, ids, m):
    """Expected arrays derived on paper from the reference's kernel (tests/golden)."""
    got = build_masks(*_dev(device, *ids), [(m["query_block"], m["kv_block"], m["kv_outer"])],
                      m["skip_pad"])[0]
    for name, x in zip(("lower", "upper", "lower_full", "upper_full"), got.flatten()):
        np.testing.assert_array_equal(x.cpu().numpy()[0, 0], np.asarray(m[name], np.int32), err_msg=name)


@pytest.mark.parametrize("case", REFERENCE_MASK_CASES)
@pytest.mark.parametrize("cp", [1, 8])
def test_reference_mask_test_family(device, case, cp):
    """Inputs of the reference's test_attention_mask; fwd 128/128, bwd 64/128, batch 2."""
    num_pad, num_segments, permute, skip_pad = case
    ids = reference_mask_case(num_pad, num_segments, permute, cp, batch=2)
    fwd = FlashAttentionParamsConfig(query_block_size=128, kv_block_size=128)
    bwd = FlashAttentionParamsConfig(query_block_size=64, kv_block_size=128)
    with attention_specs(*CP_SPECS), Mesh({"data": 1, "context": cp, "model": 1}):
        got = create_attention_mask(*_dev(device, *ids), fwd_params=fwd, bwd_params=bwd,
                                    calc_bwd_mask=True, skip_pad_tokens=skip_pad)
    want = mo.create_attention_mask(*ids, (128, 128), (64, 128), True, skip_pad, cp)
    _assert_masks_equal(got, want)
    assert tuple(got[2].lower_bounds.shape) == (2, cp, 256)


@pytest.mark.parametrize("name", ["cpu_plumbing", "dense_causal", "doc32k", "cp_shard", "block_skip"])
@pytest.mark.parametrize("block", [64, 128])
def test_measurement_workloads(device, name, block):
    w = workload(name)
    ids = (w.q_pos, w.q_seg, w.kv_pos, w.kv_seg)
    params = FlashAttentionParamsConfig(query_block_size=block, kv_block_size=block)
    with attention_specs(*TP_SPECS):
        got = create_attention_mask(*_dev(device, *ids), fwd_params=params, bwd_params=params,
                                    calc_bwd_mask=True)
    want = mo.create_attention_mask(*ids, (block, block), (block, block), True, True, 1)
    _assert_masks_equal(got, want)
    if name == "dense_causal":  # closed form
        i = torch.arange(w.q_len // block, dtype=torch.int32)
        assert (got[0].upper_bounds.cpu()[0, 0] == i + 1).all()
        assert (got[0].upper_full_bounds.cpu()[0, 0] == i).all()
        assert (got[2].lower_bounds.cpu()[0, 0] == i).all()


def test_default_params_and_single_mask(device):
    w = workload("cpu_plumbing")
    with attention_specs(*TP_SPECS):
        got = create_attention_mask(*_dev(device, w.q_pos, w.q_seg, w.kv_pos, w.kv_seg))
    assert len(got) == 1
    want = mo.create_attention_mask(w.q_pos, w.q_seg, w.kv_pos, w.kv_seg, (128, 128))
    _assert_masks_equal(got, want)


def test_specs_must_be_set(device):
    w = workload("cpu_plumbing")
    with pytest.raises(ValueError):
        create_attention_mask(*_dev(device, w.q_pos, w.q_seg, w.kv_pos, w.kv_seg))


def test_mask_diagnostics_on_device_masks(device):
    from kvax_amd.ops.mask_creator import calculate_mask_sparsity, mask_block_levels, render_mask

    w = workload("dense_causal")
    params = FlashAttentionParamsConfig(query_block_size=128, kv_block_size=128)
    with attention_specs(*TP_SPECS):
        fwd, dq, dkdv = create_attention_mask(*_dev(device, w.q_pos, w.q_seg, w.kv_pos, w.kv_seg),
                                              fwd_params=params, bwd_params=params,
                                              calc_bwd_mask=True)
    n = w.q_len // 128
    levels = mask_block_levels(fwd, n)
    want = torch.tril(torch.full((n, n), 2, dtype=torch.int8), -1) + torch.eye(n, dtype=torch.int8)
    assert torch.equal(levels, want)
    # The dK/dV mask is the transposed picture: kv block j is visited by query blocks >= j.
    assert torch.equal(mask_block_levels(dkdv, n), want.T)
    assert calculate_mask_sparsity(fwd, 128, 128, w.q_len, w.kv_len) == pytest.approx(
        (n + 1) / (2 * n))
    lines = [l for l in render_mask(fwd, n).splitlines() if l.startswith("||")]
    assert len(lines) == min(n, 32) and lines[0].count("█") == 0 and "░" in lines[0]
