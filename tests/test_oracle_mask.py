"""Pins the CPU restatements of the block-mask builder (no GPU).

What is checked, and against what:
* loop == summaries == C on random inputs, including positions that restart per document,
  unsorted segment ids, ragged lengths and mixed padding (three independent restatements);
* the dense any/all definition the reference's test asserts its kernel equal to, on that test's
  own input family regenerated exactly (tests/test_attention.py:831-841,1011-1086);
* closed forms for one causal document; invariants of the bounds.
"""
import json
from pathlib import Path

import numpy as np
import pytest

from kvax_amd.utils.benchmarking import (
    generate_random_segments_lengths,
    make_random_attention_inputs,
    workload,
)
from kvax_amd.utils.permutation import generate_shard_indices
from oracle import mask_oracle as mo


# fixed seeds per input style: every run of the randomised tests draws the same inputs
STYLE_SEEDS = {"restart": 101, "global": 202, "unsorted": 303, "shuffled_pos": 404}


def _random_ids(rng, batch, length, style):
    pos = np.zeros((batch, length), np.int32)
    seg = np.zeros((batch, length), np.int32)
    for b in range(batch):
        n_docs = int(rng.integers(1, 6))
        cuts = np.sort(rng.choice(np.arange(1, max(2, length)), size=min(n_docs - 1, max(0, length - 2)), replace=False)) if length > 2 else np.array([], int)
        bounds = np.concatenate([[0], cuts, [length]]).astype(int)
        ids = np.arange(len(bounds) - 1)
        if style == "unsorted":
            ids = rng.permutation(ids) * 3 + 1
        for i, (a, c) in enumerate(zip(bounds[:-1], bounds[1:])):
            seg[b, a:c] = ids[i]
            pos[b, a:c] = np.arange(c - a) if style != "global" else np.arange(a, c)
        if style == "shuffled_pos":
            pos[b] = rng.integers(0, length, size=length)
        n_pad = int(rng.integers(0, length // 2 + 1))
        if n_pad:
            seg[b, length - n_pad:] = -1
        if style == "unsorted" and length > 8:  # padding in the middle too
            a = int(rng.integers(0, length - 4))
            seg[b, a:a + 3] = -1
    return pos, seg


@pytest.mark.parametrize("style", ["restart", "global", "unsorted", "shuffled_pos"])
@pytest.mark.parametrize("skip_pad", [True, False])
def test_three_restatements_agree(style, skip_pad):
    rng = np.random.default_rng([STYLE_SEEDS[style], int(skip_pad)])
    for trial in range(12):
        batch = int(rng.integers(1, 3))
        sq = int(rng.integers(1, 300))
        sk = sq if trial % 2 == 0 else int(rng.integers(1, 300))
        qbs = int(rng.choice([8, 16, 32, 64]))
        kbs = int(rng.choice([8, 16, 32, 64]))
        q_pos, q_seg = _random_ids(rng, batch, sq, style)
        if sk == sq:
            kv_pos, kv_seg = q_pos.copy(), q_seg.copy()
        else:
            kv_pos, kv_seg = _random_ids(rng, batch, sk, style)
        for dkdv in (False, True):
            a = mo.block_mask_loop(q_pos, q_seg, kv_pos, kv_seg, qbs, kbs, skip_pad, dkdv)
            b = mo.block_mask_summaries(q_pos, q_seg, kv_pos, kv_seg, qbs, kbs, skip_pad, dkdv)
            c = mo.block_mask_c(q_pos, q_seg, kv_pos, kv_seg, qbs, kbs, skip_pad, dkdv)
            for x, y, z in zip(a, b, c):
                np.testing.assert_array_equal(x, y)
                np.testing.assert_array_equal(x, z)


# (num_pad_tokens, num_segments, permute, skip_pad_tokens): tests/test_attention.py:831-841
REFERENCE_MASK_CASES = [
    (0, 1, True, False),
    (10000, 1, True, False),
    (20645, 1, False, False),
    (5632, 3, True, True),
    (6759, 5, True, False),
    (1024, 12, True, False),
]


def reference_mask_case(num_pad, num_segments, permute, cp, seq_len=32768, batch=1):
    """Id arrays of the reference's mask test: arange positions, random.seed(0) documents,
    trailing padding; queries permuted for load balance when ``permute``."""
    data, _ = make_random_attention_inputs(
        batch, seq_len, seq_len, 1, 1, 1, 1, num_pad_tokens=num_pad,
        list_of_segment_lengths=generate_random_segments_lengths(seq_len, num_segments))
    q_pos, q_seg, kv_pos, kv_seg = (x.numpy() for x in data[3:])
    if permute:
        order = generate_shard_indices(2 * cp)
        chunk = seq_len // (2 * cp)
        idx = np.concatenate([np.arange(c * chunk, (c + 1) * chunk) for c in order])
        q_pos, q_seg = q_pos[:, idx], q_seg[:, idx]
    return q_pos, q_seg, kv_pos, kv_seg


@pytest.mark.parametrize("case", REFERENCE_MASK_CASES)
@pytest.mark.parametrize("cp", [1, 8])
def test_matches_reference_brute_force_definition(case, cp):
    num_pad, num_segments, permute, skip_pad = case
    if cp == 8 and not permute and num_pad == 20645:
        pass  # still a valid case: contiguous shards
    q_pos, q_seg, kv_pos, kv_seg = reference_mask_case(num_pad, num_segments, permute, cp)
    fwd, bwd = (128, 128), (64, 128)
    got = mo.create_attention_mask(q_pos, q_seg, kv_pos, kv_seg, fwd, bwd, True, skip_pad, cp,
                                   impl=mo.block_mask_summaries)
    want = mo.create_attention_mask(q_pos, q_seg, kv_pos, kv_seg, fwd, bwd, True, skip_pad, cp,
                                    impl=mo.block_mask_dense)
    for g, w in zip(got, want):
        for x, y in zip(g, w):
            np.testing.assert_array_equal(x, y)
    # and the C restatement on the unsharded query-outer masks
    c = mo.block_mask_c(q_pos, q_seg, kv_pos, kv_seg, 128, 128, skip_pad, False)
    for x, y in zip(c, got[0]):
        np.testing.assert_array_equal(x, y)


def test_closed_form_single_causal_document():
    n, bs = 16, 32
    pos = np.arange(n * bs, dtype=np.int32)[None]
    seg = np.zeros_like(pos)
    lower, upper, lower_full, upper_full = mo.block_mask_c(pos, seg, pos, seg, bs, bs, True, False)
    i = np.arange(n)
    np.testing.assert_array_equal(lower[0, 0], 0 * i)
    np.testing.assert_array_equal(upper[0, 0], i + 1)
    np.testing.assert_array_equal(lower_full[0, 0], 0 * i)
    np.testing.assert_array_equal(upper_full[0, 0], i)
    lower, upper, lower_full, upper_full = mo.block_mask_c(pos, seg, pos, seg, bs, bs, True, True)
    np.testing.assert_array_equal(lower[0, 0], i)
    np.testing.assert_array_equal(upper[0, 0], 0 * i + n)
    np.testing.assert_array_equal(lower_full[0, 0], np.minimum(i + 1, n))
    np.testing.assert_array_equal(upper_full[0, 0], 0 * i + n)


def test_all_padding_outer_block_and_empty_rows():
    bs = 16
    pos = np.arange(4 * bs, dtype=np.int32)[None]
    seg = np.zeros_like(pos)
    seg[0, 2 * bs:] = -1
    out = mo.block_mask_c(pos, seg, pos, seg, bs, bs, True, False)
    for arr in out:
        assert (arr[0, 0, 2:] == 0).all()
    # a query block whose document has no keys at all: bounds collapse to one value
    q_seg = np.full_like(pos, 7)
    out = mo.block_mask_c(pos, q_seg, pos, seg, bs, bs, True, False)
    lower, upper, lower_full, upper_full = (a[0, 0] for a in out)
    assert (lower == upper).all() and (lower_full == upper_full).all()


@pytest.mark.parametrize("name", ["cpu_plumbing", "doc32k", "block_skip"])
def test_invariants_on_workloads(name):
    w = workload(name)
    qbs, kbs = w.fwd_blocks
    lower, upper, lower_full, upper_full = mo.block_mask_summaries(
        w.q_pos, w.q_seg, w.kv_pos, w.kv_seg, qbs, kbs, True, False)
    has_full = upper_full > lower_full
    assert (lower <= upper).all()
    assert (lower[has_full] <= lower_full[has_full]).all()
    assert (upper_full[has_full] <= upper[has_full]).all()
    # every attendable element pair lies inside [lower, upper); full blocks are all-True
    b = 0
    nq = w.q_len // qbs
    rng = np.random.default_rng(1)
    for o in rng.choice(nq, size=min(nq, 24), replace=False):
        rows = slice(o * qbs, (o + 1) * qbs)
        m = mo.dense_attention_mask(w.q_pos[b:b + 1, rows], w.q_seg[b:b + 1, rows],
                                    w.kv_pos[b:b + 1], w.kv_seg[b:b + 1])[0]
        cols = np.nonzero(m.any(0))[0]
        if len(cols):
            assert cols.min() >= lower[b, 0, o] * kbs and cols.max() < upper[b, 0, o] * kbs
        f = m[:, lower_full[b, 0, o] * kbs: upper_full[b, 0, o] * kbs]
        assert f.all()


def test_heuristic_over_covers_when_positions_restart():
    """The regression input for the regime where the heuristic is not the any/all mask."""
    w = workload("cpu_plumbing")
    h = mo.block_mask_summaries(w.q_pos, w.q_seg, w.kv_pos, w.kv_seg, 64, 64, True, False)
    d = mo.block_mask_dense(w.q_pos, w.q_seg, w.kv_pos, w.kv_seg, 64, 64, True, False)
    assert (h[1] >= d[1]).all() and (h[1] != d[1]).any()      # upper runs further right
    np.testing.assert_array_equal(h[0], d[0])                 # lower is still exact here
    loop = mo.block_mask_loop(w.q_pos, w.q_seg, w.kv_pos, w.kv_seg, 64, 64, True, False)
    for x, y in zip(h, loop):
        np.testing.assert_array_equal(x, y)


# --------------------------------------------------------------------------------------------
# hand-worked vectors (tests/golden/mask_hand_worked.json): expected arrays derived on paper from
# the reference's kernel, in the regime where the heuristic is not the dense any/all mask
# --------------------------------------------------------------------------------------------
def hand_worked_mask_cases():
    """[(case name, ids (q_pos, q_seg, kv_pos, kv_seg), mask dict), ...] from the golden file."""
    with open(Path(__file__).parent / "golden" / "mask_hand_worked.json") as f:
        golden = json.load(f)
    out = []
    for case in golden["cases"]:
        ids = tuple(np.asarray(case[k], np.int32) for k in ("q_pos", "q_seg", "kv_pos", "kv_seg"))
        for m in case["masks"]:
            tag = f"{case['name']}-{m['query_block']}x{m['kv_block']}-" \
                  f"{'kv' if m['kv_outer'] else 'q'}outer-{'skip' if m['skip_pad'] else 'noskip'}"
            out.append(pytest.param(ids, m, id=tag))
    return out


@pytest.mark.parametrize("ids, m", hand_worked_mask_cases())
@pytest.mark.parametrize("impl", ["loop", "summaries", "c"])
def test_hand_worked_vectors(ids, m, impl):
    fn = {"loop": mo.block_mask_loop, "summaries": mo.block_mask_summaries, "c": mo.block_mask_c}[impl]
    got = fn(*ids, m["query_block"], m["kv_block"], m["skip_pad"], m["kv_outer"])
    for name, x in zip(("lower", "upper", "lower_full", "upper_full"), got):
        np.testing.assert_array_equal(x[0, 0], np.asarray(m[name], np.int32), err_msg=name)
