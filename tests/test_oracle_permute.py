"""Pins the permutation / capacity part of the CPU oracle: library sorts, brute force, and the
capacity tables the reference's README holds (tests/golden/capacity_tables.json)."""

import json
import math
import os

import numpy as np
import torch

from oracle import c_oracle
from oracle import moe_oracle as O

GOLD = os.path.join(os.path.dirname(__file__), "golden", "capacity_tables.json")


def test_permute_plan_three_ways():
    g = torch.Generator().manual_seed(0)
    for n, E in [(0, 4), (1, 1), (17, 4), (1000, 8), (4096, 64)]:
        e = torch.randint(0, E, (n,), generator=g)
        if n > 10:
            e[e == 1] = 0  # an empty expert
        o1, i1, c1 = O.permute_plan(e, E)
        o2, i2, c2 = O.permute_plan_fast(e, E)
        o3, i3, c3, w3 = c_oracle.permute_plan(e.numpy(), E)
        assert torch.equal(o1, o2) and torch.equal(i1, i2) and torch.equal(c1, c2)
        assert np.array_equal(o3, o1.numpy()) and np.array_equal(i3, i1.numpy()) and np.array_equal(c3, c1.numpy())
        # definition checks: grouped by expert, ascending original row inside an expert, true inverse
        se = e[o1]
        assert torch.all(se.diff() >= 0)
        same = se[1:] == se[:-1]
        assert torch.all(o1[1:][same] > o1[:-1][same])
        assert torch.equal(o1[i1], torch.arange(n))
        within, counts = O.slot_assignment(e, E)
        brute = [int((e[:r] == e[r]).sum()) for r in range(n)] if n <= 1000 else None
        if brute is not None:
            assert within.tolist() == brute
        assert np.array_equal(w3, within.numpy())


def test_compute_capacity_known_values():
    assert O.compute_capacity(512, 2, 8, 1.0) == 128
    assert O.compute_capacity(512, 2, 8, 0.5) == 64
    assert O.compute_capacity(512, 2, 8, 1.25) == 160
    assert O.compute_capacity(512, 2, 8, 2.0) == 256
    assert O.compute_capacity(16384, 6, 64, 1.25) == 1920     # the fine-grained skewed benchmark shape
    assert O.compute_capacity(8192, 1, 16, 1.0) == 512
    assert O.compute_capacity(3, 1, 64, 0.1) == 1             # floor of one slot


def _zipf_routing(T, k, E, skew, seed):
    """The synthetic routing recipe of the reference's ablation (tests/ablation_moe.py:34-46)."""
    g = torch.Generator().manual_seed(seed)
    rank_w = 1.0 / torch.arange(1, E + 1, dtype=torch.float32) ** skew
    probs = (rank_w / rank_w.sum()).expand(T, E)
    idx = torch.multinomial(probs, k, replacement=False, generator=g)
    w = torch.softmax(torch.rand(T, k, generator=g), dim=-1)
    return idx, w


def _drop_and_rounds(idx, E, C):
    e = idx.reshape(-1)
    within, counts = O.slot_assignment(e, E)
    keep = within < C
    return 100.0 * float((~keep).sum()) / e.numel(), O.capacity_rounds(counts, C, True, 64), counts


def test_capacity_tables_held_by_the_reference():
    gold = json.load(open(GOLD))
    E, k, T = gold["num_experts"], gold["top_k"], gold["num_tokens"]
    for row in gold["vary_skew_factor_1"]:
        idx, _ = _zipf_routing(T, k, E, row["skew"], seed=100 + int(row["skew"] * 10))
        C = O.compute_capacity(T, k, E, 1.0)
        drop, rounds, counts = _drop_and_rounds(idx, E, C)
        assert C == row["capacity"]
        assert int(counts.max()) == row["worst_buf"]
        assert round(drop, 1) == row["drop_pct"]
        assert rounds == row["rounds"]
        assert abs(int(counts.max()) / counts.float().mean().item() - row["max_over_mean"]) < 0.006
    idx, _ = _zipf_routing(T, k, E, 1.0, seed=110)
    for row in gold["vary_factor_skew_1"]:
        C = O.compute_capacity(T, k, E, row["factor"])
        drop, rounds, _ = _drop_and_rounds(idx, E, C)
        assert C == row["capacity"] and round(drop, 1) == row["drop_pct"] and rounds == row["rounds"]


def test_drop_formula_equals_keep_mask():
    # closed form used by the reference's ablation (tests/ablation_moe.py:64-72): dropped = sum max(count - C, 0)
    idx, _ = _zipf_routing(512, 2, 8, 1.5, seed=3)
    e = idx.reshape(-1)
    within, counts = O.slot_assignment(e, 8)
    for C in (1, 17, 128, 1000):
        assert int((within >= C).sum()) == int(torch.clamp(counts - C, min=0).sum())
        assert O.capacity_rounds(counts, C, True, 64) == min(64, max(1, math.ceil(int(counts.max()) / C)))
        assert O.capacity_rounds(counts, C, False, 64) == 1
