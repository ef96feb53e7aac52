"""Pins the integer half of the CPU checker (oracle/) and the package's own layout
builders against hand-derived vectors, closed forms and invariants, and against
the Algo rows listed in the reference's generated tables (tests/golden/algo_table.json).
"""
import json
import os

import numpy as np
import pytest
import torch

from flashoverlap_amd import layout

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


# ---------------------------------------------------------------- reorder_indices
HAND_REORDER = [
    # (S, hint, RA) worked by hand from "RA[hint[i]] = i, the rest ascending"
    (4, [2, 0], [1, 2, 0, 3]),
    (6, [4, 1, 5], [3, 1, 4, 5, 0, 2]),
    (5, [], [0, 1, 2, 3, 4]),
    (3, [2, 1, 0], [2, 1, 0]),
    (1, [0], [0]),
]


@pytest.mark.parametrize("S,hint,expect", HAND_REORDER)
def test_reorder_indices_hand_vectors(oracle, S, hint, expect):
    assert oracle.reorder_indices(S, hint).tolist() == expect
    assert layout.reorder_indices(S, hint, device="cpu").tolist() == expect


def test_reorder_indices_invariants(oracle):
    rng = np.random.default_rng(0)
    for S in (1, 7, 64, 257):
        for frac in (0.0, 0.3, 1.0):
            hint = rng.permutation(S)[: int(S * frac)].tolist()
            ra = oracle.reorder_indices(S, hint)
            assert sorted(ra.tolist()) == list(range(S))          # a permutation
            assert all(ra[h] == i for i, h in enumerate(hint))    # RA[hint[i]] == i
            rest = [t for t in range(S) if t not in set(hint)]
            assert [ra[t] for t in rest] == list(range(len(hint), S))  # others ascending
            assert layout.reorder_indices(S, hint, device="cpu").tolist() == ra.tolist()


def test_reorder_indices_rejects_bad_hint(oracle):
    with pytest.raises(ValueError):
        oracle.reorder_indices(4, [4])
    with pytest.raises(ValueError):
        layout.reorder_indices(4, [-1], device="cpu")


# ---------------------------------------------------------------- cSeg / groups
def test_cseg_from_waves(oracle):
    assert oracle.cseg_from_waves(2048, 256).tolist() == [256] * 8
    assert oracle.cseg_from_waves(10, 4).tolist() == [4, 4, 2]
    assert oracle.cseg_from_waves(3, 8).tolist() == [3]
    for T, w in [(2048, 254), (64, 16), (7, 3)]:
        assert layout.cseg_from_waves(T, w) == oracle.cseg_from_waves(T, w).tolist()
        assert sum(layout.cseg_from_waves(T, w)) == T


def test_tile_group_matches_searchsorted(oracle):
    cseg = [3, 1, 4, 2]
    by_hand = [0, 0, 0, 1, 2, 2, 2, 2, 3, 3]
    assert [oracle.tile_group(cseg, r) for r in range(10)] == by_hand
    assert layout.tile_groups(cseg).tolist() == by_hand
    assert oracle.tile_group(cseg, 10) == -1  # beyond the last slot


# ---------------------------------------------------------------- row mapping
HAND_ROWMAP = [
    # (M, N, BM, BN, cSeg, W, RE) -- worked by hand: inside each group, rows sorted stably by row % W
    (4, 4, 2, 2, [2, 2], 2, [0, 2, 1, 3, 4, 6, 5, 7]),
    (4, 4, 2, 2, [1, 3], 2, [0, 1, 2, 5, 3, 6, 4, 7]),
    (4, 4, 2, 2, [4], 1, [0, 1, 2, 3, 4, 5, 6, 7]),
]


@pytest.mark.parametrize("M,N,BM,BN,cseg,W,expect", HAND_ROWMAP)
def test_row_mapping_hand_vectors(oracle, M, N, BM, BN, cseg, W, expect):
    assert oracle.row_mapping(M, N, BM, BN, cseg, W).tolist() == expect
    assert layout.generate_row_mapping(M, N, BM, BN, cseg, W, device="cpu").tolist() == expect


def test_row_mapping_closed_form_and_invariants(oracle):
    # BM % W == 0: RE[s0 + l] = s0 + (l % W) * (R / W) + l // W with R = cSeg*BM rows per group
    M, N, BM, BN, W = 64, 32, 8, 8, 4
    cseg = [5, 11, 16]
    re_ = oracle.row_mapping(M, N, BM, BN, cseg, W)
    assert sorted(re_.tolist()) == list(range(M * N // BN))
    s0 = 0
    for c in cseg:
        R = c * BM
        for l in range(R):
            assert re_[s0 + l] == s0 + (l % W) * (R // W) + l // W
        assert set(re_[s0:s0 + R].tolist()) == set(range(s0, s0 + R))  # group-closed
        s0 += R
    assert layout.generate_row_mapping(M, N, BM, BN, cseg, W, device="cpu").tolist() == re_.tolist()


def test_row_mapping_rejects_wrong_sum(oracle):
    with pytest.raises(ValueError):
        oracle.row_mapping(4, 4, 2, 2, [1, 2], 2)
    with pytest.raises(AssertionError):
        layout.generate_row_mapping(4, 4, 2, 2, [1, 2], 2, device="cpu")


def test_rows_by_world_size(oracle):
    assert oracle.rows_by_world_size(6, 2).tolist() == [0, 2, 4, 1, 3, 5]
    x = torch.arange(12).reshape(6, 2)
    assert layout.reorder_rows_by_world_size(x, 2)[:, 0].tolist() == [0, 4, 8, 2, 6, 10]
    assert layout.reorder_rows_by_world_size(x, 3)[:, 0].tolist() == [0, 6, 2, 8, 4, 10]


# ---------------------------------------------------------------- Algo table
def test_algo_table_matches_reference_rows(oracle):
    golden = json.load(open(os.path.join(GOLDEN, "algo_table.json")))["rows"]
    assert len(golden) == 102
    assert oracle.algo_table().tolist() == golden


def test_counter_size():
    assert layout.counter_size(256, 32, 32) == 256       # more groups than tile columns
    assert layout.counter_size(8, 64, 32) == 32
    assert layout.counter_size(8, 64, 32, monitor=True) == 65 * 32


def test_unpermute_brute_force():
    # 4x4 tiles of 2x3: every element placed by the textbook formula, one by one
    M, N, BM, BN = 8, 12, 2, 3
    TM, TN = M // BM, N // BN
    rng = np.random.default_rng(1)
    ra = rng.permutation(TM * TN).astype(np.int32)
    C = np.arange(M * N, dtype=np.float32).reshape(M, N)
    for rldn in (1, 2, 4):
        ldp = rldn * BN
        Cp = np.zeros(M * N, dtype=np.float32)
        for m in range(M):
            for n in range(N):
                r = ra[(m // BM) * TN + n // BN]
                Cp[((r // rldn) * BM + m % BM) * ldp + (r % rldn) * BN + n % BN] = C[m, n]
        back = layout.unpermute(torch.from_numpy(Cp), M, N, BM, BN, torch.from_numpy(ra), rLDN=rldn)
        assert torch.equal(back, torch.from_numpy(C))
