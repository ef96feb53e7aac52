"""CPU-side checks of the product: the C-ABI library loads and exports every
symbol the header declares, validates arguments before touching a GPU, owns the
reference's Algo table and a consistent tile schedule; the Python host logic
(latency model, searches, config JSON) agrees with the CPU checker."""
import ctypes
import json
import os
import re

import numpy as np
import pytest
import torch

from flashoverlap_amd import _capi, config, layout, tune

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _header_symbols():
    text = open(os.path.join(ROOT, "include", "flashoverlap.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fo_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    L = ctypes.CDLL(_capi.KERNEL_LIB)
    names = _header_symbols()
    assert len(names) >= 25
    for n in names:
        assert hasattr(L, n), f"libfo_kernels.so does not export {n}"
    assert set(names) == set(_capi.SIGNATURES), "ctypes table and header disagree"


def test_shim_registers_reference_names():
    from flashoverlap_amd import layers
    layers.load_library()
    ov = torch.classes.flashoverlap_class.OverlapImpl()
    for m in ["nccl_init", "cutlass_init", "overlap_init", "cutlass_gemm", "gemm_allreduce_overlap",
              "gemm_reducescatter_overlap", "gemm_allreduce", "gemm_reducescatter", "gemm_all2all",
              "nccl_allreduce", "nccl_reducescatter", "nccl_all2all", "seg_allreduce",
              "gemm_allreduce_rmsnorm_overlap"]:     # the last one is an addition
        assert hasattr(ov, m), m
    bl = torch.classes.flashoverlap_class.BaselineImpl()
    for m in ["nccl_init", "cublas_init", "cublas_gemm", "gemm_allreduce", "gemm_reducescatter",
              "gemm_all2all", "nccl_allreduce", "nccl_reducescatter", "nccl_all2all"]:
        assert hasattr(bl, m), m
    ident = torch.ops.flashoverlap_op.generate_nccl_id()
    assert len(ident) == 16                       # 128 bytes as int64, src/nccl_utils.cu:7-14
    assert hasattr(torch.ops.flashoverlap_op, "reorder_rmsnorm")
    # dtype errors surface as exceptions, as data_ptr<at::Half>() does in the reference
    x = torch.zeros(4, 8)
    with pytest.raises(RuntimeError):
        torch.ops.flashoverlap_op.reorder_rmsnorm(x, x, x[0], 4, 8, 1, torch.zeros(1, 1, dtype=torch.int32))


def test_algo_table_matches_reference_rows():
    golden = json.load(open(os.path.join(GOLDEN, "algo_table.json")))["rows"]
    assert [list(r) for r in _capi.algo_table()] == golden
    assert _capi.algo_tile(0) == (128, 128) and _capi.algo_tile(54) == (128, 256)
    assert _capi.algo_tile(78) == (256, 128)
    assert _capi.find_algo(128, 256, swizzle=4) == 57


def test_schedule_order_with_a_partial_last_wave():
    """1089 workgroup tiles of 256x256 on 256 workgroups leave 65 for a fifth wave; those are walked
    in the Algo's own tile by a second launch, and the analytic hint must follow: a permutation of all
    reorder tiles whose last 65 * 4 entries are exactly the 128x128 tiles of the last 65 positions."""
    algo = _capi.find_algo(128, 128, swizzle=4)
    M = N = 8448
    order = _capi.schedule_order(algo, M, N)
    T = (M // 128) * (N // 128)
    assert sorted(order) == list(range(T))
    whole = _capi.schedule_order(_capi.find_algo(128, 128, swizzle=4), 8192, 8192)   # 1024 tiles: no tail
    assert sorted(whole) == list(range(64 * 64))
    # every group of four consecutive entries in the main part is one 256x256 tile
    tn = N // 128
    for i in range(0, (1089 - 65) * 4, 4):
        a, b, c, d = order[i:i + 4]
        assert b == a + 1 and c == a + tn and d == c + 1 and (a // tn) % 2 == 0 and (a % tn) % 2 == 0
    # 256x128 reorder tiles: two per position, tail cut in two
    order2 = _capi.schedule_order(_capi.find_algo(256, 128, swizzle=4), M, N)
    assert sorted(order2) == list(range((M // 256) * (N // 128)))


def test_cu_limit_is_accepted_and_keeps_the_hint_a_permutation():
    """fo_gemm_set_cu_limit (the reference's sm_count - 2, tune/search.py:404-407): 1024 workgroup tiles
    are four full waves on 256 CUs, and four waves of 248 plus a tail of 32 on 248 CUs.  The tail is
    walked in the Algo's own 128x128 tile, position by position, so the hint stays the raster's order
    of 256x256 blocks either way; what changes with the limit (wave sizes, resident workgroups) needs
    the GPU and is tested there."""
    L = _capi.lib()
    assert L.fo_gemm_set_cu_limit(4) == -1      # fewer than the 8 XCDs
    algo = _capi.find_algo(128, 128, swizzle=4)
    M = N = 8192
    full = _capi.schedule_order(algo, M, N)
    try:
        _capi.set_gemm_cu_limit(248)
        cut = _capi.schedule_order(algo, M, N)
        _capi.set_gemm_cu_limit(512)            # more than the device has: all of them
        assert _capi.schedule_order(algo, M, N) == full
    finally:
        _capi.set_gemm_cu_limit(0)
    assert _capi.schedule_order(algo, M, N) == full
    T = (M // 128) * (N // 128)
    tn = N // 128
    assert sorted(cut) == list(range(T))
    for i in range(0, T, 4):
        a, b, c, d = cut[i:i + 4]
        assert b == a + 1 and c == a + tn and d == c + 1


def test_argument_validation_without_gpu():
    L = _capi.lib()
    null = ctypes.c_void_p()
    one = ctypes.c_void_p(16)  # never dereferenced: validation fails first
    assert L.fo_gemm(0, 128, 128, 64, null, one, one, 0, null) == -1           # null A
    assert L.fo_gemm(0, 100, 128, 64, one, one, one, 0, null) == -2            # M % 128
    assert L.fo_gemm(0, 128, 128, 68, one, one, one, 0, null) == -2            # K % 8
    assert L.fo_gemm(0, 128, 128, 64, one, one, one, 102, null) == -3          # Algo range
    assert L.fo_gemm(7, 128, 128, 64, one, one, one, 0, null) == -4            # dtype
    assert L.fo_gemm_signal(0, 128, 128, 64, 1, one, 0, one, one, one, one, one, 0, 0, null) == -5
    # monitor mode keeps its order counter at MM[TN-1]: needs G <= TN-1
    assert L.fo_gemm_signal(0, 128, 128, 64, 1, one, 1, one, one, one, one, one, 1, 0, null) == -5
    assert L.fo_wait(1, null, null) == -1
    assert L.fo_consumer_reduce(0, one, one, 12, null) == -2                   # nelem % 8
    assert L.fo_reorder_rmsnorm(0, one, one, one, 8, 100, 4, 50, 1, one, 1e-5, null) == -2
    assert L.fo_overlap_gemm(null, 0, 128, 128, 64, one, one, one, 0) == -1
    h = ctypes.c_void_p()
    assert L.fo_overlap_create(ctypes.byref(h)) == 0
    assert L.fo_overlap_gemm(h, 0, 128, 128, 64, one, one, one, 0) == -6       # before cutlass_init
    assert L.fo_overlap_set_world(h, 2, 2) == -1
    assert L.fo_overlap_set_world(h, 1, 8) == 0
    assert L.fo_overlap_destroy(h) == 0
    assert b"Algo" in L.fo_error_string(-3)


@pytest.mark.parametrize("algo,M,N", [(0, 1024, 1024), (3, 4096, 4096), (57, 8192, 8192),
                                       (80, 8192, 8192), (5, 384, 640), (0, 128, 128)])
def test_schedule_order_is_a_permutation_with_local_waves(algo, M, N):
    order = _capi.schedule_order(algo, M, N)
    bm, bn = _capi.algo_tile(algo)
    TM, TN = M // bm, N // bn
    assert sorted(order) == list(range(TM * TN))
    # a workgroup covers `sub` reorder tiles when the 256x256 macro tile applies
    macro = M % 256 == 0 and N % 256 == 0 and (M // 256) * (N // 256) >= 128
    sub = (256 // bm) * (256 // bn) if macro else 1
    wgs = [order[i:i + sub] for i in range(0, len(order), sub)]
    if macro:
        for w in wgs:   # the tiles of one workgroup form one 256x256 block
            assert len({(t // TN) * bm // 256 for t in w}) == 1 and len({(t % TN) * bn // 256 for t in w}) == 1
    if len(wgs) >= 256 and len(wgs) % 8 == 0:
        # one wave of 256 workgroups: 32 consecutive raster positions per XCD, so each
        # XCD's share of the wave spans few distinct macro-tile rows/columns
        mt_m, mt_n = (256, 256) if macro else (bm, bn)
        for x in range(8):
            mine = [w[0] for w in wgs[:256][x::8]]
            rows = {(t // TN) * bm // mt_m for t in mine}
            cols = {(t % TN) * bn // mt_n for t in mine}
            assert len(rows) * len(cols) <= 64


@pytest.mark.parametrize("bm,bn,M,N", [(128, 256, 8192, 8192), (256, 128, 8192, 8192), (128, 128, 8192, 4096),
                                        (128, 128, 2048, 16384), (128, 128, 16384, 2048)])
def test_waves_of_the_persistent_launch_are_whole_tile_rows(bm, bn, M, N):
    """Where the 256x256 tiles are whole waves of 256 workgroups and a wave splits into eight power-of-two
    blocks, wave k of the schedule order is exactly the tile rows that follow wave k - 1's, each XCD
    (positions x, x + 8, ... of the wave) owning one block of 32 tiles with at most 12 operand panels."""
    algo = _capi.find_algo(bm, bn, swizzle=4)
    order = _capi.schedule_order(algo, M, N)
    TM, TN = M // bm, N // bn
    assert sorted(order) == list(range(TM * TN))
    sub = (256 // bm) * (256 // bn)
    gm, gn = M // 256, N // 256
    rows_per_wave = 256 // gn
    wgs = [order[i:i + sub] for i in range(0, len(order), sub)]
    macro = [((w[0] // TN) * bm // 256, (w[0] % TN) * bn // 256) for w in wgs]
    for k in range(gm * gn // 256):
        wave = macro[k * 256:(k + 1) * 256]
        assert sorted(wave) == [(k * rows_per_wave + i, j) for i in range(rows_per_wave) for j in range(gn)]
        for x in range(8):
            mine = wave[x::8]
            rows, cols = {m for m, _ in mine}, {n for _, n in mine}
            assert len(rows) * len(cols) == 32 and len(rows) + len(cols) <= 12
    # the reorder table built from this order stores wave k's tiles in the k-th stretch of slots:
    # every tile row's last slot lies in its own wave's stretch
    RA = layout.reorder_indices(TM * TN, order, device="cpu").reshape(TM, TN)
    per_wave = 256 * sub
    for tm in range(TM):
        assert int(RA[tm].max()) // per_wave == int(RA[tm].min()) // per_wave == (tm * bm // 256) // rows_per_wave
    # switched off: the panels of the Algo's swizzle, where a wave touches every tile row
    try:
        _capi.set_row_waves(False)
        panels = _capi.schedule_order(algo, M, N)
    finally:
        _capi.set_row_waves(True)
    assert sorted(panels) == list(range(TM * TN)) and _capi.schedule_order(algo, M, N) == order
    if gm > rows_per_wave and gm >= 32:
        first_wave_rows = {(w[0] // TN) * bm // 256 for w in [panels[i:i + sub] for i in range(0, 256 * sub, sub)]}
        assert first_wave_rows != set(range(rows_per_wave))


def test_row_waves_need_whole_waves_and_power_of_two_rows():
    """12288 columns are 48 tiles of 256 (no power of two), 8448^2 leaves a partial last wave: both keep the panels."""
    for bm, bn, M, N in ((128, 128, 4096, 12288), (128, 128, 8448, 8448)):
        algo = _capi.find_algo(bm, bn, swizzle=4)
        order = _capi.schedule_order(algo, M, N)
        try:
            _capi.set_row_waves(False)
            assert _capi.schedule_order(algo, M, N) == order
        finally:
            _capi.set_row_waves(True)


def test_latency_model_and_search_agree_with_checker(oracle):
    curve = np.array([[2.0 ** (20 + 0.25 * i), 0.5 + 0.1 * i] for i in range(36)])
    M = N = 8192
    tiles, wave = 2048, 256
    for gp in ([2048], [256] * 8, [512, 512, 1024], [256, 1792], [1000, 1048]):
        a = tune.predict_latency(M, N, 0.7, curve, gp, tiles, wave, 256)
        b = oracle.predict_latency(M, N, 0.7, curve[:, 0], curve[:, 1], gp, tiles, wave, 256, 6.0)
        assert a == pytest.approx(b, rel=1e-12)
    assert tune.integer_partitions(4) == oracle.compositions(4)
    assert tune.groups_to_cseg([1, 2, 1], 256, 1000) == [256, 512, 232]
    best, dur = tune.predictive_search(M, N, 0.7, curve, tiles, wave)
    assert sum(best) == tiles and all(c % wave == 0 for c in best[:-1])
    # exhaustive check of the argmin over the same candidate set
    cands = [tune.groups_to_cseg(gp, wave, tiles) for gp in tune.integer_partitions(8)
             if not (len(gp) > 5 and gp[0] > 2)]
    assert dur == pytest.approx(min(tune.predict_latency(M, N, 0.7, curve, c, tiles, wave) for c in cands))


def test_tuner_walks_down_the_gemm_candidates_until_a_hint_is_consistent():
    """tune/search.py:397-411 (exhaustive: 5 candidates) and :452-468 (predictive: 10, consistency asked in
    units of ceil(waves/10) waves): the first candidate whose monitor-mode hint is consistent is taken with
    that hint; if none is, the first candidate with the order its launch walks the tiles in."""
    M = N = 4096
    K = 512
    BMs, BNs = [128] * 12, [128] * 12
    algos = list(range(100, 112))
    asked = []

    def measure_ok_from(first_ok):
        def measure(algo, unit):
            asked.append((algo, unit))
            return algo >= first_ok, [algo]
        return measure

    kw = dict(wave_of=lambda algo: 256, order_of=lambda algo: ["walk", algo])
    # 1024 tiles, 4 waves of 256: exhaustive consistency unit = one wave
    t, hint, ok = tune.choose_candidate(M, N, K, BMs, BNs, algos, False, measure=measure_ok_from(103), **kw)
    assert (t, hint, ok) == (3, [103], True) and asked == [(100, 256), (101, 256), (102, 256), (103, 256)]
    asked.clear()
    t, hint, ok = tune.choose_candidate(M, N, K, BMs, BNs, algos, False, measure=measure_ok_from(105), **kw)
    assert (t, hint, ok) == (0, ["walk", 100], False) and len(asked) == 5      # only five are tried
    asked.clear()
    t, hint, ok = tune.choose_candidate(M, N, K, BMs, BNs, algos, True, measure=measure_ok_from(109), **kw)
    assert (t, hint, ok) == (9, [109], True) and len(asked) == 10
    asked.clear()
    t, hint, ok = tune.choose_candidate(M, N, K, BMs, BNs, algos, True, measure=measure_ok_from(110), **kw)
    assert (t, hint, ok) == (0, ["walk", 100], False) and len(asked) == 10     # only ten are tried
    # predictive unit: 40 waves of 26 tiles -> smallest group ceil(40 / 10) = 4 waves = 104 tiles
    asked.clear()
    tune.choose_candidate(M, N, K, BMs, BNs, algos, True, measure=measure_ok_from(100), wave_of=lambda a: 26,
                          order_of=kw["order_of"])
    assert asked == [(100, 104)]
    # a candidate that leaves monitor mode no counter for its order stamp is passed over:
    # 1024 tiles in waves of 16 = 64 groups > TN - 1 = 31; the next candidate (waves of 256) is measured
    asked.clear()
    t, _, ok = tune.choose_candidate(M, N, K, BMs, BNs, algos, False, measure=measure_ok_from(100),
                                     wave_of=lambda a: 16 if a == 100 else 256, order_of=kw["order_of"])
    assert (t, ok) == (1, True) and asked == [(101, 256)]


def test_config_json_two_stage_round_trip(tmp_path):
    assert config.gpu_tag("NVIDIA A800-SXM4-80GB") == "a800"      # the reference's slicing rule
    assert config.gpu_tag("AMD Instinct MI355X") == "tinc"
    d = str(tmp_path)
    p = config.save_gemm_candidates(4096, 4096, 512, [128, 128], [128, 256], [0.1, 0.2], [3, 57],
                                    gpu="tinc", directory=d)
    assert os.path.basename(p) == "m4096n4096k512_tinc.json"
    assert config.load_gemm_candidates(4096, 4096, 512, gpu="tinc", directory=d) == \
        ([128, 128], [128, 256], [0.1, 0.2], [3, 57])
    with pytest.raises(ValueError):
        config.load_solution(4096, 4096, 512, gpu="tinc", directory=d)
    config.save_solution(4096, 4096, 512, 128, 128, 0.1, 3, [1, 0], [512, 512], gpu="tinc", directory=d)
    sol = config.load_solution(4096, 4096, 512, gpu="tinc", directory=d)
    assert sol == {"BM": 128, "BN": 128, "dur": 0.1, "Algo": 3, "hint": [1, 0], "cSeg": [512, 512],
                   "rLDN": 1}


def test_layout_matches_checker_on_random_cases(oracle):
    rng = np.random.default_rng(3)
    for _ in range(10):
        BM, BN, W = int(rng.choice([4, 8])), int(rng.choice([8, 16])), int(rng.choice([1, 2, 4]))
        TM, TN = int(rng.integers(1, 6)), int(rng.integers(1, 6))
        T = TM * TN
        cuts = sorted(rng.choice(np.arange(1, T), size=min(T - 1, int(rng.integers(0, 4))), replace=False).tolist()) if T > 1 else []
        cseg = [b - a for a, b in zip([0] + cuts, cuts + [T])]
        got = layout.generate_row_mapping(TM * BM, TN * BN, BM, BN, cseg, W, device="cpu")
        assert got.tolist() == oracle.row_mapping(TM * BM, TN * BN, BM, BN, cseg, W).tolist()
        assert layout.tile_groups(cseg).tolist() == [oracle.tile_group(cseg, r) for r in range(T)]


def test_same_wave_groups_share_a_launch():
    plan = _capi.plan_batches
    # large square: 8 groups of 256 tiles, 512 tiles complete per wave -> pairs
    assert plan([256] * 8, 512) == [(0, 2), (2, 4), (4, 6), (6, 8)]
    # reduce-scatter layout: 1024 tiles per wave -> four groups per launch
    assert plan([256] * 8, 1024) == [(0, 4), (4, 8)]
    # a group that straddles a wave boundary completes with the later wave
    assert plan([300, 300, 300, 124], 512) == [(0, 1), (1, 4)]
    assert plan([300, 300, 500, 436], 512) == [(0, 1), (1, 2), (2, 4)]   # ends at 300, 600, 1100, 1536
    # groups of whole waves, and no batching without a wave size
    assert plan([512, 512, 1024], 512) == [(0, 1), (1, 2), (2, 3)]
    assert plan([4] * 6, 0) == [(i, i + 1) for i in range(6)]
    # one wave covers everything
    assert plan([1, 2, 3], 1000) == [(0, 3)]
    with pytest.raises(_capi.FlashOverlapError):
        plan([4, 0, 4], 8)


def _norm_rows_restated(RA, cseg, wave_tiles, max_runs=4):
    """The schedule of the normalisation, written down again from its description: behind every batch of
    groups, the tile rows all of whose storage slots lie in groups consumed so far, as maximal runs of
    consecutive rows in ascending order; a batch that is not the last takes at most max_runs runs."""
    TM = RA.shape[0]
    last = RA.max(axis=1)
    emitted = np.zeros(TM, dtype=bool)
    out, done = [], 0
    batches = _capi.plan_batches(cseg, wave_tiles)
    for b, (i, j) in enumerate(batches):
        done += sum(cseg[i:j])
        ready = [tm for tm in range(TM) if not emitted[tm] and last[tm] < done]
        runs = []
        for tm in ready:
            if runs and runs[-1][1] == tm:
                runs[-1][1] = tm + 1
            else:
                runs.append([tm, tm + 1])
        if b < len(batches) - 1:
            runs = runs[:max_runs]
        for f, e in runs:
            emitted[f:e] = True
            out.append((b, f, e))
    assert emitted.all()
    return out


def test_normalisation_follows_the_groups_that_complete_its_rows():
    """fo_overlap_plan_norm_rows (the planner fo_overlap_gemm_allreduce_norm enqueues from) against a restatement,
    on the large square's own tables, on scattered reorder tables and on random ones; every tile row is
    normalised exactly once and never before the batch that holds its last tile."""
    # the large square: 64 x 32 reorder tiles, 8 groups, waves of 512 tiles that cover 16 tile rows each
    algo = _capi.find_algo(128, 256, swizzle=4)
    M = N = 8192
    TM, TN = M // 128, N // 256
    hint = _capi.schedule_order(algo, M, N)
    RA = layout.reorder_indices(TM * TN, hint, device="cpu").reshape(TM, TN).numpy()
    cseg = [256] * 8
    wave = 512
    got = _capi.plan_norm_rows(RA, cseg, wave)
    assert got == [(0, 0, 16), (1, 16, 32), (2, 32, 48), (3, 48, 64)]
    assert got == _norm_rows_restated(RA, cseg, wave)
    # identity table, groups that cut through tile rows: a row is ready with the group that holds its last tile
    RA = np.arange(12, dtype=np.int32).reshape(4, 3)
    assert _capi.plan_norm_rows(RA, [4, 4, 4], 0) == [(0, 0, 1), (1, 1, 2), (2, 2, 4)]
    # every row has a tile in the last slot range: nothing before the last batch
    RA = np.array([[0, 11], [1, 10], [2, 9], [3, 8], [4, 7], [5, 6]], dtype=np.int32)
    assert _capi.plan_norm_rows(RA, [3, 3, 6], 0) == [(2, 0, 6)]
    # alternate rows complete early: six single-row runs, of which a batch that is not the last takes four
    RA = np.zeros((12, 2), dtype=np.int32)
    RA[0::2] = np.arange(12).reshape(6, 2)
    RA[1::2] = np.arange(12, 24).reshape(6, 2)
    got = _capi.plan_norm_rows(RA, [12, 12], 0)
    assert got == _norm_rows_restated(RA, [12, 12], 0)
    assert [r for r in got if r[0] == 0] == [(0, 0, 1), (0, 2, 3), (0, 4, 5), (0, 6, 7)]
    assert [r for r in got if r[0] == 1] == [(1, 1, 2), (1, 3, 4), (1, 5, 6), (1, 7, 12)]   # the last batch takes what is left
    rng = np.random.default_rng(11)
    for _ in range(60):
        TM, TN = int(rng.integers(1, 9)), int(rng.integers(1, 6))
        T = TM * TN
        RA = rng.permutation(T).astype(np.int32).reshape(TM, TN)
        if rng.random() < 0.5:            # tables that mostly follow the rows, as the schedule order does
            RA = np.sort(RA.reshape(-1)).reshape(TM, TN)[rng.permutation(TM)]
        cuts = sorted(rng.choice(np.arange(1, T), size=min(T - 1, int(rng.integers(0, 5))), replace=False).tolist()) if T > 1 else []
        cseg = [b - a for a, b in zip([0] + cuts, cuts + [T])]
        wave = int(rng.choice([0, 2, 5, T]))
        got = _capi.plan_norm_rows(RA, cseg, wave)
        assert got == _norm_rows_restated(RA, cseg, wave), (RA.tolist(), cseg, wave)
        covered = np.zeros(TM, dtype=int)
        ends = np.cumsum([sum(cseg[i:j]) for i, j in _capi.plan_batches(cseg, wave)])
        for b, f, e in got:
            covered[f:e] += 1
            assert RA[f:e].max() < ends[b]
        assert (covered == 1).all()
    with pytest.raises(_capi.FlashOverlapError):
        _capi.plan_norm_rows(np.array([[0, 5]], dtype=np.int32), [2], 0)      # an entry outside the table
    with pytest.raises(_capi.FlashOverlapError):
        _capi.plan_norm_rows(np.arange(4, dtype=np.int32).reshape(2, 2), [3], 0)  # groups do not cover the tiles


def test_front_ends_refuse_undersized_buffers():
    """MM, RA, RE and D are indexed through raw pointers by kernels that store and count through them;
    both front ends must refuse buffers that are too small before anything is launched.  The case the
    reference itself gets wrong: more groups than tile columns with MM sized TN (test/test.py:94)."""
    from flashoverlap_amd import ops
    i32 = lambda n: torch.zeros(n, dtype=torch.int32)
    algo = _capi.find_algo(128, 128)
    M, N = 512, 256                                   # 4 x 2 tiles
    ok = dict(M=M, N=N, algo=algo, rLDN=1, G=8, MM=i32(8), RA=i32(8))
    ops._check_signal_buffers(**ok)
    for bad, what in [(dict(MM=i32(2)), "MM holds 2"),           # sized TN although G = 8
                      (dict(MM=i32(9), monitor=True), "MM holds 9"),   # monitor needs (TM+1)*TN = 10
                      (dict(RA=i32(6)), "RA holds 6"),
                      (dict(rLDN=3), "rLDN"),
                      (dict(RE=i32(1023)), "RE holds 1023"),     # M*N/BN = 1024 rows
                      (dict(D=torch.zeros(100), W=4), "D holds 100"),
                      (dict(M=500), "not a multiple")]:
        with pytest.raises(ValueError, match=what):
            ops._check_signal_buffers(**{**ok, **bad})
    ops._check_signal_buffers(**{**ok, "RE": i32(1024), "D": torch.zeros(M * N // 4), "W": 4})
    with pytest.raises(ValueError, match="acc holds"):
        ops._check_rs(torch.zeros(64).half(), torch.zeros(3 * 100 + 15).half(), 4, 100)
    ops._check_rs(torch.zeros(64).half(), torch.zeros(3 * 100 + 16).half(), 4, 100)
    with pytest.raises(ValueError, match="own holds"):
        ops._check_rs(torch.zeros(64).half(), torch.zeros(400).half(), 4, 100, own=torch.zeros(8).half())
    with pytest.raises(TypeError):
        ops._check_rs(torch.zeros(64).half(), torch.zeros(400).bfloat16(), 4, 100)
    with pytest.raises(ValueError):
        ops._check_norm(torch.zeros(4, 64).half(), torch.zeros(4, 32).half(), torch.zeros(64).half())

    # the drop-in classes check the same things before they unpack a pointer (CPU tensors get that far)
    from flashoverlap_amd import layers
    layers.load_library()
    ov = torch.classes.flashoverlap_class.OverlapImpl()
    ov.nccl_init(0, 4, [0] * 16)
    A, B, C = torch.zeros(M, 64).half(), torch.zeros(N, 64).half(), torch.zeros(M, N).half()
    RA, cs = i32(8).reshape(4, 2), i32(8)
    with pytest.raises(RuntimeError, match="MM holds 2"):
        ov.gemm_allreduce_overlap(A, B, C, i32(2), RA, 1, cs, cs, algo, False)
    with pytest.raises(RuntimeError, match="MM holds 9"):
        ov.gemm_allreduce_overlap(A, B, C, i32(9), RA, 1, cs, cs, algo, True)
    with pytest.raises(RuntimeError, match="RA must be"):
        ov.gemm_allreduce_overlap(A, B, C, i32(8), RA.reshape(2, 4), 1, cs, cs, algo, False)
    with pytest.raises(RuntimeError, match="RE holds"):
        ov.gemm_reducescatter_overlap(A, B, C, torch.zeros(M // 4, N).half(), i32(8), RA, i32(100), 1, cs, cs, algo, False)
    with pytest.raises(RuntimeError, match="D holds"):
        ov.gemm_reducescatter_overlap(A, B, C, torch.zeros(M // 8, N).half(), i32(8), RA, i32(1024), 1, cs, cs, algo, False)
    with pytest.raises(RuntimeError, match="RA holds"):
        torch.ops.flashoverlap_op.reorder_rmsnorm(C, C.clone(), torch.zeros(N).half(), 128, 128, 1, i32(7))


def test_new_handle_calls_validate_without_gpu():
    L = _capi.lib()
    null = ctypes.c_void_p()
    one = ctypes.c_void_p(16)
    h = ctypes.c_void_p()
    assert L.fo_overlap_create(ctypes.byref(h)) == 0
    out = ctypes.c_int32(7)
    assert L.fo_overlap_status(h, ctypes.byref(out)) == 0 and out.value == 0    # nothing enqueued yet
    assert L.fo_overlap_status(h, null) == -1
    assert L.fo_overlap_set_wait_limit(h, -2) == -1 and L.fo_overlap_set_wait_limit(h, 1000) == 0
    assert L.fo_overlap_set_schedule(h, -1.0, -1) == 0
    assert L.fo_overlap_destroy(h) == 0
    assert b"4096" in L.fo_error_string(-7)
    # the allocation-free call validates before it touches a device: too many groups for its static counters
    assert L.fo_gemm_allreduce_overlap_static(0, 128, 128, 64, one, one, one, null, one, 1, 1, 1, one, one, 4097, 0,
                                              -1, null, null) == -7
    assert L.fo_gemm_allreduce_overlap_static(0, 128, 128, 64, one, one, one, null, one, 1, 1, 1, null, one, 1, 0,
                                              -1, null, null) == -5


def test_config1_checker_against_torch_cpu(oracle):
    """BASELINE configuration 1 on the CPU: fp16 1024^3, A and B N(0,1)/sqrt(K) from seed 0, fp32 accumulate,
    128x128 tiles, wave groups of 2 waves (a nominal wave of 8 tiles, so 16 tiles per group), reorder by
    group, then RMSNorm over N with eps 1e-6 and gamma = 1 + 0.01 N(0,1).  The checker's whole path
    (signal GEMM into the reordered buffer, counts, reorder+RMSNorm) against torch's CPU matmul and the
    RMSNorm of example/RMSNorm.py:13-18."""
    M = N = K = 1024
    bm = bn = 128
    g = torch.Generator().manual_seed(0)
    A16 = (torch.randn(M, K, generator=g) * K ** -0.5).half()
    B16 = (torch.randn(N, K, generator=g) * K ** -0.5).half()
    gamma = (1 + 0.01 * torch.randn(N, generator=g)).half()
    T = (M // bm) * (N // bn)
    cseg = layout.cseg_from_waves(T, 2 * 8)
    assert cseg == [16] * 4
    # a simulated completion order: waves of 8 tiles walking the columns of the tile grid first
    hint = [tm * (N // bn) + tn for tn in range(N // bn) for tm in range(M // bm)]
    ra = layout.reorder_indices(T, hint, device="cpu").numpy()
    bits = lambda t: t.contiguous().view(torch.int16).numpy().view(np.uint16)
    cp, mm = oracle.gemm_signal(oracle.F16, bits(A16), bits(B16), bm, bn, RA=ra, cseg=cseg)
    assert mm[:4].tolist() == cseg                                      # signal counts, bit-exact
    ref = A16.float() @ B16.float().T                                   # torch CPU, fp32 accumulate
    back = torch.from_numpy(oracle.from_bits(oracle.unpermute(cp, M, N, bm, bn, ra), oracle.F16)).reshape(M, N)
    rel = ((back - ref).abs() / ref.abs().clamp_min(ref.abs().mean())).max().item()
    assert rel <= 1e-2
    assert (back.half() == ref.half()).float().mean() > 0.99            # same fp32 sums up to summation order
    # every group's tiles are one contiguous run of the reordered buffer: group k = tile columns 2k, 2k+1
    C16 = back.half()
    run = torch.from_numpy(oracle.from_bits(cp, oracle.F16)).reshape(T, bm, bn)
    for k, t in enumerate(hint):
        tm, tn = divmod(t, N // bn)
        assert torch.equal(run[k].half(), C16[tm * bm:(tm + 1) * bm, tn * bn:(tn + 1) * bn])
    # reorder+RMSNorm of the reordered buffer against the reference formula on the row-major product
    y = oracle.from_bits(oracle.reorder_rmsnorm(oracle.F16, cp, bits(gamma), M, N, bm, bn, 1, ra, eps=1e-6), oracle.F16)
    x = C16.float()
    want = ((x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6)).half() * gamma).float()   # RMSNorm.py:13-18
    got = torch.from_numpy(y).reshape(M, N)
    rel = ((got - want).abs() / want.abs().clamp_min(want.abs().mean())).max().item()
    assert rel <= 1e-2
    assert (got == want).float().mean() > 0.98
