"""Host-side layout builders of the overlap path (integer, bit-exact contract).

Same names, argument meaning and results as the reference helpers in
example/utils.py:3-65 (duplicated there at test/test.py:23-69 and
tune/search.py:53-81, :237-253); the only interface change is that `device`
is an argument everywhere, so they also run where there is no GPU.
"""
import numpy as np
import torch


def div_up(x: int, y: int) -> int:
    return (x + y - 1) // y


def reorder_indices(S, hint, device="cuda"):
    """RA (flat, int32): original tile id -> storage slot.

    Tiles listed in `hint` take slots 0..len(hint)-1 in hint order; the others
    follow in ascending id order (example/utils.py:6-22).
    """
    hint = np.asarray(list(hint), dtype=np.int64)
    if hint.size and (hint.min() < 0 or hint.max() >= S):
        raise ValueError("hint entries must be tile ids in [0, S)")
    ra = np.full(S, -1, dtype=np.int64)
    ra[hint] = np.arange(hint.size)  # a repeated id keeps its last position, as list assignment does
    rest = np.ones(S, dtype=bool)
    rest[hint] = False
    ra[rest] = hint.size + np.arange(int(rest.sum()))
    return torch.from_numpy(ra.astype(np.int32)).to(device)


def cseg_from_waves(tile_num, wave_size):
    """Tiles per wave group; the last group takes the remainder (tune/search.py:88-94)."""
    if tile_num <= 0 or wave_size <= 0:
        raise ValueError("tile_num and wave_size must be positive")
    return [min(wave_size, tile_num - i * wave_size) for i in range(div_up(tile_num, wave_size))]


def generate_row_mapping(M, N, BM, BN, S_list, world_size, device="cuda"):
    """RE (int32, M*N/BN rows of the reshaped output): original row -> new row.

    Inside each group's row range the rows are stably sorted by row % world_size,
    so every group holds world_size contiguous chunks (example/utils.py:24-52).
    """
    total_tiles = (M * N) // (BM * BN)
    assert sum(S_list) == total_tiles, "sum(S_list) must equal total number of tiles"
    rows = np.arange(M * N // BN, dtype=np.int64)
    order = np.empty_like(rows)
    cur = 0
    for S in S_list:
        n = S * BM
        chunk = rows[cur:cur + n]
        order[cur:cur + n] = chunk[np.argsort(chunk % world_size, kind="stable")]
        cur += n
    remap = np.empty_like(rows)
    remap[order] = rows
    return torch.from_numpy(remap.astype(np.int32)).to(device)


def reorder_rows_by_world_size(tensor, world_size):
    """Rows of `tensor` stably sorted by row % world_size (example/utils.py:54-65)."""
    M = tensor.shape[0]
    idx = torch.argsort(torch.arange(M, device=tensor.device) % world_size, stable=True)
    return tensor[idx]


def tile_groups(cseg):
    """Group index of every storage slot: searchsorted(cumsum(cSeg), r, 'right')
    (the device scans the same prefix sums, src/overlap/gemm_with_signal.h:343-349)."""
    cs = np.cumsum(np.asarray(cseg, dtype=np.int64))
    return np.searchsorted(cs, np.arange(int(cs[-1])), side="right").astype(np.int32)


def counter_size(G, TM, TN, monitor=False):
    """Number of int32 the signal buffer MM needs.

    The reference allocates TN ints (test/test.py:94) or (TM+1)*TN in monitor
    mode (tune/search.py:112) and overruns when G > TN; size by max(G, TN).
    """
    return (TM + 1) * TN if monitor else max(G, TN)


def unpermute(Cp, M, N, BM, BN, RA, rLDN=1, RE=None):
    """Rebuild row-major [M, N] from the tile-reordered (optionally row-scattered)
    buffer; torch, any device.  Inverse of the signal GEMM's address map
    (src/overlap/gemm_with_signal.h:236-256, src/rmsnorm/rmsnorm.cuh:80-86)."""
    TM, TN = M // BM, N // BN
    ra = RA.reshape(-1).long()
    ldp = rLDN * BN
    Cp2 = Cp.reshape(-1, ldp)
    m = torch.arange(M, device=Cp.device)
    tn = torch.arange(TN, device=Cp.device)
    r = ra[(m[:, None] // BM) * TN + tn[None, :]]          # [M, TN]
    prow = (r // rLDN) * BM + (m % BM)[:, None]
    if RE is not None:
        prow = RE.long()[prow]
    pcol = (r % rLDN) * BN
    cols = pcol[:, :, None] + torch.arange(BN, device=Cp.device)[None, None, :]
    return Cp2[prow[:, :, None], cols].reshape(M, N)
