"""Host-side work lists of the kernels (no GPU needed)."""
import random

import numpy as np
import pytest

from photon_infer_amd.ops.fast import (MAX_TILE_CUTS, AttentionPlanner, cut_count, deal_tiles, decode_length_bucket,
                                        decode_splits)


@pytest.mark.parametrize("seed", range(5))
def test_every_tile_is_dealt_exactly_once(seed):
    rng = random.Random(seed)
    walks = [rng.randint(1, 40) for _ in range(rng.randint(1, 300))]
    seats = rng.randint(1, 70)
    order = deal_tiles(walks, seats)
    assert order.shape[1] == seats and order.dtype == np.int32
    dealt = sorted(int(t) for t in order.reshape(-1) if t >= 0)
    assert dealt == list(range(len(walks)))


def test_the_deal_evens_out_the_work():
    # a causal prompt: tile i walks i + 1 key ranges
    walks = list(range(1, 129))
    order = deal_tiles(walks, 32)
    sums = [sum(walks[t] for t in order[:, seat] if t >= 0) for seat in range(32)]
    assert max(sums) - min(sums) <= 1
    # the first round holds the longest tiles
    assert sorted(walks[t] for t in order[0]) == list(range(97, 129))


def test_fewer_tiles_than_seats():
    order = deal_tiles([3, 9], 8)
    assert order.shape == (1, 8)
    assert list(order[0][:2]) == [1, 0] and all(t == -1 for t in order[0][2:])


def test_decode_splits_fill_the_chip_but_respect_short_contexts():
    assert decode_splits(64, 8, 4096) < decode_splits(8, 8, 4096) <= 32
    assert decode_splits(1, 8, max_kv_len=100) == 1
    assert decode_splits(1, 8, max_kv_len=4096) > 1
    # the same key ranges anywhere inside a length bucket: eager steps and graph replays agree
    assert decode_length_bucket(129) == decode_length_bucket(256) == 256
    assert decode_splits(4, 8, 1025) == decode_splits(4, 8, 2048)


def test_key_ranges_of_tiles_are_cut_only_when_the_tiles_are_few():
    assert cut_count([], 64) == 1
    assert cut_count([20] * 64, 64) == 1 and cut_count([20] * 33, 64) == 1      # enough tiles: none is cut
    assert cut_count([64] * 16, 64) == 4                                        # 16 tiles, 64 blocks wanted
    assert cut_count([64] * 2, 64) == MAX_TILE_CUTS
    assert cut_count([5] * 16, 64) == 1 and cut_count([7] * 2, 64) == 1         # a share keeps four rounds at least
    assert cut_count([12] * 4, 64) == 3
    assert cut_count([8] * 8, 64) == 1 and cut_count([9] * 16, 64) == 1         # ... and the cut saves six rounds or it is not made
    assert cut_count([16] * 16, 64) == 4
    assert cut_count([1] * 4, 64) == 1


@pytest.mark.parametrize("seed", range(6))
def test_a_step_plan_covers_every_token_of_every_portion_once(seed):
    """The planner of the prompt-attention kernel, on the host: tiles (or the shares of a cut tile)
    cover each token of each portion exactly once; requests with one token go to the other kernel
    when the planner says so; every entry is dealt to a block exactly once."""
    rng = random.Random(seed)
    R = rng.randint(1, 6)
    q_lens = [rng.choice([1, 1, 2, 17, 64, 65, 300]) for _ in range(R)]
    if all(n == 1 for n in q_lens):
        q_lens[0] = 40
    kv_lens = [n + rng.choice([0, 5, 700, 3000]) for n in q_lens]
    apart = seed % 2 == 0
    planner = AttentionPlanner(tile_rows=rng.choice([16, 32, 64]), window=rng.choice([0, 0, 100]), num_kv_heads=2,
                               singles_apart=apart, units=rng.choice([8, 256]))
    arrays, finish = planner.plan(q_lens, kv_lens)
    assert all(a.dtype == np.int32 for a in arrays.values())
    singles = [r for r, n in enumerate(q_lens) if n == 1] if apart else []
    assert arrays["singles"].tolist() == singles
    n = len(arrays["req"])
    assert len(arrays["q0"]) == len(arrays["cut"]) == len(arrays["z0"]) == n
    covered = {}
    for r, q0, cut in zip(arrays["req"].tolist(), arrays["q0"].tolist(), arrays["cut"].tolist()):
        share, shares = cut & 0xff, cut >> 8
        assert 0 <= share < shares and r not in singles
        covered.setdefault((r, q0), []).append((share, shares))
    for (r, q0), shares in covered.items():
        assert q0 % planner.tile_rows == 0 and q0 < q_lens[r]
        assert sorted(s for s, _ in shares) == list(range(shares[0][1]))          # every share of a cut tile, once
    for r, qn in enumerate(q_lens):
        if r not in singles:
            assert sorted(q0 for (rr, q0) in covered if rr == r) == list(range(0, qn, planner.tile_rows))
    dealt = sorted(t for t in arrays["order"].tolist() if t >= 0)
    assert dealt == list(range(n))
    # rows of the cut tiles: one entry per token of every cut tile
    cut_rows = sum(min(planner.tile_rows, q_lens[r] - q0) for (r, q0), sh in covered.items() if sh[0][1] > 1)
    assert len(arrays["rows"]) == cut_rows


def test_steps_of_single_tokens_need_no_plan_unless_the_tile_kernel_serves_them():
    assert AttentionPlanner(16, 0, 2, True, 256).plan([1, 1, 1], [5, 900, 17]) is None
    arrays, _ = AttentionPlanner(16, 0, 2, False, 256).plan([1, 1, 1], [5, 900, 17])
    assert arrays["req"].tolist()[:3] == [0, 1, 2] or sorted(set(arrays["req"].tolist())) == [0, 1, 2]
    assert arrays["singles"].size == 0


def test_pieces_that_would_not_fit_the_workspace_are_refused():
    """The kernels write a split product's pieces without knowing the buffer's size: the host
    refuses a request beyond it, and the split rules never make one."""
    from photon_infer_amd.errors import KernelError
    from photon_infer_amd.ops import fast
    from photon_infer_amd.ops.workspace import GEMM_PART_FLOATS, KernelWorkspace
    with pytest.raises(KernelError, match="workspace holds"):
        fast._piece_buffer(KernelWorkspace("cpu"), GEMM_PART_FLOATS + 1, "cpu")
    for M, N, K in [(2048, 2048, 8192), (2048, 3072, 8192), (2048, 4096, 14336), (8192, 4096, 14336), (4096, 8192, 28672),
                    (512, 4096, 14336), (100000, 128, 4096), (129, 128256, 2048)]:
        assert fast._tile_splits(M, N, K) * M * N <= GEMM_PART_FLOATS or fast._tile_splits(M, N, K) == 1
    for M, N, K in [(8, 128256, 2048), (128, 128256, 8192), (64, 16384, 2048), (1, 2048, 8192)]:
        assert fast._skinny_splits(M, N, K) * M * N <= GEMM_PART_FLOATS or fast._skinny_splits(M, N, K) == 1
