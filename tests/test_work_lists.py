"""Host-side work lists of the kernels (no GPU needed)."""
import random

import numpy as np
import pytest

from photon_infer_amd.ops.fast import MAX_TILE_CUTS, cut_count, deal_tiles, decode_length_bucket, decode_splits


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
    assert cut_count([5] * 16, 64) == 2                                         # a share keeps two rounds at least
    assert cut_count([1] * 4, 64) == 1
