"""What the cache must hold, derived from the model's description (CPU): mixers say what they keep
per token (any named tensors, each with its own page shape) or per request; the plan groups them by
window, keys them by (run-order entry, mixer of the block) and follows ``cache_of``."""
import pytest
import torch

from photon_infer_amd.errors import ConfigError, UnsupportedModelError
from photon_infer_amd.parts import (PAGE, Block, KVCacheSpec, LMHead, Mixer, ModelSpec, PagedCacheSpec, PagedTensor, RunEntry,
                                    StateSpec, TokenEmbedding, plan_cache)
from photon_infer_amd.parts.norm import RMSNorm


class FakeMixer(Mixer):
    def __init__(self, need, own_kv=True):
        self.need, self.own_kv = need, own_kv

    def cache_spec(self):
        return self.need


class FakeBlock(Block):
    def __init__(self, *mixers):
        self._mixers = list(mixers)

    def mixers(self):
        return self._mixers


def spec_of(blocks, order=None):
    return ModelSpec(hidden_size=8, vocab_size=16, max_positions=32, embedding=("e.", TokenEmbedding(16, 8)),
                     layers=[(f"l{i}.", b) for i, b in enumerate(blocks)], final_norm=("n.", RMSNorm(8, 1e-5)),
                     head=("h.", LMHead(16, 8, tied=True)), run_order=order or [])


def test_page_shapes_and_bytes():
    k, v = KVCacheSpec(2, 16, None).tensors
    assert (k.name, k.page_shape(8)) == ("k", (2, 8, 16)) and (v.name, v.page_shape(8)) == ("v", (2, 16, 8))
    assert k.page_bytes(8, torch.bfloat16) == 2 * 8 * 16 * 2 and k.page_bytes(8, torch.float32) == 2 * 8 * 16 * 4
    latent = PagedTensor("latent", (PAGE, 24), torch.float32)
    assert latent.page_shape(4) == (4, 24) and latent.page_bytes(4, torch.bfloat16) == 4 * 24 * 4      # its own dtype wins
    for bad in ((3, 5), (PAGE, 2, PAGE)):
        with pytest.raises(UnsupportedModelError, match="page axis"):
            PagedTensor("x", bad).page_shape(4)


def test_groups_follow_the_windows_and_owners_are_keyed_by_entry_and_mixer():
    attn = lambda w: FakeMixer(KVCacheSpec(2, 16, w))
    latent = FakeMixer(PagedCacheSpec((PagedTensor("z", (PAGE, 5), torch.float32),), window=None))
    state = FakeMixer(StateSpec((7,), torch.float32))
    blocks = [FakeBlock(attn(None), latent), FakeBlock(attn(12)), FakeBlock(state, attn(12)), FakeBlock(FakeMixer(None))]
    plan = plan_cache(spec_of(blocks))
    assert [g.window for g in plan.groups] == [None, 12]
    assert plan.groups[0].owners == ((0, 0), (0, 1)) and plan.groups[1].owners == ((1, 0), (2, 1))
    assert [[t.name for t in owner] for owner in plan.groups[0].tensors] == [["k", "v"], ["z"]]
    assert [key for key, _ in plan.states] == [(2, 0)]
    assert plan.group_of == {(0, 0): 0, (0, 1): 0, (1, 0): 1, (2, 1): 1}
    assert (3, 0) not in plan.group_of and plan.owner_of[(3, 0)] == (3, 0)


def test_an_entry_may_read_an_earlier_entrys_caches_and_a_layer_may_run_twice():
    own = FakeBlock(FakeMixer(KVCacheSpec(1, 16, None)), FakeMixer(StateSpec((3,))))
    reader = FakeBlock(FakeMixer(KVCacheSpec(1, 16, None), own_kv=False), FakeMixer(StateSpec((3,))))
    plan = plan_cache(spec_of([own, reader], [RunEntry(0), RunEntry(1, cache_of=0), RunEntry(0)]))
    assert plan.groups[0].owners == ((0, 0), (2, 0))                       # the layer that runs twice owns two caches
    assert plan.owner_of[(1, 0)] == (0, 0) and plan.owner_of[(1, 1)] == (0, 1) and plan.group_of[(1, 0)] == 0
    assert [key for key, _ in plan.states] == [(0, 1), (2, 1)]
    with pytest.raises(ConfigError, match="must name the entry"):
        plan_cache(spec_of([own, reader], [RunEntry(0), RunEntry(1)]))
    with pytest.raises(ConfigError, match="not earlier"):
        spec_of([own, reader], [RunEntry(1, cache_of=1), RunEntry(0)])
    with pytest.raises(ConfigError, match="unknown cache spec"):
        plan_cache(spec_of([FakeBlock(FakeMixer("pages, please"))]))
