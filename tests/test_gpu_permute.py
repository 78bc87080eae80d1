"""Kernel 2 (histogram, prefix sum, stable permutation) against the oracle: everything bit-exact."""
import numpy as np
import pytest
import torch

from bibo_amd import ops
from oracle import bibo_moe_oracle as O

pytestmark = pytest.mark.gpu


def _check(idx_np, E):
    dev = torch.device("cuda:0")
    counts, offsets, perm_slot, perm_token = ops.permute(torch.from_numpy(idx_np).to(dev), E)
    torch.cuda.synchronize()
    oc, oo, ops_, opt = O.permute(idx_np, E)
    assert np.array_equal(counts.cpu().numpy(), oc)
    assert np.array_equal(offsets.cpu().numpy(), oo)
    assert np.array_equal(perm_slot.cpu().numpy(), ops_)
    assert np.array_equal(perm_token.cpu().numpy(), opt)


def _random_idx(T, E, k, seed):
    rng = np.random.default_rng(seed)
    scores = rng.random((T, E))
    return np.sort(np.argsort(scores, axis=1)[:, :k], axis=1).astype(np.int32)


@pytest.mark.parametrize("T,E,k", [(1, 4, 1), (3, 8, 2), (63, 64, 6), (64, 64, 6), (65, 64, 6), (512, 64, 6),
                                   (1000, 22, 2), (8192, 64, 6), (16384, 64, 6), (300, 64, 8), (129, 5, 5)])
def test_permutation_matches_oracle(T, E, k):
    _check(_random_idx(T, E, k, T + E + k), E)


@pytest.mark.parametrize("T,E,k", [(131072, 64, 6), (140001, 64, 6), (200000, 7, 2)])
def test_large_batches_take_the_block_sums(T, E, k):
    """From 1024 chunk histograms on (131072 tokens) a launch sums them in blocks of 256 and every scatter workgroup
    adds block sums plus the histograms of its own block; the permutation is the same, bit for bit."""
    _check(_random_idx(T, E, k, T + E), E)
    skew = _random_idx(T, E, k, 5)
    skew[: T // 2] = np.arange(k)                                       # half of the tokens on the first k experts
    _check(skew, E)


def test_empty_and_skewed_and_repeated():
    _check(np.zeros((0, 6), dtype=np.int32), 64)                       # no tokens: counts and offsets all zero
    idx = _random_idx(4096, 64, 6, 1)
    idx[:, :4] = np.arange(4)                                          # four hot experts take every token
    _check(np.sort(idx, axis=1), 64)
    _check(np.full((500, 2), 3, dtype=np.int32), 8)                    # one expert, repeated within a token
    only_last = np.full((200, 1), 63, dtype=np.int32)
    _check(only_last, 64)


def test_router_output_feeds_the_permutation():
    p = O.make_inputs(**O.CONFIGS["c1"])
    dev = torch.device("cuda:0")
    idx, _, _, _ = ops.router_fwd(p["x"].to(dev), p["w_router"].to(dev), p["bias"].to(dev), 6)
    counts, offsets, perm_slot, perm_token = ops.permute(idx, 64)
    idx_np = idx.cpu().numpy()
    oc, oo, ops_, opt = O.permute(idx_np, 64)
    assert np.array_equal(perm_slot.cpu().numpy(), ops_) and np.array_equal(counts.cpu().numpy(), oc)
    # size-independent properties
    ps = perm_slot.cpu().numpy()
    assert np.array_equal(np.sort(ps), np.arange(idx_np.size))
    assert (np.bincount(perm_token.cpu().numpy(), minlength=512) == 6).all()
    assert (np.diff(idx_np.reshape(-1)[ps]) >= 0).all()
