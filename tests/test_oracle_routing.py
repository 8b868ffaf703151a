"""The routing oracle against independent constructions (numpy stable argsort, counting)."""
import numpy as np
import pytest

from oracle import routing as oroute


@pytest.mark.parametrize("seed,pairs,experts,first,span", [(0, 0, 4, 0, 4), (1, 1, 1, 0, 1), (2, 777, 8, 16, 40), (3, 5000, 32, 0, 256),
                                                            (4, 3000, 1024, 0, 1024)])
def test_route_metadata_matches_argsort(seed, pairs, experts, first, span):
    rng = np.random.default_rng(seed)
    ids = rng.integers(0, span, size=pairs).astype(np.int32)
    ps, eo, bso, dst = oroute.route_metadata(ids, first, experts, 384, 512)
    local = (ids >= first) & (ids < first + experts)
    counts = np.bincount(ids[local] - first, minlength=experts)
    assert np.array_equal(ps[:, 0], counts) and (ps[:, 1] == 384).all() and (ps[:, 2] == 512).all()
    assert np.array_equal(eo, np.concatenate([[0], np.cumsum(counts)]))
    assert np.array_equal(bso, np.concatenate([[0], np.cumsum((counts + 127) // 128 * 128)]))
    assert (dst[~local] == -1).all()
    # the packed order is the stable sort of the local pairs by expert id
    order = np.flatnonzero(local)[np.argsort(ids[local], kind="stable")]
    assert np.array_equal(dst[order], np.arange(order.size))


def test_permute_rows_round_trip():
    rng = np.random.default_rng(5)
    topk, tokens, experts = 4, 50, 6
    ids = np.stack([rng.permutation(12)[:topk] for _ in range(tokens)]).astype(np.int32)   # some ids are not local
    x = rng.standard_normal((tokens, 8)).astype(np.float32)
    ps, eo, bso, dst = oroute.route_metadata(ids, 0, experts, 1, 1)
    packed = oroute.permute_rows(x, dst, topk, int(eo[-1]))
    assert not np.isnan(packed).any()
    for p, d in enumerate(dst):
        if d >= 0:
            e = ids.reshape(-1)[p]
            assert eo[e] <= d < eo[e + 1] and np.array_equal(packed[d], x[p // topk])
