"""Micro-batch allocation and split (host logic, runs without a GPU): the product's first-fit-decreasing and
Karmarkar-Karp allocators against the oracle's brute-force restatement, the known answers and the properties of the
reference's tests (tests/test_seqpack.py:412-455, tests/test_kk_allocate.py:163-340)."""
import random

import numpy as np
import pytest
import torch

from areal_amd import microbatch as M
from oracle import microbatch as OM


def _sums(values, groups):
    return [sum(values[i] for i in g) for g in groups]


# ---- pins of the oracle: known answers and closed cases ---------------------------------------------------------
def test_oracle_known_answers():
    # the input of the docstring example of kk_allocate (seqpack.py:491-492; the grouping printed there, 400 / 600,
    # is not what the differencing method returns) traced by hand through seqpack.py:337-381: 300 and 250 pair up
    # (spread 50), then 200 and 150 (50); 100 joins the 250 of the pair with the heavier first set; the two
    # remaining solutions merge heaviest with lightest into 500 {0, 4, 3} and 500 {2, 1}, the longer set first
    assert OM.kk_allocate([100, 200, 300, 150, 250], capacity=500, min_groups=2) == [[0, 4, 3], [2, 1]]
    # tests/test_kk_allocate.py:215-220: {1, 4} and {2, 3}
    assert sorted(_sums([1, 2, 3, 4], OM.kk_partition([1, 2, 3, 4], 2))) == [5, 5]
    # :173-177 perfect partition; :179-183 one group
    assert len(set(_sums([10] * 4, OM.kk_partition([10] * 4, 2)))) == 1
    assert sorted(OM.kk_partition([5, 3, 2], 1)[0]) == [0, 1, 2]
    # :204-213 equal sizes
    parts = OM.kk_partition(list(range(1, 13)), 4, equal_size=True)
    assert [len(p) for p in parts] == [3] * 4 and sorted(sum(parts, [])) == list(range(12))
    # first fit decreasing worked by hand: 9 | 8 | 7 open three groups (min_groups 3); 3 fits everywhere and joins the
    # lightest of the one-member groups (7); 2 joins the lightest group with one member (8); 1 joins the 9
    assert OM.ffd_once(np.array([9, 8, 7, 3, 2, 1]), 12, 3) == [[0, 5], [1, 4], [2, 3]]
    # capacity forces new groups: 6, 6, 5, 5 with capacity 10, one group asked for
    assert sorted(map(sorted, OM.ffd_allocate([6, 6, 5, 5], 10, 1))) == [[0], [1], [2, 3]]
    # divisor: three groups needed, a multiple of 2 wanted
    assert len(OM.ffd_allocate([6, 6, 5, 5, 1, 1], 10, 1, 2)) % 2 == 0
    with pytest.raises(RuntimeError):
        OM.ffd_allocate([11], 10, 1)
    with pytest.raises(RuntimeError):
        OM.kk_allocate([1, 2], 10, 3)


def test_oracle_properties_from_the_reference_tests():
    for seed in range(40):                                   # tests/test_kk_allocate.py:343-373
        rng = random.Random(seed)
        n = rng.randint(10, 60)
        k = rng.randint(2, min(8, n))
        values = [rng.randint(1, 500) for _ in range(n)]
        parts = OM.kk_partition(values, k)
        assert sorted(sum(parts, [])) == list(range(n)) and sum(_sums(values, parts)) == sum(values)
    rng = random.Random(123)                                 # :193-202 balance quality
    values = [rng.randint(1, 1000) for _ in range(50)]
    s = _sums(values, OM.kk_partition(values, 4))
    assert max(s) - min(s) < sum(values) / 4 * 0.2
    values = [rng.randint(1, 100) for _ in range(30)]        # tests/test_seqpack.py:416-431
    groups = OM.ffd_allocate(values, 300, 3)
    assert len(groups) >= 3 and sorted(int(i) for g in groups for i in g) == list(range(30))
    assert all(t <= 300 for t in _sums(values, groups))


# ---- the product against the oracle --------------------------------------------------------------------------------
@pytest.mark.parametrize("seed", range(60))
def test_allocators_equal_oracle(seed):
    rng = random.Random(seed)
    n = rng.randint(1, 70)
    dist = rng.choice(["uniform", "ties", "bimodal", "skewed"])
    if dist == "uniform":
        values = [rng.randint(1, 4096) for _ in range(n)]
    elif dist == "ties":
        values = [rng.choice([128, 256, 512]) for _ in range(n)]
    elif dist == "bimodal":
        values = [rng.randint(50, 200) if rng.random() < 0.5 else rng.randint(3000, 4096) for _ in range(n)]
    else:
        values = [int(min(4096, rng.expovariate(1 / 300) + 1)) for _ in range(n)]
    capacity = rng.choice([4096, 8192, 20000, int(1e12)])
    min_groups = rng.randint(1, max(1, min(n, 6)))
    divisor = rng.choice([1, 1, 2, 4])
    for name, mine, theirs in (("ffd", M.ffd_allocate, OM.ffd_allocate), ("kk", M.kk_allocate, OM.kk_allocate)):
        try:
            want = theirs(list(values), capacity, min_groups, divisor)
        except RuntimeError:
            with pytest.raises(RuntimeError):
                mine(list(values), capacity, min_groups, divisor)
            continue
        got = mine(list(values), capacity, min_groups, divisor)
        assert [[int(i) for i in g] for g in got] == [[int(i) for i in g] for g in want], (name, values, capacity)
        assert all(t <= capacity for t in _sums(values, got))
        if name == "ffd":      # KK caps the number of groups by the number of values after rounding up to the divisor
            assert len(got) % divisor == 0
    if n % 2 == 0 and n >= 2:
        assert M.kk_allocate(values, int(1e12), 2, equal_size=True) == OM.kk_allocate(values, int(1e12), 2, equal_size=True)


def test_product_known_answers_and_errors():
    assert M.kk_allocate([100, 200, 300, 150, 250], capacity=500, min_groups=2) == [[0, 4, 3], [2, 1]]
    assert [[int(i) for i in g] for g in M.ffd_allocate([9, 8, 7, 3, 2, 1], 12, 3)] == [[0, 5], [1, 4], [2, 3]]
    with pytest.raises(RuntimeError, match="larger than capacity"):
        M.ffd_allocate([11], 10, 1)
    with pytest.raises(RuntimeError, match="smaller than min_groups"):
        M.kk_allocate([1, 2], 10, 3)
    with pytest.raises(RuntimeError, match="equal_size=True requires"):
        M.kk_allocate([1, 2, 3, 4, 5], int(1e12), 3, equal_size=True)
    with pytest.raises(ValueError, match="Unknown packing algorithm"):
        M.get_allocate_fn("best")
    with pytest.raises(ValueError, match="packing_algorithm must be one of"):
        M.MicroBatchSpec(packing_algorithm="best")
    assert M.get_allocate_fn() is M.ffd_allocate and M.get_allocate_fn("kk") is M.kk_allocate
    spec = M.MicroBatchSpec.new(M.MicroBatchSpec(n_mbs=2, max_tokens_per_mb=100), n_mbs=4)
    assert (spec.n_mbs, spec.max_tokens_per_mb, spec.packing_algorithm) == (4, 100, "ffd")
    # a KK result over the capacity falls back to first fit decreasing (tests/test_kk_allocate.py:311-324)
    values = [6, 6, 5, 5]
    assert M.kk_allocate(values, 10, 1) == OM.kk_allocate(values, 10, 1)
    assert all(t <= 10 for t in _sums(values, M.kk_allocate(values, 10, 1)))


@pytest.mark.parametrize("algorithm", ["ffd", "kk"])
@pytest.mark.parametrize("granularity", [1, 2])
def test_split_equals_oracle_on_cpu_tensors(algorithm, granularity):
    g = torch.Generator().manual_seed(3)
    bs, L = 12, 40
    lens = torch.randint(1, L + 1, (bs,), generator=g)
    attn = (torch.arange(L)[None, :] < lens[:, None]).long()
    data = dict(attention_mask=attn, input_ids=torch.randint(0, 99, (bs, L), generator=g),
                logprobs=torch.randn(bs, L, generator=g), rewards=torch.randn(bs, generator=g), tag="x")
    data = M.amend_position_ids(data)
    assert torch.equal(data["position_ids"][3], torch.arange(L))
    spec = M.MicroBatchSpec(n_mbs=2, granularity=granularity, max_tokens_per_mb=150, packing_algorithm=algorithm)
    got = M.split_padded_tensor_dict_into_mb_list(data, spec)
    mbs, group_lens, fwd, bwd = OM.split_padded_tensor_dict(data, 150, 2, granularity, 1, algorithm)
    assert got.group_lens == group_lens and [int(i) for i in got.forward_indices] == fwd and got.backward_indices == bwd
    assert len(got) == len(mbs) and all(t <= 150 for t in group_lens)
    for a, b in zip(got.mbs, mbs):
        assert sorted(a) == sorted(b)
        for key in a:
            if torch.is_tensor(a[key]):
                assert torch.equal(a[key], b[key]), key
            else:
                assert a[key] == b[key]
    # rows come back in the original order through backward_indices (tests/test_utils.py:40-75 checks this round trip)
    cat = torch.cat([mb["input_ids"] for mb in got.mbs])
    assert torch.equal(cat[torch.tensor(got.backward_indices)], data["input_ids"])
    with pytest.raises(ValueError, match="attention_mask"):
        M.split_padded_tensor_dict_into_mb_list(dict(input_ids=data["input_ids"]), spec)
    with pytest.raises(RuntimeError, match="cannot divide granularity"):
        M.split_padded_tensor_dict_into_mb_list(data, M.MicroBatchSpec(granularity=5))
    with pytest.raises(ValueError, match="Call pad_mb_list first"):
        iter(got).__next__()


def test_mb_list_to_moves_every_tensor():
    attn = (torch.arange(6)[None, :] < torch.tensor([[6], [3], [2], [5]])).long()
    data = dict(attention_mask=attn, input_ids=torch.arange(24).view(4, 6), meta=dict(w=torch.ones(2)), tag="x")
    mbl = M.split_padded_tensor_dict_into_mb_list(data, M.MicroBatchSpec(n_mbs=2))
    moved = mbl.to(torch.float64)
    assert moved.mbs[0]["input_ids"].dtype == torch.float64 and moved.data["meta"]["w"].dtype == torch.float64
    assert moved.mbs[0]["tag"] == "x" and moved.forward_indices == mbl.forward_indices
    assert mbl.mbs[0]["input_ids"].dtype == torch.int64          # the original is untouched
