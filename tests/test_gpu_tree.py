"""GPU parity of the packed-tree log-prob gather and of the (row, label) pair op behind it."""
import pytest
import torch

import areal_amd
from helpers import cosine
from oracle import tree as OT
from tree_stub import Trie, random_tree

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("V,dtype,temperature", [(97, torch.float32, 1.0), (1000, torch.bfloat16, 0.7),
                                                 (151936, torch.bfloat16, 1.0)])
def test_packed_tree_matches_oracle(device, V, dtype, temperature):
    trie, T = random_tree(9, seed=V % 7)
    g = torch.Generator().manual_seed(1)
    logits = (torch.randn(T, V, generator=g) * 3).to(dtype)
    ids = torch.randint(0, V, (T,), generator=g)
    w_lp, w_ent = OT.packed_tree_logprobs_entropy(logits, trie, ids, temperature)
    lp, ent = areal_amd.gather_packed_tree_logprobs_entropy(logits.to(device), trie, ids.to(device), temperature)
    assert lp.shape == w_lp.shape and lp.dtype == torch.float32
    assert float((lp.cpu() - w_lp).abs().max()) < 2e-3 and float((ent.cpu() - w_ent).abs().max()) < 2e-3
    assert float((lp.cpu() - w_lp).abs().max()) < 1e-4
    only = areal_amd.gather_packed_tree_logprobs(logits.to(device), trie, ids.to(device), temperature)
    assert torch.equal(only, lp)
    # batch dimension of 1 on the ids, as the engines pass them
    lp2, _ = areal_amd.gather_packed_tree_logprobs_entropy(logits.to(device), trie, ids.to(device)[None], temperature)
    assert torch.equal(lp2, lp)


def test_empty_trie_and_pair_flattening(device):
    logits = torch.randn(4, 8, device=device)
    lp, ent = areal_amd.gather_packed_tree_logprobs_entropy(logits, Trie({}), torch.zeros(4, dtype=torch.long))
    assert lp.numel() == 0 and ent.numel() == 0 and lp.dtype == torch.float32
    trie = Trie({0: [(0, 1), (2, 2), (4, 4)], 1: [(0, 1), (3, 3), (5, 5)]})
    pred, lab, sel = areal_amd.tree_sequence_pairs(trie)
    assert list(zip(pred, lab)) == [(0, 1), (1, 2), (2, 4), (4, 0), (1, 3), (3, 5), (5, 0)]   # (0, 1) shared
    assert sel == [0, 1, 2, 3, 0, 4, 5, 6]


@pytest.mark.parametrize("with_entropy", [False, True])
def test_pair_op_backward_matches_autograd(device, with_entropy):
    T, V, K = 40, 300, 90
    g = torch.Generator().manual_seed(4)
    logits = torch.randn(T, V, generator=g) * 2
    flat = torch.randperm(T * V, generator=g)[:K]          # distinct pairs, several per row
    rows, labels = flat // V, flat % V
    rows[:5] = 7                                           # one row predicting five tokens
    labels[:5] = torch.arange(5)
    gl, gh = torch.randn(K, generator=g), torch.randn(K, generator=g) * 0.3
    x = logits.clone().requires_grad_(True)
    ls = torch.log_softmax(x / 0.9, -1)
    ent_rows = -(ls.exp() * ls).sum(-1)
    ref = (ls[rows, labels] * gl).sum() + ((ent_rows[rows] * gh).sum() if with_entropy else 0.0)
    ref.backward()
    y = logits.to(device).requires_grad_(True)
    lp, ent = areal_amd.gather_logprobs_entropy_pairs(y, rows.to(device), labels.to(device), 0.9)
    obj = (lp * gl.to(device)).sum() + ((ent * gh.to(device)).sum() if with_entropy else 0.0)
    obj.backward()
    assert torch.allclose(lp.detach().cpu(), ls[rows, labels].detach(), atol=1e-5)
    assert torch.allclose(y.grad.cpu(), x.grad, atol=2e-6) and cosine(y.grad.cpu(), x.grad) > 0.999999
    bad = areal_amd.gather_logprobs_entropy_pairs(logits.to(device), torch.tensor([T, 0]), torch.tensor([0, V]))
    assert torch.isnan(bad[0]).all()                        # out of range: NaN, never a fault


@pytest.mark.parametrize("V,dtype", [(97, torch.float32), (151936, torch.bfloat16)])
def test_tree_vocab_stats_match_oracle(device, V, dtype):
    trie, T = random_tree(9, seed=3)
    g = torch.Generator().manual_seed(2)
    logits = (torch.randn(T, V, generator=g) * 3).to(dtype)
    w_min, w_max = OT.packed_tree_vocab_stats(logits, trie)
    vmin, vmax = areal_amd.gather_packed_tree_vocab_stats(logits.to(device), trie)
    assert vmin.dtype == torch.float32 and torch.equal(vmin.cpu(), w_min) and torch.equal(vmax.cpu(), w_max)
    e0, e1 = areal_amd.gather_packed_tree_vocab_stats(logits.to(device), Trie({}))
    assert e0.numel() == 0 and e1.numel() == 0 and e0.device.type == "cuda"


def test_merge_packed_tree_results_matches_oracle(device):
    g = torch.Generator().manual_seed(5)
    lens = {7: 13, 0: 1, 3: 300, 4: 0, 9: 64}
    cpu = {k: torch.randn(n, generator=g) for k, n in lens.items()}
    parts_cpu = [{k: cpu[k] for k in (7, 0)}, {k: cpu[k] for k in (3, 4, 9)}]
    parts = [{k: v.to(device) for k, v in d.items()} for d in parts_cpu]
    for kw in (dict(), dict(max_seq_len=40, padding_value=-2.5), dict(max_seq_len=512)):
        want = OT.merge_tree_results(parts_cpu, 10, **kw)
        got = areal_amd.merge_packed_tree_results(parts, 10, **kw)
        assert got.device.type == "cuda" and torch.equal(got.cpu(), want), kw
    ints = [{1: torch.arange(5, device=device)}, {0: torch.arange(3, device=device)}]
    got = areal_amd.merge_packed_tree_results(ints, 2)
    assert got.dtype == torch.int64 and got.tolist() == [[0, 1, 2, 0, 0], [0, 1, 2, 3, 4]]
    assert areal_amd.merge_packed_tree_results([], 3, 2).shape == (3, 2)
    with pytest.raises(ValueError, match="Duplicate sequence_id"):
        areal_amd.merge_packed_tree_results([parts[0], parts[0]], 10)
    with pytest.raises(ValueError, match="exceeds batch_size"):
        areal_amd.merge_packed_tree_results(parts, 8)
