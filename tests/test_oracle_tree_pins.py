"""Pins of oracle/tree.py: each sequence rebuilt from the tree and scored densely, and the docstring example of
areal/models/tree_attn/functional.py:262-275."""
import pytest
import torch

import oracle
from oracle import tree as OT
from tree_stub import Trie, random_tree


def _dense(logits, ids, trie, temperature):
    out = []
    for sid in trie.all_sequence_ids:
        pos = [p for (a, b) in trie.get_sequence_tree_indices(sid) for p in range(a, b + 1)]
        if not pos:
            continue
        labels = torch.tensor([int(ids[q]) for q in pos[1:]] + [int(ids[0])])    # the last token wraps to position 0
        out.append(oracle.logprobs_entropy(logits[pos], labels, temperature))
    return torch.cat([o[0] for o in out]), torch.cat([o[1] for o in out])


def test_docstring_example():
    # [A, B, C, D] and [A, B, E, F]: shared prefix at 0..1, C at 2, E at 3, D at 4, F at 5
    trie = Trie({0: [(0, 1), (2, 2), (4, 4)], 1: [(0, 1), (3, 3), (5, 5)]})
    g = torch.Generator().manual_seed(0)
    logits = torch.randn(6, 11, generator=g)
    ids = torch.tensor([1, 2, 3, 5, 4, 6])
    lp, ent = OT.packed_tree_logprobs_entropy(logits, trie, ids)
    ls = torch.log_softmax(logits, -1)
    want = [ls[0, 2], ls[1, 3], ls[2, 4], ls[4, 1], ls[0, 2], ls[1, 5], ls[3, 6], ls[5, 1]]
    assert torch.allclose(lp, torch.stack(want), atol=1e-6) and lp.shape == (8,) and ent.shape == (8,)


def test_random_trees_against_dense_scoring():
    for seed in range(4):
        trie, T = random_tree(7, seed)
        g = torch.Generator().manual_seed(seed)
        logits = torch.randn(T, 23, generator=g) * 2
        ids = torch.randint(0, 23, (T,), generator=g)
        lp, ent = OT.packed_tree_logprobs_entropy(logits, trie, ids, 0.8)
        w_lp, w_ent = _dense(logits, ids, trie, 0.8)
        assert torch.allclose(lp, w_lp, atol=1e-6) and torch.allclose(ent, w_ent, atol=1e-6)
    empty = Trie({})
    assert OT.packed_tree_logprobs_entropy(logits, empty, ids)[0].numel() == 0


def test_vocab_stats_and_merge_hand_cases():
    """No test of the reference covers functional.py:471-639 with values; pinned by a hand-built tree and rows."""
    from tree_stub import Trie

    # two sequences sharing node (0, 1); rows 0..4 with known extrema
    logits = torch.tensor([[0.0, 5.0, -1.0], [2.0, 2.0, 2.0], [-3.0, 0.0, 1.0], [9.0, 8.0, 7.0], [0.5, -0.5, 0.0]])
    trie = Trie({0: [(0, 1), (2, 2)], 1: [(0, 1), (3, 4)]})
    vmin, vmax = OT.packed_tree_vocab_stats(logits, trie)
    assert vmin.tolist() == [-1.0, 2.0, -3.0, -1.0, 2.0, 7.0, -0.5]
    assert vmax.tolist() == [5.0, 2.0, 1.0, 5.0, 2.0, 9.0, 0.5]
    e0, e1 = OT.packed_tree_vocab_stats(logits, Trie({}))
    assert e0.numel() == 0 and e1.numel() == 0
    # merge: rows by sequence id, cut and padded
    a = {2: torch.tensor([1.0, 2.0, 3.0])}
    b = {0: torch.tensor([4.0]), 3: torch.tensor([5.0, 6.0, 7.0, 8.0])}
    out = OT.merge_tree_results([a, b], 4)
    assert out.tolist() == [[4.0, 0, 0, 0], [0, 0, 0, 0], [1.0, 2.0, 3.0, 0], [5.0, 6.0, 7.0, 8.0]]
    out = OT.merge_tree_results([a, b], 5, max_seq_len=2, padding_value=-1.0)
    assert out.tolist() == [[4.0, -1.0], [-1.0, -1.0], [1.0, 2.0], [5.0, 6.0], [-1.0, -1.0]]
    assert OT.merge_tree_results([], 3, 2).shape == (3, 2) and OT.merge_tree_results([{}], 3).shape == (3, 0)
    with pytest.raises(ValueError, match="Duplicate sequence_id 2"):
        OT.merge_tree_results([a, a], 4)
    with pytest.raises(ValueError, match="exceeds batch_size"):
        OT.merge_tree_results([b], 3)
