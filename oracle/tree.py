"""CPU oracle of the packed-tree log-prob gather.  TEST INFRASTRUCTURE ONLY.

Restates ``_gather_packed_tree_logprobs_entropy`` (areal/models/tree_attn/functional.py:320-400) without its
caches: per sequence, per node on its path, the internal predictions (position ``p`` predicts ``p + 1`` inside the
node, :135-146) followed by the transition from the node's last position to the first position of the next node,
or to position 0 after the last node (:300-310).
"""
from __future__ import annotations

import torch

from .logprobs import logprobs_entropy


def packed_tree_logprobs_entropy(logits, trie, input_ids, temperature: float = 1.0):
    input_ids = input_ids.reshape(-1)
    lps, ents = [], []
    for seq_id in trie.all_sequence_ids:
        indices = trie.get_sequence_tree_indices(seq_id)
        for i, (start, end) in enumerate(indices):
            if end - start > 0:                                                   # internal predictions
                lp, ent = logprobs_entropy(logits[start:end], input_ids[start + 1 : end + 1], temperature)
                lps.append(lp)
                ents.append(ent)
            next_start = indices[i + 1][0] if i + 1 < len(indices) else 0         # transition
            lp, ent = logprobs_entropy(logits[end : end + 1], input_ids[next_start : next_start + 1], temperature)
            lps.append(lp)
            ents.append(ent)
    if not lps:
        return torch.empty(0), torch.empty(0)
    return torch.cat(lps), torch.cat(ents)


def packed_tree_vocab_stats(logits, trie):
    """(vocab_min, vocab_max) concatenated over the sequences; functional.py:471-564: every position of every node
    on a sequence's path (inclusive ranges) contributes the extrema of its row."""
    mins, maxs = [], []
    for seq_id in trie.all_sequence_ids:
        for start, end in trie.get_sequence_tree_indices(seq_id):
            for p in range(start, end + 1):
                mins.append(logits[p].min().float())
                maxs.append(logits[p].max().float())
    if not mins:
        return torch.empty(0), torch.empty(0)
    return torch.stack(mins), torch.stack(maxs)


def merge_tree_results(results_list, batch_size, max_seq_len=None, padding_value=0.0):
    """functional.py:567-639, one element at a time."""
    combined = {}
    for results in results_list:
        for seq_id, tensor in results.items():
            if seq_id in combined:
                raise ValueError(f"Duplicate sequence_id {seq_id} found across microbatches")
            combined[seq_id] = tensor
    if not combined:
        return torch.full((batch_size, max_seq_len or 0), padding_value)
    first = next(iter(combined.values()))
    if max_seq_len is None:
        max_seq_len = max(t.shape[0] for t in combined.values())
    out = torch.full((batch_size, max_seq_len), padding_value, dtype=first.dtype)
    for seq_id, tensor in combined.items():
        if seq_id >= batch_size:
            raise ValueError(f"sequence_id {seq_id} exceeds batch_size {batch_size}")
        for j in range(min(tensor.shape[0], max_seq_len)):
            out[seq_id, j] = tensor[j]
    return out
