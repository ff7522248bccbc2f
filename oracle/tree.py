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
