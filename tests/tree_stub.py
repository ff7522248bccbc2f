"""A minimal stand-in for the reference's TrieNode (areal/models/tree_attn/tree.py): just the two members the
log-prob gather uses."""
import random


class Trie:
    def __init__(self, paths):
        self._paths = paths                       # seq_id -> list of inclusive (start, end) ranges
        self.all_sequence_ids = list(paths)

    def get_sequence_tree_indices(self, seq_id):
        return self._paths[seq_id]


def random_tree(n_seqs, seed, max_node=6, max_depth=5):
    """Random prefix tree laid out node after node: returns (trie, total packed length)."""
    rng = random.Random(seed)
    nodes = []                                    # (start, end, parent)
    pos = 0
    paths = {}
    for s in range(n_seqs):
        path = []
        parent = -1
        depth = rng.randint(1, max_depth)
        for _ in range(depth):
            children = [i for i, nd in enumerate(nodes) if nd[2] == parent]
            if children and rng.random() < 0.6:
                node = rng.choice(children)       # share an existing node
            else:
                length = rng.randint(1, max_node)
                nodes.append((pos, pos + length - 1, parent))
                pos += length
                node = len(nodes) - 1
            path.append(node)
            parent = node
        paths[s] = [(nodes[i][0], nodes[i][1]) for i in path]
    return Trie(paths), pos
