"""Host-side draft tree (struct-of-arrays) with the reference ``Tree`` interface.

Mirrors the public surface of the reference's ``specdecodes/models/utils/cpu_tree.py:32-324``
(``add_nodes`` :69, ``prune_to_depth`` :119, ``prune_to_top_n`` :175, ``find_child_index`` :232,
``get_tree_data`` :238, ``create_attention_mask`` :263) so generator code written against it keeps
working, but stores the tree as flat python lists and adds what the HIP kernels consume:
``ancestor_bits()`` (one bitset per node instead of an ``[n, n]`` boolean mask) and
``packed()`` (token / parent / depth arrays ready for a single host-to-device copy).

Nodes are kept in level order, so ``parent[i] < i`` for every non-root node.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch


class _NodeView:
    """Read/write view of one node; gives ``tree.nodes[i].children`` etc. (cpu_tree.py:3-29)."""

    __slots__ = ("_t", "_i")

    def __init__(self, tree: "Tree", index: int):
        self._t = tree
        self._i = index

    parent = property(lambda s: (None if s._t._parent[s._i] < 0 else s._t._parent[s._i]))
    children = property(lambda s: s._t._children[s._i])
    depth = property(lambda s: s._t._depth[s._i])
    token_id = property(lambda s: s._t._token[s._i])
    has_been_sampled = property(lambda s: s._t._sampled[s._i])

    @property
    def cumulative_probability(self):
        return self._t._prob[self._i]

    @cumulative_probability.setter
    def cumulative_probability(self, value):
        self._t._prob[self._i] = value

    def __repr__(self):
        return (f"TreeNode(token_id={self.token_id}, cumulative_probability="
                f"{self.cumulative_probability:.4f}, depth={self.depth}, parent={self.parent})")


class _NodeList:
    def __init__(self, tree: "Tree"):
        self._t = tree

    def __len__(self):
        return self._t.current_size

    def __getitem__(self, i):
        if isinstance(i, slice):
            return [_NodeView(self._t, j) for j in range(*i.indices(len(self)))]
        i = int(i)
        if i < 0:
            i += len(self)
        if not 0 <= i < len(self):
            raise IndexError(i)
        return _NodeView(self._t, i)

    def __iter__(self):
        return (_NodeView(self._t, j) for j in range(len(self)))


class Tree:
    def __init__(self, root_token_id, prob_dtype: torch.dtype = torch.float32):
        self.prob_dtype = prob_dtype
        root = int(root_token_id.item()) if hasattr(root_token_id, "item") else int(root_token_id)
        self._token: List[int] = [root]
        self._parent: List[int] = [-1]
        self._depth: List[int] = [0]
        self._prob: List[float] = [1.0]
        self._children: List[List[int]] = [[]]
        self._sampled: List[bool] = [False]
        self.available_leaves: List[int] = [0]

    # ------------------------------------------------------------------ basic accessors
    @property
    def current_size(self) -> int:
        return len(self._token)

    @property
    def nodes(self) -> _NodeList:
        return _NodeList(self)

    def size(self) -> int:
        return self.current_size

    def get_node(self, node_index: int) -> _NodeView:
        if node_index < 0 or node_index >= self.current_size:
            raise IndexError(f"Node index {node_index} out of bounds for tree size {self.current_size}.")
        return _NodeView(self, node_index)

    def get_depth(self) -> torch.Tensor:
        return torch.tensor(max(self._depth, default=0), dtype=torch.long)

    def get_children_indices(self, node_index) -> torch.Tensor:
        return torch.tensor(self._children[int(node_index)], dtype=torch.long)

    def get_children_ids(self, node_index) -> torch.Tensor:
        return torch.tensor([self._token[c] for c in self._children[int(node_index)]], dtype=torch.long)

    def find_child_index(self, node_index: int, match_token_id: int) -> int:
        for c in self._children[int(node_index)]:
            if self._token[c] == int(match_token_id):
                return c
        return -1

    # ------------------------------------------------------------------ growth
    def add_nodes(self, token_ids: torch.Tensor, token_probs: torch.Tensor,
                  local_parent_indices: torch.Tensor) -> None:
        """Append ``total_depth`` levels of ``num_samples`` nodes; inputs are ``[1, depth, k]``.
        ``local_parent_indices`` index into the previous level (cpu_tree.py:69-117)."""
        if token_ids.shape[0] != 1:
            raise AssertionError("Currently only batch_size=1 is supported.")
        toks = token_ids.detach().to("cpu").tolist()[0]
        prs = token_probs.detach().to("cpu").tolist()[0]
        pars = local_parent_indices.detach().to("cpu").tolist()[0]
        for lvl_tok, lvl_pr, lvl_par in zip(toks, prs, pars):
            for leaf in self.available_leaves:
                self._sampled[leaf] = True
            frontier = self.available_leaves
            first = self.current_size
            for j, (t, pr, lp) in enumerate(zip(lvl_tok, lvl_pr, lvl_par)):
                if not 0 <= lp < len(frontier):
                    raise ValueError(f"parent {lp} of a new node is not in the tree's frontier of {len(frontier)} nodes "
                                     "(it was cut off by truncate())")
                parent = frontier[lp]
                self._token.append(int(t))
                self._parent.append(parent)
                self._depth.append(self._depth[parent] + 1)
                self._prob.append(pr)
                self._children.append([])
                self._sampled.append(False)
                self._children[parent].append(first + j)
            self.available_leaves = list(range(first, self.current_size))

    # ------------------------------------------------------------------ pruning
    def _rebuild(self, keep: List[int]) -> None:
        """Keep nodes ``keep`` (old indices, in their new order) and re-index links."""
        new_of = {old: new for new, old in enumerate(keep)}
        token = [self._token[o] for o in keep]
        prob = [self._prob[o] for o in keep]
        depth = [self._depth[o] for o in keep]
        sampled = [self._sampled[o] for o in keep]
        parent = [new_of.get(self._parent[o], -1) if self._parent[o] >= 0 else -1 for o in keep]
        children = [[new_of[c] for c in self._children[o] if c in new_of] for o in keep]
        self._token, self._prob, self._depth, self._parent, self._children = token, prob, depth, parent, children
        # every node left without children becomes expandable again
        self._sampled = [s and bool(ch) for s, ch in zip(sampled, children)]
        self.available_leaves = [i for i, ch in enumerate(children) if not ch]

    def prune_to_depth(self, max_depth: int) -> torch.Tensor:
        """Drop nodes deeper than ``max_depth``; returns kept original indices (cpu_tree.py:119-173)."""
        if max_depth < 0:
            raise ValueError("max_depth must be >= 0")
        if self.current_size == 0:
            return torch.empty(0, dtype=torch.long)
        keep = [i for i, d in enumerate(self._depth) if d <= max_depth]
        if max_depth > max(self._depth) or len(keep) == self.current_size:
            return torch.arange(self.current_size)
        self._rebuild(keep)
        return torch.tensor(keep, dtype=torch.long)

    def prune_to_top_n(self, n: int) -> torch.Tensor:
        """Keep the ``n`` nodes of highest cumulative probability, in that order
        (cpu_tree.py:175-215)."""
        if n == -1 or self.current_size <= n:
            return torch.arange(self.current_size)
        probs = torch.tensor(self._prob, dtype=self.prob_dtype)
        keep = torch.topk(probs, k=n, sorted=True).indices.tolist()
        self._rebuild(keep)
        return torch.tensor(keep, dtype=torch.long)

    def truncate(self, n: int) -> torch.Tensor:
        """Keep the first ``n`` nodes (level order, so every kept node keeps its parent).  Used to cap
        the tree at ``max_verify_tokens``; the dropped nodes are the least probable of the last level."""
        if n >= self.current_size:
            return torch.arange(self.current_size)
        n = max(1, int(n))
        frontier = [i for i in self.available_leaves if i < n]
        self._rebuild(list(range(n)))
        # The frontier stays what it was, minus the nodes cut off, IN ITS ORDER: a level added later names its parents
        # by position in the previous level, and those positions must keep their meaning (a parent that was cut off
        # is refused by add_nodes).  Shallower nodes that lost all their children do not become expandable: when the
        # whole last level is cut off the frontier is empty, and a later add_nodes raises instead of re-parenting.
        self.available_leaves = frontier
        return torch.arange(self.current_size)

    # ------------------------------------------------------------------ export
    def get_tree_data(self, skip_nodes: int = 0) -> Dict[str, torch.Tensor]:
        s = int(skip_nodes)
        return {
            "token_ids": torch.tensor(self._token[s:], dtype=torch.long),
            "cumulative_probabilities": torch.tensor(self._prob[s:], dtype=self.prob_dtype),
            "depths": torch.tensor(self._depth[s:], dtype=torch.long),
            "parent_indices": torch.tensor(self._parent[s:], dtype=torch.long),
        }

    def ancestor_bits(self) -> List[int]:
        """Bit j of entry i is set iff node j is node i or one of its ancestors.  Python ints, so
        trees wider than 64 nodes are fine; the attention kernel takes them as 64-bit words."""
        bits: List[int] = []
        for i, p in enumerate(self._parent):
            bits.append((1 << i) | (bits[p] if p >= 0 else 0))
        return bits

    def create_attention_mask(self, prefix_length: int = 0, skip_nodes: int = 0, device="cpu") -> torch.Tensor:
        """Boolean ``[1, 1, n - skip_nodes, prefix_length + n]`` mask, True = may attend
        (cpu_tree.py:263-286)."""
        n = self.current_size
        if n == 0:
            return torch.empty((1, 1, 0, prefix_length), dtype=self.prob_dtype, device=device)
        bits = self.ancestor_bits()
        rows = [[True] * prefix_length + [bool((b >> j) & 1) for j in range(n)] for b in bits]
        mask = torch.tensor(rows, dtype=torch.bool, device=device)
        return mask[int(skip_nodes):, :].unsqueeze(0).unsqueeze(0)

    def packed(self, skip_nodes: int = 0) -> Dict[str, torch.Tensor]:
        """int32 token / parent / depth arrays of the whole tree for the device kernels."""
        return {
            "token_ids": torch.tensor(self._token, dtype=torch.int32),
            "parent_indices": torch.tensor(self._parent, dtype=torch.int32),
            "depths": torch.tensor(self._depth, dtype=torch.int32),
        }

    def __repr__(self):
        return f"Tree(num_nodes={self.current_size}, device='cpu')"
