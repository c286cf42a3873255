"""Prefix lookup for KV reuse: which cached sequence shares the longest token prefix with a new prompt.

Restates ``vmm_allocator/radix_cache.py`` of the reference: ``radixDict`` (:35-72), a flat list of finished
sequences' token ids searched linearly, and ``RadixCache`` (:74-253), a radix tree over token ids whose nodes own a
KV holder for the tokens from the root down to them.  A node's ``value[0]`` is whatever the caller stores for
"the KV of these ``prefix_len`` tokens" (a sequence slot, a ``KVcacheSegment``); the tree itself never touches the
GPU.  When a lookup or an insert ends inside an edge the node is split, and the upper half needs a holder of its
own for the shorter prefix: the reference calls ``vmmAllocator.split_and_copy(child.value[0], token_size *
prefix_len)`` there (:184), which its allocator never got; here the ``split`` callable given to the tree does it,
and the one this package provides (:class:`glake_amd.worker.prefix_store.PrefixStore`) starts a new slot with
``KVcacheSegment.share_prefix``: whole chunks of the prefix are mapped a second time, only the partly filled
chunk is copied.

Departures from the reference, all defects it could not have meant:
  * ``radixDict.match_prefix`` hands out (and removes) an entry only when it shares at least one token; the
    reference pops entry 0 when nothing matches (:46-58);
  * ``radixDict.get_free_slot`` returns the value it removes (the reference drops it, :66-72);
  * ``RadixCache.match_prefix`` returns ``(None, 0)`` when disabled (the reference returns a list and a node,
    which no caller can use like the enabled result, :88-90);
  * ``evict`` only counts nodes it really removed, subtracts an evicted edge's length from
    ``evictable_size`` only when it had been added, and ``insert`` of a key that ends on an existing node keeps
    the tree unchanged and reports the full length.
"""
from __future__ import annotations

import heapq
import itertools
from typing import Callable, Dict, List, Optional, Sequence, Tuple


def match(key: Sequence, seq: Sequence) -> int:
    """Length of the common prefix (radix_cache.py:27-33)."""
    i = 0
    for k, w in zip(key, seq):
        if k != w:
            break
        i += 1
    return i


class radixDict:
    """Flat prefix store (radix_cache.py:35-72): keys are token tuples, values whatever holds their KV (a slot).
    A match removes the entry: the new sequence takes the slot over and goes on behind the shared tokens."""

    def __init__(self, token_size: int):
        self.token_size = token_size
        self.key: List[Tuple] = []
        self.value: List = []

    def match_prefix(self, key: Sequence):
        if len(key) == 0 or len(self.key) == 0:
            return None, 0
        key = tuple(key)
        index, best = -1, 0
        for i, k in enumerate(self.key):
            n = match(k, key)
            if n > best:
                index, best = i, n
        if index < 0:
            return None, 0
        self.key.pop(index)
        return self.value.pop(index), best

    def insert(self, key: Sequence, value=None) -> int:
        self.key.append(tuple(key))
        self.value.append(value)
        return len(key)

    def get_free_slot(self):
        """Give up the newest entry so that its slot can serve a prompt that matched nothing."""
        if not self.key:
            return None
        self.key.pop()
        return self.value.pop()


class TreeNode:
    """radix_cache.py:14-24.  ``last_access_time`` is a logical clock (the reference uses wall time, which
    ties on fast machines)."""

    def __init__(self):
        self.children: Dict[Tuple, "TreeNode"] = {}
        self.parent: Optional["TreeNode"] = None
        self.value: List = []
        self.ref_counter = 0
        self.last_access_time = 0
        self.prefix_len = 0

    def __lt__(self, other: "TreeNode") -> bool:
        return self.last_access_time < other.last_access_time


class RadixCache:
    """Radix tree over token ids (radix_cache.py:74-253).

    ``split(value, nbytes)`` must return a holder of the first ``nbytes`` bytes of every range that ``value``
    holds (``nbytes = token_size * prefix_len``); it stands where the reference calls ``split_and_copy``."""

    def __init__(self, token_size: int, split: Callable[[object, int], object], disable: bool = False):
        self.root_node = TreeNode()
        self.root_node.ref_counter = 1
        self.evictable_size_ = 0
        self.token_size = token_size
        self.split = split
        self.disable = disable
        self._clock = itertools.count(1)

    # ------------------------------------------------------------------ public API
    def match_prefix(self, key: Sequence):
        """(holder, prefix_len) of the longest cached prefix of ``key``, (None, 0) if none.  A match that ends
        inside an edge splits it, so the holder covers exactly ``prefix_len`` tokens (:87-99)."""
        if self.disable:
            return None, 0
        last = self._match_prefix_helper(self.root_node, tuple(key), 0)
        if last is self.root_node:
            return None, 0
        return last.value[0], last.prefix_len

    def match_node(self, key: Sequence) -> TreeNode:
        """Like match_prefix, but returns the node (for inc_ref_counter / dec_ref_counter)."""
        return self.root_node if self.disable else self._match_prefix_helper(self.root_node, tuple(key), 0)

    def insert(self, key: Sequence, value=None) -> int:
        """Register ``value`` as the holder of all of ``key``; returns how many leading tokens were in the tree
        already (:101-107).  If the whole key is there, nothing changes and ``value`` is not taken."""
        if self.disable:
            return len(key)
        key = tuple(key)
        if value is None:
            value = list(key)
        return self._insert_helper(self.root_node, key, value, 0)

    def total_size(self) -> int:
        return self._total_size_helper(self.root_node)

    def evict(self, num_tokens: int, evict_callback: Callable[[List], int]) -> int:
        """Remove least recently used leaves nobody refers to until ``num_tokens`` tokens' worth has gone
        (``evict_callback(node.value)`` frees the holder and says how many, :116-137).  Returns the total."""
        if self.disable:
            raise RuntimeError("the prefix cache is disabled")
        leaves = self._collect_leaves()
        heapq.heapify(leaves)
        num_evicted = 0
        while num_evicted < num_tokens and leaves:
            x = heapq.heappop(leaves)
            if x is self.root_node:
                break
            if x.ref_counter > 0:
                continue
            num_evicted += evict_callback(x.value)
            self._delete_leaf(x)
            if len(x.parent.children) == 0:
                heapq.heappush(leaves, x.parent)
        return num_evicted

    def inc_ref_counter(self, node: TreeNode) -> int:
        delta = 0
        while node is not self.root_node:
            if node.ref_counter == 0:
                self.evictable_size_ -= self._edge_len(node)
                delta -= self._edge_len(node)
            node.ref_counter += 1
            node = node.parent
        return delta

    def dec_ref_counter(self, node: TreeNode) -> int:
        delta = 0
        while node is not self.root_node:
            if node.ref_counter == 1:
                self.evictable_size_ += self._edge_len(node)
                delta += self._edge_len(node)
            node.ref_counter -= 1
            node = node.parent
        return delta

    def evictable_size(self) -> int:
        """Tokens on edges whose nodes nobody refers to."""
        return self.evictable_size_

    # ------------------------------------------------------------------ helpers
    @staticmethod
    def _edge_len(node: TreeNode) -> int:
        return node.prefix_len - (node.parent.prefix_len if node.parent is not None else 0)

    def _touch(self, node: TreeNode) -> None:
        node.last_access_time = next(self._clock)

    def _match_prefix_helper(self, node: TreeNode, key: Tuple, p_len: int) -> TreeNode:
        self._touch(node)
        for c_key, child in list(node.children.items()):
            n = match(c_key, key)
            if n == 0:
                continue
            if n < len(c_key):
                new_node = self._split_node(c_key, child, n, p_len + n)
                self._touch(new_node)
                return new_node
            return self._match_prefix_helper(child, key[n:], p_len + n)
        return node

    def _split_node(self, key: Tuple, child: TreeNode, split_len: int, p_len: int) -> TreeNode:
        """parent -[key]-> child  becomes  parent -[key[:split_len]]-> new_node -[key[split_len:]]-> child
        (:177-188); the new node's holder is cut from the child's."""
        new_node = TreeNode()
        new_node.children = {key[split_len:]: child}
        new_node.parent = child.parent
        new_node.ref_counter = child.ref_counter
        new_node.prefix_len = p_len
        new_node.last_access_time = child.last_access_time
        # the callable may evict to make room for the new holder: not the node it is cutting from, nor its
        # ancestors (a raise leaves the tree as it was)
        child.ref_counter += 1
        try:
            new_node.value.append(self.split(child.value[0], self.token_size * p_len))
        finally:
            child.ref_counter -= 1
        child.parent = new_node
        del new_node.parent.children[key]
        new_node.parent.children[key[:split_len]] = new_node
        return new_node

    def _insert_helper(self, node: TreeNode, key: Tuple, value, p_len: int) -> int:
        self._touch(node)
        for c_key, child in list(node.children.items()):
            n = match(c_key, key)
            if n == len(c_key):
                if n == len(key):
                    self._touch(child)
                    return n
                return n + self._insert_helper(child, key[n:], value, p_len + n)
            if n:
                new_node = self._split_node(c_key, child, n, p_len + n)
                return n + self._insert_helper(new_node, key[n:], value, p_len + n)
        if len(key):
            new_node = TreeNode()
            new_node.parent = node
            new_node.value.append(value)
            new_node.prefix_len = p_len + len(key)
            self._touch(new_node)
            node.children[key] = new_node
            self.evictable_size_ += len(key)
        return 0

    def _delete_leaf(self, node: TreeNode) -> None:
        for k, v in node.parent.children.items():
            if v is node:
                break
        del node.parent.children[k]
        self.evictable_size_ -= len(k)

    def _total_size_helper(self, node: TreeNode) -> int:
        return len(node.value) + sum(self._total_size_helper(c) for c in node.children.values())

    def _collect_leaves(self) -> List[TreeNode]:
        out: List[TreeNode] = []

        def dfs(cur: TreeNode) -> None:
            if not cur.children:
                out.append(cur)
            for x in cur.children.values():
                dfs(x)

        dfs(self.root_node)
        return out
