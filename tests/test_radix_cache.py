"""The prefix lookup (glake_amd/core/radix_cache.py; reference vmm_allocator/radix_cache.py:35-253) against what a
prefix tree must do, computed independently: the longest common prefix with any inserted key (brute force), split
points exactly where keys diverge, holders cut to the split length (on and inside chunk boundaries, through a
recording `split`), LRU eviction of unreferenced leaves, the flat store's take-over semantics."""
import random

import pytest

from glake_amd.core.radix_cache import RadixCache, match, radixDict

TOKEN = 2048             # bytes of one token row: 1024 rows per 2 MiB chunk


class Holder:
    """Stands in for a KV holder: remembers how many rows it covers and where it was cut from."""
    def __init__(self, rows, parent=None):
        self.rows, self.parent = rows, parent


def make_tree():
    cuts = []

    def split(value, nbytes):
        assert nbytes % TOKEN == 0
        cuts.append((value, nbytes // TOKEN))
        return Holder(nbytes // TOKEN, value)

    return RadixCache(TOKEN, split), cuts


def lcp_brute(keys, q):
    return max((match(k, q) for k in keys), default=0)


def test_match_is_the_longest_common_prefix_with_any_inserted_key():
    rng = random.Random(3)
    tree, _ = make_tree()
    keys = []
    for _ in range(200):
        base = list(rng.choice(keys)) if keys and rng.random() < 0.7 else []
        cut = rng.randint(0, len(base))
        key = tuple(base[:cut] + [rng.randint(0, 5) for _ in range(rng.randint(1, 30))])
        tree.insert(key, Holder(len(key)))
        keys.append(key)
        for _ in range(5):
            src = list(rng.choice(keys))
            q = tuple(src[:rng.randint(0, len(src))] + [rng.randint(0, 5) for _ in range(rng.randint(0, 8))])
            holder, n = tree.match_prefix(q)
            want = lcp_brute(keys, q)
            assert n == want
            if n:
                # the holder covers exactly the matched rows: it is a whole inserted key's holder or was cut to n
                assert holder.rows == n
            else:
                assert holder is None


def test_insert_reports_what_was_known_and_splits_where_keys_diverge():
    tree, cuts = make_tree()
    a = Holder(3000)
    assert tree.insert(tuple(range(3000)), a) == 0
    # same first 2500 tokens (inside the third chunk), then different ones
    b_key = tuple(range(2500)) + tuple(range(10000, 10500))
    b = Holder(3000)
    assert tree.insert(b_key, b) == 2500
    assert cuts == [(a, 2500)]                           # one holder cut from A's at the divergence
    # a prefix that ends exactly on a chunk boundary (1024 rows), by lookup
    holder, n = tree.match_prefix(tuple(range(1024)) + (-1, -2))
    assert n == 1024 and holder.rows == 1024 and cuts[-1][1] == 1024
    assert holder.parent.rows == 2500                    # cut from the 2500-row holder, the nearest one below
    # the whole of an inserted key: nothing is cut, its own holder answers
    before = len(cuts)
    assert tree.match_prefix(b_key) == (b, 3000) and len(cuts) == before
    assert tree.insert(b_key, Holder(3000)) == 3000 and tree.total_size() == 4   # A, B, the two cuts
    assert tree.match_prefix((77, 78)) == (None, 0)


def test_eviction_takes_unreferenced_leaves_least_recently_used_first():
    tree, _ = make_tree()
    keys = {name: tuple([i] * 10 + list(range(n))) for i, (name, n) in enumerate([("a", 5), ("b", 7), ("c", 9)])}
    holders = {name: Holder(len(k)) for name, k in keys.items()}
    for name in "abc":
        tree.insert(keys[name], holders[name])
    tree.match_prefix(keys["a"])                         # a is now the most recently used
    pinned = tree.match_node(keys["b"])
    tree.inc_ref_counter(pinned)                         # b is in use
    assert tree.evictable_size() == len(keys["a"]) + len(keys["c"])
    gone = []
    assert tree.evict(1, lambda v: (gone.append(v[0]), v[0].rows)[1]) == len(keys["c"])
    assert gone == [holders["c"]]                        # c: older than a, and b is pinned
    tree.evict(10 ** 6, lambda v: (gone.append(v[0]), v[0].rows)[1])
    assert gone == [holders["c"], holders["a"]] and tree.match_prefix(keys["b"]) == (holders["b"], len(keys["b"]))
    tree.dec_ref_counter(pinned)
    tree.evict(10 ** 6, lambda v: (gone.append(v[0]), v[0].rows)[1])
    assert gone[-1] is holders["b"] and tree.total_size() == 0 and tree.evictable_size() == 0


def test_a_split_node_inherits_the_references_and_inner_nodes_are_evicted_after_their_leaves():
    tree, _ = make_tree()
    long_key = tuple(range(40))
    tree.insert(long_key, Holder(40))
    node = tree.match_node(long_key)
    tree.inc_ref_counter(node)
    _, n = tree.match_prefix(tuple(range(25)) + (99,))   # splits the pinned edge at 25
    assert n == 25
    assert tree.evict(10 ** 6, lambda v: v[0].rows) == 0  # both halves are pinned
    tree.dec_ref_counter(node)
    order = []
    tree.evict(10 ** 6, lambda v: (order.append(v[0].rows), v[0].rows)[1])
    assert order == [40, 25]                             # the leaf first, then the node that became a leaf


def test_a_split_that_must_evict_for_room_spares_the_node_it_cuts():
    """The split callable of a full store evicts to get a holder.  The least recently used leaf may be the very
    node being cut: it must survive, and when nothing else can go the lookup fails with the tree unchanged."""
    tree = None
    budget = {"free": 0}

    def split(value, nbytes):
        if budget["free"] == 0:
            tree.evict(1, lambda v: (budget.__setitem__("free", budget["free"] + 1), v[0].rows)[1])
        if budget["free"] == 0:
            raise RuntimeError("no holder left")
        budget["free"] -= 1
        return Holder(nbytes // TOKEN, value)

    tree = RadixCache(TOKEN, split)
    old, young = tuple(range(30)), (7,) * 12
    tree.insert(old, Holder(30))                         # the least recently used leaf
    tree.insert(young, Holder(12))
    _, n = tree.match_prefix(old[:20] + (99,))           # cuts `old` at 20; room comes from evicting `young`
    assert n == 20 and tree.match_prefix(young) == (None, 0)
    assert tree.match_prefix(old)[1] == 30               # the node that was cut is still there
    leaf = tree.match_node(old)
    tree.inc_ref_counter(leaf)                           # the sequence is in use: nothing can be evicted now
    with pytest.raises(RuntimeError):
        tree.match_prefix(old[:10] + (98,))
    assert tree.match_prefix(old)[1] == 30 and tree.match_prefix(old[:20])[1] == 20 and tree.total_size() == 2
    assert leaf.ref_counter == 1 and leaf.parent.ref_counter == 1


def test_disabled_tree_matches_nothing():
    tree = RadixCache(TOKEN, lambda v, n: v, disable=True)
    assert tree.insert((1, 2, 3), Holder(3)) == 3 and tree.match_prefix((1, 2, 3)) == (None, 0)
    with pytest.raises(RuntimeError):
        tree.evict(1, lambda v: 0)


def test_flat_store_hands_a_slot_over_to_the_best_match():
    d = radixDict(TOKEN)
    assert d.match_prefix((1, 2)) == (None, 0) and d.get_free_slot() is None
    d.insert((1, 2, 3, 4), "slot0")
    d.insert((1, 2, 9), "slot1")
    d.insert((7, 7), "slot2")
    assert d.match_prefix((5, 5)) == (None, 0) and len(d.key) == 3        # nothing shared: nothing handed out
    assert d.match_prefix((1, 2, 3, 8)) == ("slot0", 3) and len(d.key) == 2
    assert d.match_prefix((1, 2, 3, 8)) == ("slot1", 2)                   # slot0 is gone: the next best
    assert d.get_free_slot() == "slot2" and d.get_free_slot() is None
