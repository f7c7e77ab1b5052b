"""Prefix page cache and per-sequence page lists.

The reference's own cases for these functions
(dev/tests/engine/kv_page_cache_test.cpp:86-220: exact chained blocks and
physical ownership, deterministic LRU leaf order, recency an exposed parent
inherits, input validation) run against BOTH the oracle (oracle/prefix_oracle.py
over the oracle's page pool) and the product (libkvx over accounting-only
storage, no GPU needed); a seeded random walk then drives the two in lockstep
and compares every answer, every page list and the pool counters.
"""
import ctypes as C
import random

import numpy as np
import pytest

from oracle import kvoracle as ko
from oracle import prefix_oracle as po
from richengine_amd import kvx

KL = ko.lib()
NO_LIMIT = 0xFFFFFFFF


def page(seed):
    """A full page of tokens (the reference's tests use seed + index)."""
    return [seed * 1000 + i for i in range(32)]


# ---- the two stacks behind one interface --------------------------------------

class OraclePool:
    def __init__(self, pages, extent_pages, runway):
        self.h = KL.ko_pool_create(pages, 100, extent_pages, runway, NO_LIMIT)
        assert self.h
        self.pages, self.extent_pages = pages, extent_pages

    def acquire(self, count):
        out = np.zeros(max(count, 1), dtype=np.uint32)
        rc = KL.ko_pool_acquire(self.h, count, ko.ptr(out))
        if rc != count:
            raise po.OracleError("nomem")
        return [int(p) for p in out[:count]]

    def retain(self, page_id, prefix_owner):
        if page_id >= self.pages:
            raise po.OracleError("range")
        if KL.ko_pool_retain(self.h, page_id, int(prefix_owner)):
            raise po.OracleError("state")

    def release(self, page_id, prefix_owner):
        if KL.ko_pool_release(self.h, page_id, int(prefix_owner)):
            raise po.OracleError("state")

    def snapshot(self):
        s = ko.PoolSnapshot()
        KL.ko_pool_snapshot_get(self.h, C.byref(s))
        return (s.pages_allocated, s.pages_free, s.pages_active, s.pages_prefix)

    def compact(self):
        first, n = C.c_uint32(), C.c_uint32()
        dest = np.zeros(self.extent_pages, dtype=np.uint32)
        copies = (ko.PageCopy * self.extent_pages)()
        moved = KL.ko_pool_compact_extent(self.h, None, 0, C.byref(first), ko.ptr(dest), copies,
                                          C.byref(n))
        return (first.value, [int(d) for d in dest]) if moved > 0 else None


class OracleStack:
    name = "oracle"

    def __init__(self, pages, extent_pages=4, runway=None):
        self.pool = OraclePool(pages, extent_pages, pages if runway is None else runway)
        self.prefix = po.PrefixCache(self.pool, pages)
        self.sequences = po.SequenceCache(self.pool, self.prefix, self.pool.acquire)

    def call(self, f, *args):
        try:
            return "ok", f(*args)
        except po.OracleError as e:
            return e.kind, None

    # pool
    def acquire(self, n): return self.call(self.pool.acquire, n)
    def release_page(self, p): return self.call(self.pool.release, p, False)
    def pool_counts(self): return self.pool.snapshot()
    # prefix
    def find(self, parent, tokens, images=(0, 0)): return self.prefix.find(parent, tokens, images)
    def insert(self, parent, tokens, p, images=(0, 0)):
        return self.call(self.prefix.insert, parent, tokens, p, images)
    def chain(self, b): return self.call(self.prefix.chain, b)
    def retain_active(self, b): return self.call(self.prefix.retain_active, b)
    def release_active(self, b): return self.call(self.prefix.release_active, b)
    def touch(self, b): return self.call(self.prefix.touch, b)
    def candidate(self, after=0): return self.prefix.eviction_candidate(after)
    def erase(self, b): return self.call(self.prefix.erase, b)
    def match(self, prompt, spans=()):
        blocks = []
        hashed = self.prefix.extend_match(blocks, prompt, spans)
        return blocks, hashed
    def generation(self): return self.prefix.generation
    # sequences
    def begin(self, s): return self.call(self.sequences.begin, s)
    def end(self, s): return self.call(self.sequences.end, s)
    def restore(self, s, b): return self.call(self.sequences.restore, s, b)
    def ensure(self, s, n): return self.call(self.sequences.ensure_tokens, s, n)
    def publish(self, s, tokens, committed, spans=()):
        return self.call(self.sequences.publish, s, tokens, committed, spans)
    def truncate(self, s, tokens): return self.call(self.sequences.truncate, s, tokens)
    def view(self, s):
        q = self.sequences.sequences[s]
        return {"pages": list(q.pages), "revision": q.revision, "first_changed": q.first_changed,
                "blocks": list(q.blocks)}
    def compact(self):
        moves = self.pool.compact()
        if moves:
            self.sequences.follow(*moves)
        return moves


KINDS = {kvx.EINVAL: "invalid", kvx.ESTATE: "state", kvx.ERANGE: "range", kvx.ENOMEM: "nomem"}


class ProductStack:
    name = "product"

    def __init__(self, pages, extent_pages=4, runway=None):
        self.storage = kvx.Storage(1, 1, 64, kvx.INT8, pages, extent_pages, accounting=True)
        self.pool = kvx.Pool(self.storage, pages if runway is None else runway)
        self.prefix = kvx.Prefix(self.pool)
        self.sequences = kvx.Sequences(self.pool, self.prefix)

    def call(self, f, *args):
        try:
            return "ok", f(*args)
        except kvx.KvxError as e:
            return KINDS[e.code], None

    def acquire(self, n): return self.call(self.pool.acquire, n)
    def release_page(self, p):
        kind, _ = self.call(self.pool.release, p, False)
        return kind, None
    def pool_counts(self):
        s = self.pool.snapshot()
        return (s.pages_allocated, s.pages_free, s.pages_active, s.pages_prefix)
    def find(self, parent, tokens, images=(0, 0)): return self.prefix.find(parent, tokens, images)
    def insert(self, parent, tokens, p, images=(0, 0)):
        return self.call(self.prefix.insert, parent, tokens, p, images)
    def chain(self, b): return self.call(self.prefix.chain, b)
    def _status(self, f, *args):
        kind, _ = self.call(f, *args)
        return kind, None
    def retain_active(self, b): return self._status(self.prefix.retain_active, b)
    def release_active(self, b): return self._status(self.prefix.release_active, b)
    def touch(self, b): return self._status(self.prefix.touch, b)
    def candidate(self, after=0): return self.prefix.eviction_candidate(after)
    def erase(self, b): return self._status(self.prefix.erase, b)
    def match(self, prompt, spans=()): return self.prefix.match(prompt, spans)
    def generation(self): return self.prefix.generation()
    def begin(self, s): return self._status(self.sequences.begin, s)
    def end(self, s): return self._status(self.sequences.end, s)
    def restore(self, s, b): return self._status(self.sequences.restore, s, b)
    def ensure(self, s, n): return self._status(self.sequences.ensure_tokens, s, n)
    def publish(self, s, tokens, committed, spans=()):
        return self._status(self.sequences.publish, s, tokens, committed, spans)
    def truncate(self, s, tokens): return self.call(self.sequences.truncate, s, tokens)
    def view(self, s): return self.sequences.view(s)
    def compact(self):
        moves = self.sequences.compact_extent()
        return (moves["first"], moves["dest"]) if moves else None


STACKS = [OracleStack, ProductStack]


def ok(result):
    assert result[0] == "ok", result
    return result[1]


# ---- the reference's cases -----------------------------------------------------

@pytest.mark.parametrize("Stack", STACKS)
def test_exact_chained_blocks_and_physical_ownership(Stack):
    s = Stack(8, extent_pages=1)
    pages = ok(s.acquire(4))
    root_tokens, left_tokens, right_tokens, other_tokens = page(11), page(12), page(13), page(14)
    root, _ = ok(s.insert(0, root_tokens, pages[0]))
    left, _ = ok(s.insert(root, left_tokens, pages[1]))
    right, _ = ok(s.insert(root, right_tokens, pages[2]))
    other, _ = ok(s.insert(0, other_tokens, pages[3]))
    assert s.pool_counts()[3] == 4                      # four prefix-owned pages
    for p in pages:
        ok(s.release_page(p))
    assert s.pool_counts()[3] == 4 and s.pool_counts()[2] == 0
    wrong = list(left_tokens)
    wrong[-1] ^= 1
    assert s.find(root, left_tokens) == (left, pages[1])
    assert s.find(root, wrong) is None                  # a hash is never trusted alone
    assert ok(s.chain(left)) == ([root, left], [pages[0], pages[1]])
    assert ok(s.insert(root, left_tokens, pages[1])) == (left, pages[1])
    assert s.pool_counts()[3] == 4                      # an exact duplicate adds no block
    assert s.erase(root)[0] == "state"                  # a parent outlives its children
    ok(s.retain_active(left))
    assert s.candidate(0) == right and s.candidate(right) == other and s.candidate(other) is None
    ok(s.release_active(left))
    assert [s.candidate(0), s.candidate(right), s.candidate(other), s.candidate(left)] == \
        [right, other, left, None]
    ok(s.touch(right))
    assert [s.candidate(0), s.candidate(other), s.candidate(left), s.candidate(right)] == \
        [other, left, right, None]
    for b in (right, left, root, other):
        ok(s.erase(b))
    counts = s.pool_counts()
    assert counts[3] == 0 and counts[1] == counts[0] == 8   # nothing leaked


@pytest.mark.parametrize("Stack", STACKS)
def test_erased_leaf_parent_inherits_recency(Stack):
    s = Stack(8, extent_pages=1)
    pages = ok(s.acquire(4))
    a0, _ = ok(s.insert(0, page(21), pages[0]))
    a1, _ = ok(s.insert(a0, page(22), pages[1]))
    b0, _ = ok(s.insert(0, page(23), pages[2]))
    b1, _ = ok(s.insert(b0, page(24), pages[3]))
    for p in pages:
        ok(s.release_page(p))
    assert s.candidate(0) == a1 and s.candidate(a1) == b1
    ok(s.erase(a1))                                     # exposes a0, still colder than b1
    assert s.candidate(0) == a0 and s.candidate(a0) == b1 and s.candidate(b1) is None
    ok(s.erase(a0))
    ok(s.erase(b1))
    assert s.candidate(0) == b0 and s.candidate(b0) is None
    ok(s.erase(b0))
    counts = s.pool_counts()
    assert counts[3] == 0 and counts[1] == 8


@pytest.mark.parametrize("Stack", STACKS)
def test_input_validation(Stack):
    s = Stack(2, extent_pages=1)
    pages = ok(s.acquire(1))
    assert s.insert(0, [1], pages[0])[0] == "invalid"          # a partial page
    assert s.insert(999, page(2), pages[0])[0] == "invalid"    # an unknown parent
    assert s.insert(0, page(2), 2)[0] == "range"               # a page past the pool
    root, _ = ok(s.insert(0, page(2), pages[0]))
    assert s.insert(0, page(3), pages[0])[0] == "state"        # the page already holds a block
    assert s.chain(77)[0] == "range" and s.erase(77)[0] == "range"
    assert s.release_active(root)[0] == "state"                # no active user
    assert s.find(0, [1]) is None and s.find(999, page(2)) is None
    ok(s.release_page(pages[0]))


@pytest.mark.parametrize("Stack", STACKS)
def test_image_identity_is_part_of_the_key(Stack):
    # dev/tests/engine/kv_page_cache_test.cpp:35-84: the same tokens under
    # different image content are different blocks.
    s = Stack(4, extent_pages=1)
    pages = ok(s.acquire(2))
    text, _ = ok(s.insert(0, page(5), pages[0]))
    image, _ = ok(s.insert(0, page(5), pages[1], (0x1234, 0x5678)))
    assert text != image
    assert s.find(0, page(5)) == (text, pages[0])
    assert s.find(0, page(5), (0x1234, 0x5678)) == (image, pages[1])
    assert s.find(0, page(5), (0x1234, 0x5679)) is None


# ---- the request layer -----------------------------------------------------------

@pytest.mark.parametrize("Stack", STACKS)
def test_publish_dedups_to_the_canonical_page(Stack):
    s = Stack(16, extent_pages=4)
    prompt = [7 * i % 1013 for i in range(100)]
    ok(s.begin(1))
    ok(s.ensure(1, 100))
    first = s.view(1)
    assert len(first["pages"]) == 4 and first["revision"] == 1 and first["first_changed"] == 0
    ok(s.publish(1, prompt, 70))                 # two full pages committed
    one = s.view(1)
    assert len(one["blocks"]) == 2 and one["pages"] == first["pages"] and one["revision"] == 1
    # a second sequence writes the same tokens into pages of its own ...
    ok(s.begin(2))
    ok(s.ensure(2, 100))
    own = s.view(2)["pages"]
    ok(s.publish(2, prompt, 96))
    two = s.view(2)
    # ... and ends on the canonical pages for the shared part, keeping its own third page
    assert two["pages"][:2] == one["pages"][:2] and two["pages"][2:] == own[2:]
    assert two["blocks"][:2] == one["blocks"] and len(two["blocks"]) == 3
    assert two["revision"] == 3 and two["first_changed"] == 1
    # match leaves at least one prompt token unmatched
    assert s.match(prompt[:96]) == (two["blocks"][:2], 2)
    assert s.match(prompt[:97]) == (two["blocks"], 3)
    assert s.match(prompt[:31]) == ([], 0) and s.match([]) == ([], 0)
    # a third sequence adopts the cached chain without computing it
    ok(s.begin(3))
    ok(s.restore(3, two["blocks"][2]))
    three = s.view(3)
    assert three["pages"] == two["pages"][:3] and three["blocks"] == two["blocks"]
    assert s.restore(3, two["blocks"][0])[0] == "state"
    # errors of publish
    assert s.publish(1, prompt, 101)[0] == "invalid"
    assert s.publish(2, prompt, 64)[0] == "state"      # history moved backwards
    ok(s.begin(4))
    assert s.publish(4, prompt, 32)[0] == "state"      # committed KV without a page
    assert s.begin(4)[0] == "invalid" and s.begin(0)[0] == "invalid"
    before = s.pool_counts()
    for q in (1, 2, 3, 4):
        ok(s.end(q))
    after = s.pool_counts()
    assert after[2] == 0 and after[3] == 3 and after[1] == before[1] + (before[0] - before[1] - 3)
    assert s.candidate(0) == two["blocks"][2]          # only the chain's leaf is evictable


@pytest.mark.parametrize("Stack", STACKS)
def test_images_keep_equal_placeholder_tokens_apart(Stack):
    """Cache::publishCommittedBlocks and Cache::extendMatch key every block with the identity of
    the images that overlap it (runtime/engine/cache/Cache.cpp:186-193, :310-318): two prompts
    with the same placeholder tokens and different images neither match nor share a page, the
    same image does both, and blocks before the image are shared whatever the image is."""
    s = Stack(24, extent_pages=4)
    prompt = [3] * 40 + [9] * 50 + [5] * 20            # an image of 50 placeholder tokens at 40
    cat = [(40, 50, 5, 10, 0x1111, 0x2222)]
    dog = [(40, 50, 5, 10, 0x3333, 0x4444)]
    ok(s.begin(1))
    ok(s.ensure(1, len(prompt)))
    ok(s.publish(1, prompt, 96, cat))
    one = s.view(1)
    assert len(one["blocks"]) == 3
    # the same tokens under another image: the text-only first page is shared, the rest is not
    ok(s.begin(2))
    ok(s.ensure(2, len(prompt)))
    own = s.view(2)["pages"]
    ok(s.publish(2, prompt, 96, dog))
    two = s.view(2)
    assert two["pages"][0] == one["pages"][0] and two["blocks"][0] == one["blocks"][0]
    assert two["pages"][1:3] == own[1:3] and not set(two["blocks"][1:]) & set(one["blocks"][1:])
    # the same image again: everything is found and deduplicated
    ok(s.begin(3))
    ok(s.ensure(3, len(prompt)))
    ok(s.publish(3, prompt, 96, cat))
    three = s.view(3)
    assert three["pages"][:3] == one["pages"][:3] and three["blocks"] == one["blocks"]
    assert s.match(prompt, cat) == (one["blocks"], 3)
    assert s.match(prompt, dog) == (two["blocks"], 3)
    # without its images the prompt matches the text page only, and publishing it as text
    # makes blocks of its own for the placeholder pages
    assert s.match(prompt) == (one["blocks"][:1], 2)
    assert s.match(prompt, [(40, 50, 5, 10, 0x1111, 0x2223)]) == (one["blocks"][:1], 2)
    assert s.match(prompt, [(41, 50, 5, 10, 0x1111, 0x2222)]) == (one["blocks"][:1], 2)
    ok(s.begin(4))
    ok(s.ensure(4, len(prompt)))
    ok(s.publish(4, prompt, 96))
    four = s.view(4)
    assert four["blocks"][0] == one["blocks"][0]
    assert not set(four["blocks"][1:]) & (set(one["blocks"]) | set(two["blocks"]))


@pytest.mark.parametrize("Stack", STACKS)
def test_truncate_gives_emptied_pages_back(Stack):
    """After a speculative rollback the pages past the kept tokens go back to the pool; the
    published pages and the pages of the kept tokens stay; the next growth takes pages again."""
    s = Stack(16, extent_pages=4)
    tokens = [11 * i % 997 for i in range(200)]
    ok(s.begin(1))
    ok(s.ensure(1, 70 + 16))                       # 70 committed tokens and a tree of 16 rows
    before = s.view(1)
    assert len(before["pages"]) == 3
    ok(s.publish(1, tokens, 70))
    counts = s.pool_counts()
    assert ok(s.truncate(1, 70 + 16)) == 0 and s.view(1) == s.view(1)   # nothing past the kept tokens
    assert ok(s.truncate(1, 300)) == 0
    assert s.view(1)["revision"] == before["revision"]
    assert ok(s.truncate(1, 64)) == 1              # the third page held no kept token
    after = s.view(1)
    assert after["pages"] == before["pages"][:2] and after["blocks"] == s.view(1)["blocks"]
    assert after["revision"] == before["revision"] + 1 and after["first_changed"] == 2
    assert s.pool_counts()[2] == counts[2] - 1 and s.pool_counts()[1] == counts[1] + 1
    assert ok(s.truncate(1, 63)) == 0              # still two pages
    assert s.truncate(1, 32)[0] == "state"         # the second page is published
    assert s.truncate(9, 10)[0] == "range"
    ok(s.ensure(1, 100))                           # growth takes pages again, from the changed end
    grown = s.view(1)
    assert grown["pages"][:2] == after["pages"] and len(grown["pages"]) == 4
    assert grown["first_changed"] == 2
    # a page another sequence holds too only loses this sequence's reference
    ok(s.begin(2))
    ok(s.restore(2, after["blocks"][1]))
    ok(s.ensure(2, 96))
    ok(s.end(1))
    held = s.pool_counts()
    assert ok(s.truncate(2, 64)) == 1
    assert s.pool_counts()[2] == held[2] - 1
    assert s.view(2)["pages"] == after["pages"]
    ok(s.end(2))


def test_random_walk_in_lockstep():
    rng = random.Random(20261125)
    o, p = OracleStack(24, extent_pages=4, runway=8), ProductStack(24, extent_pages=4, runway=8)
    vocab = [rng.randrange(50) for _ in range(4)]
    streams = {}          # sequence -> (tokens, committed)
    images = {}           # sequence -> its prompt's image spans
    next_sequence = 1
    digests = [(0xA1, 0xB1), (0xA2, 0xB2)]

    def both(name, *args):
        a, b = getattr(o, name)(*args), getattr(p, name)(*args)
        assert a == b, (name, args, a, b)
        return a

    for step in range(1500):
        op = rng.random()
        live = sorted(streams)
        if op < 0.15 and len(live) < 6:
            sequence, next_sequence = next_sequence, next_sequence + 1
            assert both("begin", sequence)[0] == "ok"
            # few distinct pages, so sequences share prefixes often
            tokens = []
            for _ in range(rng.randrange(1, 5)):
                tokens += [rng.choice(vocab)] * 32
            tokens += [rng.randrange(50) for _ in range(rng.randrange(1, 32))]
            streams[sequence] = [tokens, 0]
            # a third of the prompts carry an image over some of their tokens
            images[sequence] = ()
            if rng.random() < 0.33 and len(tokens) > 40:
                offset = rng.randrange(0, len(tokens) - 8)
                images[sequence] = ((offset, rng.randrange(4, len(tokens) - offset), 2, 2) +
                                    rng.choice(digests),)
            blocks, _ = both("match", tokens, images[sequence])
            if blocks and rng.random() < 0.7:
                assert both("restore", sequence, blocks[-1])[0] == "ok"
                streams[sequence][1] = len(blocks) * 32
        elif op < 0.55 and live:
            sequence = rng.choice(live)
            tokens, committed = streams[sequence]
            target = min(len(tokens), committed + rng.randrange(1, 48))
            # room for a tree of draft rows past the target, given back after the step
            kind, _ = both("ensure", sequence, target + rng.choice((0, 16)))
            if kind == "ok":
                assert both("publish", sequence, tokens, target, images[sequence])[0] == "ok"
                streams[sequence][1] = target
                if rng.random() < 0.5:
                    assert both("truncate", sequence, target)[0] == "ok"
        elif op < 0.70 and live:
            sequence = rng.choice(live)
            assert both("end", sequence)[0] == "ok"
            del streams[sequence]
        elif op < 0.85:
            candidate = both("candidate", 0)
            if candidate is not None:
                assert both("erase", candidate)[0] == "ok"
        elif op < 0.92:
            both("compact")
        else:
            candidate = both("candidate", 0)
            if candidate is not None:
                both("touch", candidate)
        for sequence in streams:
            assert o.view(sequence) == p.view(sequence), (step, sequence)
        assert o.pool_counts() == p.pool_counts(), step
        assert o.generation() == p.generation()
    for sequence in list(streams):
        both("end", sequence)
    while True:
        candidate = both("candidate", 0)
        if candidate is None:
            break
        both("erase", candidate)
    counts = p.pool_counts()
    assert counts[2] == 0 and counts[3] == 0


# ---- verify-tree helpers ---------------------------------------------------------

def test_tree_masks_and_paths():
    none = 0xFFFFFFFF
    # the reference's comb: chain 0-1-2-3 with one sibling leaf per chain row
    parents = [none, 0, 1, 2, 0, 1, 2]
    expected = [0b1, 0b11, 0b111, 0b1111, 0b10001, 0b100011, 0b1000111]
    assert po.tree_masks(parents) == expected
    assert kvx.tree_masks(parents) == expected
    rng = random.Random(3)
    for _ in range(50):
        rows = rng.randrange(1, 17)
        parents = [none] + [rng.randrange(0, r) if rng.random() < 0.9 else none
                            for r in range(1, rows)]
        assert kvx.tree_masks(parents) == po.tree_masks(parents)
    with pytest.raises(kvx.KvxError):
        kvx.tree_masks([none, 1])                  # a parent must be an earlier row
    with pytest.raises(kvx.KvxError):
        kvx.tree_masks([none] * 33)
    parents = [none, 0, 1, 2, 0, 1, 2]
    assert kvx.tree_path_valid(parents, [0, 1, 2, 3])
    assert kvx.tree_path_valid(parents, [0, 1, 5])
    assert not kvx.tree_path_valid(parents, [0, 2])        # not a child of the row before
    assert not kvx.tree_path_valid(parents, [1, 2])        # must start at the anchor
    assert not kvx.tree_path_valid(parents, [0, 1, 1])     # rows strictly increase


# ---- image identity ---------------------------------------------------------------

def test_block_image_identity_properties_of_the_reference():
    """dev/tests/engine/kv_page_cache_test.cpp:44-69, for the product and the oracle."""
    red, blue = (8, 16, 8, 8, 0x1111, 0x2222), (8, 16, 8, 8, 0x3333, 0x4444)
    red_later, first = (40, 16, 8, 8, 0x1111, 0x2222), (0, 8, 4, 8, 0x5555, 0x6666)
    for identity in (kvx.block_image_identity, po.block_image_identity):
        assert identity(0, 32, []) == (0, 0)                    # text only
        assert identity(32, 32, [red]) == (0, 0)                # a block after the image
        r, b = identity(0, 32, [red]), identity(0, 32, [blue])
        assert r != (0, 0) and r != b                           # the content digest counts
        assert identity(32, 32, [red_later]) != r               # so does the block's alignment
        three = [first, blue, red_later]                        # only overlapping spans count
        assert identity(32, 32, three) == identity(32, 32, [red_later])
        assert identity(0, 8, three) == identity(0, 8, [first])
        assert identity(0, 32, three) != identity(0, 32, [first])   # two spans in one block
    rng = random.Random(11)
    for _ in range(300):
        spans, at = [], 0
        for _ in range(rng.randrange(0, 5)):
            at += rng.randrange(0, 40)
            tokens = rng.randrange(1, 70)
            spans.append((at, tokens, rng.randrange(1, 64), rng.randrange(1, 64),
                          rng.getrandbits(64), rng.getrandbits(64)))
            at += tokens
        begin = 32 * rng.randrange(0, 8)
        assert kvx.block_image_identity(begin, 32, spans) == po.block_image_identity(begin, 32, spans)


# ---- copy-on-write of a shared, partly filled page (no counterpart in the reference) ----

def test_fork_shares_pages_and_a_write_copies_the_partial_one():
    s = ProductStack(16, extent_pages=4)
    prompt = [3 * i % 997 for i in range(200)]
    ok(s.begin(1))
    ok(s.ensure(1, 80))                              # 2 full pages + 16 tokens of a third
    ok(s.publish(1, prompt, 80))
    one = s.view(1)
    assert len(one["pages"]) == 3 and len(one["blocks"]) == 2
    ok(s.begin(2))
    s.sequences.fork(2, 1, 80)
    two = s.view(2)
    assert two["pages"] == one["pages"] and two["blocks"] == one["blocks"]
    assert two["revision"] == 1 and two["first_changed"] == 0
    counts = s.pool_counts()
    assert counts[2] == 3                            # three pages, each held twice
    # the fork's first write: the shared partial page is copied, the whole pages stay shared
    moved = s.sequences.ensure_writable(2, 80)
    assert moved is not None and moved[0] == one["pages"][2] and moved[1] not in one["pages"]
    two = s.view(2)
    assert two["pages"] == one["pages"][:2] + [moved[1]]
    assert two["revision"] == 2 and two["first_changed"] == 2
    assert s.view(1) == one                          # the source is untouched
    assert s.pool_counts()[2] == 4
    # now both hold their last page alone: further writes go in place
    assert s.sequences.ensure_writable(2, 81) is None
    assert s.sequences.ensure_writable(1, 80) is None
    assert s.view(1) == one and s.view(2) == two
    # published pages are final; a token without a page is refused
    with pytest.raises(kvx.KvxError) as final:
        s.sequences.ensure_writable(2, 63)
    assert final.value.code == kvx.ESTATE
    with pytest.raises(kvx.KvxError) as absent:
        s.sequences.ensure_writable(2, 96)
    assert absent.value.code == kvx.EINVAL
    # the fork goes on: its own pages, published blocks continue the shared chain
    ok(s.ensure(2, 130))
    other = prompt[:80] + [5000 + i for i in range(50)]
    ok(s.publish(2, other, 128))
    two = s.view(2)
    assert two["blocks"][:2] == one["blocks"] and len(two["blocks"]) == 4
    assert two["pages"][2] == moved[1]
    # the source publishes its own third page: different tokens, a different block
    ok(s.ensure(1, 96))
    ok(s.publish(1, prompt, 96))
    assert s.view(1)["blocks"][2] != two["blocks"][2] and s.view(1)["pages"] == one["pages"]
    ok(s.end(1))
    ok(s.end(2))
    assert s.pool_counts()[2] == 0


def test_fork_errors_and_the_source_writing_first():
    s = ProductStack(8, extent_pages=4, runway=8)
    ok(s.begin(1))
    ok(s.ensure(1, 40))
    ok(s.begin(2))
    with pytest.raises(kvx.KvxError) as too_far:
        s.sequences.fork(2, 1, 65)
    assert too_far.value.code == kvx.EINVAL
    with pytest.raises(kvx.KvxError):
        s.sequences.fork(2, 9, 8)                     # unknown source
    with pytest.raises(kvx.KvxError) as itself:
        s.sequences.fork(1, 1, 8)
    assert itself.value.code == kvx.ESTATE
    s.sequences.fork(2, 1, 40)
    with pytest.raises(kvx.KvxError) as twice:
        s.sequences.fork(2, 1, 40)
    assert twice.value.code == kvx.ESTATE
    before = s.view(1)
    # the source writes first: it is the one that moves to a copy, the fork keeps the page
    moved = s.sequences.ensure_writable(1, 40)
    assert moved and moved[0] == before["pages"][1]
    assert s.view(1)["pages"] == [before["pages"][0], moved[1]]
    assert s.view(2)["pages"] == before["pages"]
    assert s.sequences.ensure_writable(2, 40) is None      # sole holder now
    # no page to be had: nothing changes
    ok(s.begin(3))
    s.sequences.fork(3, 2, 40)
    ok(s.begin(4))
    ok(s.ensure(4, 32 * 5))                          # takes the five free pages
    held = s.view(3)
    with pytest.raises(kvx.KvxError) as full:
        s.sequences.ensure_writable(3, 40)
    assert full.value.code == kvx.ENOMEM and s.view(3) == held
    for q in (1, 2, 3, 4):
        ok(s.end(q))
    assert s.pool_counts()[2] == 0 and s.pool_counts()[1] == 8
