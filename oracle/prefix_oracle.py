"""TEST INFRASTRUCTURE ONLY: a plain-Python restatement of the resident tier of
the reference's prefix page cache and of its per-request page lists.

Follows runtime/engine/cache/KvCache.cpp (find :66-86, insert :88-158,
retainActive/releaseActive/touch :227-257, chain :259-273, inherit :441-446,
evictionCandidate :480-484, erase :515-559, reindex :577-592, followPages
:393-409) and runtime/engine/cache/Cache.cpp (beginRequest/endRequest :143-166,
extendMatch :179-199, pageTable/pagesChanged :284-292, publishCommittedBlocks
:294-333, ensureTokens :381-397, compactExtent :700-731, restoreRequest
:748-785 for resident chains).  The disk tier, recurrent states and poisoning
are left out: they are not part of the KV data path.

Pinned against the reference's own cases for these functions
(dev/tests/engine/kv_page_cache_test.cpp:86-220) in tests/test_prefix_cache.py.
Nothing in the product may import this module.
"""

PAGE_TOKENS = 32
NO_PAGE = 0xFFFFFFFF


class OracleError(Exception):
    """kind: 'invalid' (std::invalid_argument), 'state' (std::logic_error),
    'range' (std::out_of_range), 'nomem' (refused allocation)."""

    def __init__(self, kind, message=""):
        super().__init__(f"{kind}: {message}")
        self.kind = kind


class Block:
    def __init__(self):
        self.id = 0
        self.parent = 0
        self.tokens = ()
        self.images = (0, 0)
        self.page = NO_PAGE
        self.depth = 0
        self.children = 0
        self.active_users = 0
        self.last_used = 0


class PrefixCache:
    """`pool` is the oracle's page pool (or anything with retain(page, prefix_owner)
    and release(page, prefix_owner) that raise OracleError): a block owns one prefix
    reference of its page."""

    def __init__(self, pool, pages):
        self.pool = pool
        self.blocks = {}
        self.index = {}          # (parent, tokens, images) -> id; the reference hashes then compares the key
        self.block_on_page = [0] * pages
        self.next_id = 1
        self.clock = 0
        self.generation = 0

    def _tick(self):
        self.clock += 1
        return self.clock

    def _block(self, block):
        if block not in self.blocks:
            raise OracleError("range", "unknown KV cache block")
        return self.blocks[block]

    def find(self, parent, tokens, images=(0, 0)):
        if len(tokens) != PAGE_TOKENS:
            return None
        if parent and parent not in self.blocks:
            return None
        found = self.index.get((parent, tuple(tokens), tuple(images)))
        if found is None:
            return None
        return found, self.blocks[found].page

    def insert(self, parent, tokens, page, images=(0, 0)):
        if len(tokens) != PAGE_TOKENS:
            raise OracleError("invalid", "KV cache block must contain one full page")
        if page >= len(self.block_on_page):
            raise OracleError("range", "KV cache physical page is out of range")
        existing = self.find(parent, tokens, images)
        if existing:
            return existing
        if parent and parent not in self.blocks:
            raise OracleError("invalid", "KV cache parent block is unknown")
        if self.block_on_page[page]:
            raise OracleError("state", "KV cache page already holds a block")
        self.pool.retain(page, True)
        b = Block()
        b.id = self.next_id
        self.next_id += 1
        b.parent, b.tokens, b.images, b.page = parent, tuple(tokens), tuple(images), page
        b.depth = self.blocks[parent].depth + 1 if parent else 1
        self.blocks[b.id] = b
        self.index[(parent, b.tokens, b.images)] = b.id
        self.block_on_page[page] = b.id
        if parent:
            self.blocks[parent].children += 1
        b.last_used = self._tick()
        self.generation += 1
        return b.id, page

    def chain(self, block):
        b = self._block(block)
        blocks, pages = [0] * b.depth, [NO_PAGE] * b.depth
        for index in range(b.depth, 0, -1):
            blocks[index - 1], pages[index - 1] = b.id, b.page
            b = self.blocks.get(b.parent)
        return blocks, pages

    def retain_active(self, block):
        b = self._block(block)
        b.active_users += 1
        b.last_used = self._tick()

    def release_active(self, block):
        b = self._block(block)
        if not b.active_users:
            raise OracleError("state", "no active user")
        b.active_users -= 1
        if not b.active_users and not b.children:
            b.last_used = self._tick()

    def touch(self, block):
        self._block(block).last_used = self._tick()

    def _leaves(self):
        return sorted((b.last_used, b.id) for b in self.blocks.values()
                      if not b.active_users and not b.children)

    def eviction_candidate(self, after=0):
        order = self._leaves()
        if not after:
            return order[0][1] if order else None
        key = (self._block(after).last_used, after)
        for entry in order:
            if entry > key:
                return entry[1]
        return None

    def erase(self, block):
        b = self._block(block)
        if b.children or b.active_users:
            raise OracleError("state", "cannot evict a referenced KV cache block")
        del self.index[(b.parent, b.tokens, b.images)]
        del self.blocks[block]
        self.generation += 1
        self.block_on_page[b.page] = 0
        if b.parent:
            p = self.blocks[b.parent]
            p.children -= 1
            if not p.children and not p.active_users:
                p.last_used = max(p.last_used, b.last_used)
        self.pool.release(b.page, True)

    def follow_pages(self, first_page, destinations):
        for offset, to in enumerate(destinations):
            source = first_page + offset
            if to == source:
                continue
            block, self.block_on_page[source] = self.block_on_page[source], 0
            if not block:
                continue
            self.blocks[block].page = to
            self.block_on_page[to] = block

    def extend_match(self, blocks, prompt, spans=()):
        """Cache::extendMatch (runtime/engine/cache/Cache.cpp:179-199); spans are the prompt's
        images, sorted by offset: each block is looked up under blockImageIdentity of the spans
        that have not ended before it (spansFrom, Cache.cpp:16-22)."""
        if not len(prompt):
            return 0
        maximum = (len(prompt) - 1) // PAGE_TOKENS
        hashed = 0
        spans = list(spans)
        for index in range(len(blocks), maximum):
            parent = blocks[-1] if blocks else 0
            hashed += 1
            begin = index * PAGE_TOKENS
            spans = spans_from(spans, begin)
            match = self.find(parent, prompt[begin:begin + PAGE_TOKENS],
                              block_image_identity(begin, PAGE_TOKENS, spans))
            if not match:
                break
            blocks.append(match[0])
        return hashed


class Sequence:
    def __init__(self):
        self.pages = []
        self.blocks = []
        self.revision = 0
        self.first_changed = 0


class SequenceCache:
    """acquire(count) -> list of page ids (or raises OracleError('nomem')) is the
    pool's acquisition, injected so the oracle can follow any pool policy."""

    def __init__(self, pool, prefix, acquire):
        self.pool, self.prefix, self.acquire = pool, prefix, acquire
        self.sequences = {}

    @staticmethod
    def _changed(s, first):
        s.revision += 1
        s.first_changed = first

    def _sequence(self, sequence):
        if sequence not in self.sequences:
            raise OracleError("range", "unknown sequence")
        return self.sequences[sequence]

    def begin(self, sequence):
        if not sequence or sequence in self.sequences:
            raise OracleError("invalid", "invalid or duplicate sequence id")
        self.sequences[sequence] = Sequence()

    def end(self, sequence):
        s = self.sequences.pop(sequence, None)
        if s is None:
            return
        for page in s.pages:
            self.pool.release(page, False)
        if s.blocks:
            self.prefix.release_active(s.blocks[-1])

    def restore(self, sequence, last_block):
        s = self._sequence(sequence)
        if s.pages or s.blocks:
            raise OracleError("state", "restore target already owns KV pages")
        blocks, pages = self.prefix.chain(last_block)
        self.prefix.retain_active(blocks[-1])
        for page in pages:
            self.pool.retain(page, False)
        s.pages, s.blocks = pages, blocks
        self._changed(s, 0)

    def ensure_tokens(self, sequence, tokens):
        s = self._sequence(sequence)
        needed = (tokens + PAGE_TOKENS - 1) // PAGE_TOKENS
        previous = len(s.pages)
        if needed <= previous:
            return
        s.pages += list(self.acquire(needed - previous))
        self._changed(s, previous)

    def truncate(self, sequence, tokens):
        """No counterpart in the reference (it never shrinks a request): the pages past those of
        the first `tokens` tokens go back to the pool; published pages may not."""
        s = self._sequence(sequence)
        keep = (tokens + PAGE_TOKENS - 1) // PAGE_TOKENS
        if keep < len(s.blocks):
            raise OracleError("state", "truncation would drop a published page")
        if keep >= len(s.pages):
            return 0
        dropped = s.pages[keep:]
        for page in dropped:
            self.pool.release(page, False)
        del s.pages[keep:]
        self._changed(s, keep)
        return len(dropped)

    def publish(self, sequence, tokens, committed, spans=()):
        """Cache::publishCommittedBlocks (Cache.cpp:294-333), images included (:310-318)."""
        s = self._sequence(sequence)
        spans = list(spans)
        if committed > len(tokens):
            raise OracleError("invalid", "committed KV exceeds exact token history")
        full = committed // PAGE_TOKENS
        if (committed + PAGE_TOKENS - 1) // PAGE_TOKENS > len(s.pages):
            raise OracleError("state", "committed KV has no physical request page")
        if full < len(s.blocks):
            raise OracleError("state", "committed KV history moved backwards")
        while len(s.blocks) < full:
            logical = len(s.blocks)
            parent = s.blocks[-1] if logical else 0
            writer = s.pages[logical]
            begin = logical * PAGE_TOKENS
            spans = spans_from(spans, begin)
            block, canonical = self.prefix.insert(
                parent, tokens[begin:begin + PAGE_TOKENS], writer,
                block_image_identity(begin, PAGE_TOKENS, spans))
            replace = canonical != writer
            if replace:
                self.pool.retain(canonical, False)
            self.prefix.retain_active(block)
            s.blocks.append(block)
            if replace:
                s.pages[logical] = canonical
                self._changed(s, logical)
                self.pool.release(writer, False)
            if parent:
                self.prefix.release_active(parent)

    def follow(self, first_page, destinations):
        """The re-pointing half of Cache::compactExtent, given the pool's moves (the
        pool moves the references with the pages itself)."""
        self.prefix.follow_pages(first_page, destinations)

        def follow(page):
            offset = page - first_page
            return destinations[offset] if 0 <= offset < len(destinations) else page

        for s in self.sequences.values():
            first = len(s.pages)
            for index, page in enumerate(s.pages):
                to = follow(page)
                if to != page:
                    s.pages[index] = to
                    first = min(first, index)
            if first < len(s.pages):
                self._changed(s, first)


def tree_masks(parents, none=0xFFFFFFFF):
    """verify_input_tree_tokens (runtime/metal/kernels/shared/embedding.metal:248-281):
    mask = 1 << row | the bits of the row's ancestors; a later row without a
    parent is dead and gets 0."""
    masks = []
    for row, parent in enumerate(parents):
        if row and parent == none:
            masks.append(0)
            continue
        mask = 1 << row
        while parent != none:
            mask |= 1 << parent
            parent = parents[parent]
        masks.append(mask)
    return masks


def spans_from(spans, block_begin):
    """spansFrom (runtime/engine/cache/Cache.cpp:16-22): the spans that can still overlap the
    block at block_begin or a later one."""
    first = 0
    while first < len(spans) and ((spans[first][0] + spans[first][1]) & 0xFFFFFFFF) <= block_begin:
        first += 1
    return spans[first:]


def block_image_identity(block_begin, block_tokens, spans):
    """Restates blockImageIdentity (runtime/engine/cache/KvCache.cpp:29-52): (lo, hi) of a block
    of `block_tokens` tokens at `block_begin`; spans are (offset, tokens, grid height, grid
    width, digest lo, digest hi) sorted by offset.  Only spans that overlap the block count;
    a block without any has identity (0, 0).

    Pinned to the bit: tests/golden/reference_vectors.npz holds what the reference's own
    compiled function returned (tests/golden/make_vectors.py through oracle/_ref), and
    tests/test_golden.py holds this restatement and the library to those values; the
    properties of dev/tests/engine/kv_page_cache_test.cpp:44-69 (zero for text, zero after the
    image, dependence on digest and alignment, spans outside the block ignored) are checked in
    tests/test_prefix_cache.py."""
    mask = (1 << 64) - 1

    def mix(h, v):
        return h ^ ((v + 0x9E3779B97F4A7C15 + ((h << 6) & mask) + (h >> 2)) & mask)

    lo = hi = 0
    end = block_begin + block_tokens
    for offset, tokens, height, width, digest_lo, digest_hi in spans:
        if offset >= end:
            break
        if ((offset + tokens) & 0xFFFFFFFF) <= block_begin:
            continue
        lo = lo or 0x243F6A8885A308D3
        hi = hi or 0x13198A2E03707344
        for value in (digest_lo, digest_hi, (height << 32) | width, (offset << 32) | tokens, block_begin):
            lo = mix(lo, value)
            hi = mix(hi, ~value & mask)
    return lo, hi
