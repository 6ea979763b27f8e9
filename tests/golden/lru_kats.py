"""Known-answer vectors for the LRU update, restated as data from the reference's
own unit tests (dram_attention/lru_triton_kernel_test.py:17-204).  Geometry of
all three: 2 heads, 8 DRAM pages, 4 HBM slots, page payload 64 floats, int32
metadata, access times arange(4) per head, current_step = 4.

Each case: initial (d2h, h2d), requests, and the entries the reference asserts
after the call, as {(head, index): value} tables.  `payload` lists
(head, slot, page): hbm[head, slot] must equal dram[head, page].
"""

EMPTY = -1

CASES = {
    # :17-76  empty cache, two requests per head
    "basic": dict(
        d2h=[[EMPTY] * 8, [EMPTY] * 8],
        h2d=[[EMPTY] * 4, [EMPTY] * 4],
        topk=[[0, 1], [1, 2]],
        time={(0, 0): 4, (0, 1): 4, (1, 0): 4, (1, 1): 4},
        d2h_after={(0, 0): 0, (0, 1): 1, (1, 1): 0, (1, 2): 1},
        h2d_after={(0, 0): 0, (0, 1): 1, (1, 0): 1, (1, 1): 2},
        payload=[(0, 0, 0), (0, 1, 1), (1, 0, 1), (1, 1, 2)],
    ),
    # :78-143  full cache (page i in slot i), requests for absent pages evict slots 0, 1
    "eviction": dict(
        d2h=[[0, 1, 2, 3, EMPTY, EMPTY, EMPTY, EMPTY]] * 2,
        h2d=[[0, 1, 2, 3]] * 2,
        topk=[[4, 5], [5, 6]],
        time={(0, 0): 4, (0, 1): 4, (1, 0): 4, (1, 1): 4},
        d2h_after={(0, 4): 0, (0, 5): 1, (1, 5): 0, (1, 6): 1},
        h2d_after={(0, 0): 4, (0, 1): 5, (1, 0): 5, (1, 1): 6},
        payload=[(0, 0, 4), (0, 1, 5), (1, 0, 5), (1, 1, 6)],
    ),
    # :145-204  heads are independent
    "multiple_heads": dict(
        d2h=[[EMPTY] * 8, [EMPTY] * 8],
        h2d=[[EMPTY] * 4, [EMPTY] * 4],
        topk=[[0, 2], [1, 3]],
        time={(0, 0): 4, (0, 1): 4, (1, 0): 4, (1, 1): 4},
        d2h_after={(0, 0): 0, (0, 2): 1, (1, 1): 0, (1, 3): 1},
        h2d_after={(0, 0): 0, (0, 1): 2, (1, 0): 1, (1, 1): 3},
        payload=[(0, 0, 0), (0, 1, 2), (1, 0, 1), (1, 1, 3)],
    ),
}

NUM_HEADS, NUM_DRAM_PAGES, NUM_HBM_PAGES, PAGE_DIM, STEP = 2, 8, 4, 64, 4

# Geometry facts asserted by dram_attention/lru_cache_test.py:16-29,60-66:
# 4 heads x 8192 tokens x 64 dims, page 16 -> 512 DRAM pages; default HBM share
# 0.2 -> 102 slots holding the LAST 102 pages in order; lru_hbm_cache_size=1024 -> 64 slots.
GEOMETRY = dict(tokens=8192, page_size=16, dram_pages=512, default_hbm_pages=102,
                hbm_pages_for_1024_tokens=64)

# Not one of the reference's tests: a hand walk of its three launches
# (dram_attention/lru_triton_kernel.py:159-194) when the caller's step EQUALS the
# stored access times.  One head, 3 slots holding pages 3, 4, 5, all times 0, step 0,
# requests [0, 1, 3]: the touch pass stamps slot 0 (page 3) with 0, the stable argsort
# of [0, 0, 0] is [0, 1, 2]; the walk gives page 0 slot 0 (evicting page 3, which was
# "hit" a moment ago), page 1 slot 1, and finds page 3 gone: a third miss, slot 2.
STAMP_TIES = dict(
    n_dram_pages=6, d2h=[[EMPTY, EMPTY, EMPTY, 0, 1, 2]], h2d=[[3, 4, 5]], time=[[0, 0, 0]], step=0,
    topk=[[0, 1, 3]],
    d2h_after=[[0, 1, EMPTY, 2, EMPTY, EMPTY]], h2d_after=[[0, 1, 3]], time_after=[[0, 0, 0]],
    hit=[[False, False, False]], misses=[[(0, 0), (1, 1), (3, 2)]],
)
