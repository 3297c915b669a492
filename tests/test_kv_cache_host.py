"""Host logic of the block KV cache: allocation, slot mapping, prefix sharing
with copy-on-write.  CPU tensors (no kernel is called)."""
import pytest
import torch

from ironcore_amd.kv_cache import BlockAllocator, OutOfBlocks, PagedKVCache


def test_allocator_refcounts():
    a = BlockAllocator(3)
    b0, b1 = a.allocate(), a.allocate()
    assert {b0, b1} == {0, 1} and a.num_free == 1
    a.share(b0)
    a.release(b0)
    assert a.ref_count(b0) == 1 and a.num_free == 1
    a.release(b0)
    assert a.num_free == 2
    with pytest.raises(ValueError):
        a.release(b0)
    a.allocate(), a.allocate()
    with pytest.raises(OutOfBlocks):
        a.allocate()


def test_prepare_builds_tables_slots_and_lengths():
    cache = PagedKVCache(2, 8, 16, 2, 8, torch.float32, "cpu")
    s0, s1 = cache.add_sequence(), cache.add_sequence()
    meta = cache.prepare([s0, s1], 20)
    assert meta.context_lens.tolist() == [20, 20] and meta.max_context_len == 20
    assert meta.block_tables.shape == (2, 2)
    t = meta.block_tables.tolist()
    assert len({*t[0], *t[1]}) == 4
    want = [t[i][p // 16] * 16 + p % 16 for i in range(2) for p in range(20)]
    assert meta.slot_mapping.tolist() == want
    meta = cache.prepare([s0, s1], 1)
    assert meta.context_lens.tolist() == [21, 21]
    assert meta.slot_mapping.tolist() == [t[0][1] * 16 + 4, t[1][1] * 16 + 4]
    cache.free_sequence(s0)
    assert cache.allocator.num_free == 6


def test_fork_aliases_full_blocks_and_copies_the_partial_one():
    cache = PagedKVCache(1, 8, 16, 1, 4, torch.float32, "cpu")
    s = cache.add_sequence()
    cache.prepare([s], 40)                      # 2 full blocks + 8 tokens
    blocks = cache.blocks(s)
    cache.k_pools[0, blocks[2]].fill_(7.0)
    c = cache.fork(s)
    cb = cache.blocks(c)
    assert cb[:2] == blocks[:2] and cb[2] != blocks[2]
    assert cache.allocator.ref_count(blocks[0]) == 2
    assert torch.equal(cache.k_pools[0, cb[2]], cache.k_pools[0, blocks[2]])
    m = cache.prepare([s, c], 1)                # both append privately
    assert m.slot_mapping.tolist() == [blocks[2] * 16 + 8, cb[2] * 16 + 8]
    cache.free_sequence(s)
    assert cache.allocator.ref_count(blocks[0]) == 1


def test_append_into_shared_block_copies_on_write():
    cache = PagedKVCache(1, 8, 16, 1, 4, torch.float32, "cpu")
    s = cache.add_sequence()
    cache.prepare([s], 32)                      # exactly 2 full blocks
    c = cache.fork(s)                           # aliases both
    # rewind the child by hand into the shared last block to force a write there
    cache._seqs[c].length = 20
    m = cache.prepare([c], 1)
    new_blk = cache.blocks(c)[1]
    assert new_blk != cache.blocks(s)[1]
    assert m.slot_mapping.tolist() == [new_blk * 16 + 4]


def test_shared_prefix_blocks_helper():
    import numpy as np
    from ironcore_amd.paged_ops import shared_prefix_blocks
    tables = np.array([[7, 8, 9, 1], [7, 8, 5, 2], [3, 4, 0, 0], [3, 4, 6, 0], [9, 0, 0, 0]], dtype=np.int32)
    ctx = np.array([64, 50, 32, 40, 10])
    assert shared_prefix_blocks(tables, ctx, 16, 2).tolist() == [2, 2, 0]
    assert shared_prefix_blocks(tables, ctx, 16, 4).tolist() == [0, 0]
    # a block is only shared if every member's context covers it entirely
    assert shared_prefix_blocks(tables, np.array([64, 20, 32, 40, 10]), 16, 2).tolist() == [1, 2, 0]


def test_prepare_reports_cohorts_of_forked_sequences():
    cache = PagedKVCache(1, 16, 16, 1, 4, torch.float32, "cpu")
    s = cache.add_sequence()
    cache.prepare([s], 40)                      # 2 full blocks + 8 tokens
    kids = [cache.fork(s) for _ in range(3)]
    lone = cache.add_sequence()
    cache.prepare([lone], 5)
    m = cache.prepare([s] + kids + [lone], 1, cohort_size=2)
    assert m.cohort_size == 2
    # (s, kid0) and (kid1, kid2) alias the two full prompt blocks; lone is alone in its cohort
    assert m.cohort_shared_blocks.tolist() == [2, 2, 0]
    assert cache.prepare([s] + kids, 1).cohort_size == 1


def test_pick_endings_groups_by_prompt_and_takes_the_lowest_loss():
    from ironcore_amd.scoring import pick_endings
    prompts = ["a", "a", "a", "b", "b", "b"]
    losses = [2.0, 1.0, 3.0, 0.5, 0.7, 0.9]
    labels = [0, 1, 0, 0, 0, 1]
    assert pick_endings(prompts, losses, labels) == {"metric": "accuracy", "score": 50.0}
    assert pick_endings([], [], []) == 0.0


def test_reserve_gives_blocks_ahead_and_unshares_the_block_in_use():
    """What a decode loop without per-step host work relies on: after
    ``reserve`` the slots that ``prepare`` would hand out one by one can be
    computed from ``block_table`` alone."""
    cache = PagedKVCache(1, 16, 16, 1, 4, torch.float32, "cpu")
    root = cache.add_sequence()
    cache.prepare([root], 20)                               # blocks: one full, one holding 4 tokens
    cache.k_pools[0, cache.blocks(root)[1]].fill_(7.0)
    child = cache.fork(root)                                # full block aliased, partial one copied
    twin = cache.add_sequence()
    cache.prepare([twin], 16)
    shared_partial = cache.fork(twin)                       # block-aligned: the whole block is aliased
    for sid, total in ((child, 50), (shared_partial, 40)):
        cache.reserve(sid, total)
        assert len(cache.blocks(sid)) * 16 >= total
    assert cache.blocks(child)[0] == cache.blocks(root)[0] and cache.blocks(child)[1] != cache.blocks(root)[1]
    assert bool((cache.k_pools[0, cache.blocks(child)[1]] == 7.0).all())
    table = cache.block_table([child, shared_partial])
    assert table.dtype == torch.int32 and table.shape == (2, 4)
    assert table[1].tolist() == cache.blocks(shared_partial) + [0]
    # the slots prepare() would give for the next tokens are the table's
    want = [int(table[0, p // 16]) * 16 + p % 16 for p in range(20, 50)]
    got = [int(cache.prepare([child], 1).slot_mapping[0]) for _ in range(30)]
    assert got == want
    # and advance() is the bookkeeping of the same appends done on the device
    cache.advance([shared_partial], 24)
    assert cache.length(shared_partial) == 40
    with pytest.raises(ValueError):
        cache.advance([shared_partial], 9)                  # 49 tokens do not fit 3 blocks


def test_reserve_copies_a_shared_block_that_is_partly_filled():
    cache = PagedKVCache(1, 8, 16, 1, 4, torch.float32, "cpu")
    a = cache.add_sequence()
    cache.prepare([a], 10)
    blk = cache.blocks(a)[0]
    cache.allocator.share(blk)                              # someone else holds the partly filled block too
    cache.k_pools[0, blk].fill_(3.0)
    cache.reserve(a, 30)
    assert cache.blocks(a)[0] != blk and cache.allocator.ref_count(blk) == 1
    assert bool((cache.k_pools[0, cache.blocks(a)[0]] == 3.0).all())
    assert len(cache.blocks(a)) == 2


@pytest.mark.parametrize("seed", range(6))
def test_random_cache_traffic_keeps_the_books(seed):
    """Random appends, forks, reservations and frees: at every step a block's
    reference count is the number of sequences that hold it, no block is both
    free and held, a block that will be written is held by one sequence only,
    and every sequence still reads back exactly the tokens written to it
    (token t of sequence s is stored as the value 1000 s' + t, s' the sequence
    that wrote it first)."""
    import random
    rng = random.Random(seed)
    bs = 16
    cache = PagedKVCache(1, 48, bs, 1, 2, torch.float32, "cpu")
    flat = cache.k_pools[0].view(-1, 2)          # [blocks * bs, hd]: gn == 1, so slot s is row s
    want = {}                                      # sid -> list of values, one per token
    next_tag = [0]

    def append(sid, n):
        meta = cache.prepare([sid], n)
        for s in meta.slot_mapping.tolist():
            want[sid].append(float(next_tag[0]))
            flat[s] = float(next_tag[0])
            next_tag[0] += 1

    for step in range(300):
        live = list(want)
        op = rng.choice(["new", "append", "append", "append", "fork", "free", "reserve"])
        try:
            if op == "new" or not live:
                sid = cache.add_sequence()
                want[sid] = []
                append(sid, rng.randint(1, 40))
            elif op == "append":
                append(rng.choice(live), rng.choice([1, 1, 1, 5, 17]))
            elif op == "fork":
                src = rng.choice(live)
                want[cache.fork(src)] = list(want[src])
            elif op == "reserve":
                sid = rng.choice(live)
                cache.reserve(sid, cache.length(sid) + rng.randint(1, 30))
                table = cache.block_table([sid])[0].tolist()
                assert table[:len(cache.blocks(sid))] == cache.blocks(sid)
                nxt = cache.length(sid)          # the block the next token goes to is this sequence's alone
                assert cache.allocator.ref_count(cache.blocks(sid)[nxt // bs]) == 1
            else:
                sid = rng.choice(live)
                cache.free_sequence(sid)
                del want[sid]
        except OutOfBlocks:                        # nothing may have changed; make room and go on
            victim = rng.choice(list(want))
            cache.free_sequence(victim)
            del want[victim]
        # the books
        holders = {}
        for sid in want:
            assert len(cache.blocks(sid)) * bs >= cache.length(sid) == len(want[sid])
            for blk in cache.blocks(sid):
                holders[blk] = holders.get(blk, 0) + 1
        for blk in range(cache.num_blocks):
            assert cache.allocator.ref_count(blk) == holders.get(blk, 0), f"step {step} block {blk}"
        assert cache.allocator.num_free == cache.num_blocks - len(holders)
        # the contents
        for sid, vals in want.items():
            blocks = cache.blocks(sid)
            got = [flat[blocks[t // bs] * bs + t % bs, 0].item() for t in range(len(vals))]
            assert got == vals, f"step {step} sequence {sid}"


def test_prepare_with_chunks_of_unequal_length():
    """One step, a chunk length per sequence: slots and positions are padded to
    the longest chunk, the true bounds and the rows that exist come with them."""
    cache = PagedKVCache(1, 16, 16, 1, 4, torch.float32, "cpu")
    a, b, c = cache.add_sequence(), cache.add_sequence(), cache.add_sequence()
    cache.prepare([a], 10)
    meta = cache.prepare([a, b, c], [3, 0, 5])
    assert meta.context_lens.tolist() == [13, 0, 5] and meta.max_context_len == 13
    assert meta.cu_seqlens_q.tolist() == [0, 3, 3, 8] and meta.max_chunk_len == 5
    assert meta.chunk_rows.tolist() == [0, 1, 2, 10, 11, 12, 13, 14]
    slots = meta.slot_mapping.view(3, 5)
    blk_a, blk_c = cache.blocks(a)[0], cache.blocks(c)[0]
    assert slots[0].tolist() == [blk_a * 16 + 10, blk_a * 16 + 11, blk_a * 16 + 12, -1, -1]
    assert slots[1].tolist() == [-1] * 5
    assert slots[2].tolist() == [blk_c * 16 + t for t in range(5)]
    assert meta.positions.view(3, 5)[0].tolist() == [10, 11, 12, 0, 0]
    with pytest.raises(ValueError):
        cache.prepare([a, b], [1, 2], cohort_size=2)


def test_attention_refuses_inputs_that_require_grad():
    """The reference's layer is differentiable (tests/test_attention.py:391-426
    backpropagates through it); the HIP path is forward only and says so
    instead of returning a tensor without a graph.  Raised on the host, before
    anything touches a device."""
    import pytest
    import torch
    from ironcore_amd import config as ic_config
    from ironcore_amd.layers import Attention
    cfg = ic_config.MainConfig(model=ic_config.ModelConfig(d_model=128, num_attention_heads=2,
                                                           num_attention_groups=2, head_dim=64, dropout_attn=0.0,
                                                           precision="bf16"),
                               trainer=ic_config.TrainerConfig(use_flash_attn=False))
    attn = Attention(cfg)
    q = torch.randn(1, 4, 2, 64, requires_grad=True)
    k, v = torch.randn(1, 4, 2, 64), torch.randn(1, 4, 2, 64)
    for args in ((q, k, v), (k, q, v), (k, v, q)):
        with pytest.raises(NotImplementedError, match="forward only"):
            attn(*args)
    with torch.no_grad():                            # not recording: passes the check (and then needs a GPU)
        with pytest.raises(RuntimeError, match="GPU only"):
            attn(q, k, v)


def test_masks_built_under_inference_mode_and_the_mask_cache_stays_small():
    """A tensor created under torch.inference_mode() keeps no version counter:
    the layer classifies such a mask on every call instead of failing on it (the
    call then goes on to the device check).  And the per-tensor cache of
    classified masks holds a few live masks at most and lets go of a mask's
    byte copy when the mask tensor dies."""
    import gc
    import pytest
    import torch
    from ironcore_amd import config as ic_config
    from ironcore_amd.layers import Attention
    from ironcore_amd.layers import attention as attention_module
    cfg = ic_config.MainConfig(model=ic_config.ModelConfig(d_model=128, num_attention_heads=2,
                                                           num_attention_groups=2, head_dim=64, dropout_attn=0.0,
                                                           precision="bf16"),
                               trainer=ic_config.TrainerConfig(use_flash_attn=False))
    attn = Attention(cfg).eval()
    with torch.inference_mode():
        q = torch.randn(1, 4, 2, 64)
        mask = torch.tril(torch.ones(1, 1, 4, 4))
        assert attn._classify_mask(mask, 1, 4, 4, 2) == ("causal", None)
        mask[0, 0, 3, 0] = 0
        kind, data = attn._classify_mask(mask, 1, 4, 4, 2)       # the edit is seen: nothing was cached
        assert kind == "general" and data[0, 0, 3].tolist() == [0, 1, 1, 1]
        with pytest.raises(RuntimeError, match="GPU only"):
            attn(q, q, q, mask)
    attention_module._MASK_CLASSES.clear()
    masks = []
    for i in range(10):
        m = torch.ones(1, 1, 4, 4)
        m[0, 0, 0, 1 + i % 3] = 0
        assert attn._classify_mask(m, 1, 4, 4, 2)[0] == "general"
        masks.append(m)
        assert len(attention_module._MASK_CLASSES) <= attention_module._MASK_CLASSES_MAX
    kept = len(attention_module._MASK_CLASSES)
    assert kept == attention_module._MASK_CLASSES_MAX
    again = attn._classify_mask(masks[-1], 1, 4, 4, 2)            # a cached answer: the same byte tensor
    assert again[1] is attention_module._MASK_CLASSES[id(masks[-1])][3]
    del masks, m, again
    gc.collect()
    assert len(attention_module._MASK_CLASSES) == 0
