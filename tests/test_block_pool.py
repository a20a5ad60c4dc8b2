"""Host logic of the paged mode: block pool bookkeeping and the paged cache's allocation rules, no GPU needed.

The cases are those of the reference's own tests (crates/hyprstream/src/runtime/kv_cache.rs):
test_block_pool_allocate_free :2424-2464, test_paged_update_exhaustion_is_fail_soft :2671-2695,
test_cross_owner_free_is_rejected :2698-2742 (the parts that run before any tensor is touched)."""
import ctypes

import pytest

from hyprstream_amd import bindings as hb
from hyprstream_amd import kv_cache as kc


def test_block_pool_allocate_free():
    pool = kc.BlockPool(4, 2, 64)
    owner = 1  # CacheOwner::Stateless(1)
    assert pool.total_blocks() == 4 and pool.free_block_count() == 4 and pool.used_blocks() == 0
    b0, b1, b2 = pool.allocate(owner), pool.allocate(owner), pool.allocate(owner)
    assert len({b0, b1, b2}) == 3
    assert pool.used_blocks() == 3 and pool.free_block_count() == 1
    b3 = pool.allocate(owner)
    assert pool.free_block_count() == 0
    with pytest.raises(kc.BlockPoolExhausted) as e:  # fail-soft typed error, not a generic failure
        pool.allocate(owner)
    assert e.value.code == hb.HS_ERR_POOL_EXHAUSTED and str(e.value) == "block pool exhausted (all 4 blocks in use)"
    pool.free(owner, b1)
    assert pool.free_block_count() == 1
    assert pool.allocate(owner) == b1  # LIFO: the block just freed comes back
    for b in (b0, b1, b2, b3):
        pool.free(owner, b)
    assert pool.free_block_count() == 4 and pool.used_memory() == 0


def test_used_memory_counts_codes_and_scales():
    pool = kc.BlockPool(3, 8, 128)
    pool.allocate("s")
    assert pool.used_memory() == 8 * 256 * (128 + 4)


def test_cross_owner_free_is_rejected():
    pool = kc.BlockPool(4, 2, 64)
    block = pool.allocate("alice")
    assert pool.owner_of(block) == "alice"
    with pytest.raises(kc.CacheError) as e:
        pool.free("bob", block)
    assert "cross-owner block free rejected" in str(e.value)
    assert pool.owner_of(block) == "alice" and pool.used_blocks() == 1  # ownership and use count untouched
    pool.free("alice", block)
    assert pool.used_blocks() == 0 and pool.owner_of(block) is None


def test_owner_identity_is_kind_id_and_name():
    pool = kc.BlockPool(4, 2, 64)
    a = pool.allocate(7)               # Stateless(7)
    b = pool.allocate(("run", 7))      # Training("run", 7)
    assert pool.owner_of(a) == 7 and pool.owner_of(b) == ("run", 7)
    with pytest.raises(kc.CacheError):
        pool.free(8, a)                # another stateless id
    with pytest.raises(kc.CacheError):
        pool.free(7, b)                # same id, different kind
    pool.free(7, a)
    pool.free(("run", 7), b)
    assert pool.used_blocks() == 0


def test_double_free_and_invalid_ids_change_nothing():
    pool = kc.BlockPool(2, 2, 64)
    b = pool.allocate(1)
    pool.free(1, b)
    with pytest.raises(kc.CacheError) as e:
        pool.free(1, b)
    assert "double-free" in str(e.value)
    for bad in (-1, 2, 99):
        with pytest.raises(kc.CacheError):
            pool.free(1, bad)
        assert pool.owner_of(bad) is None
    assert pool.free_block_count() == 2


def test_paged_update_exhaustion_is_fail_soft_and_rolls_back():
    # one block cannot hold a (K, V) pair: the key block taken first goes back (kv_cache.rs:2671-2695)
    pool = kc.BlockPool(1, 2, 64)
    L = kc.lib()
    c = ctypes.c_void_p(L.hs_paged_cache_create(1024, pool._h, 0, 1, None))
    p = ctypes.c_void_p(0x1000)  # never dereferenced: the allocation fails before any device work
    rc = L.hs_paged_cache_update(c, p, p, hb.HS_BF16, 10, ctypes.c_int64(0), None)
    assert rc == hb.HS_ERR_POOL_EXHAUSTED
    assert L.hs_paged_cache_last_error(c) == b"block pool exhausted (all 1 blocks in use)"
    assert pool.used_blocks() == 0 and L.hs_paged_cache_seq_pos(c) == 0 and L.hs_paged_cache_num_blocks(c) == 0
    L.hs_paged_cache_destroy(c)


def test_paged_update_overflow_and_empty_get():
    pool = kc.BlockPool(8, 2, 64)
    L = kc.lib()
    c = ctypes.c_void_p(L.hs_paged_cache_create(300, pool._h, 1, 0, b"s"))
    p = ctypes.c_void_p(0x1000)
    assert L.hs_paged_cache_update(c, p, p, hb.HS_BF16, 10, ctypes.c_int64(295), None) == hb.HS_ERR_OVERFLOW
    assert L.hs_paged_cache_last_error(c) == (b"Cache overflow: trying to cache 10 tokens starting at position 295, "
                                              b"but max_seq_len is 300")
    assert pool.used_blocks() == 0
    assert L.hs_paged_cache_get_dense(c, p, p, hb.HS_BF16, None) != hb.HS_OK
    assert L.hs_paged_cache_last_error(c) == b"Cache is empty"
    L.hs_paged_cache_destroy(c)


def test_pool_outlives_its_handle_while_caches_exist():
    pool = kc.BlockPool(4, 2, 64)
    L = kc.lib()
    c = ctypes.c_void_p(L.hs_paged_cache_create(512, pool._h, 0, 3, None))
    h = pool._h
    pool._h = None          # drop the Python owner without destroying twice
    L.hs_pool_destroy(h)    # the blocks live on: the cache holds the pool
    L.hs_paged_cache_clear(c)
    assert L.hs_paged_cache_seq_pos(c) == 0
    L.hs_paged_cache_destroy(c)
