"""Host side of the paged KV cache (page bookkeeping with the reference's method names) and the pins of
the paged compaction oracle.  No GPU."""
import pytest
import torch

from oracle import kv as okv
from subspec_amd.paged_cache import KvCachePool, RequestKvCache


def _pool(max_pages=12, page_len=4):
    return KvCachePool(max_pages, num_layers=2, num_heads=2, head_dim=8, page_len=page_len, dtype=torch.float32, device="cpu")


def test_pool_allocation_and_request_lengths():
    pool = _pool()
    assert int(pool.num_free_pages()) == 12
    req = RequestKvCache(pool, 4, seq_init_len=9)            # 3 pages, last one holds 1 token
    assert req.kv_page_indices == [0, 1, 2] and req.kv_last_page_len == 1 and req.get_seq_length() == 9
    other = RequestKvCache(pool, 4, seq_init_len=4)
    assert other.kv_page_indices == [3] and other.kv_last_page_len == 4
    req.increment(3)                                          # 12 tokens: still 3 pages
    assert req.kv_page_indices == [0, 1, 2] and req.kv_last_page_len == 4
    req.increment(1)                                          # 13 tokens: a fourth page, the first free one
    assert req.kv_page_indices == [0, 1, 2, 4] and req.kv_last_page_len == 1 and req.get_seq_length() == 13
    req.decrement(2)                                          # 11 tokens: the page is returned
    assert req.kv_page_indices == [0, 1, 2] and req.kv_last_page_len == 3
    assert bool(pool.free_page_mask[4])
    req.decrement(100)                                        # clamps at zero
    assert req.get_seq_length() == 0 and req.kv_page_indices == [] and req.kv_last_page_len == 0
    other.release()
    assert other.is_released and int(pool.num_free_pages()) == 12
    with pytest.raises(AssertionError):
        pool.allocate(13)
    with pytest.raises(ValueError):
        KvCachePool(4, 1, 1, 8, page_len=6, dtype=torch.float32, device="cpu")


def test_request_crop_and_pool_crop():
    pool = _pool()
    req = RequestKvCache(pool, 4, seq_init_len=14)            # 4 pages
    req.crop(6)                                               # keep 6 tokens -> 2 pages
    assert req.get_seq_length() == 6 and req.kv_page_indices == [0, 1] and req.kv_last_page_len == 2
    req.crop(-2)                                              # negative: remove from the end
    assert req.get_seq_length() == 4 and req.kv_page_indices == [0] and req.kv_last_page_len == 4
    req.crop(9)                                               # end <= start: nothing happens
    assert req.get_seq_length() == 4
    pool.cache_data.fill_(1.0)
    pool.crop(6)
    assert pool.cache_data[:, 0].min() == 1 and pool.cache_data[:, 1, :, :2].min() == 1
    assert pool.cache_data[:, 1, :, 2:].abs().max() == 0 and pool.cache_data[:, 2:].abs().max() == 0
    assert pool.free_page_mask.tolist() == [False, False] + [True] * 10
    with pytest.raises(ValueError):
        pool.crop(12 * 4 + 1)


def test_append_places_rows_through_the_page_table():
    pool = _pool(max_pages=8, page_len=4)
    pool.allocate(2)                                          # someone else owns pages 0 and 1
    req = RequestKvCache(pool, 4, seq_init_len=3)             # page 2
    g = torch.Generator().manual_seed(0)
    k, v = torch.randn(6, 2, 8, generator=g), torch.randn(6, 2, 8, generator=g)
    table = req.append(1, k, v)                               # rows 3..8 -> pages 2, 3, 4
    assert table.tolist() == [2, 3, 4] and req.get_seq_length() == 3
    kk, vv = okv.gather_paged(pool.cache_data[1], table, 9)
    assert torch.equal(kk[0, :, 3:9].transpose(0, 1), k) and torch.equal(vv[0, :, 3:9].transpose(0, 1), v)
    assert pool.cache_data[0].abs().max() == 0                # other layers untouched


@pytest.mark.parametrize("seed", range(6))
def test_paged_compaction_oracle_pins(seed):
    g = torch.Generator().manual_seed(seed)
    L, max_pages, page_len, H, D = 2, 10, 4, 2, 8
    pool = torch.randn(L, max_pages, 2, page_len, H, D, generator=g)
    offset = int(torch.randint(0, 9, (1,), generator=g))
    n = int(torch.randint(1, 12, (1,), generator=g))
    ctx = torch.sort(torch.randperm(24, generator=g)[:n]).values.tolist()      # ascending, as accepted paths are
    # identity table: the literal reference algorithm
    ident = list(range(max_pages))
    ref = okv.compact_paged_reference(pool, ctx, offset)
    assert torch.equal(okv.compact_paged(pool, ident, ctx, offset), ref)
    # rows outside [offset, offset + n) and the other plane positions are untouched
    flat_ref = ref[:, :, 0].reshape(L, -1, H, D)
    flat_in = pool[:, :, 0].reshape(L, -1, H, D)
    assert torch.equal(flat_ref[:, :offset], flat_in[:, :offset]) and torch.equal(flat_ref[:, offset + n:], flat_in[:, offset + n:])
    for j, c in enumerate(ctx):
        assert torch.equal(flat_ref[:, offset + j], flat_in[:, offset + c])
    # a permuted table: the same logical result on the request's own pages, everything else untouched
    perm = torch.randperm(max_pages, generator=g).tolist()
    got = okv.compact_paged(pool, perm, ctx, offset)
    logical_in = pool[:, perm].clone()                         # pages in sequence order
    logical_out = okv.compact_paged_reference(logical_in, ctx, offset)
    assert torch.equal(got[:, perm], logical_out)


def test_paged_cache_behind_the_static_cache_interface():
    """PagedKVCache on the CPU: pages are taken as rows are first needed, writes land where the page table says,
    prefix_kv gathers them back in logical order, crop hands whole pages back."""
    from subspec_amd.cache import create_kv_cache
    from subspec_amd.model import DecoderConfig
    cfg = DecoderConfig(num_hidden_layers=2, hidden_size=64, num_attention_heads=2, num_key_value_heads=2, head_dim=8,
                        intermediate_size=64, vocab_size=50)
    kv = create_kv_cache("paged", max_cache_len=100, config=cfg, device="cpu", dtype=torch.float32)
    c = kv.cache
    assert c.max_cache_len == 112 and not c.contiguous and not c.growable         # 7 pages of 16 rows
    held = c.pool.allocate(2)
    c.ensure(40)                                                                   # 3 pages: physical 2, 3, 4
    assert c.table().tolist() == [2, 3, 4]
    c.pool.deallocate(held)
    g = torch.Generator().manual_seed(0)
    k = torch.randn(1, 2, 40, 8, generator=g)
    v = torch.randn(1, 2, 40, 8, generator=g)
    c.write(1, torch.arange(40), k, v)
    kk, vv = c.prefix_kv(1, 40)
    assert torch.equal(kk, k) and torch.equal(vv, v)
    assert torch.equal(c.pool.cache_data[1, 3, 0, 5], k[0, :, 21])                  # row 21 = page 1 (physical 3), token 5
    c.write(1, torch.arange(33, 36), k[:, :, :3], v[:, :, :3])                     # overwrite rows in the last page
    assert torch.equal(c.prefix_kv(1, 36)[0][0, :, 33:36], k[0, :, :3])
    c.ensure(50)                                                                   # a 4th page: the lowest free one
    assert c.table().tolist() == [2, 3, 4, 0]
    c.crop(17)
    assert c.table().tolist() == [2, 3] and int(c.pool.num_free_pages()) == 5
    with pytest.raises(ValueError):
        c.ensure(113)
    kv.reset()
    assert c.table().numel() == 0 and int(c.pool.num_free_pages()) == 7
    with pytest.raises(ValueError):
        create_kv_cache("paged", config=cfg)
