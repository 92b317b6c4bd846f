"""Host half of the paged cache's decode append (no GPU): page-table growth, the fixed-address
table that a recorded decode step needs, and the error paths."""
import pytest
import torch

from twilight_amd.cache import PagedKVCache


def _cache():
    c = PagedKVCache(10, 1, torch.float16, "cpu")
    c.set_page_table(torch.tensor([0, 1, 2], dtype=torch.int32), torch.tensor([0, 2, 3], dtype=torch.int32),
                     torch.tensor([16, 5], dtype=torch.int32))
    return c


def test_advance_host_grows_the_table_when_a_last_page_is_full():
    c, free = _cache(), [5, 6, 7]
    assert c.max_pages_per_req == 2 and c._seq_lens == [32, 5]
    c.advance_host(free)                       # request 0 needs a new page, request 1 does not
    assert free == [6, 7]
    assert c.kv_page_indices.tolist() == [0, 1, 5, 2] and c.kv_page_indptr.tolist() == [0, 3, 4]
    # the device-side lengths are re-sent as they are BEFORE the token is written (the append
    # kernel adds one); the host mirror already counts the token
    assert c.kv_last_page_len.tolist() == [0, 5] and c._last == [1, 6] and c._seq_lens == [33, 6]
    assert c.max_pages_per_req == 3
    for _ in range(10):                        # request 1 fills its page after 10 more tokens
        c.advance_host(free)
    assert c._last == [11, 16] and free == [6, 7]
    c.advance_host(free)
    assert c.kv_page_indices.tolist() == [0, 1, 5, 2, 6] and c.kv_page_indptr.tolist() == [0, 3, 5]
    assert c._last == [12, 1] and free == [7]


def test_reserved_table_keeps_its_addresses_and_its_bound():
    c, free = _cache(), [5, 6]
    c.reserve_page_table(4)
    ind, ptr, last = c.kv_page_indices, c.kv_page_indptr, c.kv_last_page_len
    assert ind.numel() == 2 * 4 and ind[:3].tolist() == [0, 1, 2] and c.max_pages_per_req == 4
    c.advance_host(free)
    assert c.kv_page_indices is ind and c.kv_page_indptr is ptr and c.kv_last_page_len is last
    assert ind[:4].tolist() == [0, 1, 5, 2] and ptr.tolist() == [0, 3, 4] and c.max_pages_per_req == 4
    with pytest.raises(RuntimeError):
        c.reserve_page_table(2)                # below the longest request
    # a fresh page table drops the reservation
    c.set_page_table(torch.tensor([0], dtype=torch.int32), torch.tensor([0, 1], dtype=torch.int32),
                     torch.tensor([3], dtype=torch.int32))
    assert c._table_cap == 0 and c.max_pages_per_req == 1


def test_advance_host_error_paths():
    c = _cache()
    with pytest.raises(RuntimeError):
        c.advance_host([])                     # no free page for request 0
    c = _cache()
    c.reserve_page_table(2)
    with pytest.raises(RuntimeError):
        c.advance_host([7])                    # request 0 would outgrow the reserved table
