"""Host-side refusals: block tables and page ids that would make a kernel index outside
the pool are turned into ValueError before anything is launched (all on the CPU)."""
import pytest
import torch

from deserve_amd.execution.graph import GraphedDecodeStep
from deserve_amd.kvcache import _native
from deserve_amd.kvcache.paged.page_pool import PagePool
from deserve_amd.paged_ops import (BatchDecodeWithPagedKVCacheWrapper,
                                   BatchPrefillWithPagedKVCacheWrapper)

CPU = torch.device("cpu")


def _i32(x):
    return torch.tensor(x, dtype=torch.int32)


def _decode():
    return BatchDecodeWithPagedKVCacheWrapper(torch.empty(16, dtype=torch.uint8))


def test_decode_begin_forward_refuses_bad_block_tables():
    shape = dict(num_qo_heads=32, num_kv_heads=8, head_dim=128, page_size=16)
    with pytest.raises(ValueError, match="indptr\\[-1\\] is 3"):
        _decode().begin_forward(_i32([0, 1, 3]), _i32([5, 6]), _i32([16, 4]), **shape)
    with pytest.raises(ValueError, match="negative page id -2"):
        _decode().begin_forward(_i32([0, 1, 3]), _i32([5, -2, 7]), _i32([16, 4]), **shape)
    with pytest.raises(ValueError, match="not decrease"):
        _decode().begin_forward(_i32([0, 2, 1]), _i32([5, 6]), _i32([16, 4]), **shape)
    with pytest.raises(ValueError, match="indices_host holds 1"):
        _decode().begin_forward(_i32([0, 1, 3]), _i32([5, 6, 7]), _i32([16, 4]), indices_host=_i32([5]),
                                indptr_host=_i32([0, 1, 3]), last_page_len_host=_i32([16, 4]), **shape)
    with pytest.raises(ValueError, match="1 entries for 2 requests"):
        _decode().begin_forward(_i32([0, 1, 3]), _i32([5, 6, 7]), _i32([16]), **shape)
    with pytest.raises(ValueError, match="kv_last_page_len\\[1\\] = 17 outside \\[1, 16\\]"):
        _decode().begin_forward(_i32([0, 1, 3]), _i32([5, 6, 7]), _i32([16, 17]), **shape)


def test_forward_refuses_a_pool_that_lacks_a_named_page_or_has_another_shape():
    w = _decode()
    w._shape_args(32, 8, 128, 16)
    w._check_block_tables(_i32([0, 1, 3]), _i32([5, 40, 7]), None, _i32([16, 4]))
    assert w._max_page_id == 40
    ok = torch.empty((41, 2, 16, 8, 128), dtype=torch.bfloat16)
    w._check_pool(ok, torch.bfloat16)
    with pytest.raises(ValueError, match="name page 40, the pool has 40 pages"):
        w._check_pool(ok[:40], torch.bfloat16)
    with pytest.raises(ValueError, match="as given to begin_forward"):
        w._check_pool(torch.empty((41, 2, 8, 8, 128), dtype=torch.bfloat16), torch.bfloat16)
    with pytest.raises(ValueError, match="as given to begin_forward"):
        w._check_pool(torch.empty((41, 2, 16, 8, 64), dtype=torch.bfloat16), torch.bfloat16)
    with pytest.raises(ValueError, match="dtype"):
        w._check_pool(ok, torch.float16)
    with pytest.raises(ValueError, match="contiguous"):
        w._check_pool(torch.empty((41, 2, 16, 8, 256), dtype=torch.bfloat16)[..., ::2], torch.bfloat16)


def test_fused_append_refuses_a_plan_with_a_request_that_owns_no_page():
    """forward(k_append=) writes the step's token into the page slot the block table names
    for it (model/layer/attention.py:175-185): a request without a page has no such slot, and
    the refusal comes from the host, before anything is launched."""
    from deserve_amd import _lib

    w = _decode()
    w._shape_args(32, 8, 128, 16)
    h_indptr, h_last = _i32([0, 0, 3, 4]), _i32([16, 8, 3])
    w._check_block_tables(h_indptr, _i32([1, 2, 3, 0]), None, h_last)
    cap = int(_lib.lib().dskv_decode_plan_bound(3, 4 * 16))
    w._plan_into(torch.zeros(cap, dtype=torch.int32), cap, h_indptr, h_last, 0)
    assert w._empty_requests == [0]
    w._planned = True
    q = torch.zeros((3, 32, 128), dtype=torch.bfloat16)
    k = torch.zeros((3, 8, 128), dtype=torch.bfloat16)
    pages = torch.zeros((4, 2, 16, 8, 128), dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="\\[0\\] have no page"):
        w.forward(q, pages, k_append=k, v_append=k)
    assert not pages.any()
    # a plan whose requests all own a page passes this check
    w._plan_into(torch.zeros(cap, dtype=torch.int32), cap, _i32([0, 1, 3, 4]), h_last, 0)
    assert w._empty_requests == []


def test_prefill_begin_forward_refuses_bad_block_tables():
    w = BatchPrefillWithPagedKVCacheWrapper(torch.empty(16, dtype=torch.uint8))
    shape = dict(num_qo_heads=32, num_kv_heads=8, head_dim=128, page_size=16)
    with pytest.raises(ValueError, match="disagree about the batch"):
        w.begin_forward(_i32([0, 4]), _i32([0, 1, 2]), _i32([3, 4]), _i32([4, 4]), **shape)
    with pytest.raises(ValueError, match="negative page id"):
        w.begin_forward(_i32([0, 4, 8]), _i32([0, 1, 2]), _i32([3, -1]), _i32([4, 4]), **shape)
    with pytest.raises(ValueError, match="indptr\\[-1\\] is 2"):
        w.begin_forward(_i32([0, 4, 8]), _i32([0, 1, 2]), _i32([3]), _i32([4, 4]), **shape)
    with pytest.raises(ValueError, match="qo_indptr"):
        w.begin_forward(_i32([0, 4, 2]), _i32([0, 1, 2]), _i32([3, 4]), _i32([4, 4]), **shape)
    with pytest.raises(ValueError, match="kv_last_page_len\\[0\\] = 0 outside"):
        w.begin_forward(_i32([0, 4, 8]), _i32([0, 1, 2]), _i32([3, 4]), _i32([0, 4]), **shape)
    with pytest.raises(ValueError, match="1 entries for 2 requests"):
        w.begin_forward(_i32([0, 4, 8]), _i32([0, 1, 2]), _i32([3, 4]), _i32([4]), **shape)


def test_gather_and_scatter_refuse_page_ids_outside_the_pool():
    pool = PagePool(2, 8, 4, CPU, torch.float16, n_kv_heads=1, head_dim=8)
    for bad in ([0, 8], [-1, 3]):
        with pytest.raises(ValueError, match="page ids span"):
            _native.gather_pages(pool, _i32(bad))
        with pytest.raises(ValueError, match="page ids span"):
            pool.retrieve(_i32(bad))
        with pytest.raises(ValueError, match="page ids span"):
            _native.scatter_pages(pool, _i32(bad), torch.zeros((2 * 2, 2, 4, 1, 8), dtype=torch.float16))
    with pytest.raises(ValueError, match="hold 2 x 2 pages"):
        _native.scatter_pages(pool, _i32([1, 2]), torch.zeros((3, 2, 4, 1, 8), dtype=torch.float16))


def test_graph_key_holds_the_item_count_only_for_the_kernel_launched_per_item():
    q = [torch.empty((2, 4, 8, 64))]
    key = GraphedDecodeStep.graph_key
    # persistent kernel: 5 and 7 items of 4 requests replay the same graph ...
    assert key(4, 4, 5, q, True) == key(4, 4, 7, q, True)
    # ... unless the step changes from nothing-to-merge to merge, or to the wide merge
    assert key(4, 4, 4, q, True) != key(4, 4, 5, q, True)
    assert key(4, 4, 5, q, True) != key(4, 4, 129, q, True)
    # one workgroup per item: every item count is a graph of its own
    assert key(4, 4, 5, q, False) != key(4, 4, 7, q, False)
    assert key(4, 4, 5, q, False) == key(4, 4, 5, q, False)
    assert key(4, 4, 5, q, False) != key(4, 4, 5, q, True)
    assert key(4, 4, 5, q, True) != key(3, 4, 5, q, True) and key(4, 4, 5, q, True) != key(4, 8, 5, q, True)


@pytest.mark.gpu
def test_prefill_plan_falls_back_to_whole_tiles_when_the_workspace_cannot_hold_the_parts():
    """One 512-token chunk over 4096 tokens is planned in parts that need 34 MB of partials;
    with a 1 MiB workspace the wrapper plans whole tiles instead (no workspace needed)."""
    dev = torch.device("cuda")
    qo, kv_indptr = _i32([0, 512]).to(dev), _i32([0, 288]).to(dev)
    ids, last = torch.arange(288, dtype=torch.int32, device=dev), _i32([16]).to(dev)
    shape = dict(num_qo_heads=32, num_kv_heads=8, head_dim=128, page_size=16, target_workgroups=256)
    small = BatchPrefillWithPagedKVCacheWrapper(torch.empty(1 << 20, dtype=torch.uint8, device=dev))
    big = BatchPrefillWithPagedKVCacheWrapper(torch.empty(64 << 20, dtype=torch.uint8, device=dev))
    for w in (small, big):
        w.begin_forward(qo, kv_indptr, ids, last, **shape)
    assert (small._n_splits, small._n_tiles) == (1, 8)
    assert (big._n_splits, big._n_tiles) == (4, 32)
