"""The reference's CPU path for one decode step of one layer, restated with torch on the
host.

TEST INFRASTRUCTURE ONLY: the timed CPU baseline of the bench and a cross-check in the
tests.  Nothing in the shipped package imports it.

What the reference runs when its KV cache lives on the host (paths relative to the
reference repository's ``deserve_worker/`` package):

* storage: ``CpuPagePool`` (kvcache/paged/page_pool.py:97-107) - one torch tensor
  ``pages: (L, num_pages, 2, P, Hkv, D)`` on the CPU;
* append: the new token's K and V rows are index-assigned into slot
  ``(kv_len - 1) % P`` of the request's last page (the semantics of the append call
  site model/layer/attention.py:174-183, stated with torch indexing);
* gather: ``pages[layer, table]`` - advanced indexing with the request's block table,
  the gather of page_pool.py:78-82 / kvcache/manager.py:37-42;
* attention: ``repeat_kv`` (model/layer/attention.py:75-84), ``scores = q k^T /
  sqrt(D)``, ``softmax(scores.float())``, ``scores v`` per request, as
  ``Attention.traced_forward`` does (model/layer/attention.py:241-266; no mask: a
  decode step has one query).

Pinned by tests/test_oracle_data.py against the numpy oracle (kv_oracle.decode_attention,
itself pinned by scipy's softmax and closed forms) and the brute-force append.
"""
from __future__ import annotations

import math
from typing import Sequence

import torch


def repeat_kv(x: torch.Tensor, n_rep: int) -> torch.Tensor:
    """(bs, slen, Hkv, D) -> (bs, slen, Hkv * n_rep, D), head h of the result = kv head h // n_rep."""
    bs, slen, n_kv_heads, head_dim = x.shape
    if n_rep == 1:
        return x
    return x[:, :, :, None, :].expand(bs, slen, n_kv_heads, n_rep, head_dim).reshape(
        bs, slen, n_kv_heads * n_rep, head_dim)


def decode_step(pages: torch.Tensor, layer: int, tables: Sequence[torch.Tensor], kv_lens: Sequence[int],
                q: torch.Tensor, k_new: torch.Tensor, v_new: torch.Tensor) -> torch.Tensor:
    """pages: (L, num_pages, 2, P, Hkv, D) on the CPU; tables[b]: int64 page ids of request
    b; kv_lens[b]: its length INCLUDING the step's token; q: (B, Hq, D); k_new, v_new:
    (B, Hkv, D).  Appends in place, returns the attention output (B, Hq, D)."""
    P, Hkv, D = pages.shape[3], pages.shape[4], pages.shape[5]
    Hq = q.shape[1]
    n_rep = Hq // Hkv
    outs = []
    for b, (table, n) in enumerate(zip(tables, kv_lens)):
        # append: index-assign the new rows
        pos = n - 1
        page = table[pos // P]
        pages[layer, page, 0, pos % P] = k_new[b]
        pages[layer, page, 1, pos % P] = v_new[b]
        # gather: pages[layer, table] -> (n_pages, 2, P, Hkv, D)
        mine = pages[layer, table]
        keys = mine[:, 0].reshape(1, -1, Hkv, D)[:, :n]
        values = mine[:, 1].reshape(1, -1, Hkv, D)[:, :n]
        keys = repeat_kv(keys, n_rep).transpose(1, 2)            # (1, Hq, n, D)
        values = repeat_kv(values, n_rep).transpose(1, 2)
        xq = q[b].view(1, 1, Hq, D).transpose(1, 2)              # (1, Hq, 1, D)
        scores = torch.matmul(xq, keys.transpose(2, 3)) / math.sqrt(D)
        scores = torch.nn.functional.softmax(scores.float(), dim=-1).type_as(xq)
        out = torch.matmul(scores, values)                       # (1, Hq, 1, D)
        outs.append(out.transpose(1, 2).reshape(Hq, D))
    return torch.stack(outs)
