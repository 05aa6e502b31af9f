"""Writes tests/golden/attention_small.npz from the numpy oracle (seeded).

Run from the repository root:  python tests/golden/make_golden.py
The file pins the oracle's outputs against accidental change; it is data only.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from kvutil import make_scenario  # noqa: E402
from oracle import kv_oracle as orc  # noqa: E402


def main() -> None:
    # decode: 3 requests, ragged last pages, GQA 8q/2kv, D 32, P 4, fp32
    d = make_scenario(11, kv_lens=[5, 16, 1], qo_lens=[1, 1, 1], P=4, Hq=8, Hkv=2, D=32,
                      dtype="f32")
    d_out = orc.decode_attention(d.q, d.pages, d.kv_page_indices, d.kv_page_indptr,
                                 d.kv_last_page_lens, "f32")
    # prefill: chunk of 3 and 5 new tokens over priors of 4 and 0
    p = make_scenario(12, kv_lens=[7, 5], qo_lens=[3, 5], P=4, Hq=4, Hkv=2, D=32, dtype="f32")
    p_out = orc.prefill_attention(p.q, p.qo_indptr, p.pages, p.kv_page_indices, p.kv_page_indptr,
                                  p.kv_last_page_lens, "f32", causal=True)
    np.savez_compressed(
        os.path.join(HERE, "attention_small.npz"),
        d_q=d.q, d_pages=d.pages, d_indices=d.kv_page_indices, d_indptr=d.kv_page_indptr,
        d_last=d.kv_last_page_lens, d_out=d_out,
        p_q=p.q, p_qo=p.qo_indptr, p_pages=p.pages, p_indices=p.kv_page_indices,
        p_indptr=p.kv_page_indptr, p_last=p.kv_last_page_lens, p_out=p_out)


if __name__ == "__main__":
    main()
