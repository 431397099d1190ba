"""Writes the fixture files of this folder.  Run from the repository root: ``python tests/golden/make_fixtures.py``.

Two kinds of fixture, told apart by their ``source`` field:

* ``reference-test``: the input / expected-output vectors that the reference's own tests hold for this path, typed
  in from those tests (file and lines in ``source``).  Where such a test draws its inputs at random and expects a
  pure copy, the inputs here are seeded numpy draws of the same shape: the expected output is a function of them.
* ``oracle``: inputs of a small attention case together with the float64 oracle's output, as a regression vector
  for the GPU kernels.  The oracle's attention is pinned by mathematics only (the arithmetic lives in ejkernel,
  which is not vendored), so these vectors carry no more authority than the oracle itself.

Nothing here imports or runs the reference.
"""

from __future__ import annotations

import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(HERE))


def kv_cache_update_vectors():
    rng = np.random.default_rng(0)
    out = []
    # tests/layers/caching/test_kv_cache_update_jax.py:84-119 -- three slices of lengths 3, 2, 2 land at 10, 20, 30
    new_tokens = rng.standard_normal((16, 4, 8)).astype(np.float32)
    lens = np.array([3, 2, 2, 0, 0], dtype=np.int32)
    src = np.concatenate(([0], np.cumsum(lens[:-1]))).astype(np.int32)
    dst = np.array([10, 20, 30, 0, 0], dtype=np.int32)
    expected = np.zeros((64, 4, 8), np.float32)
    for i in range(3):
        expected[dst[i]:dst[i] + lens[i]] = new_tokens[src[i]:src[i] + lens[i]]
    out.append(dict(name="slice_mapping", source="tests/layers/caching/test_kv_cache_update_jax.py:84-119",
                    new_tokens=new_tokens.tolist(), cache_shape=[64, 4, 8], slice_indices=np.stack([dst, src, lens]).tolist(),
                    total_update_slices=3, page_size=4, page_shard_index=0, expected=expected.tolist()))
    # :149-180 -- shard 1 of a two-shard cache keeps only the slices that fall on its pages, at local offsets
    new_tokens = np.arange(6 * 2 * 4, dtype=np.float32).reshape(6, 2, 4)
    expected = np.zeros((8, 2, 4), np.float32)
    expected[0:2] = new_tokens[2:4]
    expected[4:6] = new_tokens[4:6]
    out.append(dict(name="page_shard_local_offsets", source="tests/layers/caching/test_kv_cache_update_jax.py:149-180",
                    new_tokens=new_tokens.tolist(), cache_shape=[8, 2, 4], slice_indices=[[0, 8, 12, 0], [0, 2, 4, 0], [2, 2, 2, 0]],
                    total_update_slices=3, page_size=4, page_shard_index=1, expected=expected.tolist()))
    return out


def localize_vectors():
    # test_kv_cache_update_jax.py:122-146
    return [dict(name="localize_zeroes_non_local", source="tests/layers/caching/test_kv_cache_update_jax.py:122-146",
                 slice_indices=[[0, 5, 8, 13], [0, 1, 2, 4], [1, 1, 2, 1]], total_update_slices=4, page_size=4,
                 local_flat_cache_positions=8, page_shard_index=1, expected=[[0, 0, 0, 5], [0, 0, 2, 4], [0, 0, 2, 1]])]


def request_distribution_vectors():
    src = "tests/inference/test_request_distribution_bounds.py"
    return [dict(source=src + ":31-37", scheduled=[4], context_lens=[4], expected=[0, 1, 1]),
            dict(source=src + ":38-44", scheduled=[4, 1, 0], context_lens=[4, 9, 0], expected=[1, 2, 2]),
            dict(source=src + ":47-58", scheduled=[4, 1, 0, 0], context_lens=[4, 9, 0, 0], expected=[1, 2, 2])]


def storage_layout_vectors():
    # The layout arithmetic is easydel/caching/ragged_page/cache.py:143-158 (elements per 32 bits) and :606-647
    # (combined heads aligned to the packing, groups = combined / packing, head_dim 64 stored as K|V rows of 128).
    # The reference's test of it, tests/layers/caching/test_ragged_page_dtype_compat.py:34-60, pins one consequence:
    # 4 KV heads of fp8 give 2 groups, which 4 head shards do not divide (second vector below).
    src = "easydel/caching/ragged_page/cache.py:143-158, 606-647"
    return [dict(source=src, num_kv_heads=8, head_dim=128, bits=16, packing=2, combined=16, groups=8, storage_head_dim=128),
            dict(source=src + "; tests/layers/caching/test_ragged_page_dtype_compat.py:48-56", num_kv_heads=4, head_dim=128, bits=8,
                 packing=4, combined=8, groups=2, storage_head_dim=128),
            dict(source=src, num_kv_heads=2, head_dim=64, bits=32, packing=1, combined=2, groups=2, storage_head_dim=128)]


def attention_c1():
    """The tiny fp32 configuration: 4 sequences, ctx [17,64,130,255], q_lens [1,1,8,33], Hq 8, Hkv 2, D 64, page 16."""
    import rpa_testlib as tl

    b = tl.make_batch(0, [17, 64, 130, 255], [1, 1, 8, 33], Hq=8, Hkv=2, D=64, page_size=16, num_pages=128,
                      q_dtype=tl.F32, kv_dtype=tl.F32)
    live = np.unique(b.block_tables[b.block_tables > 0])
    want = tl.oracle_out(b, softmax_scale=0.125)
    np.savez_compressed(os.path.join(HERE, "attention_c1_fp32.npz"), source=np.array("oracle"),
                        query=b.q_raw.astype(np.float32), live_pages=live.astype(np.int32),
                        live_page_values=b.kv_raw[live].astype(np.float32), num_pages=np.int32(b.kv_raw.shape[0]),
                        context_lens=b.context_lens, block_tables=b.block_tables, query_start_loc=b.query_start_loc,
                        num_seqs=b.num_seqs, softmax_scale=np.float32(0.125), expected=want.astype(np.float32))


def main():
    with open(os.path.join(HERE, "reference_vectors.json"), "w") as f:
        json.dump(dict(kv_cache_update=kv_cache_update_vectors(), localize_slice_indices=localize_vectors(),
                       request_distribution=request_distribution_vectors(), storage_layout=storage_layout_vectors()), f)
    attention_c1()


if __name__ == "__main__":
    main()
