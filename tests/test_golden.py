"""The committed fixtures of tests/golden against the oracle and the host-side code (no GPU)."""

import json
import os

import numpy as np
import torch

from easydel_amd.caching import RaggedPagesCacheConfig, request_distribution
from rpa_testlib import orc

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _vectors():
    with open(os.path.join(GOLDEN, "reference_vectors.json")) as f:
        return json.load(f)


def test_oracle_scatter_reproduces_the_reference_vectors():
    for v in _vectors()["kv_cache_update"]:
        new = np.array(v["new_tokens"], np.float32)
        got = orc.kv_cache_update_ref(new, np.array(v["slice_indices"], np.int32), np.zeros(v["cache_shape"], np.float32),
                                      [v["total_update_slices"]], page_size=v["page_size"], page_shard_index=v["page_shard_index"])
        assert np.array_equal(got, np.array(v["expected"], np.float32)), v["name"]
    for v in _vectors()["localize_slice_indices"]:
        got = orc.localize_slice_indices_ref(np.array(v["slice_indices"], np.int32), [v["total_update_slices"]], page_size=v["page_size"],
                                             local_flat_cache_positions=v["local_flat_cache_positions"], page_shard_index=v["page_shard_index"])
        assert np.array_equal(got, np.array(v["expected"], np.int32)), v["name"]


def test_request_distribution_reproduces_the_reference_vectors():
    for v in _vectors()["request_distribution"]:
        assert list(orc.request_distribution_ref(v["scheduled"], v["context_lens"])) == v["expected"], v["source"]
        assert list(request_distribution(v["scheduled"], v["context_lens"])) == v["expected"], v["source"]


def test_storage_layout_reproduces_the_reference_numbers():
    dtypes = {32: torch.float32, 16: torch.bfloat16, 8: torch.float8_e4m3fn}
    for v in _vectors()["storage_layout"]:
        lay = orc.storage_layout_ref(v["num_kv_heads"], v["head_dim"], v["bits"])
        assert (lay["packing"], lay["combined"], lay["groups"], lay["head_dim"]) == (v["packing"], v["combined"], v["groups"], v["storage_head_dim"])
        cfg = RaggedPagesCacheConfig.create(dtypes[v["bits"]], num_hidden_layers=1, num_kv_heads=v["num_kv_heads"], max_model_length=64,
                                            kv_head_dim_size=v["head_dim"], page_size=16, num_pages=2)
        assert (cfg.kv_head_packing, cfg.storage_num_combined_kv_heads, cfg.storage_num_kv_groups, cfg.storage_head_dim) == \
               (v["packing"], v["combined"], v["groups"], v["storage_head_dim"])


def test_attention_fixture_is_what_the_oracle_computes():
    z = np.load(os.path.join(GOLDEN, "attention_c1_fp32.npz"))
    pages = np.zeros((int(z["num_pages"]), 16, 4, 64), np.float32)
    pages[z["live_pages"]] = z["live_page_values"]
    got = orc.ragged_paged_attention_ref(z["query"].astype(np.float64), pages.astype(np.float64), z["context_lens"], z["block_tables"],
                                         z["query_start_loc"], z["num_seqs"], softmax_scale=float(z["softmax_scale"]))
    assert np.abs(got - z["expected"]).max() <= 1e-6
    assert list(z["query_start_loc"][:5]) == [0, 1, 2, 10, 43]
