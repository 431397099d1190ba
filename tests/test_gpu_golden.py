"""The committed fixtures of tests/golden against the HIP kernels (through the C ABI)."""

import json
import os

import numpy as np
import pytest
import torch

from easydel_amd import kernels

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def test_slice_scatter_reproduces_the_reference_vectors(gpu):
    with open(os.path.join(GOLDEN, "reference_vectors.json")) as f:
        vectors = json.load(f)["kv_cache_update"]
    for v in vectors:
        new = torch.tensor(v["new_tokens"], dtype=torch.float32, device=gpu)
        cache = torch.zeros(v["cache_shape"], dtype=torch.float32, device=gpu)
        kernels.page_scatter_slices(new, torch.tensor(v["slice_indices"], dtype=torch.int32, device=gpu),
                                    torch.tensor([v["total_update_slices"]], dtype=torch.int32, device=gpu), cache,
                                    page_size=v["page_size"], page_shard_index=v["page_shard_index"])
        torch.cuda.synchronize()
        assert np.array_equal(cache.cpu().numpy(), np.array(v["expected"], np.float32)), v["name"]


@pytest.mark.parametrize("layout", ["interleaved", "separate pools"])
def test_attention_reproduces_the_c1_fixture(gpu, layout):
    z = np.load(os.path.join(GOLDEN, "attention_c1_fp32.npz"))
    pages = np.zeros((int(z["num_pages"]), 16, 4, 64), np.float32)
    pages[z["live_pages"]] = z["live_page_values"]
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(gpu)  # noqa: E731
    args = (dev(z["context_lens"]), dev(z["block_tables"]), dev(z["query_start_loc"]), dev(z["num_seqs"]))
    if layout == "interleaved":
        out = kernels.ragged_paged_attention(dev(z["query"]), dev(pages), *args, softmax_scale=float(z["softmax_scale"]), num_kv_heads=2)
    else:
        out = kernels.unified_attention(dev(z["query"]), dev(pages[:, :, 0::2]), dev(pages[:, :, 1::2]), *args,
                                        softmax_scale=float(z["softmax_scale"]))
    torch.cuda.synchronize()
    assert np.abs(out.cpu().numpy() - z["expected"]).max() <= 1e-5
