"""Pins the multi-latent attention oracle.  The arithmetic of the operation lives in ejkernel and the reference
holds no vector for it, so the oracle is pinned to the reference's own other branch of the same layer: with the
keys and values decompressed through the up-projection and ordinary attention run on them
(layers/attention/_unified.py:1240-1248, 1380-1395), the result must equal the absorbed form (queries times the key
half of the up-projection, attention over the latent rows, output times the value half; :1280-1371).  A dropped rope
term, a wrong scale, latent and rope parts swapped or misplaced in the page row, or a wrong position all fail it."""

import numpy as np
import pytest

from rpa_testlib import orc


def _mla_case(seed, ctx_lens, q_lens, *, heads=3, lkv=32, rope=8, nope=16, vdim=12, page_size=8):
    rng = np.random.default_rng(seed)
    n = len(ctx_lens)
    lay = orc.mla_page_layout_ref(lkv, rope, page_size)
    row = lay["kv_dim_padded"]
    need = [-(-c // page_size) for c in ctx_lens]
    P = sum(need) + 3
    perm = rng.permutation(np.arange(1, P))
    M = max(need)
    bt = np.zeros((n, M), np.int32)
    k = 0
    for i, m in enumerate(need):
        bt[i, :m] = perm[k:k + m]
        k += m
    qsl = np.concatenate([[0], np.cumsum(q_lens)]).astype(np.int32)
    T = int(qsl[-1])
    c = dict(n=n, bt=bt, qsl=qsl, ctx=np.asarray(ctx_lens, np.int32), T=T, lkv=lkv, rope=rope, nope=nope, vdim=vdim,
             heads=heads, page_size=page_size, P=P, row=row, off=lay["rope_offset"])
    c["w_k"] = rng.standard_normal((lkv, heads, nope))
    c["w_v"] = rng.standard_normal((lkv, heads, vdim))
    c["q_nope"] = rng.standard_normal((T, heads, nope))
    c["q_pe"] = rng.standard_normal((T, heads, rope))
    c["new_latent"] = rng.standard_normal((T, lkv))
    c["new_k_pe"] = rng.standard_normal((T, rope))
    pages = np.full((P, page_size, row), 1e6)  # poison: slots never written and the padding of a row must not be read
    # prior context: latent and rope rows of earlier steps
    for i in range(n):
        for pos in range(int(ctx_lens[i]) - int(q_lens[i])):
            r = pages[bt[i, pos // page_size], pos % page_size]
            r[:lkv] = rng.standard_normal(lkv)
            r[c["off"]:c["off"] + rope] = rng.standard_normal(rope)
    c["pages_before"] = pages
    return c


def _absorbed(c, **kw):
    pages = orc.mla_page_scatter_ref(c["new_latent"], c["new_k_pe"], c["pages_before"], c["ctx"], c["bt"], c["qsl"], [c["n"]])
    q_abs = np.einsum("tnd,and->tna", c["q_nope"], c["w_k"])
    scale = (c["nope"] + c["rope"]) ** -0.5
    out = orc.mla_ragged_paged_attention_ref(q_abs, c["q_pe"], pages, c["ctx"], c["bt"], c["qsl"], [c["n"]],
                                             kv_lora_rank=c["lkv"], qk_rope_head_dim=c["rope"], softmax_scale=scale, **kw)
    return np.einsum("tna,anh->tnh", out, c["w_v"]), pages


def _decompressed(c, pages, **kw):
    """Ordinary attention on per-head keys [k_nope | k_pe] and values, built from the latent pages."""
    lkv, rope, nope, vdim, heads = c["lkv"], c["rope"], c["nope"], c["vdim"], c["heads"]
    d = nope + rope
    latent = np.where(np.abs(pages[..., :lkv]) > 1e5, 0.0, pages[..., :lkv])  # unwritten slots: any finite value
    k_pe = np.where(np.abs(pages[..., c["off"]:c["off"] + rope]) > 1e5, 0.0, pages[..., c["off"]:c["off"] + rope])
    dense = np.zeros(pages.shape[:2] + (2 * heads, d))
    dense[:, :, 0::2, :nope] = np.einsum("pta,and->ptnd", latent, c["w_k"])
    dense[:, :, 0::2, nope:] = k_pe[:, :, None, :]
    dense[:, :, 1::2, :vdim] = np.einsum("pta,anh->ptnh", latent, c["w_v"])
    q = np.concatenate([c["q_nope"], c["q_pe"]], axis=-1)
    out = orc.ragged_paged_attention_ref(q, dense, c["ctx"], c["bt"], c["qsl"], [c["n"]], softmax_scale=d ** -0.5,
                                         num_kv_heads=heads, **kw)
    return out[..., :vdim]


@pytest.mark.parametrize("kw", [{}, {"sliding_window": 5}, {"logits_soft_cap": 3.0},
                                {"softmax_aux": np.array([0.5, -1.0, 2.0])}])
def test_absorbed_form_equals_attention_on_decompressed_keys_and_values(kw):
    c = _mla_case(0, [17, 9, 30, 1], [1, 9, 6, 1])
    got, pages = _absorbed(c, **kw)
    want = _decompressed(c, pages, **kw)
    assert np.abs(want).max() > 0.1
    np.testing.assert_allclose(got, want, rtol=1e-9, atol=1e-9)


def test_write_places_latent_and_rope_parts_and_zeroes_the_padding():
    c = _mla_case(1, [11, 4], [3, 4], lkv=40, rope=8)  # latent width not a multiple of 128: padding inside the row
    pages = orc.mla_page_scatter_ref(c["new_latent"], c["new_k_pe"], c["pages_before"], c["ctx"], c["bt"], c["qsl"], [2])
    assert c["off"] == 128 and c["row"] == 256
    t = 0
    for i in range(2):
        q_len = int(c["qsl"][i + 1] - c["qsl"][i])
        for r in range(q_len):
            pos = int(c["ctx"][i]) - q_len + r
            row = pages[c["bt"][i, pos // 8], pos % 8]
            np.testing.assert_array_equal(row[:40], c["new_latent"][t])
            np.testing.assert_array_equal(row[128:136], c["new_k_pe"][t])
            assert not row[40:128].any() and not row[136:].any()
            t += 1
    untouched = np.ones(pages.shape[:2], bool)
    for i in range(2):
        q_len = int(c["qsl"][i + 1] - c["qsl"][i])
        for pos in range(int(c["ctx"][i]) - q_len, int(c["ctx"][i])):
            untouched[c["bt"][i, pos // 8], pos % 8] = False
    np.testing.assert_array_equal(pages[untouched], c["pages_before"][untouched])


def test_one_key_returns_its_latent_row_and_the_default_scale():
    rng = np.random.default_rng(2)
    lkv, rope = 16, 4
    pages = np.zeros((2, 4, 256))
    pages[1, 0, :lkv] = rng.standard_normal(lkv)
    pages[1, 0, 128:132] = rng.standard_normal(rope)
    qn, qp = rng.standard_normal((1, 2, lkv)), rng.standard_normal((1, 2, rope))
    out = orc.mla_ragged_paged_attention_ref(qn, qp, pages, [1], np.array([[1]]), [0, 1], [1], kv_lora_rank=lkv,
                                             qk_rope_head_dim=rope)
    np.testing.assert_allclose(out[0], np.broadcast_to(pages[1, 0, :lkv], (2, lkv)))
    # two keys: weight of the second = sigmoid of the score difference at scale (lkv + rope) ** -0.5
    pages[1, 1, :lkv] = rng.standard_normal(lkv)
    pages[1, 1, 128:132] = rng.standard_normal(rope)
    out = orc.mla_ragged_paged_attention_ref(qn, qp, pages, [2], np.array([[1]]), [0, 1], [1], kv_lora_rank=lkv,
                                             qk_rope_head_dim=rope)
    for h in range(2):
        ds = (qn[0, h] @ (pages[1, 1, :lkv] - pages[1, 0, :lkv]) + qp[0, h] @ (pages[1, 1, 128:132] - pages[1, 0, 128:132])) / np.sqrt(20.0)
        w = 1.0 / (1.0 + np.exp(-ds))
        np.testing.assert_allclose(out[0, h], (1 - w) * pages[1, 0, :lkv] + w * pages[1, 1, :lkv], rtol=1e-12)


def test_latent_page_layout_follows_the_cache_config():
    # caching/mla_ragged_page/cache.py:198-201: 512 + 64 -> 512 + 128 = 640 per token; bf16 packs two tokens a row
    lay = orc.mla_page_layout_ref(512, 64, 64, bits=16)
    assert lay["kv_dim_padded"] == 640 and lay["kv_packing"] == 2 and lay["shape_tail"] == (32, 2, 640)
    assert lay["rope_offset"] == 512
    lay = orc.mla_page_layout_ref(512, 64, 128, bits=32)
    assert lay["shape_tail"] == (128, 1, 640)
    lay = orc.mla_page_layout_ref(192, 0, 17, bits=8)  # widths padded separately; page size rounded up to the packing
    assert lay["kv_dim_padded"] == 256 and lay["shape_tail"] == (5, 4, 256)
