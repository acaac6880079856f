"""Pins of the sparse-MLA oracle (oracle/ref_dsa.py) that do not reuse its formulae: the dense
MLA oracle when every position is selected, a float64 loop on a tiny case, and hand-worked page
lists."""

import math

import numpy as np
import torch

from oracle.ref_dsa import page_level_metadata_ref, sparse_mla_ref, topk_pages_ref
from oracle.ref_mla import ref_mla_ragged_paged_attention


def small_case(seed, kv_lens, P, H, lkv, rope):
    g = torch.Generator().manual_seed(seed)
    S = len(kv_lens)
    counts = [-(-k // P) for k in kv_lens]
    pps = max(counts)
    pool = sum(counts) + 2
    perm = torch.randperm(pool, generator=g)[: sum(counts)].to(torch.int32)
    cu_kv = np.zeros(S + 1, dtype=np.int32)
    cu_kv[1:] = np.cumsum([c * P for c in counts])
    q = (torch.randn(S, H, lkv + rope, generator=g) * 0.5).to(torch.bfloat16)
    cache = (torch.randn(pool, P, lkv + rope, generator=g) * 0.5).to(torch.bfloat16)
    flat = torch.cat([perm, torch.zeros(pps, dtype=torch.int32)])  # slack for the fixed-length slices
    return dict(q=q, cache=cache, kv_lens=torch.tensor(kv_lens, dtype=torch.int32), pages=flat,
                cu_q=torch.arange(S + 1, dtype=torch.int32), cu_kv=torch.from_numpy(cu_kv), pps=pps, counts=counts)


def test_all_positions_selected_is_dense_mla():
    kv_lens, P, H, lkv, rope = [5, 33, 17], 8, 4, 32, 8
    c = small_case(3, kv_lens, P, H, lkv, rope)
    k = max(kv_lens)
    topk = torch.full((3, k), -1, dtype=torch.int32)
    for i, n in enumerate(kv_lens):
        topk[i, :n] = torch.arange(n, dtype=torch.int32)
    got = sparse_mla_ref(c["q"], c["cache"], c["kv_lens"], topk, c["pages"], c["cu_q"], c["cu_kv"], [3, 3, 3],
                         sm_scale=0.3, pages_per_seq=c["pps"], v_dim=lkv)
    # dense oracle wants the padded [S * pages_per_seq] table
    padded = torch.zeros(3 * c["pps"], dtype=torch.int32)
    o = 0
    for i, cnt in enumerate(c["counts"]):
        padded[i * c["pps"] : i * c["pps"] + cnt] = c["pages"][o : o + cnt]
        o += cnt
    want, _ = ref_mla_ragged_paged_attention(c["q"][..., :lkv], c["q"][..., lkv:], None, None, c["cache"], c["kv_lens"],
                                             padded, c["cu_q"], [3, 3, 3], sm_scale=0.3)
    torch.testing.assert_close(got.float(), want.float(), rtol=2e-2, atol=1e-2)  # dense oracle rounds P to bf16


def test_float64_loop_on_a_tiny_case():
    kv_lens, P, H, lkv, rope = [11, 6], 4, 2, 8, 4
    c = small_case(4, kv_lens, P, H, lkv, rope)
    topk = torch.tensor([[10, 0, 3, -1, -1], [5, 2, 99, 4, -1]], dtype=torch.int32)  # 99 >= kv_len: ignored
    got = sparse_mla_ref(c["q"], c["cache"], c["kv_lens"], topk, c["pages"], c["cu_q"], c["cu_kv"], [2, 2, 2],
                         sm_scale=0.7, pages_per_seq=c["pps"], v_dim=lkv)
    for t, (sel, start) in enumerate([([10, 0, 3], 0), ([5, 2, 4], c["counts"][0])]):
        rows = [c["cache"][int(c["pages"][start + p // P]), p % P].double() for p in sel]
        for h in range(H):
            qv = c["q"][t, h].double()
            lg = [float((qv * r).sum()) * 0.7 for r in rows]
            mx = max(lg)
            w = [math.exp(x - mx) for x in lg]
            want = sum(wi / sum(w) * r[:lkv] for wi, r in zip(w, rows))
            torch.testing.assert_close(got[t, h].double(), want, rtol=1e-2, atol=1e-2)


def test_page_lists_by_hand():
    topk = np.array([[0, 1, 17, 35, -1, 16], [-1, -1, -1, -1, -1, -1]], dtype=np.int32)
    got = topk_pages_ref(topk, page_size=8, pages_per_seq=6, k_pages_max=4)
    assert got.tolist() == [[0, 2, 4, -1], [-1, -1, -1, -1]]
    # sequence 0: kv_len 37 -> new token at position 36 = page 4, offset 4; touched {0, 2, 4} minus {4}
    # sequence 1: kv_len 0 (padding row): everything points at the sentinel
    kv_len, pages = page_level_metadata_ref(
        [37, 0], topk, np.array([50, 51, 52, 53, 54, 60, 61], dtype=np.int32), [0, 1, 2], [0, 40, 48],
        page_size=8, pages_per_seq=6, k_pages_max=4, sentinel_page=99)
    assert kv_len.tolist() == [2 * 8 + 4 + 1, 0 * 8 + 0 + 1]
    assert pages.tolist() == [[50, 52, 54, 99], [99, 99, 99, 99]]


def test_device_page_lists_agree_with_the_loops_on_cpu_tensors(pkg):
    """compute_topk_pages is plain tensor code: it runs on CPU tensors too and must reproduce the
    per-row loops, including rows with more touched pages than k_pages_max and empty rows."""
    rng = np.random.default_rng(9)
    topk = rng.integers(-1, 900, size=(7, 40)).astype(np.int32)
    topk[3] = -1
    for P, kp in ((16, 8), (64, 64), (1, 5)):
        pps = -(-900 // P)
        got = pkg.compute_topk_pages(torch.from_numpy(topk), page_size=P, pages_per_seq=pps, k_pages_max=kp)
        assert np.array_equal(got.numpy(), topk_pages_ref(topk, P, pps, kp))
