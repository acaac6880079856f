"""GPU parity of the sparse absorbed-MLA wrappers (sglang-jax_amd/dsa.py) against the CPU oracles:
token-level selection against the restated sparse reference (dsa/ref.py:272-337), page-level
selection against the dense MLA oracle over the page lists worked out in plain loops
(dsa/sparse_mla.py:107-175).  rtol = atol = 2e-2 (bf16)."""

import sys

import numpy as np
import pytest
import torch

from parity import assert_parity

from oracle.ref_dsa import page_level_metadata_ref, sparse_mla_ref, topk_pages_ref
from oracle.ref_mla import ref_mla_ragged_paged_attention

pytestmark = pytest.mark.gpu
TOL = dict(rtol=2e-2, atol=2e-2)


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def batch(wl, kv_lens, P, seed, Hq=16):
    b = wl.make_mla_batch("dsa", [1] * len(kv_lens), kv_lens, num_q_heads=Hq, lkv_dim=512, rope_dim=64, page_size=P,
                          seed=seed, sm_scale=192 ** -0.5)
    # one more page at the end: the padding target, owned by no sequence
    b.cache_kv = torch.cat([b.cache_kv, torch.zeros_like(b.cache_kv[:1])], dim=0)
    return b


def draw_topk(kv_lens, k, seed):
    """k positions per sequence, the newest token last among the valid ones, -1 padded."""
    rng = np.random.default_rng(seed)
    out = np.full((len(kv_lens), k), -1, dtype=np.int32)
    for i, n in enumerate(kv_lens):
        m = min(k, n)
        older = rng.choice(n - 1, size=m - 1, replace=False) if m > 1 else np.zeros(0, dtype=np.int64)
        out[i, : m - 1] = older
        out[i, m - 1] = n - 1
    return out


@pytest.mark.parametrize("P", [16, 64])
def test_topk_pages_on_the_device(pkg, gpu, P):
    kv_lens = [40, 300, 64, 1000, 130]
    topk = draw_topk(kv_lens, 48, 5)
    pps = -(-max(kv_lens) // P)
    for kp in (4, 64):
        got = pkg.compute_topk_pages(torch.from_numpy(topk).to(gpu), page_size=P, pages_per_seq=pps, k_pages_max=kp)
        assert np.array_equal(got.cpu().numpy(), topk_pages_ref(topk, P, pps, kp))


@pytest.mark.parametrize("with_new_token", [False, True])
def test_token_level_selection_through_the_dense_kernel(pkg, wl, gpu, with_new_token):
    kv_lens, P, k = [40, 300, 64, 1000, 130], 16, 64
    b = batch(wl, kv_lens, P, 81)
    topk = torch.from_numpy(draw_topk(kv_lens, k, 6))
    S = len(kv_lens)
    pps = -(-max(kv_lens) // P)
    pages = torch.cat([b.page_indices, torch.zeros(pps, dtype=torch.int32)])
    q = torch.cat([b.ql_nope, b.q_pe], dim=-1)
    say(f"dsa via dense new_token={with_new_token}")
    want = sparse_mla_ref(q, b.cache_kv, b.kv_lens, topk, pages, b.cu_q_lens, b.cu_kv_lens, [S, S, S],
                          sm_scale=b.sm_scale, pages_per_seq=pps, v_dim=512)
    g = b.to(gpu)
    cache = b.cache_kv.clone()
    new_c = new_r = None
    if with_new_token:
        # the newest row of every sequence is not in the cache yet: it arrives as new_kv_c / new_k_pe
        new_c = torch.zeros(S, 512, dtype=torch.bfloat16)
        new_r = torch.zeros(S, 64, dtype=torch.bfloat16)
        o = 0
        for i, n in enumerate(kv_lens):
            page, off = int(b.page_indices[o + (n - 1) // P]), (n - 1) % P
            new_c[i], new_r[i] = cache[page, off, :512], cache[page, off, 512:]
            cache[page, off] = float("nan")
            o += -(-n // P)
        new_c, new_r = new_c.to(gpu), new_r.to(gpu)
    got = pkg.sparse_mla_via_dense(
        g.ql_nope, g.q_pe, new_c, new_r, cache.to(gpu), g.kv_lens, topk.to(gpu), g.page_indices, g.cu_q_lens,
        g.cu_kv_lens, (S, S, S), sm_scale=b.sm_scale, page_size=P, pages_per_seq=pps, kv_lora_rank=512)
    torch.cuda.synchronize()
    assert_parity(got.cpu().float(), want.float(), **TOL)


@pytest.mark.parametrize("precomputed", [False, True])
def test_page_level_selection(pkg, wl, gpu, precomputed):
    kv_lens, P, k, kp = [40, 300, 64, 1000, 130], 16, 24, 32
    b = batch(wl, kv_lens, P, 82)
    topk_np = draw_topk(kv_lens, k, 7)
    S = len(kv_lens)
    pps = -(-max(kv_lens) // P)
    sentinel = b.cache_kv.shape[0] - 1
    sp_len, sp_pages = page_level_metadata_ref(b.kv_lens.numpy(), topk_np, b.page_indices.numpy(), b.cu_q_lens.numpy(),
                                               b.cu_kv_lens.numpy(), page_size=P, pages_per_seq=pps, k_pages_max=kp,
                                               sentinel_page=sentinel)
    want, _ = ref_mla_ragged_paged_attention(
        b.ql_nope, b.q_pe, None, None, b.cache_kv, torch.from_numpy(sp_len), torch.from_numpy(sp_pages).reshape(-1),
        torch.arange(S + 1, dtype=torch.int32), [S, S, S], sm_scale=b.sm_scale)
    # the newest row arrives as new_kv_c / new_k_pe and must land in its true slot
    cache = b.cache_kv.clone()
    new_c = torch.zeros(S, 512, dtype=torch.bfloat16)
    new_r = torch.zeros(S, 64, dtype=torch.bfloat16)
    o = 0
    for i, n in enumerate(kv_lens):
        page, off = int(b.page_indices[o + (n - 1) // P]), (n - 1) % P
        new_c[i], new_r[i] = cache[page, off, :512], cache[page, off, 512:]
        cache[page, off] = 0
        o += -(-n // P)
    g = b.to(gpu)
    topk = torch.from_numpy(topk_np).to(gpu)
    pre = pkg.compute_topk_pages(topk, page_size=P, pages_per_seq=pps, k_pages_max=kp) if precomputed else None
    say(f"dsa page level precomputed={precomputed}")
    got, cache_out = pkg.sparse_mla_page_level(
        g.ql_nope, g.q_pe, new_c.to(gpu), new_r.to(gpu), cache.to(gpu), g.kv_lens, topk, g.page_indices, g.cu_q_lens,
        g.cu_kv_lens, (S, S, S), pre, sm_scale=b.sm_scale, page_size=P, pages_per_seq=pps, kv_lora_rank=512,
        k_pages_max=kp)
    torch.cuda.synchronize()
    assert_parity(got.cpu().float(), want.float(), **TOL)
    assert torch.equal(cache_out.cpu(), b.cache_kv)  # every new row back in its slot, nothing else touched
