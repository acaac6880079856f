"""Pins of the MLA oracle (oracle/ref_mla.py): golden brute-force fixture, the
generic RPA oracle with one shared kv head, float64 non-absorbed MHA, and the
padded-vs-compact cache layouts."""

import math
import os

import numpy as np
import torch

from oracle.ref_mla import mla_update_kv_cache, ref_mla_ragged_paged_attention
from oracle.ref_rpa import ref_ragged_paged_attention

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def small(seed=0, Hq=4, lkv=32, rope=8, P=4, kv_lens=(9, 16, 5), q_lens=None):
    g = torch.Generator().manual_seed(seed)
    rng = np.random.default_rng(seed)
    S = len(kv_lens)
    q_lens = q_lens or [1] * S
    counts = [-(-k // P) for k in kv_lens]
    pool = sum(counts) + 2
    perm = rng.permutation(pool)[: sum(counts)].astype(np.int32)
    pps = max(counts)
    table = np.zeros((S, pps), dtype=np.int32)
    o = 0
    for i, c in enumerate(counts):
        table[i, :c] = perm[o : o + c]
        o += c
    T = sum(q_lens)
    cu_q = np.zeros(S + 1, dtype=np.int32)
    cu_q[1:] = np.cumsum(q_lens)
    return dict(
        ql=(torch.randn(T, Hq, lkv, generator=g) * 0.5).to(torch.bfloat16),
        qp=(torch.randn(T, Hq, rope, generator=g) * 0.5).to(torch.bfloat16),
        cache=(torch.randn(pool, P, lkv + rope, generator=g) * 0.5).to(torch.bfloat16),
        kv_lens=torch.tensor(kv_lens, dtype=torch.int32), table=torch.from_numpy(table),
        cu_q=torch.from_numpy(cu_q), S=S, lkv=lkv, rope=rope, P=P)


def run(c, **kw):
    out, _ = ref_mla_ragged_paged_attention(c["ql"], c["qp"], None, None, c["cache"], c["kv_lens"],
                                            c["table"].reshape(-1), c["cu_q"], [c["S"]] * 3, **kw)
    return out


def test_golden_fixture():
    z = np.load(os.path.join(GOLDEN, "mla_small.npz"))
    f = lambda n: torch.from_numpy(z[n])
    S = len(z["kv_lens"])
    out, _ = ref_mla_ragged_paged_attention(
        f("ql_nope_bits").view(torch.bfloat16), f("q_pe_bits").view(torch.bfloat16), None, None,
        f("cache_bits").view(torch.bfloat16), f("kv_lens"), f("page_indices"), f("cu_q_lens"), [S, S, S],
        sm_scale=float(z["sm_scale"]))
    # P and the output are rounded to bf16 by the reference (kernels/mla/v1/ref.py:237-240)
    np.testing.assert_allclose(out.double().numpy(), z["expected_f64"], rtol=2e-2, atol=1e-2)


def test_equals_generic_oracle_with_one_shared_kv_head():
    c = small(seed=1, q_lens=[1, 3, 2], kv_lens=(9, 16, 5))
    sm = 1.0 / math.sqrt(24.0)
    for window, cap in [(None, None), (5, None), (None, 4.0)]:
        got = run(c, sm_scale=sm, sliding_window=window, soft_cap=cap)
        q = torch.cat([c["ql"], c["qp"]], dim=-1)
        k_pages = c["cache"][:, :, None, :]
        v_pages = torch.zeros_like(k_pages)
        v_pages[..., : c["lkv"]] = c["cache"][:, :, None, : c["lkv"]]
        ref = ref_ragged_paged_attention(q, k_pages, v_pages, c["kv_lens"], c["table"], c["cu_q"], [c["S"]],
                                         sm_scale=sm, sliding_window=window, soft_cap=cap)[..., : c["lkv"]]
        # the only difference: MLA rounds P to bf16 before the value product
        torch.testing.assert_close(got.float(), ref.float(), rtol=2e-2, atol=1e-2)


def test_absorbed_equals_plain_mha_in_float64():
    """models/deepseek_v3.py:349-366 (absorbed) vs :370-409 (plain): with
    k_nope = c W_uk and v = c W_uv per head, attention over (k_nope|k_pe) equals
    latent attention with q absorbed through W_uk, then projected by W_uv."""
    g = torch.Generator().manual_seed(2)
    Hq, lkv, rope, dn, dv, kv = 3, 16, 4, 6, 5, 11
    c_kv = torch.randn(kv, lkv, generator=g, dtype=torch.float64)
    k_pe = torch.randn(kv, rope, generator=g, dtype=torch.float64)
    q_nope = torch.randn(Hq, dn, generator=g, dtype=torch.float64)
    q_pe = torch.randn(Hq, rope, generator=g, dtype=torch.float64)
    w_uk = torch.randn(lkv, Hq, dn, generator=g, dtype=torch.float64)
    w_uv = torch.randn(lkv, Hq, dv, generator=g, dtype=torch.float64)
    sm = 1.0 / math.sqrt(dn + rope)
    k_nope = torch.einsum("kr,rhd->khd", c_kv, w_uk)
    v = torch.einsum("kr,rhd->khd", c_kv, w_uv)
    s = (torch.einsum("hd,khd->hk", q_nope, k_nope) + torch.einsum("hd,kd->hk", q_pe, k_pe)) * sm
    plain = torch.einsum("hk,khd->hd", torch.softmax(s, -1), v)
    ql = torch.einsum("hd,rhd->hr", q_nope, w_uk)
    cache = torch.cat([c_kv, k_pe], dim=-1).reshape(1, kv, lkv + rope)
    out, _ = ref_mla_ragged_paged_attention(ql[None], q_pe[None], None, None, cache, torch.tensor([kv], dtype=torch.int32),
                                            torch.tensor([0], dtype=torch.int32), torch.tensor([0, 1], dtype=torch.int32),
                                            [1, 1, 1], sm_scale=sm)
    absorbed = torch.einsum("hr,rhd->hd", out[0], w_uv)
    torch.testing.assert_close(absorbed, plain, rtol=1e-5, atol=1e-5)  # oracle computes in f32


def test_padded_layout_equals_compact_layout():
    """kernels/mla/v2/kernel.py:74-86 pads kv_c and k_pe to multiples of 128; zero
    padding adds nothing to q.k."""
    c = small(seed=3, lkv=32, rope=8)
    pool, P, _ = c["cache"].shape
    padded = torch.zeros(pool, P, 256, dtype=torch.bfloat16)
    padded[..., :32] = c["cache"][..., :32]
    padded[..., 128:136] = c["cache"][..., 32:]
    a = run(c, sm_scale=0.2)
    b, _ = ref_mla_ragged_paged_attention(c["ql"], c["qp"], None, None, padded, c["kv_lens"], c["table"].reshape(-1),
                                          c["cu_q"], [c["S"]] * 3, sm_scale=0.2, layout="padded")
    assert torch.equal(a, b)


def test_cache_update_places_new_rows():
    """kernels/mla/v1/ref.py:56-105: new token j of sequence i lands at kv_len-q_len+j."""
    c = small(seed=4, q_lens=[2, 1, 3], kv_lens=(9, 16, 5))
    T = 6
    g = torch.Generator().manual_seed(5)
    new_c = torch.randn(T, c["lkv"], generator=g).to(torch.bfloat16)
    new_r = torch.randn(T, c["rope"], generator=g).to(torch.bfloat16)
    upd = mla_update_kv_cache(new_c, new_r, c["cache"], c["kv_lens"], c["table"].reshape(-1), c["cu_q"], c["S"], c["lkv"])
    pps = c["table"].shape[1]
    t = 0
    for i, (ql, kv) in enumerate(zip([2, 1, 3], [9, 16, 5])):
        for j in range(ql):
            pos = kv - ql + j
            page = int(c["table"][i, pos // c["P"]])
            assert torch.equal(upd[page, pos % c["P"], : c["lkv"]], new_c[t])
            assert torch.equal(upd[page, pos % c["P"], c["lkv"] :], new_r[t])
            t += 1
    # with the rows written, attention equals attention on a cache that already held them
    a, _ = ref_mla_ragged_paged_attention(c["ql"], c["qp"], new_c, new_r, c["cache"], c["kv_lens"], c["table"].reshape(-1),
                                          c["cu_q"], [c["S"]] * 3, sm_scale=0.2)
    b, _ = ref_mla_ragged_paged_attention(c["ql"], c["qp"], None, None, upd, c["kv_lens"], c["table"].reshape(-1),
                                          c["cu_q"], [c["S"]] * 3, sm_scale=0.2)
    assert torch.equal(a, b)
