"""Pins of the CPU oracle (oracle/ref_rpa.py) that do not retype its formulae.

The reference ships no stored vectors for attention (its tests compare kernel
and jnp oracle on fresh random inputs), so the oracle is pinned by
  * torch.nn.functional.scaled_dot_product_attention with an explicit boolean
    mask (a library routine),
  * a float64 scalar-loop brute force (tests/bruteforce.py),
  * closed forms and invariants of masked softmax attention,
  * the committed fixtures under tests/golden/ (brute-force outputs).
softmax_dtype has no such pin: parity unpinned.
"""

import math
import os

import numpy as np
import pytest
import torch

from oracle import ref_rpa
from oracle.ref_rpa import (
    DEFAULT_MASK_VALUE,
    lse_combine,
    merge_kv,
    ragged_to_padded_page_table,
    ref_forward_metadata,
    ref_ragged_paged_attention,
    ref_ragged_paged_attention_fused,
    split_fused_cache,
)
from tests.bruteforce import brute_attention

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def make_case(q_lens, kv_lens, Hq, Hkv, D, P, seed, dtype=torch.bfloat16, pool_extra=3, canary=None):
    g = torch.Generator().manual_seed(seed)
    rng = np.random.default_rng(seed)
    S = len(q_lens)
    counts = [-(-k // P) for k in kv_lens]
    pool = sum(counts) + pool_extra
    perm = rng.permutation(pool)[: sum(counts)].astype(np.int32)
    width = max(counts)
    table = np.zeros((S, width), dtype=np.int32)
    o = 0
    for i, c in enumerate(counts):
        table[i, :c] = perm[o : o + c]
        o += c
    T = sum(q_lens)
    q = torch.randn(T, Hq, D, generator=g).to(dtype)
    k_pages = torch.randn(pool, P, Hkv, D, generator=g).to(dtype)
    v_pages = torch.randn(pool, P, Hkv, D, generator=g).to(dtype)
    if canary is not None:
        used = np.zeros((pool, P), dtype=bool)
        for i, kv in enumerate(kv_lens):
            for t in range(kv):
                used[table[i, t // P], t % P] = True
        mask = torch.from_numpy(~used)
        k_pages[mask] = canary
        v_pages[mask] = canary
    cu_q = np.zeros(S + 1, dtype=np.int32)
    cu_q[1:] = np.cumsum(q_lens)
    return dict(q=q, k_pages=k_pages, v_pages=v_pages, kv_lens=torch.tensor(kv_lens, dtype=torch.int32),
                page_indices=torch.from_numpy(table), cu_q_lens=torch.from_numpy(cu_q), num_seqs=[S])


def run(c, **kw):
    return ref_ragged_paged_attention(c["q"], c["k_pages"], c["v_pages"], c["kv_lens"], c["page_indices"],
                                      c["cu_q_lens"], c["num_seqs"], **kw)


def gathered(c, i):
    P = c["k_pages"].shape[1]
    kv = int(c["kv_lens"][i])
    idx = c["page_indices"][i].long()
    k = c["k_pages"][idx].reshape(-1, *c["k_pages"].shape[2:])[:kv]
    v = c["v_pages"][idx].reshape(-1, *c["v_pages"].shape[2:])[:kv]
    return k, v


# ---------------------------------------------------------------- library routine
@pytest.mark.parametrize("window", [None, 7])
def test_matches_torch_sdpa(window):
    q_lens, kv_lens = [1, 5, 16, 3], [37, 5, 40, 20]
    Hq, Hkv, D, P = 8, 2, 32, 8
    c = make_case(q_lens, kv_lens, Hq, Hkv, D, P, seed=1, dtype=torch.float32)
    sm = 1.0 / math.sqrt(D)
    out = run(c, sm_scale=sm, sliding_window=window)
    o = 0
    for i, (ql, kv) in enumerate(zip(q_lens, kv_lens)):
        k, v = gathered(c, i)
        qi = c["q"][o : o + ql]
        pos = (kv - ql) + torch.arange(ql)[:, None]
        t = torch.arange(kv)[None, :]
        visible = t <= pos
        if window is not None:
            visible &= t > pos - window
        kk = k.repeat_interleave(Hq // Hkv, dim=1)
        vv = v.repeat_interleave(Hq // Hkv, dim=1)
        ref = torch.nn.functional.scaled_dot_product_attention(
            qi.permute(1, 0, 2)[None], kk.permute(1, 0, 2)[None], vv.permute(1, 0, 2)[None],
            attn_mask=visible[None, None], scale=sm)[0].permute(1, 0, 2)
        torch.testing.assert_close(out[o : o + ql], ref, rtol=1e-5, atol=1e-5)
        o += ql


# ---------------------------------------------------------------- brute force
@pytest.mark.parametrize("window,cap", [(None, None), (5, None), (None, 3.0), (4, 2.5)])
def test_matches_float64_brute_force(window, cap):
    q_lens, kv_lens = [1, 4, 7], [23, 9, 7]
    Hq, Hkv, D, P = 4, 2, 8, 4
    c = make_case(q_lens, kv_lens, Hq, Hkv, D, P, seed=2, dtype=torch.float32)
    sm = 0.3
    out = run(c, sm_scale=sm, sliding_window=window, soft_cap=cap).double().numpy()
    o = 0
    for i, (ql, kv) in enumerate(zip(q_lens, kv_lens)):
        k, v = gathered(c, i)
        ref = brute_attention(c["q"][o : o + ql].double().numpy(), k.double().numpy(), v.double().numpy(), ql, kv,
                              sm_scale=sm, window=window, soft_cap=cap)
        np.testing.assert_allclose(out[o : o + ql], ref, rtol=2e-5, atol=2e-6)
        o += ql


def test_attention_sink_matches_brute_force():
    # numpy RandomState sink vectors, as the reference's tests draw them
    # (python/sgl_jax/test/test_flashattention_misc.py:72)
    q_lens, kv_lens = [2, 1], [6, 11]
    Hq, Hkv, D, P = 4, 2, 8, 4
    sink = np.random.RandomState(123).randn(Hq)
    c = make_case(q_lens, kv_lens, Hq, Hkv, D, P, seed=3, dtype=torch.float32)
    out = run(c, sm_scale=0.5, attention_sink=torch.from_numpy(sink)).double().numpy()
    o = 0
    for i, (ql, kv) in enumerate(zip(q_lens, kv_lens)):
        k, v = gathered(c, i)
        ref = brute_attention(c["q"][o : o + ql].double().numpy(), k.double().numpy(), v.double().numpy(), ql, kv,
                              sm_scale=0.5, sink=sink)
        np.testing.assert_allclose(out[o : o + ql], ref, rtol=2e-5, atol=2e-6)
        o += ql


def test_golden_fixtures():
    """Brute-force outputs committed under tests/golden (made by make_golden.py)."""
    z = np.load(os.path.join(GOLDEN, "rpa_small.npz"))
    n = int(z["n_cases"])
    for ci in range(n):
        pre = f"c{ci}_"
        f = lambda name: torch.from_numpy(z[pre + name])
        q = f("q_bf16_bits").view(torch.bfloat16)
        kp = f("k_pages_bf16_bits").view(torch.bfloat16)
        vp = f("v_pages_bf16_bits").view(torch.bfloat16)
        window = int(z[pre + "window"]) or None
        cap = float(z[pre + "soft_cap"]) or None
        out = ref_ragged_paged_attention(q, kp, vp, f("kv_lens"), f("page_indices"), f("cu_q_lens"),
                                         [int(z[pre + "num_seqs"])], sm_scale=float(z[pre + "sm_scale"]),
                                         sliding_window=window, soft_cap=cap)
        want = z[pre + "expected_f64"]
        # the oracle rounds its output to bf16; the fixture is exact float64
        np.testing.assert_allclose(out.double().numpy(), want, rtol=1e-2, atol=1e-2)
        assert np.abs(out.double().numpy() - want).max() < 2.0 ** -7 * max(1.0, np.abs(want).max())


# ---------------------------------------------------------------- hand-computed order of operations
def test_hand_computed_two_by_three():
    """1 head, D=1, q=[2], keys=[1,2,3], values=[10,20,40], scale 0.5, cap 1:
    s = 0.5*2*k = [1,2,3]; capped = tanh([1,2,3]); softmax; dot values."""
    q = torch.tensor([[[2.0]]])
    k_pages = torch.tensor([1.0, 2.0, 3.0, 99.0]).reshape(1, 4, 1, 1)
    v_pages = torch.tensor([10.0, 20.0, 40.0, 99.0]).reshape(1, 4, 1, 1)
    args = (q, k_pages, v_pages, torch.tensor([3], dtype=torch.int32), torch.tensor([[0]], dtype=torch.int32),
            torch.tensor([0, 1], dtype=torch.int32), [1])
    out = ref_ragged_paged_attention(*args, sm_scale=0.5, soft_cap=1.0)
    e = [math.exp(math.tanh(x)) for x in (1.0, 2.0, 3.0)]
    want = (10 * e[0] + 20 * e[1] + 40 * e[2]) / sum(e)
    assert abs(out.item() - want) < 1e-5
    # scale BEFORE the cap: cap(0.5*s) differs from 0.5*cap(s)
    wrong = [math.exp(0.5 * math.tanh(2 * x)) for x in (1.0, 2.0, 3.0)]
    assert abs(want - (10 * wrong[0] + 20 * wrong[1] + 40 * wrong[2]) / sum(wrong)) > 1e-2
    # window 2 keeps keys 2,3 only (position 2 sees t > 0)
    out_w = ref_ragged_paged_attention(*args, sm_scale=0.5, sliding_window=2)
    ew = [math.exp(x) for x in (2.0, 3.0)]
    assert abs(out_w.item() - (20 * ew[0] + 40 * ew[1]) / sum(ew)) < 1e-5


# ---------------------------------------------------------------- closed forms
def test_kv_len_one_returns_value_bit_exact():
    c = make_case([1, 1], [1, 1], 4, 2, 16, 4, seed=4)
    out = run(c, sm_scale=0.7)
    for i in range(2):
        _, v = gathered(c, i)
        assert torch.equal(out[i], v[0].repeat_interleave(2, dim=0))


def test_equal_keys_give_mean_of_visible_values():
    c = make_case([3], [10], 2, 1, 8, 4, seed=5, dtype=torch.float32)
    c["k_pages"][:] = c["k_pages"][0, 0, 0]
    out = run(c, sm_scale=1.0, sliding_window=4)
    _, v = gathered(c, 0)
    for j in range(3):
        pos = 10 - 3 + j
        want = v[pos - 3 : pos + 1, 0].mean(dim=0)
        torch.testing.assert_close(out[j, 0], want, rtol=1e-5, atol=1e-6)


def test_window_at_least_kv_len_is_no_window():
    c = make_case([5, 1], [12, 30], 4, 2, 16, 8, seed=6)
    assert torch.equal(run(c, sm_scale=0.2), run(c, sm_scale=0.2, sliding_window=30))
    assert not torch.equal(run(c, sm_scale=0.2), run(c, sm_scale=0.2, sliding_window=3))


def test_soft_cap_limits():
    c = make_case([4], [9], 2, 2, 8, 4, seed=7, dtype=torch.float32)
    base = run(c, sm_scale=0.1)
    torch.testing.assert_close(run(c, sm_scale=0.1, soft_cap=1e6), base, rtol=1e-4, atol=1e-5)
    assert (run(c, sm_scale=0.1, soft_cap=0.05) - base).abs().max() > 1e-3


def test_prefill_rows_equal_decode_at_that_position():
    """Row j of a chunk with kv_len L equals a 1-token decode with kv_len L-q_len+j+1."""
    ql, kv = 6, 21
    c = make_case([ql], [kv], 4, 2, 16, 4, seed=8)
    full = run(c, sm_scale=0.25, sliding_window=9)
    for j in range(ql):
        d = dict(c)
        d["q"] = c["q"][j : j + 1]
        d["kv_lens"] = torch.tensor([kv - ql + j + 1], dtype=torch.int32)
        d["cu_q_lens"] = torch.tensor([0, 1], dtype=torch.int32)
        torch.testing.assert_close(run(d, sm_scale=0.25, sliding_window=9)[0].float(), full[j].float(), rtol=0, atol=0)


def test_gqa_equals_mha_on_repeated_kv():
    c = make_case([3, 1], [17, 8], 8, 2, 16, 4, seed=9)
    d = dict(c)
    d["k_pages"] = c["k_pages"].repeat_interleave(4, dim=2)
    d["v_pages"] = c["v_pages"].repeat_interleave(4, dim=2)
    assert torch.equal(run(c, sm_scale=0.3), run(d, sm_scale=0.3))


def test_page_permutation_and_canaries_do_not_matter():
    q_lens, kv_lens = [2, 1, 5], [13, 30, 5]
    a = make_case(q_lens, kv_lens, 4, 2, 16, 8, seed=10)
    # same logical content, different physical placement, NaN in every unused slot
    b = make_case(q_lens, kv_lens, 4, 2, 16, 8, seed=10, pool_extra=9, canary=float("nan"))
    P = 8
    for i, kv in enumerate(kv_lens):
        for t in range(kv):
            src = (int(a["page_indices"][i, t // P]), t % P)
            dst = (int(b["page_indices"][i, t // P]), t % P)
            b["k_pages"][dst] = a["k_pages"][src]
            b["v_pages"][dst] = a["v_pages"][src]
    b["q"] = a["q"]
    out_a, out_b = run(a, sm_scale=0.3), run(b, sm_scale=0.3)
    assert torch.isfinite(out_b.float()).all()
    assert torch.equal(out_a, out_b)


def test_fused_layout_equals_split_layout():
    c = make_case([2, 1], [9, 20], 4, 2, 16, 4, seed=11)
    pool, P, Hkv, D = c["k_pages"].shape
    fused = merge_kv(c["k_pages"].reshape(-1, Hkv, D), c["v_pages"].reshape(-1, Hkv, D)).reshape(pool, P, 2 * Hkv, D)
    k2, v2 = split_fused_cache(fused)
    assert torch.equal(k2, c["k_pages"]) and torch.equal(v2, c["v_pages"])
    # K0,V0,K1,V1 order (kernels/ragged_paged_attention/ragged_paged_attention.py:74-76)
    assert torch.equal(fused[:, :, 0], c["k_pages"][:, :, 0]) and torch.equal(fused[:, :, 1], c["v_pages"][:, :, 0])
    out = ref_ragged_paged_attention_fused(c["q"], fused, c["kv_lens"], c["page_indices"], c["cu_q_lens"], [2], sm_scale=0.3)
    assert torch.equal(out, run(c, sm_scale=0.3))


def test_fp8_scale_semantics():
    """x representable in e4m3 and scale 1 => identical to the bf16 path; per-head
    scales equal dequantise-then-attend (ragged_paged_attention_v3.py:140-145)."""
    c = make_case([1, 3], [19, 7], 4, 2, 16, 4, seed=12)
    k8 = c["k_pages"].to(torch.float8_e4m3fn)
    v8 = c["v_pages"].to(torch.float8_e4m3fn)
    d = dict(c, k_pages=k8, v_pages=v8)
    e = dict(c, k_pages=k8.to(torch.bfloat16), v_pages=v8.to(torch.bfloat16))
    assert torch.equal(run(d, sm_scale=0.3, k_scale=1.0, v_scale=1.0), run(e, sm_scale=0.3))
    ks, vs = torch.tensor([0.5, 2.0]), torch.tensor([4.0, 0.25])
    f = dict(c, k_pages=(k8.float() * ks.reshape(1, 1, 2, 1)).to(torch.bfloat16),
             v_pages=(v8.float() * vs.reshape(1, 1, 2, 1)).to(torch.bfloat16))
    assert torch.equal(run(d, sm_scale=0.3, k_scale=ks, v_scale=vs), run(f, sm_scale=0.3))


def test_lse_combine_equals_unsplit_softmax():
    g = torch.Generator().manual_seed(13)
    s = torch.randn(3, 50, generator=g) * 4
    v = torch.randn(50, 8, generator=g)
    full = torch.softmax(s, dim=-1) @ v
    parts = [(0, 7), (7, 32), (32, 50)]
    po, pl, pm = [], [], []
    for a, b in parts:
        m = s[:, a:b].max(dim=-1).values
        p = torch.exp(s[:, a:b] - m[:, None])
        po.append(p @ v[a:b]); pl.append(p.sum(-1)); pm.append(m)
    out = lse_combine(torch.stack(po), torch.stack(pl), torch.stack(pm))
    torch.testing.assert_close(out, full, rtol=1e-5, atol=1e-6)


def test_mask_value_constant():
    assert DEFAULT_MASK_VALUE == -0.7 * float(np.finfo(np.float32).max)


# ---------------------------------------------------------------- metadata
def test_forward_metadata_closed_forms():
    """page_indices = cache_loc[::P] // P; cu_kv = cumsum(ceil(len/P)*P)
    (layers/attention/flashattention_backend.py:168-224)."""
    P = 4
    seq_lens = np.array([5, 8, 1, 0], dtype=np.int32)
    # sequence i occupies whole pages; slots inside a page are contiguous
    pages = [[7, 2], [3, 9], [5], []]
    cache_loc = np.concatenate([np.arange(p * P, p * P + P) for ps in pages for p in ps]).astype(np.int32)
    pi, cu_q, cu_kv, dist = ref_forward_metadata(cache_loc, seq_lens, None, P, is_decode=True)
    assert pi.tolist() == [7, 2, 3, 9, 5]
    assert cu_q.tolist() == [0, 1, 2, 3, 4]
    assert cu_kv.tolist() == [0, 8, 16, 20, 20]
    assert dist.tolist() == [3, 3, 3]
    pi, cu_q, cu_kv, dist = ref_forward_metadata(cache_loc, seq_lens, np.array([2, 8, 1, 0]), P, is_decode=False)
    assert cu_q.tolist() == [0, 2, 10, 11, 11]
    assert dist.tolist() == [0, 3, 3]
    table = ragged_to_padded_page_table(pi, cu_kv, P, 3)
    assert table.tolist() == [[7, 2], [3, 9], [5, 0]]


# ---------------------------------------------------------------- temperature (rpa_v3:171-177)
def test_temperature_reduces_to_a_per_row_scale():
    """With T = 4 a query at position 16 has factor log2(16)/log2(4) = 2 exactly and a query at
    position 64 has 3: each such row equals the plain oracle with sm_scale doubled / tripled;
    rows at positions <= T are unchanged."""
    D = 16
    # decode rows at chosen positions (position = kv_len - 1) and one chunk crossing T
    q_lens, kv_lens = [1, 1, 1, 1, 3], [17, 65, 5, 3, 6]
    c = make_case(q_lens, kv_lens, 4, 2, D, 4, seed=31, dtype=torch.float32)
    out = run(c, sm_scale=0.25, xai_temperature_len=4.0)
    plain = run(c, sm_scale=0.25)
    x2 = run(c, sm_scale=0.5)
    x3 = run(c, sm_scale=0.75)
    torch.testing.assert_close(out[0], x2[0], rtol=1e-5, atol=1e-6)      # position 16
    torch.testing.assert_close(out[1], x3[1], rtol=1e-5, atol=1e-6)      # position 64
    torch.testing.assert_close(out[2], plain[2], rtol=0, atol=0)         # position 4 == T: not beyond
    torch.testing.assert_close(out[3], plain[3], rtol=0, atol=0)         # position 2
    # chunk rows at positions 3, 4, 5: only the last is beyond T (factor log2(5)/2)
    torch.testing.assert_close(out[4:6], plain[4:6], rtol=0, atol=0)
    f = math.log2(5.0) / 2.0
    scaled = run(c, sm_scale=0.25 * f)
    torch.testing.assert_close(out[6], scaled[6], rtol=1e-5, atol=1e-6)


def test_temperature_applies_after_the_soft_cap():
    """cap*tanh(s/cap) is bounded by cap; with factor 2 the logits reach 2*cap, which a factor
    applied before the cap could never produce: compare with the float64 brute force fed the
    doubled cap-ed scores through its own scale/cap arguments."""
    q_lens, kv_lens = [1], [17]
    c = make_case(q_lens, kv_lens, 2, 1, 8, 4, seed=32, dtype=torch.float32)
    cap, sm = 1.5, 0.9
    out = run(c, sm_scale=sm, soft_cap=cap, xai_temperature_len=4.0).double().numpy()
    k, v = gathered(c, 0)
    q = c["q"].double().numpy()
    kk, vv = k.double().numpy(), v.double().numpy()
    want = np.zeros_like(out)
    for h in range(2):
        sc = np.array([2.0 * cap * math.tanh(sm * float(q[0, h] @ kk[t, 0]) / cap) for t in range(17)])
        w = np.exp(sc - sc.max())
        want[0, h] = (w / w.sum()) @ vv[:, 0]
    np.testing.assert_allclose(out, want, rtol=2e-5, atol=2e-6)


# ---------------------------------------------------------------- custom mask (rpa_v3:152-165)
def _flat_mask(masks):
    return torch.from_numpy(np.concatenate([m.reshape(-1) for m in masks]).astype(np.int32))


def test_custom_mask_special_cases_and_brute_force():
    q_lens, kv_lens = [3, 1, 5], [9, 6, 5]
    Hq, Hkv, D, P = 4, 2, 8, 4
    c = make_case(q_lens, kv_lens, Hq, Hkv, D, P, seed=33, dtype=torch.float32)
    sm = 0.4
    # (1) a mask that spells out the causal pattern reproduces causal attention
    causal = [(np.arange(kv)[None, :] <= (kv - ql) + np.arange(ql)[:, None]) for ql, kv in zip(q_lens, kv_lens)]
    out = run(c, sm_scale=sm, causal=False, custom_mask=_flat_mask(causal))
    torch.testing.assert_close(out, run(c, sm_scale=sm), rtol=1e-6, atol=1e-6)
    # (2) an all-ones mask equals causal=False without a mask
    ones = [np.ones((ql, kv)) for ql, kv in zip(q_lens, kv_lens)]
    torch.testing.assert_close(run(c, sm_scale=sm, causal=False, custom_mask=_flat_mask(ones)),
                               run(c, sm_scale=sm, causal=False), rtol=0, atol=0)
    # (3) a random tree-like mask (every row keeps at least one token) against a float64 loop
    rng = np.random.default_rng(5)
    masks = []
    for ql, kv in zip(q_lens, kv_lens):
        mk = rng.integers(0, 2, size=(ql, kv))
        mk[:, 0] = 1
        masks.append(mk)
    out = run(c, sm_scale=sm, causal=False, custom_mask=_flat_mask(masks)).double().numpy()
    o = 0
    for i, (ql, kv) in enumerate(zip(q_lens, kv_lens)):
        k, v = gathered(c, i)
        q = c["q"][o:o + ql].double().numpy()
        kk, vv = k.double().numpy(), v.double().numpy()
        for j in range(ql):
            for h in range(Hq):
                keep = [t for t in range(kv) if masks[i][j, t] >= 1]
                sc = np.array([sm * float(q[j, h] @ kk[t, h // 2]) for t in keep])
                w = np.exp(sc - sc.max())
                want = (w / w.sum()) @ vv[keep, h // 2]
                np.testing.assert_allclose(out[o + j, h], want, rtol=2e-5, atol=2e-6)
        o += ql


def test_query_quantisation_lands_on_the_cache_grid():
    """rpa_v3:463-470.  Pins: results are values of the cache's element type, inside its finite
    range, unchanged by a second pass at scale 1, and equal to the input when that is already
    on the grid; the clip makes 1e4 / 2 saturate at 448 instead of overflowing e4m3."""
    from oracle.ref_rpa import quantise_queries
    g = torch.Generator().manual_seed(5)
    q = (torch.randn(64, 4, 128, generator=g) * 3).to(torch.bfloat16)
    q[0, 0, 0] = 1.0e4
    x = quantise_queries(q, 2.0, torch.float8_e4m3fn)
    assert x.dtype == torch.bfloat16 and float(x.abs().max()) == 448.0
    assert torch.equal(x.to(torch.float8_e4m3fn).to(torch.bfloat16), x)
    assert torch.equal(quantise_queries(x, 1.0, torch.float8_e4m3fn), x)
    # nearest grid point: error at most half a grid step (2^-4 relative for 3 mantissa bits)
    ref = (q.float() / 2.0).clamp(-448, 448)
    big = ref.abs() > 2.0 ** -6  # normal range of e4m3
    assert float(((x.float() - ref).abs()[big] / ref.abs()[big]).max()) <= 2.0 ** -4 + 2.0 ** -8
    # a bf16 cache: the quotient rounded to bf16, nothing else
    y = quantise_queries(q, 3.0, torch.bfloat16)
    assert torch.equal(y, (q.float() / 3.0).to(torch.bfloat16))


def test_softmax_dtype_rounds_logits_and_probabilities():
    """rpa_v3:181-199 with softmax_dtype = bfloat16: the masked logits become bf16 values and so do
    the probabilities that multiply V.  Checked against a float64 loop with the two roundings done
    by hand, and against the f32 softmax, from which it may differ by bf16 rounding only.  The
    reduction order inside jax's bf16 softmax is not reproducible here: parity unpinned below
    one bf16 ulp of the probabilities."""
    c = make_case([3, 1], [9, 17], Hq=4, Hkv=2, D=8, P=4, seed=21)
    base = run(c, sm_scale=0.5)
    rnd = run(c, sm_scale=0.5, softmax_dtype=torch.bfloat16)
    torch.testing.assert_close(rnd.float(), base.float(), rtol=2e-2, atol=2e-2)

    def bf(x):
        return float(torch.tensor(x, dtype=torch.float32).to(torch.bfloat16))

    o = 0
    for i, (ql, kv) in enumerate([(3, 9), (1, 17)]):
        k, v = gathered(c, i)
        for j in range(ql):
            for h in range(4):
                qv = c["q"][o + j, h].double()
                vis = range(kv - ql + j + 1)
                logit = [bf(float((qv * k[t, h // 2].double()).sum()) * 0.5) for t in vis]
                mx = max(logit)
                e = [math.exp(x - mx) for x in logit]
                p = [bf(x / sum(e)) for x in e]
                want = sum(pt * v[t, h // 2].double() for pt, t in zip(p, vis))
                torch.testing.assert_close(rnd[o + j, h].double(), want, rtol=2e-2, atol=2e-2)
        o += ql
