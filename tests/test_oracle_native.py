"""The restated native attention (oracle/ref_native.py, the reference engine's own CPU path)
against the restated ragged paged attention (oracle/ref_rpa.py) and the float64 brute force.

The two restatements follow different reference files with different structure -- one dense
block-diagonal score matrix over a token-gathered cache here, a per-sequence loop over pages
there -- so agreement between them is a cross-check neither gets from its own formulae.
"""

import math

import numpy as np
import pytest
import torch

from oracle.ref_native import ref_forward_attention
from oracle.ref_rpa import ref_ragged_paged_attention
from tests.bruteforce import brute_attention
from tests.test_oracle_rpa import make_case


def token_view(case, kv_lens):
    """The paged cache as the native path sees it: one row per cached token, row 0 unused (a
    location of 0 means padding there), and the rows of every sequence's tokens in order."""
    q, k_pages, v_pages, table = case
    pool, P, Hkv, D = k_pages.shape
    k_rows = torch.cat([torch.zeros(1, Hkv, D, dtype=k_pages.dtype), k_pages.reshape(pool * P, Hkv, D)])
    v_rows = torch.cat([torch.zeros(1, Hkv, D, dtype=v_pages.dtype), v_pages.reshape(pool * P, Hkv, D)])
    loc = [1 + int(table[i, t // P]) * P + t % P for i, kv in enumerate(kv_lens) for t in range(kv)]
    return k_rows, v_rows, torch.tensor(loc, dtype=torch.int64)


def both(q_lens, kv_lens, *, Hq=8, Hkv=2, D=64, P=16, seed=0, dtype=torch.float32, pad_kv=0, **opt):
    c = make_case(q_lens, kv_lens, Hq, Hkv, D, P, seed, dtype=dtype)
    q, k_pages, v_pages, table = c["q"], c["k_pages"], c["v_pages"], c["page_indices"].numpy()
    sm_scale = 1.0 / math.sqrt(D)
    paged = ref_ragged_paged_attention(
        q, k_pages, v_pages, c["kv_lens"], c["page_indices"], c["cu_q_lens"], c["num_seqs"],
        sm_scale=sm_scale, sliding_window=opt.get("sliding_window_size"),
        xai_temperature_len=opt.get("xai_temperature_len"), attention_sink=opt.get("attention_sink"),
        softmax_dtype=opt.get("softmax_dtype"))
    k_rows, v_rows, loc = token_view((q, k_pages, v_pages, table), kv_lens)
    if pad_kv:
        loc = torch.cat([loc, torch.zeros(pad_kv, dtype=torch.int64)])
    decode = all(x == 1 for x in q_lens)
    native = ref_forward_attention(
        q, k_rows, v_rows, torch.tensor(kv_lens), loc,
        torch.tensor([k - x for k, x in zip(kv_lens, q_lens)]), torch.tensor(q_lens), Hq, Hkv, scale=sm_scale,
        is_causal=not decode, mode="decode" if decode else "extend", **opt)
    return paged, native.reshape(paged.shape), (q, k_pages, v_pages, table)


@pytest.mark.parametrize("opt", [
    {},
    {"sliding_window_size": 7},
    {"attention_sink": torch.tensor([0.3, -1.0, 2.0, 0.0, 1.5, -0.5, 0.1, 0.9])},
    {"xai_temperature_len": 8.0},
    {"sliding_window_size": 5, "attention_sink": torch.linspace(-1, 1, 8), "xai_temperature_len": 4.0},
])
def test_extend_batches_agree_with_the_paged_restatement(opt):
    """Chunks with and without a cached prefix, in f32 (both paths keep f32 scores then, so the
    only differences are summation order and the mask constant)."""
    paged, native, _ = both([5, 1, 9, 3], [5, 20, 30, 17], seed=11, pad_kv=3, **opt)
    torch.testing.assert_close(native, paged, rtol=2e-5, atol=2e-5)


@pytest.mark.parametrize("window", [None, 6, 64])
def test_decode_batches_agree_with_the_paged_restatement(window):
    opt = {"sliding_window_size": window} if window else {}
    paged, native, _ = both([1, 1, 1, 1, 1], [1, 16, 17, 40, 33], seed=12, pad_kv=5, **opt)
    torch.testing.assert_close(native, paged, rtol=2e-5, atol=2e-5)


def test_native_against_the_scalar_brute_force():
    """float64 loops (tests/bruteforce.py): independent of both restatements."""
    q_lens, kv_lens = [4, 2], [9, 12]
    paged, native, (q, k_pages, v_pages, table) = both(q_lens, kv_lens, Hq=4, Hkv=2, D=16, P=4, seed=13)
    P = k_pages.shape[1]
    t0 = 0
    for i, (ql, kv) in enumerate(zip(q_lens, kv_lens)):
        k = torch.stack([k_pages[int(table[i, t // P]), t % P] for t in range(kv)])
        v = torch.stack([v_pages[int(table[i, t // P]), t % P] for t in range(kv)])
        want = brute_attention(q[t0:t0 + ql].double().numpy(), k.double().numpy(), v.double().numpy(), ql, kv,
                               sm_scale=1.0 / math.sqrt(16))
        np.testing.assert_allclose(native[t0:t0 + ql].numpy(), want, rtol=1e-5, atol=1e-5)
        t0 += ql


def test_bf16_scores_stay_inside_the_parity_tolerance():
    """The native path keeps its scores in bf16 (no wider accumulator type is requested at
    native:256) where the paged path keeps f32: the two differ by bf16 rounding of the logits,
    which the parity tolerance of the bf16 kernels (2e-2) covers on inputs of this scale."""
    paged, native, _ = both([6, 1, 4], [6, 50, 31], seed=14, dtype=torch.bfloat16)
    torch.testing.assert_close(native.float(), paged.float(), rtol=2e-2, atol=2e-2)
    paged32, native32, _ = both([6, 1, 4], [6, 50, 31], seed=14, dtype=torch.bfloat16, softmax_dtype=torch.float32)
    torch.testing.assert_close(native32.float(), paged32.float(), rtol=2e-2, atol=2e-2)


def test_decode_temperature_uses_the_length_not_the_last_position():
    """native:273 takes seq_lengths as the decode query's position; the ragged kernel takes
    kv_len - 1 (rpa_v3:171-180).  At kv_len = xai_len + 1 only the native path scales."""
    paged, native, _ = both([1], [9], seed=15, xai_temperature_len=8.0)
    plain, _, _ = both([1], [9], seed=15)
    torch.testing.assert_close(paged, plain, rtol=1e-6, atol=1e-6)  # position 8 is not beyond 8
    assert (native - plain).abs().max() > 1e-4  # length 9 is
