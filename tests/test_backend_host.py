"""Host metadata builder of the attention backend (no GPU): the product builder
``build_forward_metadata`` against the oracle restatement of
layers/attention/flashattention_backend.py:146-237 and against hand-computed cases."""

import numpy as np
import pytest
from hypothesis import given, settings
from hypothesis import strategies as st

from oracle.ref_rpa import ref_forward_metadata


def make_cache_loc(rng, seq_lens, P, pool_pages):
    """Page-aligned slots per sequence, pages drawn without replacement (schedule_batch.py:2433-2454)."""
    n_pages = [-(-int(s) // P) for s in seq_lens]
    perm = rng.permutation(pool_pages)[: sum(n_pages)]
    loc, k = [], 0
    for n in n_pages:
        for p in perm[k:k + n]:
            loc.append(np.arange(p * P, p * P + P))
        k += n
    return (np.concatenate(loc) if loc else np.zeros(0)).astype(np.int32), perm


@settings(max_examples=60, deadline=None)
@given(st.integers(0, 2**31 - 1), st.sampled_from([1, 4, 16, 64]), st.integers(1, 9), st.booleans())
def test_builder_equals_oracle(pkg, seed, P, bs, is_decode):
    rng = np.random.default_rng(seed)
    seq_lens = rng.integers(0, 5 * P + 3, size=bs).astype(np.int32)
    seq_lens[::-1].sort()  # padded (zero-length) sequences sit at the end
    ext = np.minimum(seq_lens, rng.integers(1, 2 * P + 2, size=bs)).astype(np.int32)
    cache_loc, _ = make_cache_loc(rng, seq_lens, P, 64)
    got = pkg.build_forward_metadata(forward_mode="DECODE" if is_decode else pkg.ForwardMode.EXTEND,
                                     seq_lens=seq_lens, cache_loc=cache_loc, extend_seq_lens=ext, page_size=P)
    pi, cu_q, cu_kv, dist = ref_forward_metadata(cache_loc, seq_lens, ext, P, is_decode=is_decode)
    assert got["page_indices"].tolist() == pi.tolist()
    assert got["cu_q_lens"].tolist() == cu_q.tolist()
    assert got["cu_kv_lens"].tolist() == cu_kv.tolist()
    assert got["distribution"].tolist() == dist.tolist()
    for k in ("page_indices", "cu_q_lens", "cu_kv_lens", "distribution", "seq_lens"):
        assert got[k].dtype == np.int32


def test_hand_computed_case(pkg):
    P = 4
    seq_lens = np.array([5, 8, 1, 0], dtype=np.int32)
    pages = [[7, 2], [3, 9], [5], []]
    cache_loc = np.concatenate([np.arange(p * P, p * P + P) for ps in pages for p in ps]).astype(np.int32)
    md = pkg.build_forward_metadata(forward_mode=pkg.ForwardMode.DECODE, seq_lens=seq_lens, cache_loc=cache_loc,
                                    page_size=P)
    assert md["page_indices"].tolist() == [7, 2, 3, 9, 5]
    assert md["cu_q_lens"].tolist() == [0, 1, 2, 3, 4]
    assert md["cu_kv_lens"].tolist() == [0, 8, 16, 20, 20]
    assert md["distribution"].tolist() == [3, 3, 3]
    md = pkg.build_forward_metadata(forward_mode=pkg.ForwardMode.EXTEND, seq_lens=seq_lens, cache_loc=cache_loc,
                                    extend_seq_lens=np.array([2, 8, 1, 0]), page_size=P)
    assert md["cu_q_lens"].tolist() == [0, 2, 10, 11, 11]
    assert md["distribution"].tolist() == [0, 3, 3]


def test_data_parallel_sections_restart_at_zero(pkg):
    """flashattention_backend.py:190-224: every DP rank's section of cu_q / cu_kv starts at 0
    and distribution holds one triple per rank."""
    P = 2
    seq_lens = np.array([3, 0, 2, 4], dtype=np.int32)  # rank 0: [3, 0]; rank 1: [2, 4]
    cache_loc = np.array([4, 5, 6, 7, 0, 0, 10, 11, 20, 21, 22, 23], dtype=np.int32)  # 6 slots per rank
    md = pkg.build_forward_metadata(forward_mode="EXTEND", seq_lens=seq_lens, cache_loc=cache_loc,
                                    extend_seq_lens=np.array([3, 0, 1, 2]), page_size=P, dp_size=2, per_dp_bs_size=2)
    assert md["page_indices"].tolist() == [2, 3, 0, 5, 10, 11]
    assert md["cu_q_lens"].tolist() == [0, 3, 3, 0, 1, 3]
    assert md["cu_kv_lens"].tolist() == [0, 4, 4, 0, 2, 6]
    assert md["distribution"].tolist() == [0, 1, 1, 0, 2, 2]
    md = pkg.build_forward_metadata(forward_mode="DECODE", seq_lens=seq_lens, cache_loc=cache_loc, page_size=P,
                                    dp_size=2, per_dp_bs_size=2)
    assert md["cu_q_lens"].tolist() == [0, 1, 2, 0, 1, 2]
    assert md["distribution"].tolist() == [1, 1, 1, 2, 2, 2]


def test_sliding_window_pool_mapping(pkg):
    """flashattention_backend.py:178-188: full-pool slot -> window-pool slot, then // P."""
    P = 4
    cache_loc = np.array([8, 9, 10, 11, 0, 1, 2, 3], dtype=np.int32)
    mapping = np.arange(64, dtype=np.int32)[::-1].copy()  # slot s -> 63 - s
    md = pkg.build_forward_metadata(forward_mode="DECODE", seq_lens=np.array([4, 3], dtype=np.int32),
                                    cache_loc=cache_loc, page_size=P, swa_index_mapping=mapping)
    assert md["page_indices"].tolist() == [2, 0]
    assert md["swa_page_indices"].tolist() == [(63 - 8) // 4, (63 - 0) // 4]


def test_error_messages(pkg):
    kw = dict(seq_lens=np.array([1, 2], dtype=np.int32), cache_loc=np.arange(8, dtype=np.int32), page_size=4)
    with pytest.raises(ValueError, match="Invalid dp_size"):
        pkg.build_forward_metadata(forward_mode="DECODE", dp_size=0, **kw)
    with pytest.raises(ValueError, match="Inconsistent DP batch metadata"):
        pkg.build_forward_metadata(forward_mode="DECODE", dp_size=1, per_dp_bs_size=3, **kw)
    with pytest.raises(ValueError, match="not divisible by dp_size"):
        pkg.build_forward_metadata(forward_mode="DECODE", dp_size=2, per_dp_bs_size=1,
                                   seq_lens=kw["seq_lens"], cache_loc=np.arange(7, dtype=np.int32), page_size=4)
    with pytest.raises(ValueError, match="Invalid forward mode"):
        pkg.build_forward_metadata(forward_mode="IDLE", **kw)


def test_max_running_requests(pkg):
    """flashattention_backend.py:770-777."""
    assert pkg.FlashAttention.get_max_running_reqests(4096, 64) == 1024 * 1024 // 2 // 64 // 4
    with pytest.raises(AssertionError):
        pkg.FlashAttention.get_max_running_reqests(1 << 30, 1)


def test_mla_extend_distribution(pkg):
    """mla_backend.py:192-199: an extend batch is declared (0, 0, n)."""
    md = pkg.build_forward_metadata(forward_mode="EXTEND", seq_lens=np.array([5, 8, 0], dtype=np.int32),
                                    cache_loc=np.arange(16, dtype=np.int32), extend_seq_lens=np.array([2, 8, 0]),
                                    page_size=4, extend_distribution_is_mixed=True)
    assert md["distribution"].tolist() == [0, 0, 2]
    md = pkg.build_forward_metadata(forward_mode="DECODE", seq_lens=np.array([5, 8, 0], dtype=np.int32),
                                    cache_loc=np.arange(16, dtype=np.int32), page_size=4,
                                    extend_distribution_is_mixed=True)
    assert md["distribution"].tolist() == [2, 2, 2]


def test_pad_page_indices_buckets(pkg):
    """flashattention_backend.py:42-69, worked by hand: 4 slots, 70 pages -> 18 per slot -> 32 per
    slot -> 128 entries; 3 pages -> the floor of 16 per slot; a fixed capacity wins over both."""
    pad = pkg.backend.pad_page_indices
    out = pad(np.arange(1, 71), 4)
    assert out.dtype == np.int32 and len(out) == 128
    assert np.array_equal(out[:70], np.arange(1, 71)) and not out[70:].any()
    assert len(pad(np.arange(3), 4)) == 64
    assert len(pad(np.arange(64), 4)) == 64  # exactly 16 per slot stays
    assert len(pad(np.arange(65), 4)) == 128  # 17 -> 32
    assert len(pad(np.arange(0), 4)) == 0
    assert len(pad(np.arange(5), 4, fixed_capacity=24)) == 24
    with pytest.raises(ValueError, match="exceed fixed capacity: required=5, capacity=4"):
        pad(np.arange(5), 4, fixed_capacity=4)


def test_verify_metadata_hand_case(pkg):
    """Target-verify (flashattention_backend.py:298-376): 3 slots, the middle one padding, 2 draft
    tokens, pages of 4.  Verified lengths 3 and 1 become kv lengths 5 and 3; mask rows widen to 8
    and 4 entries; the padding slot's 2*(2-1) mask entries vanish."""
    m0 = np.array([1, 1, 1, 1, 0, 1, 1, 1, 1, 1], dtype=np.int32)  # 2 rows of 5
    pad_slot = np.array([7, 7], dtype=np.int32)  # dropped
    m2 = np.array([1, 1, 0, 1, 1, 1], dtype=np.int32)  # 2 rows of 3
    md = pkg.backend.build_verify_metadata(
        seq_lens=[3, 0, 1], draft_token_num=2, logits_indices_selector=[0, 2],
        custom_mask=np.concatenate([m0, pad_slot, m2]), page_size=4,
    )
    assert md["extend_seq_lens"].tolist() == [2, 0, 2]
    assert md["seq_lens"].tolist() == [5, 0, 3]
    assert md["cu_q_lens"].tolist() == [0, 2, 2, 4]
    assert md["cu_kv_lens"].tolist() == [0, 8, 8, 12]
    assert md["distribution"].tolist() == [0, 2, 2]
    want = [1, 1, 1, 1, 0, 0, 0, 0, 1, 1, 1, 1, 1, 0, 0, 0, 1, 1, 0, 0, 1, 1, 1, 0]
    assert md["custom_mask"].tolist() == want  # 24 entries: 18 in, rounded to 24, equals the packed length
    assert md["custom_mask"].dtype == np.int32


def test_verify_metadata_two_ranks_share_one_length(pkg):
    """dp_size 2: each rank's packed mask is padded to the longer one (or to the original length per
    rank rounded up to 8 when that is more), and the cumulative lengths restart per rank."""
    q, P = 2, 4
    kv = [9, 2]  # after the draft tokens: verified 7 and 0 -> second slot is padding?  no: verified 0 means padding
    mask = np.concatenate([np.ones(q * 9, np.int32), np.full(q * (q - 1), 5, np.int32)])
    md = pkg.backend.build_verify_metadata(
        seq_lens=[7, 0], draft_token_num=q, logits_indices_selector=[0], custom_mask=mask, page_size=P, dp_size=2,
    )
    assert md["seq_lens"].tolist() == [9, 0]
    assert md["cu_q_lens"].tolist() == [0, 2, 0, 0]
    assert md["cu_kv_lens"].tolist() == [0, 12, 0, 0]
    assert md["distribution"].tolist() == [0, 1, 1, 0, 0, 0]
    cm = md["custom_mask"].reshape(2, -1)
    assert cm.shape == (2, 24)  # rank 0 packs 2 rows of 12; 20 // 2 -> 16 is less
    assert cm[0].reshape(2, 12)[:, :9].all() and not cm[0].reshape(2, 12)[:, 9:].any()
    assert not cm[1].any()
    with pytest.raises(ValueError, match="bool dtype is not supported"):
        pkg.backend.build_verify_metadata(
            seq_lens=[7, 0], draft_token_num=q, logits_indices_selector=[0],
            custom_mask=np.ones(22, dtype=bool), page_size=P, dp_size=2,
        )


def test_verify_mask_runs_through_the_oracle_shapes(pkg):
    """The packed mask has exactly the layout the kernel's aligned mode indexes:
    row t of slot s starts at q * cu_kv_aligned[s] + t * aligned_len[s]."""
    rng = np.random.default_rng(3)
    q, P = 4, 16
    verified = np.array([33, 0, 7, 120], dtype=np.int32)
    kv = np.where(verified > 0, verified + q, 0)
    parts = [rng.integers(0, 2, q * (k if k > 0 else q - 1)).astype(np.int32) for k in kv]
    md = pkg.backend.build_verify_metadata(
        seq_lens=verified, draft_token_num=q, logits_indices_selector=np.flatnonzero(verified),
        custom_mask=np.concatenate(parts), page_size=P,
    )
    cu = md["cu_kv_lens"]
    for s, k in enumerate(kv):
        if k == 0:
            continue
        width = cu[s + 1] - cu[s]
        for t in range(q):
            row = md["custom_mask"][q * cu[s] + t * width :][:width]
            assert np.array_equal(row[:k], parts[s].reshape(q, k)[t]) and not row[k:].any()
