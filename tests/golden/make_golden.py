"""Writes tests/golden/rpa_small.npz and tests/golden/mla_small.npz.

Inputs are seeded bf16 tensors (stored as int16 bit patterns: numpy has no
bfloat16); expected outputs are EXACT float64 results of the scalar-loop brute
force in tests/bruteforce.py, which shares no code with the oracle.  Lengths walk
page boundaries the way the reference's decode sweep does
(python/sgl_jax/test/test_flashattention_gqa.py:61-71: P-1, P, P+1, ...), scaled
to sizes a Python triple loop finishes in seconds.

Run from the repository root:  python tests/golden/make_golden.py
"""

import math
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from tests.bruteforce import brute_attention  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def bits(t):
    return t.view(torch.int16).numpy()


def rpa_cases():
    # (q_lens, kv_lens, Hq, Hkv, D, P, window, soft_cap)
    return [
        ([1, 1, 1, 1, 1], [7, 8, 9, 15, 17], 4, 2, 16, 8, 0, 0.0),     # decode, page-boundary sweep
        ([1, 3, 8, 5], [16, 20, 8, 5], 4, 1, 16, 4, 0, 0.0),           # mixed, (3,20) (8,8) (5,5) style
        ([1, 6, 2], [25, 19, 30], 6, 2, 8, 8, 6, 0.0),                 # sliding window
        ([1, 4], [11, 12], 4, 4, 8, 4, 0, 2.0),                        # soft cap, MHA
        ([1, 5], [23, 14], 8, 2, 8, 1, 5, 3.0),                        # page_size 1, window + cap
    ]


def build(case, seed):
    q_lens, kv_lens, Hq, Hkv, D, P, window, cap = case
    g = torch.Generator().manual_seed(seed)
    rng = np.random.default_rng(seed)
    S = len(q_lens)
    counts = [-(-k // P) for k in kv_lens]
    pool = sum(counts) + 2
    perm = rng.permutation(pool)[: sum(counts)].astype(np.int32)
    table = np.zeros((S, max(counts)), dtype=np.int32)
    o = 0
    for i, c in enumerate(counts):
        table[i, :c] = perm[o : o + c]
        o += c
    q = torch.randn(sum(q_lens), Hq, D, generator=g).to(torch.bfloat16)
    kp = torch.randn(pool, P, Hkv, D, generator=g).to(torch.bfloat16)
    vp = torch.randn(pool, P, Hkv, D, generator=g).to(torch.bfloat16)
    sm = 1.0 / math.sqrt(D)
    outs = []
    o = 0
    for i in range(S):
        idx = torch.from_numpy(table[i]).long()
        k = kp[idx].reshape(-1, Hkv, D)[: kv_lens[i]].double().numpy()
        v = vp[idx].reshape(-1, Hkv, D)[: kv_lens[i]].double().numpy()
        qi = q[o : o + q_lens[i]].double().numpy()
        outs.append(brute_attention(qi, k, v, q_lens[i], kv_lens[i], sm_scale=sm,
                                    window=window or None, soft_cap=cap or None))
        o += q_lens[i]
    cu_q = np.zeros(S + 1, dtype=np.int32)
    cu_q[1:] = np.cumsum(q_lens)
    return dict(q_bf16_bits=bits(q), k_pages_bf16_bits=bits(kp), v_pages_bf16_bits=bits(vp),
                kv_lens=np.asarray(kv_lens, dtype=np.int32), page_indices=table, cu_q_lens=cu_q,
                num_seqs=np.int32(S), sm_scale=np.float64(sm), window=np.int32(window),
                soft_cap=np.float64(cap), expected_f64=np.concatenate(outs, axis=0))


def mla_case(seed):
    """Absorbed MLA: Hq heads, latent 32 + rope 8 (scaled-down 512 + 64), one shared row per token."""
    g = torch.Generator().manual_seed(seed)
    rng = np.random.default_rng(seed)
    Hq, lkv, rope, P = 4, 32, 8, 4
    kv_lens = [9, 16, 5]
    S = len(kv_lens)
    counts = [-(-k // P) for k in kv_lens]
    pool = sum(counts) + 2
    perm = rng.permutation(pool)[: sum(counts)].astype(np.int32)
    pps = max(counts)
    table = np.zeros((S, pps), dtype=np.int32)
    o = 0
    for i, c in enumerate(counts):
        table[i, :c] = perm[o : o + c]
        o += c
    ql = (torch.randn(S, Hq, lkv, generator=g) * 0.5).to(torch.bfloat16)
    qp = (torch.randn(S, Hq, rope, generator=g) * 0.5).to(torch.bfloat16)
    cache = (torch.randn(pool, P, lkv + rope, generator=g) * 0.5).to(torch.bfloat16)
    sm = 1.0 / math.sqrt(24.0)
    outs = []
    for i in range(S):
        idx = torch.from_numpy(table[i]).long()
        rows = cache[idx].reshape(-1, lkv + rope)[: kv_lens[i]].double().numpy()
        q = torch.cat([ql[i], qp[i]], dim=-1).double().numpy()[None]  # [1, Hq, 40]
        k = rows[:, None, :]                                         # one shared kv head
        v = rows[:, None, :lkv]
        outs.append(brute_attention(q, k, v, 1, kv_lens[i], sm_scale=sm))
    return dict(ql_nope_bits=bits(ql), q_pe_bits=bits(qp), cache_bits=bits(cache),
                kv_lens=np.asarray(kv_lens, dtype=np.int32), page_indices=table.reshape(-1),
                cu_q_lens=np.arange(S + 1, dtype=np.int32), sm_scale=np.float64(sm),
                expected_f64=np.concatenate(outs, axis=0))


def main():
    blob = {"n_cases": np.int32(len(rpa_cases()))}
    for ci, case in enumerate(rpa_cases()):
        for k, v in build(case, 100 + ci).items():
            blob[f"c{ci}_{k}"] = v
    np.savez_compressed(os.path.join(HERE, "rpa_small.npz"), **blob)
    np.savez_compressed(os.path.join(HERE, "mla_small.npz"), **mla_case(200))
    print("wrote", os.listdir(HERE))


if __name__ == "__main__":
    main()
