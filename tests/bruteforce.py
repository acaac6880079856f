"""Float64 scalar-loop attention used to pin the oracle on tiny inputs.

Written from the definition of masked softmax attention, independently of
oracle/ref_rpa.py: no einsum, no shared helpers.  The only conventions taken
from the reference are the ones under test -- query j of a sequence sits at
position kv_len - q_len + j, sees keys t <= position and (with a window W)
t > position - W, query head h reads kv head h // G, scores are
scale -> soft-cap -> mask."""

import math

import numpy as np


def brute_attention(q, k, v, q_len, kv_len, *, sm_scale, window=None, soft_cap=None, sink=None):
    """q [q_len, Hq, D], k/v [kv_len, Hkv, D] float64 arrays -> [q_len, Hq, Dv]."""
    Hq, D = q.shape[1], q.shape[2]
    Hkv = k.shape[1]
    G = Hq // Hkv
    out = np.zeros((q_len, Hq, v.shape[2]))
    for j in range(q_len):
        pos = kv_len - q_len + j
        for h in range(Hq):
            hk = h // G
            scores = []
            toks = []
            for t in range(kv_len):
                if t > pos:
                    continue
                if window is not None and t <= pos - window:
                    continue
                s = 0.0
                for d in range(D):
                    s += q[j, h, d] * k[t, hk, d]
                s *= sm_scale
                if soft_cap is not None:
                    s = soft_cap * math.tanh(s / soft_cap)
                scores.append(s)
                toks.append(t)
            mx = max(scores + ([sink[h]] if sink is not None else []))
            den = sum(math.exp(s - mx) for s in scores)
            if sink is not None:
                den += math.exp(sink[h] - mx)
            for s, t in zip(scores, toks):
                w = math.exp(s - mx) / den
                out[j, h] += w * v[t, hk]
    return out


def bf16_round(x):
    """Round a float64/float32 array to bfloat16 precision (round to nearest even)."""
    import torch

    return torch.from_numpy(np.asarray(x, dtype=np.float32)).to(torch.bfloat16).to(torch.float64).numpy()
