"""Seeded synthetic batches for the five benchmark configurations.

Lengths, page permutations and page tables come from
``numpy.random.Generator(PCG64(seed))`` so the metadata is identical on every
machine; tensor values come from a seeded torch generator on the requested
device (CPU for parity tests, the GPU for full-size bench runs, where drawing
gigabytes of normals on the host would dominate the run time).

Layouts follow the reference's KV pools:
  * MHA/GQA cache: ``[pages, P, 2*Hkv, D]`` with heads stored K0,V0,K1,V1,...
    (python/sgl_jax/srt/mem_cache/memory_pool.py:56-91, 580-588);
  * page table: flat, sequence i owns ``cdiv(kv_len_i, P)`` consecutive entries
    starting at ``cu_kv_lens[i] // P`` where ``cu_kv_lens`` is the cumulative sum
    of page-aligned lengths
    (python/sgl_jax/srt/layers/attention/flashattention_backend.py:168-212);
  * sequences ordered decode-only first, then prefill/mixed, described by
    ``distribution = (decode_end, prefill_end, total)``
    (python/sgl_jax/srt/kernels/ragged_paged_attention/ragged_paged_attention_v3.py:82-91).
"""

from __future__ import annotations

import math
from dataclasses import dataclass, field

import numpy as np
import torch

FP8_E4M3_MAX = 448.0


@dataclass
class Batch:
    name: str
    q: torch.Tensor  # [T, Hq, D] bf16
    kv_cache: torch.Tensor  # [pages, P, 2*Hkv, D] bf16 / float8_e4m3fn
    kv_lens: torch.Tensor  # i32[S]
    page_indices: torch.Tensor  # i32[flat]
    cu_q_lens: torch.Tensor  # i32[S+1]
    cu_kv_lens: torch.Tensor  # i32[S+1]
    distribution: torch.Tensor  # i32[3]
    sm_scale: float
    page_size: int
    num_kv_heads: int
    sliding_window: int | None = None
    soft_cap: float | None = None
    k_scale: torch.Tensor | None = None  # f32[Hkv]
    v_scale: torch.Tensor | None = None
    meta: dict = field(default_factory=dict)

    @property
    def num_seqs(self) -> int:
        return int(self.kv_lens.shape[0])

    def to(self, device) -> "Batch":
        kw = {}
        for k, v in self.__dict__.items():
            kw[k] = v.to(device) if isinstance(v, torch.Tensor) else v
        return Batch(**kw)

    def q_lens(self) -> np.ndarray:
        cu = self.cu_q_lens.cpu().numpy()
        return cu[1:] - cu[:-1]

    def padded_page_table(self) -> torch.Tensor:
        """The flat table re-laid as the zero-padded [S, pages_per_seq] table the
        pure-jnp reference consumes (ragged_paged_attention_v3.py:99)."""
        P = self.page_size
        kv = self.kv_lens.cpu().numpy()
        cu = self.cu_kv_lens.cpu().numpy()
        flat = self.page_indices.cpu().numpy()
        counts = -(-kv // P)
        width = max(int(counts.max()) if len(counts) else 1, 1)
        table = np.zeros((len(kv), width), dtype=np.int32)
        for i in range(len(kv)):
            s = cu[i] // P
            table[i, : counts[i]] = flat[s : s + counts[i]]
        return torch.from_numpy(table)


@dataclass
class MlaBatch:
    name: str
    ql_nope: torch.Tensor  # [T, Hq, lkv] bf16
    q_pe: torch.Tensor  # [T, Hq, rope] bf16
    cache_kv: torch.Tensor  # [pages, P, lkv+rope] bf16 (compact latent rows)
    kv_lens: torch.Tensor
    page_indices: torch.Tensor  # flat ragged
    cu_q_lens: torch.Tensor
    cu_kv_lens: torch.Tensor
    distribution: torch.Tensor
    sm_scale: float
    page_size: int
    sliding_window: int | None = None
    soft_cap: float | None = None
    meta: dict = field(default_factory=dict)

    def to(self, device) -> "MlaBatch":
        kw = {}
        for k, v in self.__dict__.items():
            kw[k] = v.to(device) if isinstance(v, torch.Tensor) else v
        return MlaBatch(**kw)

    def padded_page_indices(self):
        """Flat ragged table -> the padded ``[S * pages_per_seq]`` layout the MLA
        reference indexes with ``i * pages_per_seq`` (kernels/mla/v1/ref.py:197-200)."""
        P = self.page_size
        kv = self.kv_lens.cpu().numpy()
        cu = self.cu_kv_lens.cpu().numpy()
        flat = self.page_indices.cpu().numpy()
        counts = -(-kv // P)
        width = max(int(counts.max()) if len(counts) else 1, 1)
        table = np.zeros((len(kv), width), dtype=np.int32)
        for i in range(len(kv)):
            s = cu[i] // P
            table[i, : counts[i]] = flat[s : s + counts[i]]
        return torch.from_numpy(table.reshape(-1))


def _normal(shape, std, dtype, device, seed):
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    n = int(np.prod(shape))
    # draw in slabs so the f32 staging buffer stays small next to a multi-GiB pool
    out = torch.empty(n, dtype=dtype, device=device)
    slab = 1 << 26
    for s in range(0, n, slab):
        e = min(n, s + slab)
        out[s:e] = (torch.randn(e - s, generator=g, device=device, dtype=torch.float32) * std).to(dtype)
    return out.reshape(shape)


def _paging(rng: np.random.Generator, kv_lens: np.ndarray, page_size: int, pool_pages: int | None, canary: int = 1):
    """Random physical placement: the pages a batch needs are the first entries of
    a seeded permutation of the pool, skipping ``canary`` guard pages at each end."""
    counts = -(-kv_lens // page_size)
    need = int(counts.sum())
    if pool_pages is None:
        pool_pages = need + 2 * canary
        usable = np.arange(canary, canary + need)
    else:
        usable = np.arange(pool_pages)
        assert need <= pool_pages
    perm = rng.permutation(usable)[:need].astype(np.int32)
    aligned = counts * page_size
    cu_kv = np.zeros(len(kv_lens) + 1, dtype=np.int32)
    cu_kv[1:] = np.cumsum(aligned)
    return perm, cu_kv, pool_pages


def make_batch(
    name: str,
    q_lens,
    kv_lens,
    *,
    num_q_heads: int,
    num_kv_heads: int,
    head_dim: int,
    page_size: int,
    seed: int,
    device="cpu",
    pool_pages: int | None = None,
    kv_dtype=torch.bfloat16,
    sliding_window: int | None = None,
    soft_cap: float | None = None,
    sm_scale: float | None = None,
    std: float = 1.0,
    pad_tokens: int = 0,
    pad_seqs: int = 0,
) -> Batch:
    """General ragged batch.  Sequences must already be ordered decode-first."""
    rng = np.random.Generator(np.random.PCG64(seed))
    q_lens = np.asarray(q_lens, dtype=np.int64)
    kv_lens = np.asarray(kv_lens, dtype=np.int64)
    S = len(q_lens)
    assert np.all(q_lens > 0) and np.all(q_lens <= kv_lens)
    decode_end = 0
    while decode_end < S and q_lens[decode_end] == 1:
        decode_end += 1
    perm, cu_kv, pool_pages = _paging(rng, kv_lens, page_size, pool_pages)
    T = int(q_lens.sum())
    cu_q = np.zeros(S + 1 + pad_seqs, dtype=np.int32)
    cu_q[1 : S + 1] = np.cumsum(q_lens)
    cu_q[S + 1 :] = T
    kv_pad = np.concatenate([kv_lens, np.zeros(pad_seqs, dtype=np.int64)]).astype(np.int32)
    cu_kv = np.concatenate([cu_kv, np.full(pad_seqs, cu_kv[-1], dtype=np.int32)])

    q = _normal((T + pad_tokens, num_q_heads, head_dim), std, torch.bfloat16, device, seed * 7 + 1)
    shape = (pool_pages, page_size, 2 * num_kv_heads, head_dim)
    k_scale = v_scale = None
    if kv_dtype == torch.bfloat16:
        cache = _normal(shape, std, torch.bfloat16, device, seed * 7 + 2)
    else:
        raw = _normal(shape, std, torch.bfloat16, device, seed * 7 + 2).to(torch.float32)
        k_amax = raw[:, :, 0::2].abs().amax(dim=(0, 1, 3))
        v_amax = raw[:, :, 1::2].abs().amax(dim=(0, 1, 3))
        k_scale = (k_amax / FP8_E4M3_MAX).to(torch.float32)
        v_scale = (v_amax / FP8_E4M3_MAX).to(torch.float32)
        scale = torch.stack([k_scale, v_scale], dim=1).reshape(1, 1, 2 * num_kv_heads, 1)
        cache = (raw / scale).to(torch.float8_e4m3fn)
        del raw
    return Batch(
        name=name,
        q=q,
        kv_cache=cache,
        kv_lens=torch.from_numpy(kv_pad).to(device),
        page_indices=torch.from_numpy(perm).to(device),
        cu_q_lens=torch.from_numpy(cu_q).to(device),
        cu_kv_lens=torch.from_numpy(cu_kv).to(device),
        distribution=torch.tensor([decode_end, decode_end, S], dtype=torch.int32, device=device),
        sm_scale=float(sm_scale if sm_scale is not None else 1.0 / math.sqrt(head_dim)),
        page_size=page_size,
        num_kv_heads=num_kv_heads,
        sliding_window=sliding_window,
        soft_cap=soft_cap,
        k_scale=k_scale,
        v_scale=v_scale,
        meta={"q_lens": q_lens.tolist(), "kv_lens": kv_lens.tolist(), "seed": seed},
    )


def _scaled(x: int, scale: float, lo: int = 1) -> int:
    return max(lo, int(round(x * scale)))


def config_c1(device="cpu", scale: float = 1.0) -> Batch:
    """Decode-only, Qwen3-0.6B shape: 8 seqs x 1 token, Hq16/Hkv8/D128, P=16,
    kv_len ~ U[64,512], 512-page pool."""
    seed = 1001
    rng = np.random.Generator(np.random.PCG64(seed))
    S = 8
    kv = rng.integers(_scaled(64, scale), _scaled(512, scale), size=S, endpoint=True)
    return make_batch("c1_qwen3_0p6b_decode", np.ones(S, int), kv, num_q_heads=16, num_kv_heads=8,
                      head_dim=128, page_size=16, seed=seed, device=device, pool_pages=512)


def config_c2(device="cpu", scale: float = 1.0) -> Batch:
    """Mixed ragged batch, Llama-3-8B shape: 56 decode rows (kv ~ U[512,4096]) then
    8 prefill chunks (q ~ U[128,2048], prefix ~ U[0,2048]); Hq32/Hkv8/D128, P=64."""
    seed = 1002
    rng = np.random.Generator(np.random.PCG64(seed))
    kv_d = rng.integers(_scaled(512, scale), _scaled(4096, scale), size=56, endpoint=True)
    q_p = rng.integers(_scaled(128, scale), _scaled(2048, scale), size=8, endpoint=True)
    pre = rng.integers(0, _scaled(2048, scale), size=8, endpoint=True)
    q_lens = np.concatenate([np.ones(56, int), q_p])
    kv_lens = np.concatenate([kv_d, pre + q_p])
    return make_batch("c2_llama3_8b_mixed", q_lens, kv_lens, num_q_heads=32, num_kv_heads=8,
                      head_dim=128, page_size=64, seed=seed, device=device)


def config_c3(device="cpu", scale: float = 1.0) -> Batch:
    """Long-context decode, Llama-3-8B shape: 16 seqs x 1 token, kv_len 32768, P=64."""
    seed = 1003
    S = 16
    kv = np.full(S, _scaled(32768, scale), dtype=np.int64)
    return make_batch("c3_llama3_8b_long_decode", np.ones(S, int), kv, num_q_heads=32, num_kv_heads=8,
                      head_dim=128, page_size=64, seed=seed, device=device)


def config_c4(device="cpu", scale: float = 1.0, window: bool = False) -> Batch:
    """fp8-e4m3 KV decode, Qwen3-32B shape: 128 seqs x 1 token, Hq64/Hkv8/D128,
    kv ~ U[1024,8192], P=64, per-kv-head scale max|x|/448; sliding window 4096 on
    alternating layers (``window=True`` selects that layer kind)."""
    seed = 1004
    rng = np.random.Generator(np.random.PCG64(seed))
    S = 128
    kv = rng.integers(_scaled(1024, scale), _scaled(8192, scale), size=S, endpoint=True)
    return make_batch("c4_qwen3_32b_fp8_decode" + ("_swa" if window else ""), np.ones(S, int), kv,
                      num_q_heads=64, num_kv_heads=8, head_dim=128, page_size=64, seed=seed,
                      device=device, kv_dtype=torch.float8_e4m3fn,
                      sliding_window=_scaled(4096, scale) if window else None)


def make_mla_batch(name, q_lens, kv_lens, *, num_q_heads, lkv_dim, rope_dim, page_size, seed,
                   device="cpu", sm_scale=None, std=0.5, sliding_window=None, soft_cap=None,
                   kv_dtype=torch.bfloat16) -> MlaBatch:
    rng = np.random.Generator(np.random.PCG64(seed))
    q_lens = np.asarray(q_lens, dtype=np.int64)
    kv_lens = np.asarray(kv_lens, dtype=np.int64)
    S = len(q_lens)
    decode_end = 0
    while decode_end < S and q_lens[decode_end] == 1:
        decode_end += 1
    perm, cu_kv, pool_pages = _paging(rng, kv_lens, page_size, None)
    T = int(q_lens.sum())
    cu_q = np.zeros(S + 1, dtype=np.int32)
    cu_q[1:] = np.cumsum(q_lens)
    return MlaBatch(
        name=name,
        ql_nope=_normal((T, num_q_heads, lkv_dim), std, torch.bfloat16, device, seed * 7 + 1),
        q_pe=_normal((T, num_q_heads, rope_dim), std, torch.bfloat16, device, seed * 7 + 3),
        cache_kv=_normal((pool_pages, page_size, lkv_dim + rope_dim), std, kv_dtype, device, seed * 7 + 2),
        kv_lens=torch.from_numpy(kv_lens.astype(np.int32)).to(device),
        page_indices=torch.from_numpy(perm).to(device),
        cu_q_lens=torch.from_numpy(cu_q).to(device),
        cu_kv_lens=torch.from_numpy(cu_kv).to(device),
        distribution=torch.tensor([decode_end, decode_end, S], dtype=torch.int32, device=device),
        sm_scale=float(sm_scale if sm_scale is not None else 1.0 / math.sqrt(lkv_dim + rope_dim)),
        page_size=page_size,
        sliding_window=sliding_window,
        soft_cap=soft_cap,
        meta={"q_lens": q_lens.tolist(), "kv_lens": kv_lens.tolist(), "seed": seed},
    )


def config_c5(device="cpu", scale: float = 1.0, num_q_heads: int = 128, kv_dtype=torch.bfloat16) -> MlaBatch:
    """Absorbed-MLA decode, DeepSeek-V3 shape: 64 seqs x 1 token, 128 q heads,
    latent 512 + rope 64 (one shared 576-wide row per token), kv ~ U[2048,16384],
    P=64, values ~ N(0, 0.5), sm_scale 1/sqrt(192)."""
    seed = 1005
    rng = np.random.Generator(np.random.PCG64(seed))
    S = 64
    kv = rng.integers(_scaled(2048, scale), _scaled(16384, scale), size=S, endpoint=True)
    name = ("c5_deepseek_v3_mla_decode" + ("" if kv_dtype == torch.bfloat16 else "_fp8") +
            ("" if num_q_heads == 128 else f"_{num_q_heads}_heads"))
    return make_mla_batch(name, np.ones(S, int), kv, num_q_heads=num_q_heads,
                          lkv_dim=512, rope_dim=64, page_size=64, seed=seed, device=device,
                          sm_scale=1.0 / math.sqrt(192.0), kv_dtype=kv_dtype)


def config_c5_prefill(device="cpu", scale: float = 1.0, num_q_heads: int = 128, num_seqs: int = 4) -> MlaBatch:
    """Absorbed-MLA prefill chunks, DeepSeek-V3 shape: `num_seqs` sequences, each a 512-token chunk
    on a 4096-token prefix (kv_len 4608); 128 q heads, latent 512 + rope 64, P=64."""
    seed = 1006
    q = _scaled(512, scale)
    kv = _scaled(4096, scale) + q
    name = "c5p_deepseek_v3_mla_prefill" + ("" if num_q_heads == 128 else f"_{num_q_heads}_heads")
    return make_mla_batch(name, np.full(num_seqs, q), np.full(num_seqs, kv),
                          num_q_heads=num_q_heads, lkv_dim=512, rope_dim=64, page_size=64, seed=seed, device=device,
                          sm_scale=1.0 / math.sqrt(192.0))


# --------------------------------------------------------------------------
# Peaked inputs: a few keys per (sequence, kv head) that every query of that head attends to
# --------------------------------------------------------------------------
def needle_positions(rng: np.random.Generator, kv_len: int, window: int | None, count: int = 4) -> list[int]:
    """Token positions worth a needle: the first and last tiles of the row, tile / page / piece
    borders inside it (multiples of 32 ... 4096 and their neighbours) and the edge of the sliding
    window.  One position always comes from the first 64 tokens and one from the last 64."""
    cand = {0, 1, 31, 32, 63, 64, kv_len - 1, kv_len - 2, kv_len - 32, kv_len - 33, kv_len - 64, kv_len - 65}
    for step in (32, 64, 128, 256, 512, 1024, 4096):
        for k in rng.integers(1, max(2, kv_len // step + 1), size=2):
            cand.update({int(k) * step - 1, int(k) * step})
    if window:
        cand.update({kv_len - window - 1, kv_len - window, kv_len - window + 1})
    cand = sorted(t for t in cand if 0 <= t < kv_len)
    first = [t for t in cand if t < 64]
    last = [t for t in cand if t >= kv_len - 64]
    picks = {int(rng.choice(first)), int(rng.choice(last))}
    picks.update(int(t) for t in rng.choice(cand, size=min(count, len(cand)), replace=False))
    return sorted(picks)


def plant_needles(b: Batch, *, logit: float = 14.0, seed: int = 0, count: int = 4) -> dict:
    """Make the batch peaked, in place: for every (sequence, kv head) draw a
    direction u of +-1/sqrt(D) entries, add a*u to the queries of that head group and overwrite the
    K rows of a few tokens with a*u, a = sqrt(logit / sm_scale), so that those tokens score about
    `logit` above the random ones and carry most of the softmax weight: output rows are O(1)
    whatever the row length, and losing the tile, split or partial row that holds a needle
    changes them by tens of per cent.  Returns {(seq, kv head): positions}."""
    rng = np.random.Generator(np.random.PCG64(77000 + seed))
    dev = b.q.device
    P, Hkv = b.page_size, b.num_kv_heads
    Hq, D = b.q.shape[1], b.q.shape[2]
    G = Hq // Hkv
    a = math.sqrt(logit / b.sm_scale)
    kv = b.kv_lens.cpu().numpy()
    cu_q = b.cu_q_lens.cpu().numpy()
    cu_kv = b.cu_kv_lens.cpu().numpy()
    pages = b.page_indices.cpu().numpy()
    n = int(b.distribution[2])
    k_scale = None if b.k_scale is None else b.k_scale.cpu()
    fp8 = b.kv_cache.dtype != torch.bfloat16
    placed = {}
    q = b.q.float()
    for i in range(n):
        for h in range(Hkv):
            u = torch.from_numpy(rng.choice([-1.0, 1.0], size=D).astype(np.float32)) / math.sqrt(D)
            q[cu_q[i]:cu_q[i + 1], h * G:(h + 1) * G] += (a * u).to(dev)
            pos = needle_positions(rng, int(kv[i]), b.sliding_window, count)
            for t in pos:
                page = int(pages[cu_kv[i] // P + t // P])
                row = a * u
                if fp8:
                    row = row / k_scale[h]
                b.kv_cache[page, t % P, 2 * h] = row.to(b.kv_cache.dtype).to(dev)
            placed[(i, h)] = pos
    b.q = q.to(torch.bfloat16)
    return placed


def plant_mla_needles(b: MlaBatch, *, logit: float = 14.0, seed: int = 0, count: int = 4) -> dict:
    """`plant_needles` for the latent cache: one direction per sequence over the whole 576-wide
    row, shared by every query head (they all read the same latent rows)."""
    rng = np.random.Generator(np.random.PCG64(78000 + seed))
    dev = b.ql_nope.device
    P = b.page_size
    lkv, rope = b.ql_nope.shape[2], b.q_pe.shape[2]
    W = lkv + rope
    a = math.sqrt(logit / b.sm_scale)
    kv = b.kv_lens.cpu().numpy()
    cu_q = b.cu_q_lens.cpu().numpy()
    cu_kv = b.cu_kv_lens.cpu().numpy()
    pages = b.page_indices.cpu().numpy()
    placed = {}
    qn, qp = b.ql_nope.float(), b.q_pe.float()
    for i in range(int(b.distribution[2])):
        u = (torch.from_numpy(rng.choice([-1.0, 1.0], size=W).astype(np.float32)) / math.sqrt(W)).to(dev)
        qn[cu_q[i]:cu_q[i + 1]] += a * u[:lkv]
        qp[cu_q[i]:cu_q[i + 1]] += a * u[lkv:]
        pos = needle_positions(rng, int(kv[i]), b.sliding_window, count)
        for t in pos:
            page = int(pages[cu_kv[i] // P + t // P])
            # the row is K and V at once: keep its random part (the value), add the needle
            b.cache_kv[page, t % P, :W] = (b.cache_kv[page, t % P, :W].float() + a * u).to(b.cache_kv.dtype)
        placed[i] = pos
    b.ql_nope, b.q_pe = qn.to(torch.bfloat16), qp.to(torch.bfloat16)
    return placed


def sub_batch(b: Batch, seqs, last_rows: int | None = None) -> Batch:
    """The sequences `seqs` of `b` as a compact CPU batch of their own (pages renumbered 0..n-1,
    same page contents).  With `last_rows`, a chunk keeps only its last `last_rows` query tokens
    (their results do not depend on the tokens dropped: a causal row sees its own past only)."""
    P = b.page_size
    kv = b.kv_lens.cpu().numpy()
    cu_q = b.cu_q_lens.cpu().numpy()
    cu_kv = b.cu_kv_lens.cpu().numpy()
    pages = b.page_indices.cpu().numpy()
    q_rows, new_pages, q_lens, kv_lens = [], [], [], []
    for i in seqs:
        q0, q1 = int(cu_q[i]), int(cu_q[i + 1])
        if last_rows is not None:
            q0 = max(q0, q1 - last_rows)
        q_rows.append(torch.arange(q0, q1))
        cnt = -(-int(kv[i]) // P)
        new_pages.append(pages[cu_kv[i] // P: cu_kv[i] // P + cnt])
        q_lens.append(q1 - q0)
        kv_lens.append(int(kv[i]))
    q_rows = torch.cat(q_rows)
    old = np.concatenate(new_pages).astype(np.int64)
    counts = np.array([len(x) for x in new_pages])
    cu_kv_new = np.zeros(len(seqs) + 1, dtype=np.int32)
    cu_kv_new[1:] = np.cumsum(counts * P)
    cu_q_new = np.zeros(len(seqs) + 1, dtype=np.int32)
    cu_q_new[1:] = np.cumsum(q_lens)
    dec = 0
    while dec < len(seqs) and q_lens[dec] == 1:
        dec += 1
    dev = b.q.device
    return Batch(
        name=b.name + "_sample", q=b.q[q_rows.to(dev)].cpu(), kv_cache=b.kv_cache[torch.from_numpy(old).to(dev)].cpu(),
        kv_lens=torch.tensor(kv_lens, dtype=torch.int32), page_indices=torch.arange(len(old), dtype=torch.int32),
        cu_q_lens=torch.from_numpy(cu_q_new), cu_kv_lens=torch.from_numpy(cu_kv_new),
        distribution=torch.tensor([dec, dec, len(seqs)], dtype=torch.int32), sm_scale=b.sm_scale, page_size=P,
        num_kv_heads=b.num_kv_heads, sliding_window=b.sliding_window, soft_cap=b.soft_cap,
        k_scale=None if b.k_scale is None else b.k_scale.cpu(), v_scale=None if b.v_scale is None else b.v_scale.cpu(),
        meta={"q_lens": q_lens, "kv_lens": kv_lens, "rows": q_rows.tolist()})


def mla_sub_batch(b: MlaBatch, seqs) -> MlaBatch:
    """`sub_batch` for the latent cache: the sequences `seqs` of `b` as a compact CPU batch of their own
    (pages renumbered 0..n-1, same page contents, every query token kept)."""
    P = b.page_size
    kv = b.kv_lens.cpu().numpy()
    cu_q = b.cu_q_lens.cpu().numpy()
    cu_kv = b.cu_kv_lens.cpu().numpy()
    pages = b.page_indices.cpu().numpy()
    q_rows, new_pages, q_lens, kv_lens = [], [], [], []
    for i in seqs:
        q_rows.append(torch.arange(int(cu_q[i]), int(cu_q[i + 1])))
        cnt = -(-int(kv[i]) // P)
        new_pages.append(pages[cu_kv[i] // P: cu_kv[i] // P + cnt])
        q_lens.append(int(cu_q[i + 1] - cu_q[i]))
        kv_lens.append(int(kv[i]))
    q_rows = torch.cat(q_rows)
    old = np.concatenate(new_pages).astype(np.int64)
    cu_kv_new = np.zeros(len(seqs) + 1, dtype=np.int32)
    cu_kv_new[1:] = np.cumsum(np.array([len(x) for x in new_pages]) * P)
    cu_q_new = np.zeros(len(seqs) + 1, dtype=np.int32)
    cu_q_new[1:] = np.cumsum(q_lens)
    dec = 0
    while dec < len(seqs) and q_lens[dec] == 1:
        dec += 1
    dev = b.ql_nope.device
    return MlaBatch(
        name=b.name + "_sample", ql_nope=b.ql_nope[q_rows.to(dev)].cpu(), q_pe=b.q_pe[q_rows.to(dev)].cpu(),
        cache_kv=b.cache_kv[torch.from_numpy(old).to(dev)].cpu(), kv_lens=torch.tensor(kv_lens, dtype=torch.int32),
        page_indices=torch.arange(len(old), dtype=torch.int32), cu_q_lens=torch.from_numpy(cu_q_new),
        cu_kv_lens=torch.from_numpy(cu_kv_new), distribution=torch.tensor([dec, dec, len(seqs)], dtype=torch.int32),
        sm_scale=b.sm_scale, page_size=P, sliding_window=b.sliding_window, soft_cap=b.soft_cap,
        meta={"q_lens": q_lens, "kv_lens": kv_lens, "rows": q_rows.tolist()})


# --------------------------------------------------------------------------
# Algorithmic bytes / FLOPs of a batch (the numerators of every roofline figure)
# --------------------------------------------------------------------------
def decode_bytes(b: Batch, lo: int = 0, hi: int | None = None) -> int:
    """Bytes a decode pass must move for sequences [lo, hi): each visible KV token
    once (all heads, K and V), q in, out out, the page ids and lengths touched."""
    kv = np.asarray(b.meta["kv_lens"][lo:hi], dtype=np.int64)
    n = len(kv)
    eff = np.minimum(kv, b.sliding_window) if b.sliding_window else kv
    Hq, D = b.q.shape[1], b.q.shape[2]
    token_bytes = 2 * b.num_kv_heads * D * b.kv_cache.element_size()
    total = int(eff.sum()) * token_bytes
    total += 2 * n * Hq * D * 2  # q + out
    total += int((-(-eff // b.page_size)).sum()) * 4 + (2 * n + 1) * 4
    if b.k_scale is not None:
        total += 2 * b.num_kv_heads * 4
    return total


def prefill_flops(b: Batch, lo: int = 0, hi: int | None = None) -> int:
    """4*Hq*D FLOP per visible (query, key) pair: 2D for q.k, 2D for p.v."""
    ql = np.asarray(b.meta["q_lens"][lo:hi], dtype=np.int64)
    kv = np.asarray(b.meta["kv_lens"][lo:hi], dtype=np.int64)
    Hq, D = b.q.shape[1], b.q.shape[2]
    pairs = 0
    for q, k in zip(ql, kv):
        prefix = k - q
        if b.sliding_window:
            j = np.arange(q)
            pairs += int(np.minimum(prefix + j + 1, b.sliding_window).sum())
        else:
            pairs += int(q * prefix + q * (q + 1) // 2)
    return 4 * Hq * D * pairs


def mla_decode_bytes(b: MlaBatch) -> int:
    kv = np.asarray(b.meta["kv_lens"], dtype=np.int64)
    T, Hq, lkv = b.ql_nope.shape
    width = b.cache_kv.shape[-1]
    total = int(kv.sum()) * width * b.cache_kv.element_size()
    total += T * Hq * width * 2 + T * Hq * lkv * 2
    total += int((-(-kv // b.page_size)).sum()) * 4 + (2 * len(kv) + 1) * 4
    return total


def mla_attention_flops(b: MlaBatch) -> int:
    """Any batch composition: Hq * (2 * 576 + 2 * 512) FLOP per visible (query token, cached token) pair."""
    ql = np.asarray(b.meta["q_lens"], dtype=np.int64)
    kv = np.asarray(b.meta["kv_lens"], dtype=np.int64)
    _, Hq, lkv = b.ql_nope.shape
    width = b.cache_kv.shape[-1]
    pairs = int((ql * (kv - ql) + ql * (ql + 1) // 2).sum())
    return pairs * Hq * (2 * width + 2 * lkv)


def mla_decode_flops(b: MlaBatch) -> int:
    kv = np.asarray(b.meta["kv_lens"], dtype=np.int64)
    _, Hq, lkv = b.ql_nope.shape
    width = b.cache_kv.shape[-1]
    return int(kv.sum()) * Hq * (2 * width + 2 * lkv)
