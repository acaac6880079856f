"""GPU parity of the absorbed-MLA decode kernel against the CPU oracle
(oracle/ref_mla.py), rtol = atol = 2e-2 (bf16).  Shapes follow the reference's
MLA tests (python/sgl_jax/test/test_mla_attention.py:346-696: 16 heads, latent 512,
rope 64, page sizes 8..64, window 128, soft cap 30) and the DeepSeek-V3 decode
configuration."""

import sys

import numpy as np
import pytest
import torch

from parity import assert_parity, row_rel_error

from oracle.ref_mla import ref_mla_ragged_paged_attention

pytestmark = pytest.mark.gpu
TOL = dict(rtol=2e-2, atol=2e-2)


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def oracle(b, **kw):
    n = int(b.distribution[2])
    out, _ = ref_mla_ragged_paged_attention(
        b.ql_nope, b.q_pe, None, None, b.cache_kv, b.kv_lens, b.padded_page_indices(), b.cu_q_lens, [n, n, n],
        sm_scale=b.sm_scale, sliding_window=b.sliding_window, soft_cap=b.soft_cap, **kw)
    return out


def run_gpu(pkg, b, dev, cache=None, **kw):
    g = b.to(dev)
    out, _ = pkg.mla_ragged_paged_attention(
        g.ql_nope, g.q_pe, None, None, g.cache_kv if cache is None else cache.to(dev), g.kv_lens, g.page_indices,
        g.cu_q_lens, g.cu_kv_lens, b.distribution.cpu().numpy(), sm_scale=b.sm_scale,
        sliding_window=b.sliding_window, soft_cap=b.soft_cap, max_kv_len=int(max(b.meta["kv_lens"])), **kw)
    torch.cuda.synchronize()
    return out.cpu()


@pytest.mark.parametrize("P", [8, 16, 32, 64])
@pytest.mark.parametrize("Hq", [16, 128])
def test_mla_decode_page_sizes(pkg, wl, gpu, P, Hq):
    kv_lens = [1, 31, 32, 33, 129, 500, 1025]
    say(f"mla decode P={P} Hq={Hq} kv={kv_lens}")
    b = wl.make_mla_batch("mla", [1] * len(kv_lens), kv_lens, num_q_heads=Hq, lkv_dim=512, rope_dim=64,
                          page_size=P, seed=71, sm_scale=192 ** -0.5)
    got = run_gpu(pkg, b, gpu)
    assert_parity(got.float(), oracle(b).float(), **TOL)


@pytest.mark.parametrize("P", [4, 8, 16])
@pytest.mark.parametrize("f8", [False, True])
def test_mla_long_rows_on_pages_smaller_than_a_tile(pkg, wl, gpu, P, f8):
    """Pages that do not hold whole 32-token tiles: the lanes look their rows' pages up in the wave's LDS window of
    256 page ids, which moves on several times along these rows.  One long row (cut over the GPU, forced counts
    included) and a ragged batch on the balanced plan, planted keys."""
    kw = dict(num_q_heads=128, lkv_dim=512, rope_dim=64, page_size=P, sm_scale=192 ** -0.5,
              kv_dtype=torch.float8_e4m3fn if f8 else torch.bfloat16)
    ref = fp8_oracle if f8 else oracle
    say(f"mla small pages P={P} f8={f8}: one long row")
    b = wl.make_mla_batch("mla_small_pages", [1], [6001], seed=410 + P, **kw)
    wl.plant_mla_needles(b, seed=4)
    want = ref(b)
    for ns in (0, 1, 5):
        got = run_gpu(pkg, b, gpu, **({"num_splits": ns} if ns else {}))
        assert_parity(got.float(), want.float(), **TOL)
    say(f"mla small pages P={P} f8={f8}: ragged batch")
    lens = [int(x) for x in np.random.default_rng(P).integers(1, 3000, size=24)] + [1, 31, 32, 33, 2049]
    b = wl.make_mla_batch("mla_small_pages_ragged", [1] * len(lens), lens, seed=420 + P, **kw)
    wl.plant_mla_needles(b, seed=5)
    assert_parity(run_gpu(pkg, b, gpu).float(), ref(b).float(), **TOL)


@pytest.mark.parametrize("Hq", [8, 16, 32, 48, 64])
@pytest.mark.parametrize("f8", [False, True])
def test_mla_waves_share_tiles_when_heads_are_few(pkg, wl, gpu, monkeypatch, Hq, f8):
    """At most 64 heads (a tensor-parallel share of the 128): the eight waves of a workgroup share each tile of a
    block of 16 heads -- partial scores per (token half, k-step group) summed through LDS, output chunks dealt out
    -- instead of one wave per block.  Against the oracle and against RPA_MLA_SHARED_TILES=0: a long row cut over
    the GPU, a ragged batch on the balanced plan, a sliding window, planted keys, a short chunk (token rows)."""
    kw = dict(num_q_heads=Hq, lkv_dim=512, rope_dim=64, page_size=64, sm_scale=192 ** -0.5,
              kv_dtype=torch.float8_e4m3fn if f8 else torch.bfloat16)
    ref = fp8_oracle if f8 else oracle
    lens = [int(x) for x in np.random.default_rng(Hq).integers(1, 3000, size=20)] + [1, 31, 32, 33, 7001]
    for name, q_lens, kv_lens, window in (("long", [1], [9001], None), ("ragged", [1] * len(lens), lens, None),
                                          ("window", [1, 1, 1], [100, 700, 5000], 600), ("chunk", [1, 9], [800, 2100], None)):
        say(f"mla shared tiles Hq={Hq} f8={f8} {name}")
        b = wl.make_mla_batch("mla_shared_" + name, q_lens, kv_lens, seed=430 + Hq, sliding_window=window, **kw)
        wl.plant_mla_needles(b, seed=6)
        want = ref(b)
        T = sum(q_lens)
        shared = run_gpu(pkg, b, gpu)[:T]
        monkeypatch.setenv("RPA_MLA_SHARED_TILES", "0")
        single = run_gpu(pkg, b, gpu)[:T]
        monkeypatch.delenv("RPA_MLA_SHARED_TILES")
        assert_parity(shared.float(), want.float(), **TOL)
        assert_parity(single.float(), want.float(), **TOL)
        assert torch.equal(shared, run_gpu(pkg, b, gpu)[:T])


@pytest.mark.parametrize("Hq", [16, 32, 64])
@pytest.mark.parametrize("f8", [False, True])
def test_mla_prefill_rows_share_tiles_among_query_tokens_when_heads_are_few(pkg, wl, gpu, monkeypatch, Hq, f8):
    """Prefill / mixed batches with 16 / 32 / 64 heads (the reference's own MLA test shape has 16,
    test_mla_attention.py:346): a workgroup holds 8 / 4 / 2 consecutive query tokens of a sequence over shared
    latent tiles, each wave masking with its own token's length (the reference's kernel shares a tile among 16
    query tokens, kernels/mla/v2/kernel.py:1448-1459).  bf16 latents without a window run the groups on wide
    workgroups (four waves, each with two blocks of heads that may belong to two tokens), everything else on eight
    waves.  Against the oracle, against one token per workgroup (RPA_MLA_TOKEN_GROUPS=0) and against the
    eight-wave groups (RPA_MLA_WIDE=0): chunk lengths that leave partial groups, windows of tokens that span the border
    between two sequences, decode rows in front, a chunk with no prefix, a sliding window shorter than the chunk,
    pages of 32 and 128 tokens, planted keys."""
    ref = fp8_oracle if f8 else oracle
    cases = (("chunks", [300, 77, 130], [1500, 77, 4230], None, 64),
             ("mixed", [1, 1, 1, 259, 64], [900, 33, 2000, 1259, 3064], None, 32),
             ("window", [200, 45], [3000, 700], 150, 128),
             ("long_chunk", [1024], [1024 + 4096], None, 64))
    for name, q_lens, kv_lens, window, P in cases:
        say(f"mla token groups Hq={Hq} f8={f8} {name}")
        b = wl.make_mla_batch("mla_tg_" + name, q_lens, kv_lens, num_q_heads=Hq, lkv_dim=512, rope_dim=64, page_size=P,
                              seed=470 + Hq, sm_scale=192 ** -0.5, sliding_window=window,
                              kv_dtype=torch.float8_e4m3fn if f8 else torch.bfloat16)
        wl.plant_mla_needles(b, seed=7)
        want = ref(b)
        T = sum(q_lens)
        grouped = run_gpu(pkg, b, gpu)[:T]
        assert_parity(grouped.float(), want.float(), **TOL)
        monkeypatch.setenv("RPA_MLA_TOKEN_GROUPS", "0")
        single = run_gpu(pkg, b, gpu)[:T]
        monkeypatch.delenv("RPA_MLA_TOKEN_GROUPS")
        assert_parity(single.float(), want.float(), **TOL)
        assert_parity(grouped.float(), single.float(), **TOL)
        monkeypatch.setenv("RPA_MLA_WIDE", "0")
        eight = run_gpu(pkg, b, gpu)[:T]
        monkeypatch.delenv("RPA_MLA_WIDE")
        assert_parity(eight.float(), want.float(), **TOL)
        assert_parity(grouped.float(), eight.float(), **TOL)
        monkeypatch.setenv("RPA_MLA_PIPE", "0")  # the compiled tile loop under the same grouping
        compiled = run_gpu(pkg, b, gpu)[:T]
        monkeypatch.delenv("RPA_MLA_PIPE")
        assert_parity(compiled.float(), want.float(), **TOL)


@pytest.mark.parametrize("window,cap", [(128, None), (None, 30.0), (128, 30.0)])
def test_mla_window_and_soft_cap(pkg, wl, gpu, window, cap):
    kv_lens = [100, 128, 129, 700]
    b = wl.make_mla_batch("mla_swa", [1] * 4, kv_lens, num_q_heads=16, lkv_dim=512, rope_dim=64, page_size=16,
                          seed=72, sm_scale=192 ** -0.5, sliding_window=window, soft_cap=cap)
    got = run_gpu(pkg, b, gpu)
    assert_parity(got.float(), oracle(b).float(), **TOL)


def test_mla_split_count_does_not_matter(pkg, wl, gpu):
    b = wl.make_mla_batch("mla_splits", [1] * 3, [40, 1000, 3000], num_q_heads=32, lkv_dim=512, rope_dim=64,
                          page_size=64, seed=73, sm_scale=192 ** -0.5)
    want = oracle(b)
    base = None
    for ns in (1, 2, 5, 16):
        say(f"mla num_splits {ns}")
        got = run_gpu(pkg, b, gpu, num_splits=ns)
        assert_parity(got.float(), want.float(), **TOL)
        base = got if base is None else base
        torch.testing.assert_close(got.float(), base.float(), rtol=1e-2, atol=4e-3)


def test_mla_many_ragged_rows_are_dealt_out_evenly(pkg, wl, gpu):
    """More rows than workgroup slots, none long enough for the fixed plan to cut: the batch still
    takes the balanced plan (at most two whole-row jobs per slot would end with the longest rows);
    pieces are padded, so workgroups that cross into new rows get fewer tiles.  Against the
    oracle and against whole rows (num_splits = 1)."""
    rng = np.random.default_rng(79)
    kv_lens = [int(x) for x in rng.integers(100, 900, size=300)]
    say("mla 300 ragged rows")
    b = wl.make_mla_batch("mla_many", [1] * len(kv_lens), kv_lens, num_q_heads=16, lkv_dim=512, rope_dim=64,
                          page_size=64, seed=80, sm_scale=192 ** -0.5)
    want = oracle(b)
    auto = run_gpu(pkg, b, gpu)
    whole = run_gpu(pkg, b, gpu, num_splits=1)
    assert_parity(auto.float(), want.float(), **TOL)
    torch.testing.assert_close(auto.float(), whole.float(), rtol=1e-2, atol=4e-3)
    assert not torch.equal(auto, whole)  # merged rows differ from whole ones in the last bits somewhere


def test_mla_reference_padded_cache_layout(pkg, wl, gpu):
    """The reference stores rope padded to 128 (kernels/mla/v2/kernel.py:74-86): 640-wide rows."""
    b = wl.make_mla_batch("mla_padded", [1] * 3, [70, 300, 64], num_q_heads=16, lkv_dim=512, rope_dim=64,
                          page_size=16, seed=74, sm_scale=192 ** -0.5)
    pool, P, _ = b.cache_kv.shape
    padded = torch.zeros(pool, P, 640, dtype=torch.bfloat16)
    padded[..., :512] = b.cache_kv[..., :512]
    padded[..., 512:576] = b.cache_kv[..., 512:]
    a = run_gpu(pkg, b, gpu)
    c = run_gpu(pkg, b, gpu, cache=padded)
    assert torch.equal(a.view(torch.int16), c.view(torch.int16))
    d = run_gpu(pkg, b, gpu, cache=padded.view(pool, P // 2, 2, 640))
    assert torch.equal(a.view(torch.int16), d.view(torch.int16))


def test_mla_nan_canaries(pkg, wl, gpu):
    kv_lens = [5, 64, 65, 300]
    b = wl.make_mla_batch("mla_canary", [1] * 4, kv_lens, num_q_heads=16, lkv_dim=512, rope_dim=64, page_size=64,
                          seed=75, sm_scale=192 ** -0.5)
    clean = run_gpu(pkg, b, gpu)
    used = torch.zeros(b.cache_kv.shape[:2], dtype=torch.bool)
    table = b.padded_page_indices().reshape(len(kv_lens), -1)
    for i, kv in enumerate(kv_lens):
        for t in range(kv):
            used[table[i, t // 64], t % 64] = True
    b.cache_kv[~used] = float("nan")
    dirty = run_gpu(pkg, b, gpu)
    assert torch.isfinite(dirty.float()).all()
    assert torch.equal(clean.view(torch.int16), dirty.view(torch.int16))


def test_c5_scaled_against_oracle(pkg, wl, gpu):
    b = wl.config_c5(scale=0.06)
    got = run_gpu(pkg, b, gpu)
    assert_parity(got.float(), oracle(b).float(), **TOL)


# ------------------------------------------------------------------ prefill / mixed rows, fused latent write
@pytest.mark.parametrize("P,window,cap", [(16, None, None), (64, None, None), (64, 128, 30.0)])
def test_mla_prefill_and_mixed_rows(pkg, wl, gpu, P, window, cap):
    """Decode rows, chunks with a prefix and whole prompts in one batch
    (kernels/mla/v2/kernel.py:1338-1744 runs them as three launches)."""
    q_lens = [1, 1, 5, 64, 33, 130]
    kv_lens = [77, 1, 5, 300, 33, 131]
    say(f"mla mixed P={P} window={window} cap={cap} q={q_lens} kv={kv_lens}")
    b = wl.make_mla_batch("mla_mixed", q_lens, kv_lens, num_q_heads=16, lkv_dim=512, rope_dim=64, page_size=P,
                          seed=81, sliding_window=window, soft_cap=cap)
    want = oracle(b)
    got = run_gpu(pkg, b, gpu)
    T = sum(q_lens)
    assert torch.isfinite(got[:T].float()).all()
    assert_parity(got[:T].float(), want.float(), **TOL)
    # any split count gives the same rows
    got4 = run_gpu(pkg, b, gpu, num_splits=3)
    torch.testing.assert_close(got4[:T].float(), got[:T].float(), rtol=1e-2, atol=1e-2)


def test_mla_token_rows_equal_sequence_rows_on_a_decode_batch(pkg, wl, gpu):
    kv_lens = [40, 1000, 257, 64]
    b = wl.make_mla_batch("mla_dec", [1] * 4, kv_lens, num_q_heads=32, lkv_dim=512, rope_dim=64, page_size=64, seed=82)
    seq_rows = run_gpu(pkg, b, gpu)
    # the same batch declared as "mixed" takes the one-row-per-token entry point
    g = b.to(gpu)
    out, _ = pkg.mla_ragged_paged_attention(
        g.ql_nope, g.q_pe, None, None, g.cache_kv, g.kv_lens, g.page_indices, g.cu_q_lens, g.cu_kv_lens,
        [0, 0, 4], sm_scale=b.sm_scale, max_kv_len=1000)
    torch.cuda.synchronize()
    assert torch.equal(out.cpu(), seq_rows)


@pytest.mark.parametrize("padded", [False, True])
def test_mla_new_rows_are_written_into_the_cache(pkg, wl, gpu, padded):
    """The cache holds kv_len - q_len rows, new_kv_c / new_k_pe bring the rest
    (kernels/mla/v1/ref.py:56-105): cache bit for bit, output within tolerance."""
    q_lens, kv_lens, P = [1, 1, 20, 65], [64, 200, 20, 300], 16
    b = wl.make_mla_batch("mla_write", q_lens, kv_lens, num_q_heads=16, lkv_dim=512, rope_dim=64, page_size=P, seed=83)
    say(f"mla write padded={padded}")
    cache = b.cache_kv
    if padded:  # the reference's 128-aligned rows: [kv_c 512 | k_pe 64 | 64 unused]
        wide = torch.zeros(cache.shape[0], P, 640, dtype=cache.dtype)
        wide[..., :576] = cache
        cache = wide
    table = b.padded_page_indices().view(len(q_lens), -1)
    T = sum(q_lens)
    new_c = torch.empty(T, 512, dtype=torch.bfloat16)
    new_r = torch.empty(T, 64, dtype=torch.bfloat16)
    holed = cache.clone()
    t = 0
    for i, (ql, kv) in enumerate(zip(q_lens, kv_lens)):
        for j in range(ql):
            pos = kv - ql + j
            page, row = int(table[i, pos // P]), pos % P
            new_c[t], new_r[t] = cache[page, row, :512], cache[page, row, 512:576]
            holed[page, row] = float("nan")
            if padded:
                holed[page, row, 576:] = 0
            t += 1
    n = len(q_lens)
    want, want_cache = ref_mla_ragged_paged_attention(
        b.ql_nope, b.q_pe, new_c, new_r, holed, b.kv_lens, b.padded_page_indices(), b.cu_q_lens, [0, 0, n],
        sm_scale=b.sm_scale, layout="padded" if padded else "compact")
    assert torch.equal(want_cache.view(torch.int16), cache.view(torch.int16))
    g = b.to(gpu)
    out, got_cache = pkg.mla_ragged_paged_attention(
        g.ql_nope, g.q_pe, new_c.to(gpu), new_r.to(gpu), holed.to(gpu), g.kv_lens, g.page_indices, g.cu_q_lens,
        g.cu_kv_lens, b.distribution.numpy(), sm_scale=b.sm_scale, max_kv_len=300)
    torch.cuda.synchronize()
    assert torch.equal(got_cache.cpu().view(torch.int16), cache.view(torch.int16))
    assert_parity(out.cpu()[:T].float(), want.float(), **TOL)


@pytest.mark.parametrize("f8", [False, True], ids=["bf16", "e4m3"])
def test_c5_full_size_page_permutation_invariance(pkg, wl, gpu, f8):
    """DeepSeek-V3 decode configuration at full size (64 rows of 2048-16384 tokens, 128 heads), peaked inputs:
    the output must not depend, bit for bit, on where pages physically live; a sample of rows (first,
    longest, shortest, last), re-run by the oracle on a compact copy of their pages, must match; and the split
    plans must agree with a single pass row by row, relative to each row's own size."""
    b = wl.config_c5(device=gpu, **({"kv_dtype": torch.float8_e4m3fn} if f8 else {}))
    wl.plant_mla_needles(b, seed=23)
    n = int(b.distribution[2])
    kw = dict(sm_scale=b.sm_scale, max_kv_len=int(max(b.meta["kv_lens"])))

    def run(x, **extra):
        out, _ = pkg.mla_ragged_paged_attention(x.ql_nope, x.q_pe, None, None, x.cache_kv, x.kv_lens, x.page_indices,
                                                x.cu_q_lens, x.cu_kv_lens, (n, n, n), **kw, **extra)
        torch.cuda.synchronize()
        return out

    a = run(b)
    assert torch.isfinite(a.float()).all()
    kv = np.asarray(b.meta["kv_lens"])
    seqs = sorted({0, int(np.argmax(kv)), int(np.argmin(kv)), n - 1})
    sample = wl.mla_sub_batch(b, seqs)
    say(f"c5 f8={f8}: oracle sample of sequences {seqs}, kv {sample.meta['kv_lens']}")
    want = (fp8_oracle if f8 else oracle)(sample)
    got = a[torch.tensor(sample.meta["rows"], device=gpu)].cpu()
    assert float(want.float().norm(dim=-1).min()) > 0.3  # peaked rows: the outputs are O(1), not averages near zero
    assert_parity(got.float(), want.float(), **TOL)
    pool = b.cache_kv.shape[0]
    perm = torch.randperm(pool, generator=torch.Generator().manual_seed(11)).to(gpu)
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(pool, device=gpu)
    c = b.to(gpu)
    c.cache_kv = b.cache_kv[perm]  # new page j holds old page perm[j]
    c.page_indices = inv[b.page_indices.long()].to(torch.int32)
    assert torch.equal(a.view(torch.int16), run(c).view(torch.int16))
    one = run(b, num_splits=1)
    assert_parity(a.float(), one.float(), **TOL)  # element-wise and every row relative to its own norm


def test_mla_more_rows_than_a_grid_dimension_holds(pkg, wl, gpu):
    """A prefill call of 66000 query tokens (one kernel row each; the reference loops over any number,
    kernels/mla/v2/kernel.py:1722-1739): rows are folded onto the first grid dimension.  16 heads, short prefixes;
    a sample of sequences against the oracle."""
    q_lens = [3000] * 22
    kv_lens = [3000 + 64 * i for i in range(22)]
    b = wl.make_mla_batch("mla_many_rows", q_lens, kv_lens, num_q_heads=16, lkv_dim=512, rope_dim=64, page_size=64,
                          seed=93, sm_scale=192 ** -0.5, device=gpu)
    g = b
    out, _ = pkg.mla_ragged_paged_attention(
        g.ql_nope, g.q_pe, None, None, g.cache_kv, g.kv_lens, g.page_indices, g.cu_q_lens, g.cu_kv_lens,
        b.distribution.cpu().numpy(), sm_scale=b.sm_scale, max_kv_len=max(kv_lens))
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()
    sample = wl.mla_sub_batch(b, [21])
    # the last 64 tokens of the last sequence hold the highest row numbers (65936 ..)
    want = oracle(sample)
    got = out[torch.tensor(sample.meta["rows"], device=gpu)].cpu()
    assert_parity(got[-64:].float(), want[-64:].float(), **TOL)
    first = wl.mla_sub_batch(b, [0])
    assert_parity(out[torch.tensor(first.meta["rows"][:64], device=gpu)].cpu().float(), oracle(first)[:64].float(), **TOL)


@pytest.mark.parametrize("seed", list(range(8)))
def test_random_mla_batches_against_oracle(pkg, wl, gpu, seed):
    """Seeded random decode and mixed batches, head counts, page sizes, window and soft cap."""
    import numpy as np
    rng = np.random.default_rng(3000 + seed)
    Hq = int(rng.choice([16, 48, 128, 160]))
    P = int(rng.choice([8, 16, 32, 64]))
    n_dec, n_pre = int(rng.integers(0, 6)), int(rng.integers(0, 3))
    if seed % 2 == 0:
        n_pre = 0  # decode batches take the one-row-per-sequence entry point
    if n_dec + n_pre == 0:
        n_dec = 2
    kv_dec = rng.integers(1, 2500, size=n_dec)
    q_pre = rng.integers(2, 60, size=n_pre)
    kv_pre = q_pre + rng.integers(0, 400, size=n_pre)
    q_lens = [1] * n_dec + [int(x) for x in q_pre]
    kv_lens = [int(x) for x in kv_dec] + [int(x) for x in kv_pre]
    window = int(rng.integers(1, 300)) if rng.integers(0, 3) == 0 else None
    cap = 30.0 if rng.integers(0, 3) == 0 else None
    say(f"mla random seed={seed} Hq={Hq} P={P} q={q_lens} kv={kv_lens} window={window} cap={cap}")
    b = wl.make_mla_batch("mla_rand", q_lens, kv_lens, num_q_heads=Hq, lkv_dim=512, rope_dim=64, page_size=P,
                          seed=4000 + seed, sliding_window=window, soft_cap=cap)
    want = oracle(b)
    got = run_gpu(pkg, b, gpu)
    T = sum(q_lens)
    assert torch.isfinite(got[:T].float()).all()
    assert_parity(got[:T].float(), want.float(), **TOL)


@pytest.mark.parametrize("seed", list(range(8)))
def test_random_large_mla_batches_against_oracle(pkg, wl, gpu, seed):
    """Seeded random batches large enough for the balanced plan: up to 39 decode rows of up to 9000
    tokens, sometimes one of 15000-40000, with chunks behind them on odd seeds."""
    rng = np.random.default_rng(70000 + seed)
    Hq = int(rng.choice([16, 32, 48, 64, 128, 160]))
    P = int(rng.choice([8, 16, 32, 64, 128]))
    n_dec, n_pre = int(rng.integers(6, 40)), (int(rng.integers(0, 3)) if seed % 2 else 0)
    kv_dec = rng.integers(1, 9000, size=n_dec)
    if rng.integers(0, 2):
        kv_dec[rng.integers(0, n_dec)] = int(rng.integers(15000, 40000))
    q_pre = rng.integers(2, 60, size=n_pre)
    kv_pre = q_pre + rng.integers(0, 400, size=n_pre)
    q_lens = [1] * n_dec + [int(x) for x in q_pre]
    kv_lens = [int(x) for x in kv_dec] + [int(x) for x in kv_pre]
    window = int(rng.integers(1, 3000)) if rng.integers(0, 3) == 0 else None
    cap = 30.0 if rng.integers(0, 3) == 0 else None
    say(f"mla random large seed={seed} Hq={Hq} P={P} n_dec={n_dec} max_kv={max(kv_lens)} q={q_lens[n_dec:]} window={window} cap={cap}")
    b = wl.make_mla_batch("mla_rand_large", q_lens, kv_lens, num_q_heads=Hq, lkv_dim=512, rope_dim=64, page_size=P,
                          seed=5000 + seed, sliding_window=window, soft_cap=cap)
    if seed % 2 == 0:
        wl.plant_mla_needles(b, seed=seed)  # peaked rows: O(1) outputs whatever the length
    want = oracle(b)
    got = run_gpu(pkg, b, gpu)
    T = sum(q_lens)
    assert torch.isfinite(got[:T].float()).all()
    assert_parity(got[:T].float(), want.float(), **TOL)


@pytest.mark.parametrize("Hq", [8, 24, 40, 100, 136])
def test_mla_head_counts_off_the_sixteen_head_tile(pkg, wl, gpu, Hq):
    """Head counts that do not fill the last 16-head MFMA tile (a tensor-parallel share of 8 heads,
    say): the spare columns read a clamped head and write nothing.  Decode rows (both plans) and
    a mixed batch."""
    say(f"mla heads Hq={Hq}")
    b = wl.make_mla_batch("mla_heads", [1] * 5, [3, 700, 64, 2049, 130], num_q_heads=Hq, lkv_dim=512, rope_dim=64,
                          page_size=32, seed=610 + Hq)
    want = oracle(b)
    for kw in ({}, {"num_splits": 1}, {"num_splits": 4}):
        got = run_gpu(pkg, b, gpu, **kw)
        assert_parity(got[:5].float(), want.float(), **TOL)
    q_lens, kv_lens = [1, 1, 9, 33], [40, 900, 9, 133]
    b = wl.make_mla_batch("mla_heads_mixed", q_lens, kv_lens, num_q_heads=Hq, lkv_dim=512, rope_dim=64, page_size=16,
                          seed=620 + Hq)
    got = run_gpu(pkg, b, gpu)
    T = sum(q_lens)
    assert torch.isfinite(got[:T].float()).all()
    assert_parity(got[:T].float(), oracle(b).float(), **TOL)


MLA_NEEDLE_CASES = {
    # name: (q_lens, kv_lens, Hq, P, window)
    "few_long_rows": ([1] * 3, [16384, 20000, 9000], 128, 64, None),
    "one_row_40000": ([1], [40000], 128, 64, None),
    "balanced_ragged_rows": ([1] * 48, [2048 + 301 * i for i in range(48)], 128, 64, None),
    "ragged_small_pages_window": ([1] * 20, [3000 + 707 * i for i in range(20)], 64, 16, 2500),
    "chunk_on_a_prefix": ([1, 1, 40], [5000, 9000, 4136], 128, 64, None),
}


@pytest.mark.parametrize("case", list(MLA_NEEDLE_CASES))
def test_mla_peaked_long_rows_against_oracle(pkg, wl, gpu, case):
    """Latent rows of 2000-40000 tokens with a few planted keys that carry the softmax weight
    (first and last tiles, tile / page / piece borders, the window edge): outputs are O(1), so a lost
    tile or piece or a wrong merge weight shows up.  Fixed and balanced plans, any split count."""
    q_lens, kv_lens, Hq, P, window = MLA_NEEDLE_CASES[case]
    say(f"mla needles {case}: q={q_lens} kv={kv_lens} Hq={Hq} P={P} window={window}")
    b = wl.make_mla_batch(case, q_lens, kv_lens, num_q_heads=Hq, lkv_dim=512, rope_dim=64, page_size=P, seed=8200,
                          sliding_window=window)
    placed = wl.plant_mla_needles(b, seed=len(case))
    say(f"  needles of seq 0: {placed[0]}")
    want = oracle(b)
    T = sum(q_lens)
    assert float(want.float().pow(2).mean().sqrt()) > 0.1
    got = run_gpu(pkg, b, gpu)
    assert_parity(got[:T].float(), want.float(), **TOL)
    if all(q == 1 for q in q_lens):
        for ns in (1, 3):
            say(f"  num_splits {ns}")
            assert_parity(run_gpu(pkg, b, gpu, num_splits=ns)[:T].float(), want.float(), **TOL)


@pytest.mark.parametrize("window", [None, 3000])
def test_mla_assembly_loop_against_compiled_loop(pkg, wl, gpu, window, monkeypatch):
    """128 heads and 64-token pages: whole unmasked tiles run inside the assembly loop
    (rpa_mla_pipe_loop.inc), the first tile, window-edge tiles and the last tiles of a row in the
    compiled step.  Rows from one tile to 400, ends on and off tile borders, with and without planted
    keys (which send the loop through its reference-raising path), every plan: against the oracle
    and against the same call with the loop switched off (RPA_MLA_PIPE=0)."""
    kv_lens = [1, 31, 32, 33, 96, 127, 128, 129, 160, 161, 1000, 2048, 4097, 6001, 12800, 9999]
    for needles in (False, True):
        b = wl.make_mla_batch("mla_pipe", [1] * len(kv_lens), kv_lens, num_q_heads=128, lkv_dim=512, rope_dim=64,
                              page_size=64, seed=8600 + needles, sliding_window=window)
        if needles:
            wl.plant_mla_needles(b, seed=5)
        want = oracle(b)
        for kw in ({}, {"num_splits": 1}, {"num_splits": 3}, {"num_splits": 40}):
            say(f"mla assembly loop window={window} needles={needles} {kw}")
            monkeypatch.setenv("RPA_MLA_PIPE", "1")
            on = run_gpu(pkg, b, gpu, **kw)[:len(kv_lens)]
            monkeypatch.setenv("RPA_MLA_PIPE", "0")
            off = run_gpu(pkg, b, gpu, **kw)[:len(kv_lens)]
            assert_parity(on.float(), want.float(), **TOL)
            assert_parity(off.float(), want.float(), **TOL)
            assert float(row_rel_error(on.float(), off.float()).max()) < 1e-2
    # chunks on long prefixes: one row per query token
    monkeypatch.setenv("RPA_MLA_PIPE", "1")
    q_lens, kv_lens = [1, 70, 33], [5000, 4170, 1033]
    b = wl.make_mla_batch("mla_pipe_chunks", q_lens, kv_lens, num_q_heads=128, lkv_dim=512, rope_dim=64, page_size=64,
                          seed=8610, sliding_window=window)
    assert_parity(run_gpu(pkg, b, gpu)[:sum(q_lens)].float(), oracle(b).float(), **TOL)


@pytest.mark.parametrize("window", [None, 3000])
def test_mla_wide_workgroups_against_eight_wave_workgroups(pkg, wl, gpu, window, monkeypatch):
    """128 heads, 64-token pages, bf16 cache: by default four waves of 32 heads run every tile of a
    segment inside the assembly loop of rpa_mla_wide_loop.inc (masks of the first and last tile, clamped
    copies of the row's last tile and the reference-raising path included); RPA_MLA_WIDE=0 keeps the
    eight-wave kernels.  Rows from one token to 12800, ends on and off tile borders, with and without
    planted keys, every plan: against the oracle and against each other."""
    kv_lens = [1, 31, 32, 33, 96, 127, 128, 129, 160, 161, 256, 416, 1000, 2048, 4097, 6001, 12800, 9999]
    for needles in (False, True):
        b = wl.make_mla_batch("mla_wide", [1] * len(kv_lens), kv_lens, num_q_heads=128, lkv_dim=512, rope_dim=64,
                              page_size=64, seed=8620 + needles, sliding_window=window)
        if needles:
            wl.plant_mla_needles(b, seed=6)
        want = oracle(b)
        for kw in ({}, {"num_splits": 1}, {"num_splits": 3}, {"num_splits": 40}):
            say(f"mla wide workgroups window={window} needles={needles} {kw}")
            monkeypatch.delenv("RPA_MLA_WIDE", raising=False)
            on = run_gpu(pkg, b, gpu, **kw)[:len(kv_lens)]
            monkeypatch.setenv("RPA_MLA_WIDE", "0")
            off = run_gpu(pkg, b, gpu, **kw)[:len(kv_lens)]
            monkeypatch.delenv("RPA_MLA_WIDE")
            assert_parity(on.float(), want.float(), **TOL)
            assert_parity(off.float(), want.float(), **TOL)
            assert float(row_rel_error(on.float(), off.float()).max()) < 1e-2
            assert not torch.equal(on, off)  # two kernels: the last bits differ somewhere
    # chunks on long prefixes (one row per query token), 256 heads (two workgroups per row), 32-token pages
    for Hq, P, q_lens, kv_lens in ((128, 64, [1, 70, 33], [5000, 4170, 1033]), (256, 32, [40, 1], [1500, 700])):
        b = wl.make_mla_batch("mla_wide_chunks", q_lens, kv_lens, num_q_heads=Hq, lkv_dim=512, rope_dim=64, page_size=P,
                              seed=8630, sliding_window=window)
        assert_parity(run_gpu(pkg, b, gpu)[:sum(q_lens)].float(), oracle(b).float(), **TOL)


@pytest.mark.parametrize("window", [None, 3000])
def test_mla_wide_workgroups_on_32x32_matrix_instructions(pkg, wl, gpu, window, monkeypatch):
    """RPA_MLA_WIDE=32: the wide loop generated for 32x32x16 matrix instructions (one head per lane and half,
    rpa_mla_wide32_loop.inc; opt-in): same cases, against the oracle and the default loop."""
    kv_lens = [1, 31, 32, 33, 96, 127, 128, 129, 160, 161, 256, 416, 1000, 2048, 4097, 6001, 12800, 9999]
    for needles in (False, True):
        b = wl.make_mla_batch("mla_wide32", [1] * len(kv_lens), kv_lens, num_q_heads=128, lkv_dim=512, rope_dim=64,
                              page_size=64, seed=8640 + needles, sliding_window=window)
        if needles:
            wl.plant_mla_needles(b, seed=7)
        want = oracle(b)
        for kw in ({}, {"num_splits": 1}, {"num_splits": 3}):
            say(f"mla wide 32x32 window={window} needles={needles} {kw}")
            monkeypatch.setenv("RPA_MLA_WIDE", "32")
            on = run_gpu(pkg, b, gpu, **kw)[:len(kv_lens)]
            monkeypatch.delenv("RPA_MLA_WIDE")
            off = run_gpu(pkg, b, gpu, **kw)[:len(kv_lens)]
            assert_parity(on.float(), want.float(), **TOL)
            assert float(row_rel_error(on.float(), off.float()).max()) < 1e-2
            assert not torch.equal(on, off)
    monkeypatch.setenv("RPA_MLA_WIDE", "32")
    q_lens, kv_lens = [1, 70, 33], [5000, 4170, 1033]
    b = wl.make_mla_batch("mla_wide32_chunks", q_lens, kv_lens, num_q_heads=128, lkv_dim=512, rope_dim=64, page_size=64,
                          seed=8650, sliding_window=window)
    assert_parity(run_gpu(pkg, b, gpu)[:sum(q_lens)].float(), oracle(b).float(), **TOL)


FP8 = torch.float8_e4m3fn
FP8_TOL = dict(rtol=5e-2, atol=5e-2)


def fp8_oracle(b, **kw):
    """The oracle on the cache's values widened to bf16 (exact): what the kernels compute.  The
    reference's jnp oracle itself rounds the NORMALISED probabilities to the cache's element type
    (mla/v1/ref.py:237), which in e4m3 flushes every row of more than a few hundred tokens to zero;
    its kernel keeps them in f32 (mla/v2/kernel.py:401-404), and so does this one."""
    wide = b.to("cpu")
    wide.cache_kv = wide.cache_kv.to(torch.bfloat16)
    return oracle(wide, **kw)


@pytest.mark.parametrize("P", [16, 32, 64])
@pytest.mark.parametrize("Hq", [16, 128])
def test_mla_fp8_latent_cache_decode(pkg, wl, gpu, P, Hq):
    """e4m3 latent rows with k_scale / v_scale (mla/v2/kernel.py:1354-1356): decode rows of one to
    sixty tiles, fixed and balanced plans."""
    kv_lens = [1, 31, 32, 33, 129, 500, 1025, 1900]
    say(f"mla fp8 decode P={P} Hq={Hq}")
    b = wl.make_mla_batch("mla_fp8", [1] * len(kv_lens), kv_lens, num_q_heads=Hq, lkv_dim=512, rope_dim=64,
                          page_size=P, seed=8700 + P, kv_dtype=FP8)
    scales = dict(k_scale=0.75, v_scale=1.5)
    want = fp8_oracle(b, **scales)
    for kw in ({}, {"num_splits": 1}, {"num_splits": 3}):
        got = run_gpu(pkg, b, gpu, **scales, **kw)[:len(kv_lens)]
        assert torch.isfinite(got.float()).all()
        assert_parity(got.float(), want.float(), **FP8_TOL, rel=1e-2)  # exact widening: the bf16 bar holds


def test_mla_fp8_latent_cache_long_rows_and_chunks(pkg, wl, gpu):
    """Balanced plan over ragged long rows with planted keys, then chunks on prefixes (one row per
    query token) with a sliding window, all on an e4m3 cache."""
    kv_lens = [3000 + 911 * i for i in range(24)]
    b = wl.make_mla_batch("mla_fp8_long", [1] * len(kv_lens), kv_lens, num_q_heads=128, lkv_dim=512, rope_dim=64,
                          page_size=64, seed=8710, kv_dtype=FP8)
    wl.plant_mla_needles(b, seed=3)
    want = fp8_oracle(b, k_scale=0.5)
    assert float(want.float().pow(2).mean().sqrt()) > 0.1
    say("mla fp8 long rows")
    assert_parity(run_gpu(pkg, b, gpu, k_scale=0.5)[:len(kv_lens)].float(), want.float(), **FP8_TOL, rel=1e-2)
    q_lens, kv_lens = [1, 1, 37, 64], [700, 90, 1200, 64]
    for window in (None, 500):
        say(f"mla fp8 chunks window={window}")
        b = wl.make_mla_batch("mla_fp8_mixed", q_lens, kv_lens, num_q_heads=32, lkv_dim=512, rope_dim=64, page_size=32,
                              seed=8711, kv_dtype=FP8, sliding_window=window)
        assert_parity(run_gpu(pkg, b, gpu)[:sum(q_lens)].float(), fp8_oracle(b).float(), **FP8_TOL, rel=1e-2)


def test_mla_fp8_new_rows_are_written_into_the_cache(pkg, wl, gpu):
    """rpa_mla_kv_write on an e4m3 cache: the new rows (bytes) land in their slots, bit for bit."""
    q_lens, kv_lens, P = [1, 5, 33], [40, 5, 100], 16
    b = wl.make_mla_batch("mla_fp8_write", q_lens, kv_lens, num_q_heads=16, lkv_dim=512, rope_dim=64, page_size=P,
                          seed=8720, kv_dtype=FP8)
    cache = b.cache_kv
    table = b.padded_page_indices().view(len(q_lens), -1)
    T = sum(q_lens)
    new_c = torch.empty(T, 512, dtype=FP8)
    new_r = torch.empty(T, 64, dtype=FP8)
    holed = cache.clone()
    t = 0
    for i, (ql, kv) in enumerate(zip(q_lens, kv_lens)):
        for j in range(ql):
            pos = kv - ql + j
            page, row = int(table[i, pos // P]), pos % P
            new_c[t], new_r[t] = cache[page, row, :512], cache[page, row, 512:576]
            holed.view(torch.uint8)[page, row] = 0x7F  # NaN in e4m3fn
            t += 1
    g = b.to(gpu)
    out, got_cache = pkg.mla_ragged_paged_attention(
        g.ql_nope, g.q_pe, new_c.to(gpu), new_r.to(gpu), holed.to(gpu), g.kv_lens, g.page_indices, g.cu_q_lens,
        g.cu_kv_lens, b.distribution.numpy(), sm_scale=b.sm_scale, max_kv_len=100)
    torch.cuda.synchronize()
    assert torch.equal(got_cache.cpu().view(torch.uint8), cache.view(torch.uint8))
    assert_parity(out.cpu()[:T].float(), fp8_oracle(b).float(), **FP8_TOL, rel=1e-2)


@pytest.mark.parametrize("cap", [None, 30.0])
def test_mla_scalar_scales(pkg, wl, gpu, cap):
    """q_scale, k_scale and v_scale of kernels/mla/v2/kernel.py:1354-1356: the logits are multiplied by
    k_scale and q_scale (before the soft cap), the output by v_scale; decode rows whole and split, and
    chunks (token rows)."""
    q_lens = [1, 1, 1, 9, 40]
    kv_lens = [700, 33, 5000, 300, 40]
    b = wl.make_mla_batch("mla_scales", q_lens, kv_lens, num_q_heads=32, lkv_dim=512, rope_dim=64, page_size=32,
                          seed=8301, soft_cap=cap)
    wl.plant_mla_needles(b, seed=2, logit=9.0)
    T = sum(q_lens)
    scales = dict(q_scale=0.61, k_scale=1.7, v_scale=0.37)
    say(f"mla scales cap={cap} {scales}")
    want = oracle(b, **scales)
    got = run_gpu(pkg, b, gpu, **scales)
    assert_parity(got[:T].float(), want.float(), **TOL)
    # each scale alone does what the formula says: v_scale scales the rows, q_scale * k_scale acts like sm_scale
    plain = run_gpu(pkg, b, gpu)
    half = run_gpu(pkg, b, gpu, v_scale=0.5)
    assert float(row_rel_error(half[:T].float(), 0.5 * plain[:T].float()).max()) <= 1e-2
    folded = run_gpu(pkg, b, gpu, q_scale=0.61 * 1.7)
    both = run_gpu(pkg, b, gpu, q_scale=0.61, k_scale=1.7)
    assert float(row_rel_error(folded[:T].float(), both[:T].float()).max()) <= 1e-2
    # decode rows only, split
    d = wl.make_mla_batch("mla_scales_dec", [1, 1], [6000, 900], num_q_heads=128, lkv_dim=512, rope_dim=64, page_size=64,
                          seed=8302)
    wl.plant_mla_needles(d, seed=3)
    want = oracle(d, **scales)
    for ns in (0, 1, 4):
        assert_parity(run_gpu(pkg, d, gpu, num_splits=ns, **scales)[:2].float(), want.float(), **TOL)


def test_mla_device_side_distribution(pkg, wl, gpu):
    """Static-shape mode: the number of sequences read on the device (a bucket padded with empty
    sequences and spare tokens); same results as with host integers, new rows written first."""
    q_lens = [1, 1, 1, 9, 40]
    kv_lens = [700, 33, 2100, 300, 40]
    b = wl.make_mla_batch("mla_static", q_lens, kv_lens, num_q_heads=32, lkv_dim=512, rope_dim=64, page_size=32, seed=8303)
    wl.plant_mla_needles(b, seed=6, logit=9.0)
    T, S = sum(q_lens), len(q_lens)
    pad_s, pad_t = 11, 12
    g = b.to(gpu)
    kv_pad = torch.cat([g.kv_lens, torch.zeros(pad_s, dtype=torch.int32, device=gpu)])
    cu_q_pad = torch.cat([g.cu_q_lens, torch.full((pad_s,), T, dtype=torch.int32, device=gpu)])
    cu_kv_pad = torch.cat([g.cu_kv_lens, g.cu_kv_lens[-1:].expand(pad_s)])
    qn = torch.cat([g.ql_nope, torch.zeros(pad_t, 32, 512, dtype=torch.bfloat16, device=gpu)])
    qp = torch.cat([g.q_pe, torch.zeros(pad_t, 32, 64, dtype=torch.bfloat16, device=gpu)])
    want = oracle(b)
    host, _ = pkg.mla_ragged_paged_attention(qn, qp, None, None, g.cache_kv, kv_pad, g.page_indices, cu_q_pad, cu_kv_pad,
                                             b.distribution.cpu().numpy(), sm_scale=b.sm_scale, max_kv_len=max(kv_lens),
                                             num_splits=1)
    dev, _ = pkg.mla_ragged_paged_attention(qn, qp, None, None, g.cache_kv, kv_pad, g.page_indices, cu_q_pad, cu_kv_pad,
                                            g.distribution, sm_scale=b.sm_scale, num_splits=1)
    auto, _ = pkg.mla_ragged_paged_attention(qn, qp, None, None, g.cache_kv, kv_pad, g.page_indices, cu_q_pad, cu_kv_pad,
                                             g.distribution, sm_scale=b.sm_scale)
    torch.cuda.synchronize()
    assert_parity(dev[:T].cpu().float(), want.float(), **TOL)
    assert_parity(auto[:T].cpu().float(), want.float(), **TOL)
    # whole rows in both modes: the same arithmetic, bit for bit
    assert torch.equal(dev[:T].view(torch.int16), host[:T].view(torch.int16))


def test_mla_token_groups_with_the_composition_on_the_device(pkg, wl, gpu):
    """16 heads, chunks whose tokens run eight to a workgroup, in static-shape mode: the token total and the number of
    sequences are bounds (a bucket padded with empty sequences and spare tokens), windows of tokens past the real
    total leave at once."""
    q_lens = [1, 300, 77]
    kv_lens = [900, 1500, 77]
    b = wl.make_mla_batch("mla_tg_static", q_lens, kv_lens, num_q_heads=16, lkv_dim=512, rope_dim=64, page_size=64, seed=8307,
                          sm_scale=192 ** -0.5)
    wl.plant_mla_needles(b, seed=8)
    T = sum(q_lens)
    pad_s, pad_t = 5, 130
    g = b.to(gpu)
    kv_pad = torch.cat([g.kv_lens, torch.zeros(pad_s, dtype=torch.int32, device=gpu)])
    cu_q_pad = torch.cat([g.cu_q_lens, torch.full((pad_s,), T, dtype=torch.int32, device=gpu)])
    cu_kv_pad = torch.cat([g.cu_kv_lens, g.cu_kv_lens[-1:].expand(pad_s)])
    qn = torch.cat([g.ql_nope, torch.zeros(pad_t, 16, 512, dtype=torch.bfloat16, device=gpu)])
    qp = torch.cat([g.q_pe, torch.zeros(pad_t, 16, 64, dtype=torch.bfloat16, device=gpu)])
    want = oracle(b)
    dev, _ = pkg.mla_ragged_paged_attention(qn, qp, None, None, g.cache_kv, kv_pad, g.page_indices, cu_q_pad, cu_kv_pad,
                                            g.distribution, sm_scale=b.sm_scale)
    host, _ = pkg.mla_ragged_paged_attention(qn, qp, None, None, g.cache_kv, kv_pad, g.page_indices, cu_q_pad, cu_kv_pad,
                                             b.distribution.cpu().numpy(), sm_scale=b.sm_scale, max_kv_len=max(kv_lens))
    torch.cuda.synchronize()
    assert_parity(dev[:T].cpu().float(), want.float(), **TOL)
    assert torch.equal(dev[:T].view(torch.int16), host[:T].view(torch.int16))

