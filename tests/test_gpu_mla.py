"""GPU parity of the absorbed-MLA decode kernel against the CPU oracle
(oracle/ref_mla.py), rtol = atol = 2e-2 (bf16).  Shapes follow the reference's
MLA tests (python/sgl_jax/test/test_mla_attention.py:346-696: 16 heads, latent 512,
rope 64, page sizes 8..64, window 128, soft cap 30) and the DeepSeek-V3 decode
configuration."""

import sys

import pytest
import torch

from oracle.ref_mla import ref_mla_ragged_paged_attention

pytestmark = pytest.mark.gpu
TOL = dict(rtol=2e-2, atol=2e-2)


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def oracle(b):
    n = int(b.distribution[2])
    out, _ = ref_mla_ragged_paged_attention(
        b.ql_nope, b.q_pe, None, None, b.cache_kv, b.kv_lens, b.padded_page_indices(), b.cu_q_lens, [n, n, n],
        sm_scale=b.sm_scale, sliding_window=b.sliding_window, soft_cap=b.soft_cap)
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
    torch.testing.assert_close(got.float(), oracle(b).float(), **TOL)


@pytest.mark.parametrize("window,cap", [(128, None), (None, 30.0), (128, 30.0)])
def test_mla_window_and_soft_cap(pkg, wl, gpu, window, cap):
    kv_lens = [100, 128, 129, 700]
    b = wl.make_mla_batch("mla_swa", [1] * 4, kv_lens, num_q_heads=16, lkv_dim=512, rope_dim=64, page_size=16,
                          seed=72, sm_scale=192 ** -0.5, sliding_window=window, soft_cap=cap)
    got = run_gpu(pkg, b, gpu)
    torch.testing.assert_close(got.float(), oracle(b).float(), **TOL)


def test_mla_split_count_does_not_matter(pkg, wl, gpu):
    b = wl.make_mla_batch("mla_splits", [1] * 3, [40, 1000, 3000], num_q_heads=32, lkv_dim=512, rope_dim=64,
                          page_size=64, seed=73, sm_scale=192 ** -0.5)
    want = oracle(b)
    base = None
    for ns in (1, 2, 5, 16):
        say(f"mla num_splits {ns}")
        got = run_gpu(pkg, b, gpu, num_splits=ns)
        torch.testing.assert_close(got.float(), want.float(), **TOL)
        base = got if base is None else base
        torch.testing.assert_close(got.float(), base.float(), rtol=1e-2, atol=4e-3)


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
    torch.testing.assert_close(got.float(), oracle(b).float(), **TOL)
