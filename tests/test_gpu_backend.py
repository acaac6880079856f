"""The attention backend end to end on the GPU: metadata from a scheduler-shaped batch,
per-layer calls that write the new tokens into the layer's cache and attend over it
(flashattention_backend.py:146-237, 603-760), checked against the CPU oracle run on the
complete cache."""

import sys
from types import SimpleNamespace

import numpy as np
import pytest
import torch

from parity import assert_parity

from oracle.ref_rpa import ref_ragged_paged_attention_fused

pytestmark = pytest.mark.gpu

TOL = dict(rtol=2e-2, atol=2e-2)


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


class Pool:
    """Per-layer fused caches [pages, P, 2*Hkv, D] (memory_pool.py:566-611)."""

    def __init__(self, layers, pages, P, Hkv, D, device, seed):
        g = torch.Generator().manual_seed(seed)
        # unused slots hold NaN canaries: nothing may read them
        self.host = [torch.full((pages, P, 2 * Hkv, D), float("nan"), dtype=torch.bfloat16) for _ in range(layers)]
        self.dev = [h.to(device) for h in self.host]
        self.g = g

    def get_fused_kv_buffer(self, layer_id):
        return self.dev[layer_id]


def padded_table(page_lists, width):
    t = np.zeros((len(page_lists), width), dtype=np.int32)
    for i, ps in enumerate(page_lists):
        t[i, :len(ps)] = ps
    return torch.from_numpy(t)


@pytest.mark.parametrize("P,window,cap", [(16, None, None), (64, 48, 30.0)])
def test_extend_then_decode_steps(pkg, gpu, P, window, cap):
    Hq, Hkv, D, layers, pool_pages = 8, 2, 128, 2, 96
    rng = np.random.default_rng(7)
    gen = torch.Generator().manual_seed(11)
    pool = Pool(layers, pool_pages, P, Hkv, D, gpu, 3)
    backend = pkg.FlashAttention(Hq, Hkv, D, page_size=P, device=gpu)
    layer_objs = [SimpleNamespace(layer_id=i, scaling=D ** -0.5, head_dim=D, sliding_window_size=window,
                                  logit_cap=cap, xai_temperature_len=-1, softmax_dtype=None, attn_type=None)
                  for i in range(layers)]
    free = list(rng.permutation(pool_pages))
    prompt = [37, 70, 5]
    bs_pad = 4  # one padded (empty) request slot, as the scheduler's bucketing leaves them
    pages = [[] for _ in range(bs_pad)]
    seq_lens = np.zeros(bs_pad, dtype=np.int32)
    # what each layer's cache holds per sequence (host truth), for the oracle
    truth = [[torch.zeros(0, 2 * Hkv, D, dtype=torch.bfloat16) for _ in range(bs_pad)] for _ in range(layers)]

    def run_step(mode, new_lens):
        nonlocal seq_lens
        new_lens = np.asarray(new_lens, dtype=np.int32)
        seq_lens = seq_lens + new_lens
        for i in range(bs_pad):
            while len(pages[i]) * P < seq_lens[i]:
                pages[i].append(int(free.pop()))
        cache_loc = np.concatenate([np.arange(p * P, p * P + P) for ps in pages for p in ps]).astype(np.int32)
        batch = SimpleNamespace(forward_mode=mode, seq_lens=seq_lens.copy(), cache_loc=cache_loc,
                                extend_seq_lens=new_lens, dp_size=1, per_dp_bs_size=bs_pad)
        backend.forward_metadata = backend.get_forward_metadata(batch)
        T = int(new_lens.sum())
        n_real = int((seq_lens > 0).sum())
        for L in range(layers):
            q = torch.randn(T, Hq * D, generator=gen).to(torch.bfloat16)
            k = torch.randn(T, Hkv * D, generator=gen).to(torch.bfloat16)
            v = torch.randn(T, Hkv * D, generator=gen).to(torch.bfloat16)
            out, cache = backend(q.to(gpu), k.to(gpu), v.to(gpu), layer_objs[L], batch, pool)
            torch.cuda.synchronize()
            assert out.shape == (T, Hq * D)
            assert cache.data_ptr() == pool.dev[L].data_ptr()
            # host truth: append the new tokens (K0,V0,K1,V1,... head order)
            t = 0
            for i in range(bs_pad):
                for _ in range(int(new_lens[i])):
                    row = torch.stack([k[t].view(Hkv, D), v[t].view(Hkv, D)], dim=1).reshape(1, 2 * Hkv, D)
                    truth[L][i] = torch.cat([truth[L][i], row])
                    t += 1
            full = torch.zeros(pool_pages, P, 2 * Hkv, D, dtype=torch.bfloat16)
            for i in range(bs_pad):
                for j, pg in enumerate(pages[i]):
                    rows = truth[L][i][j * P:(j + 1) * P]
                    full[pg, :len(rows)] = rows
            cu_q = np.concatenate([[0], np.cumsum(new_lens)]).astype(np.int32)
            want = ref_ragged_paged_attention_fused(
                q.view(T, Hq, D), full, torch.from_numpy(seq_lens.copy()), padded_table(pages, 8),
                torch.from_numpy(cu_q), [n_real], sm_scale=D ** -0.5, sliding_window=window, soft_cap=cap)
            assert_parity(out.cpu().float().view(T, Hq, D), want.float(), **TOL)
            # every written slot equals the host truth bit for bit; the rest is untouched (NaN)
            got_cache = pool.dev[L].cpu()
            for i in range(bs_pad):
                for j, pg in enumerate(pages[i]):
                    rows = truth[L][i][j * P:(j + 1) * P]
                    assert torch.equal(got_cache[pg, :len(rows)].view(torch.int16), rows.view(torch.int16))
                    assert torch.isnan(got_cache[pg, len(rows):].float()).all()

    say(f"extend P={P} window={window} cap={cap}")
    run_step(pkg.ForwardMode.EXTEND, prompt + [0])
    assert backend.forward_metadata.host_distribution.tolist() == [0, 3, 3]
    for step in range(3):
        say(f"decode step {step}")
        run_step(pkg.ForwardMode.DECODE, [1, 1, 1, 0])
        assert backend.forward_metadata.host_distribution.tolist() == [3, 3, 3]
    say("chunked extend on top of the existing prefix")
    run_step(pkg.ForwardMode.EXTEND, [9, 4, 33, 0])


def test_mla_backend_extend_then_decode(pkg, gpu):
    """MLAAttentionBackend (mla_backend.py:83-389): prompt, then decode steps, on the
    reference's 640-wide latent rows; output and cache against the CPU oracle."""
    from oracle.ref_mla import ref_mla_ragged_paged_attention

    Hq, P, pool_pages, W = 16, 16, 48, 640
    rng = np.random.default_rng(17)
    gen = torch.Generator().manual_seed(19)
    host_cache = torch.zeros(pool_pages, P, W, dtype=torch.bfloat16)
    pool = SimpleNamespace(buf=host_cache.to(gpu))
    pool.get_fused_kv_buffer = lambda layer_id: pool.buf
    backend = pkg.MLAAttentionBackend(Hq, 512, 128, 64, 128, page_size=P, device=gpu)
    layer = SimpleNamespace(layer_id=0, scaling=None, sliding_window_size=None, logit_cap=None)
    free = list(rng.permutation(pool_pages))
    bs = 3
    pages = [[] for _ in range(bs)]
    seq_lens = np.zeros(bs, dtype=np.int32)

    def step(mode, new_lens):
        nonlocal seq_lens, host_cache
        new_lens = np.asarray(new_lens, dtype=np.int32)
        seq_lens = seq_lens + new_lens
        for i in range(bs):
            while len(pages[i]) * P < seq_lens[i]:
                pages[i].append(int(free.pop()))
        cache_loc = np.concatenate([np.arange(p * P, p * P + P) for ps in pages for p in ps]).astype(np.int32)
        batch = SimpleNamespace(forward_mode=mode, seq_lens=seq_lens.copy(), cache_loc=cache_loc,
                                extend_seq_lens=new_lens, dp_size=1, per_dp_bs_size=bs)
        backend.forward_metadata = backend.get_forward_metadata(batch)
        T = int(new_lens.sum())
        q = (torch.randn(T, Hq, 512, generator=gen) * 0.5).to(torch.bfloat16)
        qr = (torch.randn(T, Hq, 64, generator=gen) * 0.5).to(torch.bfloat16)
        kc = (torch.randn(T, 1, 512, generator=gen) * 0.5).to(torch.bfloat16)
        kr = (torch.randn(T, 1, 64, generator=gen) * 0.5).to(torch.bfloat16)
        out, cache = backend(q.to(gpu), kc.to(gpu), kc.to(gpu), layer, batch, pool, q_rope=qr.to(gpu), k_rope=kr.to(gpu))
        torch.cuda.synchronize()
        width = max(len(p) for p in pages)
        table = np.zeros((bs, width), dtype=np.int32)
        for i, ps in enumerate(pages):
            table[i, :len(ps)] = ps
        cu_q = np.concatenate([[0], np.cumsum(new_lens)]).astype(np.int32)
        want, host_cache = ref_mla_ragged_paged_attention(
            q, qr, kc[:, 0], kr[:, 0], host_cache, torch.from_numpy(seq_lens.copy()),
            torch.from_numpy(table.reshape(-1)), torch.from_numpy(cu_q), [0, 0, bs],
            sm_scale=1.0 / np.sqrt(192.0), layout="padded")
        assert torch.equal(cache.cpu().view(torch.int16), host_cache.view(torch.int16))
        assert_parity(out.cpu().float(), want.float(), **TOL)

    say("mla extend")
    step(pkg.ForwardMode.EXTEND, [37, 70, 5])
    assert backend.forward_metadata.host_distribution.tolist() == [0, 0, 3]
    for s_ in range(2):
        say(f"mla decode {s_}")
        step(pkg.ForwardMode.DECODE, [1, 1, 1])
