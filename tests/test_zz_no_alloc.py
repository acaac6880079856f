"""GPU test of rpa_attention_noalloc, the entry point that allocates nothing: through the C ABI,
against rpa_attention on the same inputs, bit for bit, on two calls in a row, the second on a
smaller batch (the built-in workspace keeps the first call's contents)."""

import ctypes
import importlib
import sys

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def _call(pkg, b):
    m = importlib.import_module("sglang_jax_amd.ragged_paged_attention")
    n = int(b.distribution[2])
    dec_end = int(b.distribution[0])
    q_lens = b.q_lens()[:n]
    return m.RpaCall(b.q, b.kv_cache, None, b.kv_lens, b.page_indices, b.cu_q_lens, b.cu_kv_lens, num_seqs=n,
                     decode_end=dec_end, sm_scale=b.sm_scale, sliding_window=b.sliding_window, soft_cap=b.soft_cap,
                     k_scale=b.k_scale, v_scale=b.v_scale, max_kv_len=int(max(b.meta["kv_lens"])),
                     max_q_len=int(q_lens[dec_end:].max()) if n > dec_end else 0,
                     sum_decode_kv_len=int(sum(b.meta["kv_lens"][:dec_end])))


def test_no_alloc_entry_point_matches_rpa_attention(pkg, wl, gpu):
    lib = importlib.import_module("sglang_jax_amd._lib").load()
    limit = lib.rpa_noalloc_max_workspace_bytes()
    assert limit == 40 << 20
    # first a mixed batch whose decode rows are split and merged (balanced plan), then a smaller
    # decode-only batch on the fixed split plan, then a tiny one that needs no workspace at all
    batches = [
        wl.make_batch("na_big", [1] * 40 + [300, 70], [3000 + 411 * i for i in range(40)] + [900, 70], num_q_heads=32,
                      num_kv_heads=8, head_dim=128, page_size=64, seed=9101, device=gpu),
        wl.make_batch("na_small", [1] * 3, [9000, 2000, 5000], num_q_heads=32, num_kv_heads=8, head_dim=128,
                      page_size=64, seed=9102, device=gpu),
        wl.make_batch("na_tiny", [1, 5], [40, 33], num_q_heads=16, num_kv_heads=8, head_dim=128, page_size=16,
                      seed=9103, device=gpu),
    ]
    for b in batches:
        wl.plant_needles(b, seed=5)
    for n_call, b in enumerate(batches):
        call = _call(pkg, b)
        need = call.lib.rpa_workspace_bytes(ctypes.byref(call.params))
        say(f"no-alloc {b.name}: workspace {need} bytes of {limit}")
        assert need <= limit
        call.attention()
        torch.cuda.synchronize()
        want = call.out.clone()
        call.out.fill_(float("nan"))
        free_before = torch.cuda.mem_get_info()[0]
        call.attention_noalloc()
        torch.cuda.synchronize()
        if n_call > 0:  # the first call on a device is the set-up that makes the built-in array resident
            assert torch.cuda.mem_get_info()[0] == free_before  # nothing was allocated on the device
        T = int(b.cu_q_lens[int(b.distribution[2])])
        assert torch.isfinite(call.out[:T].float()).all()
        assert torch.equal(call.out[:T].view(torch.int16), want[:T].view(torch.int16))


def test_no_alloc_entry_point_refuses_what_does_not_fit(pkg, wl, gpu):
    lib = importlib.import_module("sglang_jax_amd._lib").load()
    limit = lib.rpa_noalloc_max_workspace_bytes()
    # 600 decode rows of 32 query heads, 256 wide, each cut in four: 600 * 4 * 32 * 258 * 4 bytes of partial rows
    S = 600
    b = wl.make_batch("na_refuse", [1] * S, [300] * S, num_q_heads=32, num_kv_heads=4, head_dim=256, page_size=64,
                      seed=9104, device=gpu)
    m = importlib.import_module("sglang_jax_amd.ragged_paged_attention")
    call = m.RpaCall(b.q, b.kv_cache, None, b.kv_lens, b.page_indices, b.cu_q_lens, b.cu_kv_lens, num_seqs=S,
                     decode_end=S, sm_scale=b.sm_scale, max_kv_len=300, num_splits=4)
    need = call.lib.rpa_workspace_bytes(ctypes.byref(call.params))
    say(f"no-alloc refuse: workspace {need} bytes of {limit}")
    assert need > limit
    with pytest.raises(ValueError, match="built-in one holds"):
        call.attention_noalloc()
    call.attention()  # the same batch with a workspace of the caller's
    torch.cuda.synchronize()
    assert torch.isfinite(call.out.float()).all()
