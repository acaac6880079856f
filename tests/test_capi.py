"""Host-side checks that need no GPU: the library loads, exports every symbol
include/rpa.h declares, and its validation mirrors the reference's
static/dynamic_validate_inputs
(python/sgl_jax/srt/kernels/ragged_paged_attention/ragged_paged_attention_v3.py:1314-1487)."""

import ctypes
import os
import re
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_functions():
    text = open(os.path.join(ROOT, "include", "rpa.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(rpa_[a-z_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(pkg):
    lib = pkg._lib.load()
    names = header_functions()
    assert set(names) == set(pkg._lib.EXPORTED_SYMBOLS)
    for n in names:
        assert hasattr(lib, n), n
    assert lib.rpa_version() == 100


def test_header_links_from_two_translation_units(tmp_path):
    """A consumer with several translation units (C or C++) must link: the header may define no
    object, only types and declarations."""
    import subprocess

    inc = os.path.join(ROOT, "include")
    for cc, ext in (("gcc", "c"), ("g++", "cc")):
        a, b = tmp_path / f"a.{ext}", tmp_path / f"b.{ext}"
        a.write_text('#include "rpa.h"\nint from_a(void) { RpaMaskMode m = RPA_MASK_CUSTOM; return (int)m + RPA_VERSION; }\n')
        b.write_text('#include "rpa.h"\nint from_a(void);\nint main(void) { RpaLayout l = RPA_LAYOUT_SPLIT; '
                     'return from_a() + (int)l + (int)sizeof(RpaParams) == 0; }\n')
        out = tmp_path / f"two_units_{ext}"
        r = subprocess.run([cc, "-Wall", "-Werror", "-I", inc, str(a), str(b), "-o", str(out)],
                           capture_output=True, text=True)
        assert r.returncode == 0, r.stderr
        assert subprocess.run([str(out)]).returncode == 0


def test_library_exports_nothing_but_the_declared_entry_points(pkg):
    """The library is built with hidden visibility: its dynamic symbol table holds the functions rpa.h
    declares and nothing else (no data object, no C++ helper a host process could collide with or interpose)."""
    import subprocess

    r = subprocess.run(["nm", "-D", "--defined-only", pkg._lib.LIB_PATH], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    defined = {}
    for ln in r.stdout.splitlines():
        parts = ln.split()
        if len(parts) == 3:
            defined[parts[2]] = parts[1]
    stray = {n: k for n, k in defined.items() if n not in header_functions() and not n.startswith("__hip_")}
    assert not stray, stray
    assert all(defined[n] == "T" for n in header_functions())


def test_measurement_library_exports_its_three_kernels(pkg):
    """lib/librpa_ceilings.so (bench.py --ceilings) is a library of its own: three launchers, nothing else."""
    import subprocess

    path = os.path.join(os.path.dirname(pkg._lib.LIB_PATH), "librpa_ceilings.so")
    assert os.path.exists(path), "build it with __graft_entry__.build()"
    r = subprocess.run(["nm", "-D", "--defined-only", path], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    names = {ln.split()[2] for ln in r.stdout.splitlines() if len(ln.split()) == 3 and not ln.split()[2].startswith("__hip_")}
    assert names == {"rpa_ceiling_stream_read", "rpa_ceiling_lds_dma_read", "rpa_ceiling_mfma"}, names


def _header_struct_fields(name):
    """Field names of a struct of rpa.h, in declaration order, read from the header's text."""
    text = open(os.path.join(ROOT, "include", "rpa.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    body = re.search(r"typedef struct %s \{(.*?)\} %s;" % (name, name), text, flags=re.S).group(1)
    fields = []
    for decl in body.split(";"):
        decl = decl.strip()
        if decl:
            fields.append(re.search(r"([A-Za-z_][A-Za-z0-9_]*)$", decl).group(1))
    return fields


@pytest.mark.parametrize("struct", ["RpaParams", "RpaMlaParams"])
def test_struct_layout_matches_header(pkg, tmp_path, struct):
    """sizeof and every offsetof as the C compiler lays the header's struct out, against the ctypes mirror:
    a field reordered or retyped on one side only fails here even when the total size stays the same."""
    import subprocess

    fields = _header_struct_fields(struct)
    mirror = getattr(pkg._lib, struct)
    assert fields == [f[0] for f in mirror._fields_]
    src = tmp_path / "layout.c"
    lines = ['#include <stdio.h>', '#include <stddef.h>', '#include "rpa.h"', "int main(void) {",
             '  printf("sizeof %%zu\\n", sizeof(%s));' % struct]
    for f in fields:
        lines.append('  printf("%s %%zu %%zu\\n", offsetof(%s, %s), sizeof(((%s*)0)->%s));' % (f, struct, f, struct, f))
    lines += ["  return 0;", "}"]
    src.write_text("\n".join(lines) + "\n")
    exe = tmp_path / "layout"
    r = subprocess.run(["gcc", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    out = subprocess.run([str(exe)], capture_output=True, text=True).stdout.split("\n")
    assert int(out[0].split()[1]) == ctypes.sizeof(mirror)
    for ln in out[1:]:
        if ln:
            name, off, size = ln.split()
            assert getattr(mirror, name).offset == int(off), name
            assert getattr(mirror, name).size == int(size), name


def base_params(pkg):
    p = pkg._lib.RpaParams()
    for f in ("q", "out", "kv_cache", "kv_lens", "page_indices", "cu_q_lens", "cu_kv_lens"):
        setattr(p, f, 0x1000)  # never dereferenced by the validators
    p.num_tokens, p.num_seqs, p.num_q_heads, p.num_kv_heads = 8, 3, 8, 2
    p.head_dim, p.page_size, p.total_pages = 128, 4, 16
    p.decode_end = 1
    p.sm_scale = 1.0
    return p


def status(pkg, code):
    return pkg._lib.STATUS_NAMES[code]


def test_static_validation_codes(pkg):
    lib = pkg._lib.load()
    p = base_params(pkg)
    assert lib.rpa_validate(ctypes.byref(p)) == 0
    p.num_q_heads = 7
    assert status(pkg, lib.rpa_validate(ctypes.byref(p))) == "RPA_EINVAL_HEADS"
    assert b"divisible" in lib.rpa_last_error()
    p = base_params(pkg); p.sliding_window = -1
    assert status(pkg, lib.rpa_validate(ctypes.byref(p))) == "RPA_EINVAL_WINDOW"
    p = base_params(pkg); p.kv_dtype = 5
    assert status(pkg, lib.rpa_validate(ctypes.byref(p))) == "RPA_EINVAL_DTYPE"
    p = base_params(pkg); p.decode_end = 4
    assert status(pkg, lib.rpa_validate(ctypes.byref(p))) == "RPA_EINVAL_DISTRIBUTION"
    p = base_params(pkg); p.head_dim = 64
    assert status(pkg, lib.rpa_validate(ctypes.byref(p))) == "RPA_EUNSUPPORTED"
    # 256-wide heads: accepted (q_scale too), no workspace for short rows
    p = base_params(pkg); p.head_dim = 256
    assert lib.rpa_validate(ctypes.byref(p)) == 0
    p.decode_end = p.num_seqs
    assert lib.rpa_workspace_bytes(ctypes.byref(p)) == 0
    p.q_scale = 0.5
    assert lib.rpa_validate(ctypes.byref(p)) == 0
    p = base_params(pkg); p.softmax_dtype = 7
    assert status(pkg, lib.rpa_validate(ctypes.byref(p))) == "RPA_EINVAL_DTYPE"
    p = base_params(pkg); p.q_scale = -1.0
    assert status(pkg, lib.rpa_validate(ctypes.byref(p))) == "RPA_EINVAL_SHAPE"
    p = base_params(pkg); p.q = None
    assert status(pkg, lib.rpa_validate(ctypes.byref(p))) == "RPA_EINVAL_NULL"
    p = base_params(pkg); p.layout = 1
    assert status(pkg, lib.rpa_validate(ctypes.byref(p))) == "RPA_EINVAL_NULL"  # split layout without v_pages
    assert lib.rpa_validate(None) == -12


def host_check(pkg, p, kv_lens, pages, cu_q, cu_kv, dist):
    lib = pkg._lib.load()
    arr = lambda a: None if a is None else np.ascontiguousarray(a, dtype=np.int32)
    a = [arr(x) for x in (kv_lens, pages, cu_q, cu_kv, dist)]
    ptr = lambda x: None if x is None else x.ctypes.data_as(ctypes.POINTER(ctypes.c_int32))
    rc = lib.rpa_validate_host(ctypes.byref(p), ptr(a[0]), ptr(a[1]), len(a[1]), ptr(a[2]), ptr(a[3]), ptr(a[4]))
    return pkg._lib.STATUS_NAMES[rc], lib.rpa_last_error().decode()


def test_dynamic_validation_codes(pkg):
    p = base_params(pkg)
    kv, cu_q, cu_kv = [5, 8, 6], [0, 1, 4, 8], [0, 8, 16, 24]
    pages = [1, 2, 3, 4, 5, 6]
    ok = host_check(pkg, p, kv, pages, cu_q, cu_kv, [1, 1, 3])
    assert ok[0] == "RPA_OK", ok
    assert host_check(pkg, p, kv, pages, cu_q, cu_kv, [2, 1, 3])[0] == "RPA_EINVAL_DISTRIBUTION"
    # q_len > kv_len (message of ragged_paged_attention_v3.py:1475-1476)
    st, msg = host_check(pkg, p, [5, 2, 6], pages, cu_q, cu_kv, [1, 1, 3])
    assert st == "RPA_EINVAL_QLEN_GT_KVLEN" and "q_len=3 > kv_len=2" in msg
    # q_len == 0
    assert host_check(pkg, p, kv, pages, [0, 1, 1, 8], cu_kv, [1, 1, 3])[0] == "RPA_EINVAL_QLEN_GT_KVLEN"
    # page index out of range
    st, msg = host_check(pkg, p, kv, [1, 2, 3, 16, 5, 6], cu_q, cu_kv, [1, 1, 3])
    assert st == "RPA_EINVAL_PAGE_RANGE" and "out of [0, 16)" in msg
    assert host_check(pkg, p, kv, [1, 2, -1, 4, 5, 6], cu_q, cu_kv, [1, 1, 3])[0] == "RPA_EINVAL_PAGE_RANGE"
    # page list runs off the end of page_indices
    assert host_check(pkg, p, kv, pages[:5], cu_q, cu_kv, [1, 1, 3])[0] == "RPA_EINVAL_PAGE_RANGE"
    # tokens exceed T
    assert host_check(pkg, p, [5, 8, 9], pages + [7], [0, 1, 4, 9], [0, 8, 16, 28], [1, 1, 3])[0] == "RPA_EINVAL_SHAPE"
    # decode row with q_len 2
    assert host_check(pkg, p, kv, pages, [0, 2, 4, 8], cu_kv, [1, 1, 3])[0] == "RPA_EINVAL_DISTRIBUTION"
    # padded 2-D table: page_cnt > pages_per_seq
    p2 = base_params(pkg); p2.cu_kv_lens = None; p2.pages_per_seq = 1
    st, msg = host_check(pkg, p2, kv, [1, 2, 3], cu_q, None, [1, 1, 3])
    assert st == "RPA_EINVAL_PAGE_RANGE" and "pages_per_seq=1" in msg


def test_workspace_size_is_deterministic(pkg):
    lib = pkg._lib.load()
    p = base_params(pkg)
    p.num_seqs = p.decode_end = 16
    p.num_tokens = 16
    p.num_q_heads, p.num_kv_heads, p.page_size, p.total_pages = 32, 8, 64, 8192
    p.max_kv_len = 32768
    # lengths unknown to the host: the balanced plan, two groups of 16 partial rows per wave slot
    # plus the prefix sum of blocks (17 words, padded to 8 bytes) and one 8-byte arrival word per
    # (row, unit, wave): 16 rows x 2 units x 4 waves; its size does not depend on the batch
    a = lib.rpa_workspace_bytes(ctypes.byref(p))
    assert a > 0 and a == lib.rpa_workspace_bytes(ctypes.byref(p))
    assert (a - 18 * 4 - 16 * 2 * 4 * 8) % (2 * 16 * 130 * 4) == 0
    p.max_kv_len = 8192
    assert lib.rpa_workspace_bytes(ctypes.byref(p)) == a
    # all rows of one known length: the fixed plan, one partial row per (row, split, head)
    p.max_kv_len = 32768
    p.sum_decode_kv_len = 16 * 32768
    f = lib.rpa_workspace_bytes(ctypes.byref(p))
    assert f > 0 and f % (16 * 32 * 130 * 4) == 0
    p.num_splits = 1
    assert lib.rpa_workspace_bytes(ctypes.byref(p)) == 0


def test_workspace_for_prefill_launches_that_leave_the_gpu_idle(pkg, monkeypatch):
    """rpa_workspace_bytes also reports the room that lets an under-filled prefill launch cut its K/V
    ranges into pieces: (tokens x heads x pieces) partial rows of 128 + 2 floats.  Nothing for launches
    that fill the GPU, for calls whose composition is on the device, without a bound on the lengths,
    or with RPA_PREFILL_SPLITS=0; the forced count is honoured."""
    lib = pkg._lib.load()
    monkeypatch.delenv("RPA_PREFILL_SPLITS", raising=False)

    def params(tokens, hq, hkv, max_kv):
        p = base_params(pkg)
        p.num_seqs, p.decode_end, p.num_tokens = 1, 0, tokens
        p.num_q_heads, p.num_kv_heads, p.page_size, p.total_pages = hq, hkv, 64, 8192
        p.max_q_len, p.max_kv_len = tokens, max_kv
        return p

    row = (128 + 2) * 4
    p = params(512, 8, 2, 16384)  # one 512-token chunk on a long prefix, 32 workgroups
    need = lib.rpa_workspace_bytes(ctypes.byref(p))
    assert need > 0 and need % (512 * 8 * row) == 0
    pieces = need // (512 * 8 * row)
    assert 2 <= pieces <= 64
    p.max_kv_len = 0  # no bound on the lengths: no cut
    assert lib.rpa_workspace_bytes(ctypes.byref(p)) == 0
    p = params(512, 8, 2, 16384)
    p.distribution = 0x1000  # composition on the device: the same rule on the bounds (every workgroup fits the count to its range)
    monkeypatch.setenv("RPA_PREFILL_SPLITS", "0")
    dyn = lib.rpa_workspace_bytes(ctypes.byref(p))  # what the decode plan of such a call asks for
    monkeypatch.setenv("RPA_PREFILL_SPLITS", "7")
    assert lib.rpa_workspace_bytes(ctypes.byref(p)) == max(dyn, 512 * 8 * 7 * row)
    monkeypatch.delenv("RPA_PREFILL_SPLITS")
    assert lib.rpa_workspace_bytes(ctypes.byref(p)) == max(dyn, need)
    p = params(2048, 32, 8, 8192)  # 512 workgroups: the GPU is full
    assert lib.rpa_workspace_bytes(ctypes.byref(p)) == 0
    p = params(1000, 8, 4, 1000)  # a short range: the merge would cost what the cut saves
    assert lib.rpa_workspace_bytes(ctypes.byref(p)) == 0
    p = params(16, 8, 2, 32768)  # a verify step on a long context: the short-chunk tile, many pieces
    assert lib.rpa_workspace_bytes(ctypes.byref(p)) // (16 * 8 * row) >= 16
    p.kv_dtype = 1  # e4m3 caches take the compiled kernels (128 positions per workgroup), which cut too
    assert lib.rpa_workspace_bytes(ctypes.byref(p)) // (16 * 8 * row) >= 16
    p = params(200, 4, 1, 3000)  # 256-wide heads: rows of 256 + 2 floats
    p.head_dim = 256
    need = lib.rpa_workspace_bytes(ctypes.byref(p))
    assert need > 0 and need % (200 * 4 * (256 + 2) * 4) == 0
    p = params(512, 8, 2, 16384)
    monkeypatch.setenv("RPA_PREFILL_SPLITS", "0")
    assert lib.rpa_workspace_bytes(ctypes.byref(p)) == 0
    monkeypatch.setenv("RPA_PREFILL_SPLITS", "5")
    assert lib.rpa_workspace_bytes(ctypes.byref(p)) == 512 * 8 * 5 * row


def test_workspace_for_a_custom_mask_as_bits(pkg, monkeypatch):
    """Custom masks: rpa_workspace_bytes adds one bit per (query token, kv token up to the bound on the lengths),
    rows of whole 64-bit words, behind the partial rows of a cut launch (256-byte aligned).  Not without a bound on
    the lengths, not for 256-wide heads, not with RPA_MASK_BITS=0."""
    lib = pkg._lib.load()
    monkeypatch.delenv("RPA_PREFILL_SPLITS", raising=False)
    monkeypatch.delenv("RPA_MASK_BITS", raising=False)
    p = base_params(pkg)
    p.num_seqs, p.decode_end, p.num_tokens = 64, 0, 1024
    p.num_q_heads, p.num_kv_heads, p.page_size, p.total_pages = 32, 8, 64, 8192
    p.max_q_len, p.max_kv_len = 16, 4112
    p.mask_mode = 1
    p.custom_mask = 0x1000
    p.cu_mask_lens = 0x1000
    bits = 1024 * ((4112 + 63) // 64) * 8
    monkeypatch.setenv("RPA_PREFILL_SPLITS", "0")
    assert lib.rpa_workspace_bytes(ctypes.byref(p)) == bits
    monkeypatch.setenv("RPA_PREFILL_SPLITS", "3")
    partial = 1024 * 32 * 3 * (128 + 2) * 4
    assert lib.rpa_workspace_bytes(ctypes.byref(p)) == ((partial + 255) // 256) * 256 + bits
    monkeypatch.setenv("RPA_MASK_BITS", "0")
    assert lib.rpa_workspace_bytes(ctypes.byref(p)) == partial
    monkeypatch.delenv("RPA_MASK_BITS")
    monkeypatch.setenv("RPA_PREFILL_SPLITS", "0")
    p.max_kv_len = 0
    assert lib.rpa_workspace_bytes(ctypes.byref(p)) == 0
    p.max_kv_len = 4112
    p.head_dim = 256
    assert lib.rpa_workspace_bytes(ctypes.byref(p)) == 0


def test_python_wrapper_raises_like_the_reference(pkg):
    import torch

    q = torch.zeros(4, 8, 128, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="no CPU path"):
        pkg.ragged_paged_attention(q, None, None, torch.zeros(2, 4, 4, 128, dtype=torch.bfloat16),
                                   torch.zeros(2, dtype=torch.int32), torch.zeros(2, dtype=torch.int32),
                                   torch.zeros(3, dtype=torch.int32), torch.zeros(3, dtype=torch.int32), [0, 0, 2], None)
    m = __import__("sglang_jax_amd.ragged_paged_attention", fromlist=["x"])
    i32 = lambda *s: torch.zeros(*s, dtype=torch.int32)
    cache = torch.zeros(2, 4, 4, 128, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="must be positive"):
        m.static_validate_inputs(q, None, None, cache, i32(2), i32(2), i32(3), i32(3), i32(3), sliding_window=0)
    with pytest.raises(ValueError, match="must not be 0.0"):
        m.static_validate_inputs(q, None, None, cache, i32(2), i32(2), i32(3), i32(3), i32(3), soft_cap=0.0)
    with pytest.raises(ValueError, match="divisible"):
        m.static_validate_inputs(q, None, None, torch.zeros(2, 4, 6, 128, dtype=torch.bfloat16), i32(2), i32(2), i32(3),
                                 i32(3), i32(3))
    with pytest.raises(ValueError, match=r"cu_q_lens.shape"):
        m.static_validate_inputs(q, None, None, cache, i32(2), i32(2), i32(4), i32(3), i32(3))
    with pytest.raises(ValueError, match="int32"):
        m.static_validate_inputs(q, None, None, cache, torch.zeros(2, dtype=torch.int64), i32(2), i32(3), i32(3), i32(3))
    with pytest.raises(ValueError, match="Expected 3D"):
        m.static_validate_inputs(q, torch.zeros(4, 2), torch.zeros(4, 2), cache, i32(2), i32(2), i32(3), i32(3), i32(3))


def test_generated_assembly_is_up_to_date(tmp_path):
    """The generated include files (the assembly loops of the prefill and MLA kernels) are what
    their generators write today, with no experiment switch set."""
    import shutil
    import subprocess

    csrc = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "sglang-jax_amd", "csrc")
    work = tmp_path / "csrc"
    work.mkdir()
    for name in ("gen_prefill_pipe_loop.py", "gen_mla_pipe_loop.py", "gen_mla_wide_loop.py", "gen_mla_wide32_loop.py"):
        shutil.copy(os.path.join(csrc, name), work / name)
    env = {k: v for k, v in os.environ.items() if not k.startswith(("RPA_PIPE_", "RPA_MLA_PIPE_", "RPA_MLA_WIDE_"))}
    env["PYTHONDONTWRITEBYTECODE"] = "1"
    for gen, inc in (("gen_prefill_pipe_loop.py", "rpa_prefill_pipe_loop.inc"), ("gen_mla_pipe_loop.py", "rpa_mla_pipe_loop.inc"),
                     ("gen_mla_wide_loop.py", "rpa_mla_wide_loop.inc"), ("gen_mla_wide32_loop.py", "rpa_mla_wide32_loop.inc")):
        subprocess.run([sys.executable, str(work / gen)], check=True, env=env, stdout=subprocess.DEVNULL)
        with open(work / inc) as f, open(os.path.join(csrc, inc)) as g:
            assert f.read() == g.read(), f"{inc} is stale: run {gen}"


# ------------------------------------------------------------------ the shape table (csrc/rpa_shapes.h)
def _shape_params(pkg, *, S, decode_end, T, Hq, Hkv, D=128, P=64, fp8=False, max_q=0, max_kv=0, sum_dec=0, **opts):
    p = base_params(pkg)
    p.num_tokens, p.num_seqs, p.num_q_heads, p.num_kv_heads = T, S, Hq, Hkv
    p.head_dim, p.page_size, p.total_pages = D, P, 1 << 20
    p.decode_end, p.max_q_len, p.max_kv_len, p.sum_decode_kv_len = decode_end, max_q, max_kv, sum_dec
    p.kv_dtype = pkg._lib.RPA_KV_FP8_E4M3 if fp8 else pkg._lib.RPA_KV_BF16
    for k, v in opts.items():
        setattr(p, k, v)
    return p


def test_shape_table_rows_of_the_benchmark_configurations(pkg):
    """rpa_describe_plan: which row of the shape table, which kernel and which split plan a call takes (the
    reference answers the same question with get_tuned_block_sizes, tuned_block_sizes_v3.py:2163-2229).
    The five benchmark shapes and the option / head-width / chunk-length branches of the table."""
    d = pkg._lib.describe_plan
    c1 = d(_shape_params(pkg, S=8, decode_end=8, T=8, Hq=16, Hkv=8, P=16, max_kv=512, sum_dec=2300))
    assert "shape=decode_bf16_small" in c1 and "rpa_decode_splitkv_kernel" in c1 and "waves_per_wg=2" in c1
    assert "prefill" not in c1
    c2 = d(_shape_params(pkg, S=64, decode_end=56, T=8760, Hq=32, Hkv=8, max_q=2048, max_kv=4096, sum_dec=130000))
    assert "shape=decode_bf16_stream kernel=rpa_decode_balanced_kernel rows=56 waves_per_wg=4 resident_waves=1024" in c2
    assert "shape=prefill_pipe kernel=rpa_prefill_pipe_kernel tile=128x1x64 kv_pieces_with_workspace=1" in c2
    c3 = d(_shape_params(pkg, S=16, decode_end=16, T=16, Hq=32, Hkv=8, max_kv=32768, sum_dec=16 * 32768))
    assert "shape=decode_bf16_stream kernel=rpa_decode_splitkv_kernel" in c3 and "merge=rpa_combine_kernel" in c3
    c4 = d(_shape_params(pkg, S=128, decode_end=128, T=128, Hq=64, Hkv=8, fp8=True, max_kv=8192, sum_dec=590000))
    assert "shape=decode_fp8_stream kernel=rpa_decode_balanced_kernel" in c4 and "resident_waves=1024" in c4
    # chunks of at most 64 tokens with heads in fours: the short-chunk tile; a long prompt on few heads is cut
    short = d(_shape_params(pkg, S=64, decode_end=0, T=1024, Hq=32, Hkv=8, max_q=16, max_kv=4096))
    assert "shape=prefill_pipe_short" in short and "tile=32x4x64" in short
    one = d(_shape_params(pkg, S=1, decode_end=0, T=16, Hq=8, Hkv=2, max_q=16, max_kv=32768))
    assert "kv_pieces_with_workspace=1 " not in one  # an under-filled launch cuts its K/V range
    # options and cache types leave the assembly kernel
    assert "shape=prefill_options kernel=rpa_prefill_async_kernel" in d(_shape_params(
        pkg, S=2, decode_end=0, T=600, Hq=32, Hkv=8, max_q=300, max_kv=600, soft_cap=30.0))
    assert "shape=prefill_fp8 kernel=rpa_prefill_staged_kernel" in d(_shape_params(
        pkg, S=2, decode_end=0, T=600, Hq=32, Hkv=8, max_q=300, max_kv=600, fp8=True))
    assert "shape=prefill_pipe " not in d(_shape_params(pkg, S=2, decode_end=0, T=600, Hq=32, Hkv=8, P=48, max_q=300, max_kv=600))
    wide = d(_shape_params(pkg, S=6, decode_end=4, T=304, Hq=16, Hkv=4, D=256, max_q=200, max_kv=900, sum_dec=3000))
    assert "shape=decode_256 kernel=rpa_rows256_kernel" in wide and "shape=prefill_256 kernel=rpa_prefill_async_kernel" in wide


def test_shape_table_environment_overrides(pkg, monkeypatch):
    d = pkg._lib.describe_plan
    p = _shape_params(pkg, S=64, decode_end=56, T=8760, Hq=32, Hkv=8, max_q=2048, max_kv=4096, sum_dec=130000)
    assert "rpa_prefill_pipe_kernel" in d(p)
    monkeypatch.setenv("RPA_PREFILL_PIPE", "0")  # the switches are read again whenever the environment changes
    assert "shape=prefill_options kernel=rpa_prefill_async_kernel" in d(p)
    monkeypatch.delenv("RPA_PREFILL_PIPE")
    monkeypatch.setenv("RPA_DECODE_BALANCED", "0")
    monkeypatch.setenv("RPA_DECODE_WAVES_PER_WG", "2")
    text = d(p)
    assert "rpa_decode_splitkv_kernel" in text and "waves_per_wg=2" in text and "rpa_prefill_pipe_kernel" in text
    monkeypatch.delenv("RPA_DECODE_BALANCED")
    monkeypatch.delenv("RPA_DECODE_WAVES_PER_WG")
    assert "rpa_decode_balanced_kernel" in d(p)


def test_mla_shape_table_rows(pkg, monkeypatch):
    def params(Hq, P=64, fp8=False, S=64, T=64, max_kv=16384, sum_kv=590000, soft_cap=0.0):
        p = pkg._lib.RpaMlaParams()
        for f in ("ql_nope", "q_pe", "out", "cache_kv", "kv_lens", "page_indices", "cu_q_lens", "cu_kv_lens"):
            setattr(p, f, 0x1000)
        p.num_tokens, p.num_seqs, p.num_q_heads = T, S, Hq
        p.lkv_dim, p.rope_dim, p.page_size, p.total_pages = 512, 64, P, 1 << 16
        p.row_stride, p.rope_offset = 576, 512
        p.max_kv_len, p.sum_kv_len, p.sm_scale, p.soft_cap = max_kv, sum_kv, 0.07, soft_cap
        p.cache_dtype = pkg._lib.RPA_KV_FP8_E4M3 if fp8 else pkg._lib.RPA_KV_BF16
        return p

    d = pkg._lib.describe_mla_plan
    c5 = d(params(128), False)
    assert "shape=mla_wide" in c5 and "waves_per_wg=4" in c5 and "plan=balanced" in c5 and "workgroups=256" in c5
    assert "shape=mla_pipe" in d(params(128, fp8=True), False)
    assert "shape=mla_shared_16" in d(params(16), False) and "share=8" in d(params(16), False)
    assert "shape=mla_shared_64" in d(params(48), False)
    assert "shape=mla_compiled" in d(params(128, P=16), False)
    assert "shape=mla_compiled" in d(params(128, soft_cap=30.0), False)
    assert "shape=mla_compiled" in d(params(160), False)
    # query tokens of a chunk with few heads share a workgroup: on the wide loop for bf16 latents without a window
    chunk = dict(S=4, T=4096, max_kv=8192, sum_kv=20000)
    assert "token_groups=off" in d(params(16), False) and "token_groups=off" in d(params(16), True)  # decode rows
    assert "token_groups=wide" in d(params(16, **chunk), True) and "waves_per_wg=4" in d(params(16, **chunk), True)
    assert "token_groups=eight_waves " in d(params(32, fp8=True, **chunk), True)
    windowed = params(64, **chunk)
    windowed.sliding_window = 512
    assert "token_groups=eight_waves " in d(windowed, True)
    assert "token_groups=off" in d(params(48, **chunk), True) and "token_groups=off" in d(params(128, **chunk), True)
    monkeypatch.setenv("RPA_MLA_TOKEN_GROUPS", "0")
    assert "token_groups=off" in d(params(16, **chunk), True)
    monkeypatch.delenv("RPA_MLA_TOKEN_GROUPS")
    monkeypatch.setenv("RPA_MLA_WIDE", "0")
    assert "token_groups=eight_waves " in d(params(16, **chunk), True)
    assert "shape=mla_pipe" in d(params(128), False)
    monkeypatch.setenv("RPA_MLA_PIPE", "0")
    assert "shape=mla_compiled" in d(params(128), False)
    assert "token_groups=eight_waves_compiled" in d(params(16, **chunk), True)
