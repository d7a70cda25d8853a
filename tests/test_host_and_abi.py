"""CPU-only checks of the boundary: the C-ABI library loads and exports every symbol declared in
include/flash_decode.h, argument validation returns error codes (no compute call is made without
a GPU), the ctypes mirror of fd_params matches the header, and the host-side helpers behave."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "flash_decode.h")


def _header_text():
    with open(HEADER) as f:
        return f.read()


def test_library_exports_every_declared_symbol(fd):
    lib = fd.load_library()
    declared = re.findall(r"FD_API\s+[\w\s\*]+?\b(fd_\w+)\s*\(", _header_text())
    assert set(declared) == set(fd._lib.EXPORTED_SYMBOLS), declared
    for name in declared:
        assert getattr(lib, name) is not None
    assert lib.fd_abi_version() == int(re.search(r"#define FD_ABI_VERSION (\d+)", _header_text()).group(1))


def test_enums_and_params_struct_mirror_the_header(fd):
    text = _header_text()
    L = fd._lib
    enums = dict(re.findall(r"\b(FD_[A-Z0-9_]+)\s*=\s*(-?\d+)", text))
    for name in ("FD_F32", "FD_F16", "FD_BF16", "FD_FP8_E4M3", "FD_PATH_AUTO", "FD_PATH_VALU", "FD_PATH_MFMA",
                 "FD_COMBINE_SPLIT", "FD_COMBINE_SPLIT_LSE", "FD_COMBINE_RANK"):
        assert int(enums[name]) == getattr(L, name), name
    simple = {"int32_t": ctypes.c_int32, "int64_t": ctypes.c_int64, "float": ctypes.c_float}
    for cname, struct in (("fd_params", L.FdParams), ("fd_rank_merge", L.FdRankMerge), ("fd_qk_prep", L.FdQkPrep)):
        fields = _struct_fields(cname)
        mirror = [(n, t) for n, t in struct._fields_]
        assert [f[2] for f in fields] == [n for n, _ in mirror], cname
        for (ctype, ptr, name, _), (_, pytype) in zip(fields, mirror):
            assert pytype is (ctypes.c_void_p if ptr else simple[ctype]), (cname, name)


def test_stand_alone_reference_binding_mirrors_the_same_structs(fd):
    """reference_binding.py repeats the struct layouts on purpose (it imports nothing from the package): they must be
    the package's, field for field, and its argtypes must be those of the package's binding."""
    import importlib.util
    path = os.path.join(ROOT, "triton-distributed_amd", "reference_binding.py")
    spec = importlib.util.spec_from_file_location("fd_reference_binding_cpu", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    L = fd._lib
    assert mod.FdParams._fields_ == L.FdParams._fields_ and ctypes.sizeof(mod.FdParams) == ctypes.sizeof(L.FdParams)
    assert mod.FdQkPrep._fields_ == L.FdQkPrep._fields_ and ctypes.sizeof(mod.FdQkPrep) == ctypes.sizeof(L.FdQkPrep)
    lib = fd.load_library()
    for fn in ("fd_decode", "fd_kv_append"):
        theirs, ours = getattr(mod._lib, fn).argtypes, getattr(lib, fn).argtypes
        assert len(theirs) == len(ours), fn
        for i, (a, b) in enumerate(zip(theirs, ours)):
            both_pointers = hasattr(a, "contents") and hasattr(b, "contents")
            assert a is b or both_pointers, (fn, i, a, b)


def test_invalid_arguments_return_error_codes_without_touching_a_gpu(fd):
    lib = fd.load_library()
    L = fd._lib
    p = L.FdParams()
    # NULL tensors
    rc = lib.fd_split_kv(None, None, None, None, None, None, 1.0, None, None, 1, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, None,
                         ctypes.byref(p))
    assert rc == -1 and b"NULL" in lib.fd_last_error()
    rc = lib.fd_split_kv(None, None, None, None, None, None, 1.0, None, None, 1, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, None, None)
    assert rc == -1 and b"params" in lib.fd_last_error()
    fake = ctypes.c_void_p(0x1000)   # never dereferenced: validation fails first
    p.q_heads, p.kv_heads = 6, 4     # not a multiple
    rc = lib.fd_split_kv(None, fake, fake, fake, fake, None, 1.0, fake, fake, 1, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, None,
                         ctypes.byref(p))
    assert rc == -1 and b"multiple" in lib.fd_last_error()
    p.q_heads, p.kv_heads, p.head_dim, p.page_size, p.num_splits, p.num_pages, p.max_pages_per_seq = 8, 2, 96, 16, 4, 8, 4
    rc = lib.fd_split_kv(None, fake, fake, fake, fake, None, 1.0, fake, fake, 1, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, None,
                         ctypes.byref(p))
    assert rc == -2 and b"head_dim" in lib.fd_last_error()
    p.head_dim, p.q_dtype, p.kv_dtype, p.mid_dtype = 128, L.FD_BF16, L.FD_FP8_E4M3, L.FD_F32
    rc = lib.fd_split_kv(None, fake, fake, fake, fake, None, 1.0, fake, fake, 1, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, None,
                         ctypes.byref(p))
    assert rc == -1 and b"k_scale" in lib.fd_last_error()
    p.kv_dtype = L.FD_BF16
    rc = lib.fd_split_kv(None, fake, ctypes.c_void_p(0x1008), fake, fake, None, 1.0, fake, fake, 1, 1024, 128, 1024,
                         128, 1024, 128, 0, 0, 0, 4, None, ctypes.byref(p))
    assert rc == -3 and b"aligned" in lib.fd_last_error()
    p.num_pages, p.page_size = 1 << 20, 1 << 12
    rc = lib.fd_split_kv(None, fake, fake, fake, fake, None, 1.0, fake, fake, 1, 1024, 128, 1024, 128, 1024, 128, 0, 0,
                         0, 4, None, ctypes.byref(p))
    assert rc == -5
    # combine / schedule / decode
    assert lib.fd_combine(None, None, None, None, None, None, 1, 1, 1, 0, 0, 0, 0, 0, 0, None, None, 0,
                          ctypes.byref(p)) == -1
    assert lib.fd_combine(None, fake, None, fake, None, fake, 1, 8, 4, 0, 0, 0, 0, 0, 7, None, None, 0,
                          ctypes.byref(p)) == -1 and b"mode" in lib.fd_last_error()
    assert lib.fd_schedule(None, None, 4, None) == -1
    assert lib.fd_decode(None, fake, fake, fake, fake, None, None, None, 1.0, fake, fake, 1, 0, 0, 0, 0, 0, 0, 0, 0, 0,
                         0, 0, 0, None, 0, None, None, 0, None, ctypes.byref(p)) == -1
    # batch == 0 is a no-op success
    p2 = L.FdParams()
    assert lib.fd_schedule(None, fake, 0, fake) == 0


def test_wrappers_refuse_cpu_tensors_loudly(fd):
    wl = fd.utils.make_config(1, scale_down=8)
    with pytest.raises(RuntimeError, match="no CPU path"):
        fd.gqa_fwd_batch_decode(wl.q, wl.k_cache, wl.v_cache, None, [1], wl.kv_lens, wl.block_table, wl.scale)
    with pytest.raises(RuntimeError, match="no CPU path"):
        fd.schedule_sequences(wl.kv_lens)
    layer = fd.SpGQAFlashDecodeAttention(0, 0, 2, 1, 8, 2, 128, 128, page_size=128, max_allowed_batch=1)
    with pytest.raises(RuntimeError, match="remote_partials"):
        layer(wl.q, wl.k_cache, wl.v_cache, torch.ones(2, 1, dtype=torch.int32), wl.block_table)


def test_missing_library_is_an_error_not_a_fallback(fd, tmp_path, monkeypatch):
    monkeypatch.setattr(fd._lib, "_lib", None)
    with pytest.raises(RuntimeError, match="not built"):
        fd._lib.load_library(str(tmp_path / "nope.so"))
    monkeypatch.undo()
    fd.load_library()


def test_product_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "triton-distributed_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                with open(os.path.join(dirpath, f)) as fh:
                    text = fh.read()
                assert not re.search(r"^\s*(import|from)\s+oracle\b", text, re.M), f


def test_reference_names_are_exported(fd):
    for name in ("gqa_fwd_batch_decode", "gqa_fwd_batch_decode_aot", "gqa_fwd_batch_decode_intra_rank",
                 "gqa_fwd_batch_decode_intra_rank_aot", "gqa_fwd_batch_decode_persistent",
                 "gqa_fwd_batch_decode_persistent_aot", "kernel_inter_rank_gqa_fwd_batch_decode_combine_kv",
                 "get_triton_combine_kv_algo_info"):
        assert hasattr(fd.kernels, name)
    assert hasattr(fd.layers, "SpGQAFlashDecodeAttention")
    import triton_dist_amd
    from triton_dist_amd.kernels import gqa_fwd_batch_decode  # noqa: F401
    assert triton_dist_amd is fd
    info = fd.kernels.get_triton_split_kv_algo_info(32, 8, 128, 128, 16)
    assert info["kv_group_num"] == 4 and info["NUM_KV_SPLITS"] == 32 and info["path"] == "mfma"
    assert fd.kernels.get_triton_combine_kv_algo_info(split_kv=16)["NUM_KV_SPLITS"] == 16


def test_workload_generators_and_algorithmic_bytes(fd):
    wl = fd.utils.make_config(2, scale_down=64)
    assert wl.q.shape == (8, 32, 128) and wl.k_cache.shape[1:] == (16, 8, 128) and wl.kv_split == 32
    # every page referenced exactly once (a permutation of the pool)
    used = torch.cat([wl.block_table[b, :8] for b in range(8)])
    assert sorted(used.tolist()) == list(range(64))
    # bytes formula: K+V once, Q, used table entries, kv_lens, output, fp32 LSE
    n = 128
    expect = 8 * n * 8 * 256 * 2 + 8 * 32 * 128 * 2 + 8 * (n // 16) * 4 + 8 * 4 + 8 * 32 * 128 * 2 + 8 * 32 * 4
    assert wl.algorithmic_bytes() == expect
    wl5 = fd.utils.make_config(5, scale_down=64)
    assert wl5.k_cache.dtype == torch.float8_e4m3fn and wl5.k_scale.shape == (8,)
    assert wl5.algorithmic_bytes() == (wl5.kv_lens.sum().item() * 8 * 256 + 64 * 128 * 2 * wl5.q.shape[0] +
                                       sum(-(-int(x) // 16) for x in wl5.kv_lens) * 4 + 4 * wl5.q.shape[0] +
                                       wl5.q.shape[0] * 64 * 128 * 2 + wl5.q.shape[0] * 64 * 4 + 64)
    wl3 = fd.utils.make_config(3, scale_down=64)
    assert wl3.extra_out.shape == (7, 1, 32, 128) and float(wl3.extra_lse.min()) >= 5 and float(wl3.extra_lse.max()) <= 15
    wl4 = fd.utils.make_config(4, scale_down=16)
    assert len(set(wl4.kv_lens.tolist())) > 1          # ragged


def test_sp_layer_staging_ring_grows_and_shrinks(fd):
    layer = fd.SpGQAFlashDecodeAttention(1, 0, 4, 1, 8, 2, 128, 128, max_allowed_batch=64,
                                         thrink_buffer_threshold=3, stages=2)
    base = layer.max_allgather_buffer_size
    assert base == 4 * 8 * 128 * 8                        # sp_flash_decode_layer.py:68
    st = layer._stage(base + 1, torch.device("cpu"))
    assert layer.max_allgather_buffer_size == 2 * base and st.numel() == base + 1
    for _ in range(3):
        layer._stage(16, torch.device("cpu"))
    assert layer.max_allgather_buffer_size == base
    layer.finalize()
    assert layer.ag_buffer is None


def test_split_plan_policy(fd):
    """fd_plan_splits: an upper-bounded split count from host-known sizes only (no kv_lens read)."""
    import ctypes
    lib = fd.load_library()
    L = fd._lib

    def plan(B, Hq, Hkv, S, max_pages, P=16, kv=L.FD_BF16, D=128):
        p = L.FdParams()
        p.q_heads, p.kv_heads, p.head_dim, p.page_size, p.num_splits = Hq, Hkv, D, P, S
        p.num_pages, p.max_pages_per_seq, p.q_dtype, p.kv_dtype = 10, max_pages, L.FD_BF16, kv
        return lib.fd_plan_splits(ctypes.byref(p), B)

    assert plan(8, 32, 8, 32, 512) == 8            # config 2: 256 workgroups of 2 sibling heads x 2 waves
    assert plan(1, 32, 8, 32, 8192) == 32          # config 3: one sequence, all the splits the caller allows
    assert plan(64, 32, 8, 32, 2048) == 8          # config 4: <= 4096 tokens per split of a full-length sequence
    assert plan(32, 64, 8, 64, 1024, kv=L.FD_FP8_E4M3) == 4
    assert plan(8, 32, 8, 32, 512, D=256) == 4     # head_dim 256: 512-byte rows, no sibling heads -> 256 workgroups
    assert plan(8, 32, 8, 32, 512, D=64) == 16     # head_dim 64: four sibling heads per workgroup
    assert plan(8, 8, 8, 32, 512) == 8             # MHA runs on the MFMA kernels too
    # fp8 rows of head_dim 64: a wave takes two adjacent KV heads (4 pairs, all in one workgroup) ...
    assert plan(64, 32, 8, 32, 256, kv=L.FD_FP8_E4M3, D=64) == 4
    assert plan(8, 32, 8, 64, 512, kv=L.FD_FP8_E4M3, D=64) == 32
    # ... but not with an odd number of KV heads or more than 16 query heads per KV head
    assert plan(64, 24, 3, 32, 256, kv=L.FD_FP8_E4M3, D=64) == 4     # 192 single heads: 2 splits = 1.5 per CU -> 4
    assert plan(64, 40, 2, 32, 256, kv=L.FD_FP8_E4M3, D=64) == 2
    assert plan(8, 8, 8, 32, 512, kv=L.FD_F32) == 8  # VALU path (fp32 cache): 2048 waves with 4 waves per (head, split)
    assert plan(2, 8, 8, 32, 512) == 32
    # groups that do not divide the CU count: the count just under one workgroup per CU, without sibling heads
    # where a split would otherwise hold fewer than 512 tokens
    assert plan(3, 32, 8, 32, 512) == 10           # 24 groups x 10 = 240 workgroups
    assert plan(3, 32, 8, 8, 512) == 8             # ... or what the caller allows
    assert plan(1, 96, 12, 128, 65536, P=1) == 42  # 12 KV heads: 12 x 42 / 2 sibling heads = 252 workgroups
    assert plan(1, 96, 12, 128, 16384, P=1) == 21  # short splits: 12 x 21 = 252 workgroups of one head
    assert plan(1, 96, 12, 32, 65536, P=1) == 32   # the caller's bound wins
    assert plan(1, 8, 1, 256, 65536) == 256        # one KV head: one split per CU
    assert plan(1, 96, 12, 128, 1 << 20, P=1) == 42
    # short tables with 12 and 24 (KV head, head block) groups keep that rule: one- and two-tile splits were measured
    # level with or ahead of fewer, longer ones (3 x 512 tokens: 7.5 us with 10 splits, 8.4 / 9.3 us with 4 / 2)
    assert plan(3, 32, 8, 32, 32) == 10 and plan(3, 32, 8, 32, 64) == 10       # 512- and 1024-token tables, 24 groups
    assert plan(1, 96, 12, 32, 2048, P=1) == 21 and plan(1, 96, 12, 32, 512, P=1) == 21   # 12 groups
    assert plan(2, 96, 12, 32, 1024, P=1) == 10                                 # 24 groups of one head
    assert plan(1, 8, 8, 1, 4) == 1                # never below 1, never above what the caller asked for
    assert plan(4096, 32, 8, 32, 1) == 1
    # the part of the plan that fills the chip, without the bound on the length of a split: what a sequence gets
    # however short it is (fd_params.split_adapt)
    def fill(B, Hq, Hkv, S, max_pages, P=16, kv=L.FD_BF16, D=128):
        p = L.FdParams()
        p.q_heads, p.kv_heads, p.head_dim, p.page_size, p.num_splits = Hq, Hkv, D, P, S
        p.num_pages, p.max_pages_per_seq, p.q_dtype, p.kv_dtype = 1 << 20, max_pages, L.FD_BF16, kv
        return lib.fd_plan_min_splits(ctypes.byref(p), B)
    assert fill(8, 32, 8, 32, 512) == 8 and fill(8, 32, 8, 32, 8192) == 8      # config 2, whatever the table's width
    assert plan(8, 32, 8, 32, 8192) == 32                                      # ... while the grid covers the capacity
    assert fill(64, 32, 8, 32, 8192) == 1 and plan(64, 32, 8, 32, 8192) == 32  # a batch fills the chip by itself
    assert fill(1, 8, 1, 256, 65536) == 256
    assert fill(1, 96, 12, 128, 65536, P=1) == 64   # split_adapt is a power of two: the next one above 42
    assert plan(64, 32, 8, 256, 65536) == 32       # a table for 1 M tokens: not more than 32 slots per sequence for balance
    assert plan(2, 32, 8, 256, 65536) == 32 and plan(1, 32, 8, 256, 65536) == 64
    assert fill(0, 32, 8, 32, 512) < 0 and lib.fd_plan_min_splits(None, 1) < 0
    for args in [(3, 16, 16, 32, 83), (7, 6, 1, 5, 1000), (2, 64, 8, 64, 100000)]:
        got = plan(*args)
        assert 1 <= got <= args[3]
    assert plan(0, 32, 8, 32, 512) < 0 and b"fd_plan_splits" in lib.fd_last_error()
    assert lib.fd_plan_splits(None, 1) < 0


def test_a_stale_library_is_rebuilt_not_silently_used(fd, monkeypatch):
    """ensure_built() compares the build id inside the library with the hash of the sources beside it."""
    import importlib
    b = importlib.import_module("triton-distributed_amd.build")
    assert b.built_id() == b.source_id() == fd.load_library().fd_build_id().decode()
    assert b.ensure_built() == b.LIB_PATH           # up to date: used as it is
    calls = []
    monkeypatch.setattr(b, "source_id", lambda: "0123456789abcdef")          # as if a source had been edited
    monkeypatch.setattr(b, "build", lambda force=False, verbose=True: calls.append(force) or b.LIB_PATH)
    with pytest.raises(RuntimeError, match="does not match the sources"):
        b.ensure_built()                            # the (stubbed) rebuild did not produce a matching library
    assert calls == [True]
    monkeypatch.setenv("FD_LIBRARY_PATH", "/somewhere/else.so")            # an explicit library is the caller's business
    assert b.ensure_built() == "/somewhere/else.so"


def _struct_fields(name):
    """(ctype, is_pointer, field, array length) of the members of a struct in the header, in order."""
    body = re.search(r"typedef struct %s \{(.*?)\} %s;" % (name, name), _header_text(), re.S).group(1)
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    out = []
    for decl in body.split(";"):
        decl = decl.strip()
        if not decl:
            continue
        m = re.match(r"(?:const\s+)?(\w+)\s*(\*?)\s*(.*)$", decl, re.S)
        ctype, ptr, names = m.group(1), m.group(2), m.group(3)
        for n in names.split(","):
            n = n.strip()
            star = ptr or ("*" if n.startswith("*") else "")
            n = n.lstrip("* ")
            arr = re.match(r"(\w+)\[(\d+)\]", n)
            out.append((ctype, bool(star), arr.group(1) if arr else n, int(arr.group(2)) if arr else 0))
    return out


def test_plan_and_step_structs_mirror_the_header(fd):
    L = fd._lib
    simple = {"int32_t": ctypes.c_int32, "int64_t": ctypes.c_int64, "float": ctypes.c_float, "fd_params": L.FdParams}
    for cname, mirror in (("fd_launch_plan", L.FdLaunchPlan), ("fd_decode_args", L.FdDecodeArgs)):
        fields = _struct_fields(cname)
        assert [f[2] for f in fields] == [n for n, _ in mirror._fields_], cname
        for (ctype, ptr, name, arr), (_, pytype) in zip(fields, mirror._fields_):
            expect = ctypes.c_void_p if ptr else simple[ctype]
            if arr:
                expect = expect * arr
            assert pytype is expect or (arr and pytype._type_ is expect._type_ and pytype._length_ == arr), (cname, name)
    enums = dict(re.findall(r"\b(FD_[A-Z0-9_]+)\s*=\s*(-?\d+)", _header_text()))
    for name in ("FD_STEP_EXACT_SPLITS", "FD_STEP_SCHEDULE", "FD_STEP_NO_ORDER", "FD_STEP_FUSED", "FD_STEP_LSE_TWICE",
                 "FD_STEP_CALLER_PARTIALS", "FD_STEP_ORDER_FROM_APPEND", "FD_ORDER_NONE", "FD_ORDER_SEQUENCES",
                 "FD_ORDER_ITEMS"):
        assert int(enums[name]) == getattr(L, name), name
    # the stand-alone binding repeats fd_decode_args
    import importlib.util
    spec = importlib.util.spec_from_file_location(
        "fd_reference_binding_cpu2", os.path.join(ROOT, "triton-distributed_amd", "reference_binding.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    assert [(n, t) for n, t in mod.FdDecodeArgs._fields_[:-1]] == [(n, t) for n, t in L.FdDecodeArgs._fields_[:-1]]
    assert ctypes.sizeof(mod.FdDecodeArgs) == ctypes.sizeof(L.FdDecodeArgs)


def _plan(fd, B, Hq, Hkv, S, max_pages, P=16, kv=None, D=128, flags=0, out=None, extra=0, mid=0, max_kv_len=0):
    L = fd._lib
    lib = fd.load_library()
    kv = L.FD_BF16 if kv is None else kv
    out = L.FD_BF16 if out is None else out
    p = L.FdParams()
    p.q_heads, p.kv_heads, p.head_dim, p.page_size, p.num_splits = Hq, Hkv, D, P, S
    p.num_pages, p.max_pages_per_seq, p.q_dtype, p.kv_dtype, p.out_dtype, p.mid_dtype = max_pages * B, max_pages, out, kv, out, mid
    p.max_kv_len = max_kv_len
    lp = L.FdLaunchPlan()
    rc = lib.fd_plan_decode(ctypes.byref(p), B, extra, flags, ctypes.byref(lp))
    assert rc == 0, lib.fd_last_error()
    assert lib.fd_workspace_bytes(ctypes.byref(p), B, extra, flags) == lp.workspace_bytes
    return lp


def test_launch_plan_of_the_five_configs_and_the_published_sweep(fd):
    """fd_plan_decode pins the whole launch shape -- splits, ranges, partial type, order kind, waves, members, chunk,
    grid -- for the benchmark configurations and for the shapes of the reference's published sweep (one query,
    96 / 12 heads, fp16, page size 1, test_decode_attn.py:303-312)."""
    L = fd._lib
    F32, F16, BF16, FP8 = L.FD_F32, L.FD_F16, L.FD_BF16, L.FD_FP8_E4M3

    def shape(lp):
        return (lp.num_splits, lp.split_adapt, lp.split_align, lp.mid_dtype, lp.direct, lp.order_kind, lp.mfma, lp.tile,
                lp.waves_per_head, lp.members, lp.chunk, tuple(lp.grid))

    # config 2: planned, exactly 32 splits (chunked work items, 16-bit partials), caller-visible fp32 / bf16 partials
    assert shape(_plan(fd, 8, 32, 8, 32, 512)) == (8, 8, 64, F32, 0, 0, 1, 32, 2, 2, 1, (4, 8, 8))
    assert shape(_plan(fd, 8, 32, 8, 32, 512, flags=L.FD_STEP_EXACT_SPLITS)) == (32, 0, 64, BF16, 0, 0, 1, 32, 2, 2, 4, (4, 8, 8))
    for mid in (F32, BF16):
        lp = _plan(fd, 8, 32, 8, 32, 512, flags=L.FD_STEP_CALLER_PARTIALS, mid=mid)
        assert shape(lp) == (32, 0, 0, mid, 0, 0, 1, 32, 2, 2, 4, (4, 8, 8)) and lp.workspace_bytes == 0
    # config 3: one sequence of 131072 tokens + 7 extra partials
    assert shape(_plan(fd, 1, 32, 8, 32, 8192, extra=7)) == (64, 64, 64, F32, 0, 0, 1, 32, 2, 2, 1, (4, 1, 64))
    # config 4: ragged batch of 64 -- from 64 sequences on a step orders its (sequence, range) items whether it was asked
    # to or not; below that only when asked
    for flags in (0, L.FD_STEP_SCHEDULE):
        lp = _plan(fd, 64, 32, 8, 32, 2048, flags=flags)
        assert shape(lp) == (8, 1, 64, BF16, 0, L.FD_ORDER_ITEMS, 1, 32, 2, 2, 1, (4, 8, 64)) and lp.order_bytes == 2 * 64 * 8 * 4
    assert _plan(fd, 63, 32, 8, 32, 2048).order_kind == L.FD_ORDER_NONE
    assert _plan(fd, 63, 32, 8, 32, 2048, flags=L.FD_STEP_SCHEDULE).order_kind == L.FD_ORDER_ITEMS
    assert _plan(fd, 193, 32, 8, 32, 2048).order_kind == L.FD_ORDER_SEQUENCES   # beyond 192 sequences the per-sequence order
    assert _plan(fd, 64, 32, 8, 32, 2048, flags=L.FD_STEP_NO_ORDER).order_kind == L.FD_ORDER_NONE
    # config 5: fp8 cache, four sibling KV heads per workgroup; exactly 64 splits: written-through 16-bit partials
    assert shape(_plan(fd, 32, 64, 8, 64, 1024, kv=FP8)) == (4, 4, 64, BF16, 0, 0, 1, 64, 2, 4, 1, (2, 32, 4))
    lp = _plan(fd, 32, 64, 8, 64, 1024, kv=FP8, flags=L.FD_STEP_EXACT_SPLITS)
    assert shape(lp) == (64, 0, 64, BF16, 0, 0, 1, 64, 1, 4, 4, (2, 16, 32)) and lp.store_through == 1
    # config 1: fp32 plumbing on the VALU kernel
    lp = _plan(fd, 1, 8, 2, 4, 1, P=1024, kv=F32, out=F32)
    assert (lp.mfma, lp.mid_dtype, lp.num_splits, lp.waves_per_head) == (0, F32, 32, 8)
    # the published sweep: the library's own split count
    for tokens, expect in ((8192, (21, 32, 4, 1, (12, 1, 21))), (16384, (21, 32, 4, 1, (12, 1, 21))),
                           (32768, (42, 64, 2, 2, (6, 1, 42))), (65536, (42, 64, 2, 2, (6, 1, 42))),
                           (131072, (42, 64, 2, 2, (6, 1, 42))), (1048576, (42, 64, 2, 2, (6, 1, 42)))):
        lp = _plan(fd, 1, 96, 12, -1, tokens, P=1, kv=F16, out=F16)
        assert (lp.num_splits, lp.split_adapt, lp.waves_per_head, lp.members, tuple(lp.grid)) == expect, tokens
        assert (lp.mid_dtype, lp.order_kind, lp.direct, lp.chunk, lp.tile) == (F32, 0, 0, 1, 32)
    # a large batch of short sequences: one split, written straight to the output
    lp = _plan(fd, 64, 32, 8, 32, 128)
    assert (lp.num_splits, lp.direct, lp.partial_bytes > 0) == (1, 1, True)
    assert _plan(fd, 64, 32, 8, 32, 128, flags=L.FD_STEP_LSE_TWICE).direct == 0
    assert _plan(fd, 64, 32, 8, 32, 128, extra=1).direct == 0
    # the host-side length hint replaces the capacity, in steps of 1024 tokens
    wide = _plan(fd, 64, 32, 8, 32, 8192, max_kv_len=1000)
    assert (wide.max_kv_len, wide.num_splits) == (1024, 1) and _plan(fd, 64, 32, 8, 32, 8192).num_splits == 32
    # an order that costs no launch pays from 16 sequences on
    assert _plan(fd, 16, 32, 8, 32, 2048, flags=L.FD_STEP_ORDER_FROM_APPEND).order_kind == L.FD_ORDER_ITEMS
    assert _plan(fd, 15, 32, 8, 32, 2048, flags=L.FD_STEP_ORDER_FROM_APPEND).order_kind == L.FD_ORDER_NONE
    assert _plan(fd, 256, 32, 8, 32, 2048, flags=L.FD_STEP_SCHEDULE).order_kind == L.FD_ORDER_SEQUENCES
    assert _plan(fd, 5000, 32, 8, 32, 64, flags=L.FD_STEP_SCHEDULE).order_kind == L.FD_ORDER_NONE


def test_decode_planned_validates_before_it_launches(fd):
    L = fd._lib
    lib = fd.load_library()
    assert lib.fd_decode_planned(None, None) == -1
    a = L.FdDecodeArgs()
    a.batch = 2
    fake = 0x10000
    a.q = a.k_cache = a.v_cache = a.out = a.block_table = a.kv_lens = fake
    p = a.params
    p.q_heads, p.kv_heads, p.head_dim, p.page_size, p.num_splits, p.num_pages, p.max_pages_per_seq = 32, 8, 128, 16, 32, 64, 32
    p.q_dtype = p.kv_dtype = p.out_dtype = L.FD_BF16
    a.flags = 1 << 10
    assert lib.fd_decode_planned(None, ctypes.byref(a)) == -1 and b"flags" in lib.fd_last_error()
    a.flags, a.combine_mode = 0, L.FD_COMBINE_RANK
    assert lib.fd_decode_planned(None, ctypes.byref(a)) == -1 and b"combine_mode" in lib.fd_last_error()
    a.combine_mode = L.FD_COMBINE_SPLIT
    need = lib.fd_workspace_bytes(ctypes.byref(p), 2, 0, 0)
    assert need > 0
    assert lib.fd_decode_planned(None, ctypes.byref(a)) == -1 and str(need).encode() in lib.fd_last_error()   # no workspace
    a.workspace, a.workspace_bytes = fake + 16, need
    assert lib.fd_decode_planned(None, ctypes.byref(a)) == -1 and b"aligned" in lib.fd_last_error()
    a.workspace, a.workspace_bytes = fake, need - 1
    assert lib.fd_decode_planned(None, ctypes.byref(a)) == -1 and b"workspace" in lib.fd_last_error()
    p.q_heads = 30
    assert lib.fd_decode_planned(None, ctypes.byref(a)) == -1
    assert lib.fd_workspace_bytes(ctypes.byref(p), 2, 0, 0) == -1
    assert lib.fd_plan_decode(ctypes.byref(p), 2, 0, 0, None) == -1
    a.batch = 0
    assert lib.fd_decode_planned(None, ctypes.byref(a)) == 0   # an empty batch is a no-op
