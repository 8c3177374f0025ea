"""CPU-only checks of the drop-in boundary: the C ABI library loads and exports
exactly what include/energon_hip.h declares, the ctypes table matches the
header, the Python mirror keeps the reference's names and signatures, and host
argument checks fire before anything reaches the device."""
import ctypes
import inspect
import os
import re
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "energon_hip.h")


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(en_[a-z0-9_]+)\s*\(", text)))


def _arg_count(name):
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    m = re.search(r"\b%s\s*\((.*?)\)\s*;" % re.escape(name), text, flags=re.S)
    args = m.group(1).strip()
    return 0 if args in ("", "void") else len(args.split(","))


def test_library_exports_every_declared_symbol():
    from energonai_amd import _lib
    lib = _lib.load()
    declared = _declared_symbols()
    assert len(declared) >= 20
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in the header but not exported"
    assert sorted(_lib.SIGNATURES) == declared, "ctypes table and header disagree"
    for name, (_, argtypes) in _lib.SIGNATURES.items():
        assert len(argtypes) == _arg_count(name), f"{name}: ctypes arity differs from the header"
    assert lib.en_version() >= 100
    assert lib.en_status_string(0) == b"ok"
    assert b"NULL" in lib.en_status_string(-1)


def test_linear_library_exports_every_declared_symbol():
    from energonai_amd import _lib
    lib = _lib.load_linear()
    header = os.path.join(ROOT, "include", "energon_linear.h")
    text = re.sub(r"/\*.*?\*/", "", open(header).read(), flags=re.S)
    declared = sorted(set(re.findall(r"\b(en_linear[a-z0-9_]*)\s*\(", text)))
    assert sorted(_lib.LINEAR_SIGNATURES) == declared
    for name, (_, argtypes) in _lib.LINEAR_SIGNATURES.items():
        assert hasattr(lib, name)
        m = re.search(r"\b%s\s*\((.*?)\)\s*;" % re.escape(name), text, flags=re.S)
        args = m.group(1).strip()
        assert len(argtypes) == (0 if args in ("", "void") else len(args.split(","))), name
    assert lib.en_linear_status_string(0) == b"ok"
    # argument errors are found before any hipBLASLt or GPU call
    assert lib.en_linear(None, None, None, None, 1, 1, 1, 0, 1, -1, None, 0, None) == -1
    assert lib.en_linear(16, 32, None, 48, 0, 1, 1, 0, 1, -1, None, 0, None) == -1


def test_entry_points_validate_before_launch():
    """NULL pointers and bad extents are refused on the host: no GPU is touched."""
    from energonai_amd import _lib
    lib = _lib.load()
    assert lib.en_prefix_sum(None, 0, 4, None, None, None) == -1
    assert lib.en_prefix_sum(1, 0, 0, 1, None, None) == -2
    assert lib.en_depad(None, None, None, 1, 1, 1, 2, 0, None) == -1
    assert lib.en_depad(16, 32, 48, 1, 1, 1, 3, 0, None) == -3          # element size 3
    assert lib.en_transpose_pad(16, 32, 48, 0, 1, 1, 1, 2, None) == -2   # batch 0
    assert lib.en_scale_mask_softmax(16, 32, None, 1, 1, 1, 1, 1.0, 1, 0, 7, None) == -3   # dtype tag 7
    assert lib.en_scale_mask_softmax(16, 32, None, 1, 1, 1, 1, 1.0, 1, 96, 1, None) == -2  # tile not a power of two
    assert lib.en_layernorm_fwd(16, None, None, None, 32, None, None, 48, 64, 1, 8, 1e-5, 1, 0, None) == -3  # (f16 -> f32)
    assert lib.en_layernorm_fwd(16, None, None, None, 32, None, 80, 48, 64, 1, 8, 1e-5, 1, 1, None) == -1   # offsets, no residual
    assert lib.en_padding_offsets(16, 0, 8, 0, 32, None) == -2           # batch 0
    assert lib.en_attn_qk(16, 32, 48, 64, None, 1, 1, 8, 8, 200, 0, 0, 200, 0, 0, 200, 1.0, 1, 1, None, None, 0,
                          None, None) == -5                              # D > 128
    assert lib.en_attn_qk(16, 32, 48, 64, None, 1, 1, 8, 8, 64, 0, 0, 64, 0, 0, 64, 1.0, 0, 1, None, None, 1,
                          None, None) == -5                              # packed scores are those of a causal mask
    assert lib.en_attn_qk(16, 32, 48, 64, 80, 1, 1, 8, 8, 64, 0, 0, 64, 0, 0, 64, 1.0, 1, 1, None, None, 0,
                          96, None) == -5                                # a tile table is built from the key lengths alone
    assert lib.en_attn_pv(16, 32, 48, 64, None, 1, 1, 8, 8, 64, 0, 0, 64, 0, 0, 64, 1, 1, 1, 80, None, 0,
                          None, None) == -5                              # a packed context has no padding rows to zero
    assert lib.en_attn_tile_table_elems(16, 56, 1024, 0) == 16 * 56 * 8 and lib.en_attn_tile_table_elems(3, 3, 130, 128) == 16 * 2
    assert lib.en_attn_tile_table_elems(16, 56, 1024, 256) == 16 * 56 * 4 and lib.en_attn_tile_table_elems(3, 3, 130, 64) == 0
    assert lib.en_attn_tile_table(None, 1, 1, 8, 0, 0, 16, None) == -1
    assert lib.en_attn_tile_table(16, 0, 1, 8, 1, 128, 32, None) == -2
    assert lib.en_attn_tile_table(16, 1, 1, 8, 1, 64, 32, None) == -5            # tiles of 128 or 256 rows
    assert lib.en_packed_scores_elems(2, 3, 16, 1) == 2 * 3 * 16 * 64 and lib.en_packed_scores_elems(1, 1, 130, 1) == 64 * (64 * 3 + 2 * 3) and lib.en_packed_scores_elems(0, 3, 16, 1) == 0
    assert lib.en_scale_mask_softmax_packed(16, 32, 1, 1, 4096, 1.0, 1, None) == -5     # rows of more than 256 vectors
    assert lib.en_copy_bytes(16, 32, 24, None) == -2                     # not a multiple of 16
    # entry points added beside the reference's own surface
    i64x3 = (ctypes.c_int64 * 3)(0, 64, 768)
    assert lib.en_repad(None, 32, 48, 1, 1, 1, 2, 0, None) == -1
    assert lib.en_repad(16, 32, 48, 1, 0, 1, 2, 0, None) == -2           # max_seq_len 0
    assert lib.en_transpose_pad_heads(16, 32, 48, 1, 1, 4, 8, 6, 4, 1, 2, None) == -2   # heads 4..7 of a 6-row source
    assert lib.en_kv_append(16, 32, 48, 64, None, 1, 1, 1, 8, 8, 8, 8, 8, 8, 2, None, None) == -1
    assert lib.en_kv_append(16, 32, 48, 64, 80, 1, 1, 1, 8, 8, 8, 8, 8, 8, 3, None, None) == -3   # element size 3
    assert lib.en_decode_attn(16, 32, None, 64, 80, 1, 1, 8, 64, i64x3, i64x3, 1.0, 1, None, 0, None) == -1    # no V cache
    assert lib.en_decode_attn(16, 32, 48, 64, 80, 1, 1, 8, 64, i64x3, i64x3, 0.0, 1, None, 0, None) == -5      # scale must be positive
    assert lib.en_decode_attn(16, 32, 48, 64, 80, 1, 1, 8, 60, i64x3, i64x3, 1.0, 1, None, 0, None) == -5      # D not a multiple of 8
    assert lib.en_decode_attn(16, 32, 48, 64, 80, 1, 1, 2 ** 24, 64, i64x3, i64x3, 1.0, 1, None, 0, None) == -5   # 32-bit offsets inside a unit
    # paged caches: q, k_pool, v_pool, ctx, lens, table, batch, heads, max_pages, page, num_pages, D, ...
    assert lib.en_decode_attn_paged(16, 32, 48, 64, 80, None, 1, 1, 4, 64, 8, 64, i64x3, i64x3, 1.0, 1, None, 0, None) == -1   # no table
    assert lib.en_decode_attn_paged(16, 32, 48, 64, 80, 96, 1, 1, 4, 48, 8, 64, i64x3, i64x3, 1.0, 1, None, 0, None) == -5    # page not a power of two
    assert lib.en_decode_attn_paged(16, 32, 48, 64, 80, 96, 1, 1, 4, 8, 8, 64, i64x3, i64x3, 1.0, 1, None, 0, None) == -5     # page below 16
    assert lib.en_decode_attn_paged(16, 32, 48, 64, 80, 96, 1, 1, 0, 64, 8, 64, i64x3, i64x3, 1.0, 1, None, 0, None) == -2    # no pages per sequence
    assert lib.en_decode_attn_paged(16, 32, 48, 64, 80, 96, 1, 1, 4, 64, 8, 64, i64x3, i64x3, -1.0, 1, None, 0, None) == -5   # scale must be positive
    assert lib.en_kv_append_paged(16, 32, 48, 64, 80, None, 1, 1, 4, 64, 8, 64, 64, 64, i64x3, 2, None, None) == -1            # no table
    assert lib.en_kv_append_paged(16, 32, 48, 64, 80, 96, 1, 1, 4, 24, 8, 64, 64, 64, i64x3, 2, None, None) == -5              # page not a power of two
    assert lib.en_kv_append_paged(16, 32, 48, 64, 80, 96, 1, 1, 4, 64, 8, 60, 64, 64, i64x3, 2, None, None) == -4              # rows of 120 bytes
    assert lib.en_kv_fill_paged(16, 32, 48, None, 1, 8, 1, 64, 3, 0, 4, 64, 8, i64x3, 2, None, None) == -1                     # no table
    assert lib.en_kv_fill_paged(16, 32, 48, 64, 1, 8, 4, 64, 6, 4, 4, 64, 8, i64x3, 2, None, None) == -2                       # heads 4..7 of a 6-row source
    assert lib.en_kv_fill_paged(16, 32, 48, 64, 1, 8, 1, 64, 3, 0, 4, 64, 8, i64x3, 3, None, None) == -3                       # element size 3
    assert lib.en_decode_attn_workspace_bytes(64, 72, 2048, 128) == 0          # 4608 units fill the chip
    assert lib.en_decode_attn_workspace_bytes(1, 72, 2048, 128) == 72 * 4 * 130 * 4   # 72 units: four shares of 512 keys each
    assert lib.en_decode_attn_workspace_bytes(4, 72, 300, 128) == 0            # short caches are not shared
    assert lib.en_attn_fused(16, 32, 48, 64, 80, None, 1, 1, 8, 8, 128, i64x3, i64x3, i64x3, i64x3, None, None, 1.0, 1, 0,
                             None, 0, None) == -5                        # fp32: heads of up to 64 channels
    assert lib.en_attn_fused(16, 32, 48, 64, 80, None, 1, 1, 8, 8, 64, i64x3, i64x3, i64x3, i64x3, None, None, 1.0, 1, 0,
                             96, 0, None) == -5                          # fp32: 64-row tiles, no table of 128-row ones
    assert lib.en_attn_fused(16, 32, 48, 64, 80, None, 1, 1, 8, 8, 64, i64x3, i64x3, i64x3, i64x3, None, None, 1.0, 1, 3,
                             None, 0, None) == -3                        # no such dtype
    assert lib.en_attn_fused_query_tile(128, 128, 64, 0, 0) == 64
    assert lib.en_attn_fused(16, 32, 48, 64, 80, None, 1, 1, 8, 8, 64, i64x3, i64x3, i64x3, i64x3, None, None, 0.0, 1, 1,
                             None, 0, None) == -5                        # scale must be positive
    assert lib.en_attn_fused(16, 32, 48, 64, 80, None, 1, 1, 8, 8, 64, i64x3, i64x3, i64x3, i64x3, None, None, 1.0, 1, 1,
                             None, 256, None) == -5                      # 64 queries per wave: heads of 65..128 channels
    assert lib.en_attn_fused(16, 32, 48, 64, 80, None, 1, 1, 8, 8, 128, i64x3, i64x3, i64x3, i64x3, None, None, 1.0, 1, 1,
                             None, 64, None) == -5                       # no such tile
    assert lib.en_attn_fused_query_tile(1024, 1024, 128, 1, 1) in (128, 256)
    assert lib.en_attn_fused(16, 32, 48, 64, 80, None, 1, 1, 8, 8, 200, i64x3, i64x3, i64x3, i64x3, None, None, 1.0, 1, 1,
                             None, 0, None) == -5                        # head size above 128
    assert lib.en_padding_removal_layer(16, 32, None, 48, 64, 80, 96, 112, 128, 144, 160, 176, 192, 1, 8, 2, 8, 16, 4,
                                        1.0, 1e-5, 1, 0, 5, None, 1, None, None) == -5   # unknown attention form
    assert lib.en_padding_removal_layer(16, 32, None, 48, 64, 80, 96, 112, 128, 144, 160, 176, 192, 1, 8, 2, 8, 32, 4,
                                        1.0, 1e-5, 1, 0, 0, None, 1, None, None) == -2   # LayerNorm width 32 != 2 heads x 8, no dense_out
    assert lib.en_padding_removal_layer(16, 32, None, 48, 64, 80, None, 112, 128, 144, 160, 176, 192, 1, 8, 2, 8, 16, 4,
                                        1.0, 1e-5, 1, 0, 0, None, 1, None, None) == -1   # unfused form without the padded buffer
    # the entry point that allocates nothing sizes its pieces without wrapping: absurd extents whose products
    # overflow 64-bit arithmetic are refused before anything is launched (arguments: ..., y, seq_lens, i64, B, S, H,
    # D, hidden, T, scale, eps, causal, left, form, fold, dtype, stream)
    for form in (0, 1, 2, 3, 4):
        for fold in (0, 1):
            assert lib.en_padding_removal_layer_noalloc(16, 32, None, 48, 64, 80, 96, 0, 65536, 2 ** 31 - 1, 2 ** 31 - 1,
                                                        2 ** 31 - 1, 2 ** 62, 65536 * (2 ** 31 - 1), 1.0, 1e-5, 1, 0,
                                                        form, fold, 1, None) == -7
    assert lib.en_padding_removal_layer_noalloc(16, 32, None, 48, 64, 80, 96, 0, 4, 2 ** 20, 2 ** 20, 2 ** 20, 2 ** 40,
                                                4, 1.0, 1e-5, 1, 0, 0, 0, 1, None) == -7


def test_python_api_keeps_reference_names_and_signatures():
    from energonai_amd import kernel
    from energonai_amd.kernel import cuda_native
    want = {   # energonai/kernel/cuda_native/transpose_pad.py:12-87, scale_mask_softmax.py:10
        "transpose_pad": ["src", "batch_size", "max_seq_len", "seq_len_list", "head_num", "size_per_head"],
        "transpose_depad": ["src", "batch_size", "sum_seq", "max_seq_len", "seq_len_list", "head_num",
                            "size_per_head"],
        "depad": ["src", "batch_size", "seq_lens"],
        "scale_mask_softmax": ["batch_size", "batch_seq_len", "head_num", "src", "seq_len_list"],
        "ft_build_padding_offsets": ["seq_lens", "batch_size", "max_seq_len", "valid_word_num", "tmp_mask_offset"],
        "ft_remove_padding": ["src", "tmp_mask_offset", "mask_offset", "valid_word_num", "hidden_dim"],
        "ft_rebuild_padding": ["src", "mask_offset", "valid_word_num", "hidden_dim", "batch_size", "max_seq_len"],
        "ft_transpose_rebuild_padding": ["Q", "K", "V", "q_buf", "k_buf", "v_buf", "batch_size", "seq_len",
                                         "head_num", "size_per_head", "valid_word_num", "mask_offset"],
        "ft_transpose_remove_padding": ["src", "valid_word_num", "batch_size", "seq_len", "head_num",
                                        "size_per_head", "mask_offset"],
    }
    for name, params in want.items():
        fn = getattr(kernel, name)
        got = [p.name for p in inspect.signature(fn).parameters.values()
               if p.kind is p.POSITIONAL_OR_KEYWORD and p.default is p.empty]
        assert got == params, (name, got)
    for name in ("linear", "find_algo"):
        assert callable(getattr(kernel, name))
    assert cuda_native.LayerNorm is cuda_native.MixedFusedLayerNorm
    sig = inspect.signature(cuda_native.LayerNorm.__init__)
    assert list(sig.parameters)[1:] == ["normalized_shape", "eps", "device", "dtype"]


def test_extension_name_shims_register_under_reference_names():
    from energonai_amd import ext
    ext.install()
    import importlib
    tp = importlib.import_module("energonai_transpose_pad")
    for sym in ("transpose_pad_wrapper", "transpose_depad_wrapper", "ft_build_padding_offsets_wrapper",
                "ft_remove_padding_wrapper", "ft_rebuild_padding_wrapper", "ft_transpose_remove_padding_wrapper",
                "ft_transpose_rebuild_padding_wrapper"):
        assert callable(getattr(tp, sym))    # csrc/transpose_pad_fusion_wrapper.cpp:246-263
    assert callable(importlib.import_module("energonai_scale_mask").scale_mask_softmax_wrapper)
    assert callable(importlib.import_module("energonai_layer_norm").forward_affine)
    assert callable(importlib.import_module("energonai_linear_func").mlp_gemm)


def test_host_side_argument_errors_without_gpu():
    from energonai_amd import kernel
    lens = torch.tensor([1, 2], dtype=torch.int32)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        kernel.transpose_pad(torch.zeros(1, 3, 2, 4), 2, 4, lens, 2, 4)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        kernel.scale_mask_softmax(2, 4, 1, torch.zeros(2, 1, 4, 4), lens)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        kernel.layer_norm_forward(torch.zeros(2, 8), torch.ones(8), torch.zeros(8), (8,))
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        kernel.depad(torch.zeros(2, 4, 8), 2, lens)


def test_public_attention_calls_pass_the_tile_table_when_there_are_no_query_lengths():
    """attn_qk / attn_pv / attn_fused get the raw pointer of the query lengths as 0 when the caller gives none; the
    workgroup order of the batch must then be handed to the kernels (it once was not: 0 is not None)."""
    from energonai_amd.kernel import attention

    class Table:
        def data_ptr(self):
            return 4096

    class Info:
        def __init__(self):
            self.asked = []

        def tile_table_ptr(self, head_num, q_seq_len, unit_kv_bytes, query_tile=128):
            self.asked.append((head_num, q_seq_len, unit_kv_bytes))
            return Table().data_ptr()

    info = Info()
    assert attention._tile_table_ptr(info, 0, 12, 512, 1 << 17) == 4096 and info.asked == [(12, 512, 1 << 17)]
    assert attention._tile_table_ptr(info, None, 12, 512, 1 << 17) == 4096
    assert attention._tile_table_ptr(info, 0x7f0000001000, 12, 512, 1 << 17) is None and len(info.asked) == 2


def test_missing_library_fails_loudly(tmp_path, monkeypatch):
    """No CPU fallback: without the shared object the product refuses to load."""
    from energonai_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libenergon_hip.so"))
    with pytest.raises(RuntimeError, match="requires cuda extensions"):
        _lib.load()


def test_library_built_from_other_sources_is_refused(monkeypatch):
    """The libraries carry a digest of their sources; one that differs from the sources in the tree (an edited
    kernel without a rebuild) is refused at load instead of being tested in place of the code beside it."""
    from energonai_amd import _lib, build
    lib = _lib.load()
    assert lib.en_source_hash().decode() == build.source_hash()
    assert _lib.load_linear().en_linear_source_hash().decode() == build.linear_source_hash()
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(build, "source_hash", lambda: "0" * 32)
    with pytest.raises(RuntimeError, match="built from other sources"):
        _lib.load()
    monkeypatch.setattr(_lib, "_linear_lib", None)
    monkeypatch.setattr(build, "linear_source_hash", lambda: "0" * 32)
    with pytest.raises(RuntimeError, match="built from other sources"):
        _lib.load_linear()


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "energonai_amd")
    for base, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(base, f)).read()
                assert not re.search(r"^\s*(from|import)\s+oracle\b", text, flags=re.M), f


def test_workload_definitions():
    from energonai_amd import workloads as wl
    totals = {"c1": 698, "c2": 8538, "c3": 9244, "c4": 20142, "c5": 70929}
    for w in wl.WORKLOADS:
        lens = wl.make_lens(w)
        assert lens.dtype == torch.int32 and lens.numel() == w.batch
        assert int(lens.sum()) == totals[w.name]
        assert int(lens.min()) >= w.len_lo and int(lens.max()) <= w.len_hi
    w = wl.BY_NAME["c1"]
    inp = wl.make_inputs(w)
    assert inp["hidden_padded"].shape == (8, 128, 768) and inp["qkv_packed"].shape == (1, 698, 12, 192)
    for b, n in enumerate(inp["lens_list"]):
        assert bool((inp["hidden_padded"][b, n:] == 0).all())        # right padded, zero padding
    w2 = wl.BY_NAME["c2"]
    small = wl.make_inputs(w2, lens=torch.tensor([3, 5], dtype=torch.int32)) if False else None
    alg = wl.algorithmic_bytes(w, inp["lens_list"])
    assert alg["depad"] == 2 * 698 * 768 * 4
    assert alg["transpose_pad"] == 698 * 12 * 192 * 4 + 8 * 128 * 12 * 192 * 4
    assert alg["layernorm_residual"] == 3 * 698 * 768 * 4
    vis = sum(n * n for n in inp["lens_list"])
    assert wl.algorithmic_flops(w, inp["lens_list"]) == 2.0 * 12 * 64 * vis


def test_paged_cache_bookkeeping_on_the_host():
    """Which pages a sequence holds is decided on the host: pages are taken at prefill and at page boundaries,
    handed back on release, and an exhausted pool or a full table row raises before any kernel runs."""
    import torch
    from energonai_amd.model.kv_cache import PagedKVCache
    c = PagedKVCache(3, 2, 64, 16, torch.float16, "cpu", page_size=16, pool_pages=7)
    assert c.max_pages == 4 and c.max_seq_len == 64 and c.pages_in_use() == 0
    c._assign([(0, 2), (1, 1), (2, 3)])
    assert c.pages_in_use() == 6
    t = c.table.tolist()
    held = [p for row in t for p in row if p >= 0]
    assert len(held) == 6 and len(set(held)) == 6 and all(0 <= p < 7 for p in held)
    assert [sum(p >= 0 for p in row) for row in t] == [2, 1, 3]
    assert t[0][2] == -1 and t[1][1] == -1
    c._assign([(1, 2)])
    assert c.pages_in_use() == 7
    with pytest.raises(RuntimeError, match="used up"):
        c._assign([(0, 3)])
    c.release(2)
    assert c.pages_in_use() == 4 and c.table[2].tolist() == [-1] * 4
    c._assign([(0, 4)])
    with pytest.raises(RuntimeError, match="max_seq_len"):
        c._assign([(0, 5)])
    with pytest.raises(ValueError):
        PagedKVCache(1, 1, 64, 16, torch.float16, "cpu", page_size=24)
