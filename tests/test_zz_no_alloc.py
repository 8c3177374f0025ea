"""The entry point that allocates nothing: en_padding_removal_layer_noalloc against en_padding_removal_layer.

Both run the same kernels; the first keeps every intermediate in the library's static device array.  Outputs
are compared bit for bit on two calls in a row, the second with a smaller batch (so the array still holds the
larger call's contents), and a step that does not fit the array must be refused before anything runs.
"""
import pytest
import torch

from gpu_util import announce

pytestmark = pytest.mark.gpu

# (workload the shape is cut from, dtype, form, fold_depad, lens of the first call, lens of the second)
CASES = [
    ("c2", torch.float16, "packed", True, [512, 64, 301, 97, 200, 511], [130, 33]),
    ("c2", torch.float16, "varlen_packed", True, [512, 64, 301, 97, 200, 511], [130, 33]),
    ("c2", torch.bfloat16, "varlen", False, [256, 64, 201], [97, 5]),
    ("c1", torch.float32, "varlen", True, [128, 16, 77, 100], [25, 119]),
    ("c2", torch.float16, False, False, [256, 64, 201], [97, 5]),
    ("c2", torch.bfloat16, True, False, [300, 17, 128], [64]),
    ("c1", torch.float32, False, False, [128, 16, 77, 100], [25, 119]),
    ("c1", torch.float32, False, True, [128, 16, 77, 100], [25, 119]),
]


def _inputs(name, dtype, lens):
    from energonai_amd import workloads
    w = workloads.BY_NAME[name]
    S = max(128, -(-max(lens) // 128) * 128) if name == "c2" else w.seq
    w = workloads.Workload(w.index, name, w.title, dtype, len(lens), S, w.heads, w.head_dim, w.hidden, 1, S, w.causal,
                           w.left_padded)
    d = workloads.make_inputs(w, device="cuda", lens=torch.tensor(lens, dtype=torch.int32))
    return w, d


@pytest.mark.parametrize("name,dtype,form,fold,lens_a,lens_b", CASES)
def test_noalloc_layer_matches_the_allocating_entry_point(name, dtype, form, fold, lens_a, lens_b):
    from energonai_amd import layer, workloads
    announce("noalloc layer", name, dtype, form, fold, lens_a, lens_b)
    for lens in (lens_a, lens_b):          # the second call is smaller and finds the first one's leftovers
        w, d = _inputs(name, dtype, lens)
        T = d["total"]
        lens_dev = d["lens"].cuda()
        want = layer.padding_removal_layer(d["hidden_padded"], d["qkv_packed"], lens_dev, w.heads, w.head_dim,
                                           d["gamma"], d["beta"], workloads.EPS, w.scale, w.causal, w.left_padded,
                                           dense_out=d["dense_out"], sum_seq=T, fused_attention=form, fold_depad=fold)
        out = torch.full((1, T, w.hidden), float("nan"), dtype=dtype, device="cuda")
        torch.cuda.synchronize()
        before = torch.cuda.memory_stats()["allocation.all.allocated"]     # allocations made so far, cumulative
        got = layer.padding_removal_layer_noalloc(d["hidden_padded"], d["qkv_packed"], lens_dev, w.heads, w.head_dim,
                                                  d["gamma"], d["beta"], out, T, workloads.EPS, w.scale, w.causal,
                                                  w.left_padded, dense_out=d["dense_out"], fused_attention=form,
                                                  fold_depad=fold)
        assert torch.cuda.memory_stats()["allocation.all.allocated"] == before   # torch's allocator was not asked either
        torch.cuda.synchronize()
        assert got.data_ptr() == out.data_ptr()
        assert torch.equal(got, want), float((got.float() - want.float()).abs().max())
        # int64 lengths, as the reference's own test passes them
        out2 = torch.empty_like(out)
        layer.padding_removal_layer_noalloc(d["hidden_padded"], d["qkv_packed"], lens_dev.long(), w.heads, w.head_dim,
                                            d["gamma"], d["beta"], out2, T, workloads.EPS, w.scale, w.causal,
                                            w.left_padded, dense_out=d["dense_out"], fused_attention=form,
                                            fold_depad=fold)
        assert torch.equal(out2, want)


def test_noalloc_layer_refuses_what_does_not_fit():
    """The c2 batch with the three separate attention ops needs a 201 MB score tensor: more than the array."""
    from energonai_amd import _lib, layer, workloads
    announce("noalloc layer too large")
    w = workloads.BY_NAME["c2"]
    d = workloads.make_inputs(w, device="cuda")
    T = d["total"]
    out = torch.zeros((1, T, w.hidden), dtype=w.dtype, device="cuda")
    with pytest.raises(RuntimeError, match="static scratch"):
        layer.padding_removal_layer_noalloc(d["hidden_padded"], d["qkv_packed"], d["lens"].cuda(), w.heads, w.head_dim,
                                            d["gamma"], d["beta"], out, T, workloads.EPS, w.scale, w.causal,
                                            w.left_padded, fused_attention=False)
    torch.cuda.synchronize()
    assert not out.any()                   # nothing was launched
    # the same batch fits when the scores never exist and no padded tensor is built
    want = layer.padding_removal_layer(d["hidden_padded"], d["qkv_packed"], d["lens"].cuda(), w.heads, w.head_dim,
                                       d["gamma"], d["beta"], workloads.EPS, w.scale, w.causal, w.left_padded,
                                       sum_seq=T, fused_attention="packed", fold_depad=True)
    got = layer.padding_removal_layer_noalloc(d["hidden_padded"], d["qkv_packed"], d["lens"].cuda(), w.heads,
                                              w.head_dim, d["gamma"], d["beta"], out, T, workloads.EPS, w.scale,
                                              w.causal, w.left_padded, fused_attention="packed", fold_depad=True)
    assert torch.equal(got, want)
    assert _lib.load().en_status_string(-7).decode().startswith("the call needs more")
