"""GPU parity: depad / transpose_pad / transpose_depad / ft_* against the oracle, bit-exact.

Every call goes through the Python mirror of the reference API and from there
through the C ABI of libenergon_hip.so.
"""
import pytest
import torch

from gpu_util import announce, packed_randn, ragged_lens
from oracle import eager

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.float16, torch.bfloat16]


def _kernel():
    from energonai_amd import kernel
    return kernel


CASES = [
    # B, S, H, D, lens (None -> seeded ragged)
    (8, 128, 12, 64, [24, 127, 31, 65, 24, 127, 31, 65]),   # the reference test's shape
    (2, 3, 2, 2, [3, 1]),                                    # tiny, 4-byte rows
    (3, 7, 5, 3, [7, 0, 2]),                                 # odd sizes, an empty sequence
    (4, 33, 3, 40, [1, 33, 17, 32]),                         # full-length sequence, 80/160-byte rows
    (5, 64, 4, 192, None),                                   # fused QKV width
    (1, 1, 1, 8, [1]),                                       # minimum
    (6, 257, 2, 128, None),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("B,S,H,D,lens", CASES)
def test_transpose_pad_depad(dtype, B, S, H, D, lens):
    k = _kernel()
    lens_t = ragged_lens(B, 0, S, 77 + B + S) if lens is None else torch.tensor(lens, dtype=torch.int32)
    lens_l = [int(v) for v in lens_t]
    T = sum(lens_l)
    announce("transpose_pad/depad", dtype, B, S, H, D, lens_l)
    src = packed_randn(max(T, 1), H * D, dtype, 5)[:T].reshape(1, T, H, D)
    ref_pad = eager.transpose_pad(src, B, S, lens_l, H, D)
    for lens_dtype in (torch.int32, torch.int64):
        got = k.transpose_pad(src.cuda(), B, S, lens_t.to(lens_dtype).cuda(), H, D)
        assert got.shape == (B, H, S, D) and got.dtype == dtype
        assert torch.equal(got.cpu(), ref_pad), f"transpose_pad mismatch (lens {lens_dtype})"
    # valid rows only: same bits on every row below a length (the padding rows are left unwritten)
    got = k.transpose_pad(src.cuda(), B, S, lens_t.cuda(), H, D, zero_padding=False).cpu()
    for b, n in enumerate(lens_l):
        assert torch.equal(got[b, :, :n], ref_pad[b, :, :n])
    # inverse
    ref_depad = eager.transpose_depad(ref_pad, B, T, S, lens_l, H, D)
    assert torch.equal(ref_depad, src)
    got = k.transpose_depad(ref_pad.cuda(), B, T, S, lens_t.cuda(), H, D)
    assert got.shape == (1, T, H, D)
    assert torch.equal(got.cpu(), src)
    # sum_seq as a 0-d tensor, as the reference caller passes it (examples/bert/bert.py:122-123)
    got = k.transpose_depad(ref_pad.cuda(), B, torch.sum(lens_t.cuda()), S, lens_t.cuda(), H, D)
    assert torch.equal(got.cpu(), src)


def test_transpose_pad_fused_qkv_chunks(ref_test_shape):
    """Dk = 3D: chunks of the fused result equal three separate transpose_pads."""
    k = _kernel()
    B, S, H, D, lens = (ref_test_shape[x] for x in ("batch", "seq", "heads", "head_dim", "lens"))
    T = sum(lens)
    announce("transpose_pad fused", B, S, H, D)
    src = packed_randn(T, H * 3 * D, torch.float16, 9).reshape(1, T, H, 3 * D)
    lens_t = torch.tensor(lens, dtype=torch.int32).cuda()
    fused = k.transpose_pad(src.cuda(), B, S, lens_t, H, 3 * D)
    parts = torch.chunk(src, 3, dim=-1)
    for got, part in zip(torch.chunk(fused, 3, dim=-1), parts):
        want = k.transpose_pad(part.contiguous().cuda(), B, S, lens_t, H, D)
        assert torch.equal(got, want)
        assert torch.equal(want.cpu(), eager.transpose_pad(part.contiguous(), B, S, lens, H, D))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("left", [False, True])
@pytest.mark.parametrize("B,S,hid,lens", [
    (8, 128, 768, [24, 127, 31, 65, 24, 127, 31, 65]),
    (3, 5, 6, [5, 0, 1]),
    (2, 9, 7, [4, 9]),            # 14/28-byte rows: scalar vector path
    (4, 40, 12288, None),         # a row wider than one tile
])
def test_depad(dtype, left, B, S, hid, lens):
    k = _kernel()
    lens_t = ragged_lens(B, 0, S, 31 + S) if lens is None else torch.tensor(lens, dtype=torch.int32)
    lens_l = [int(v) for v in lens_t]
    announce("depad", dtype, left, B, S, hid, lens_l)
    g = torch.Generator().manual_seed(3)
    src = torch.randn(B, S, hid, generator=g).to(dtype)
    want = eager.depad(src, B, lens_l, left_padded=left)
    got = k.depad(src.cuda(), B, lens_t.cuda(), left_padded=left)
    assert got.shape == want.shape
    assert torch.equal(got.cpu(), want)
    # host-known lengths: no device round trip for the total
    got = k.depad(src.cuda(), B, lens_l, left_padded=left)
    assert torch.equal(got.cpu(), want)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("B,S,H,D,lens", [
    (8, 128, 12, 64, [24, 127, 31, 65, 24, 127, 31, 65]),   # tests/test_kernel/test_ft_transpose_pad.py:6-11
    (3, 6, 2, 4, [6, 0, 3]),
    (4, 50, 56, 128, None),                                  # hidden 7168: above the reference's block-size limit
])
def test_ft_family(dtype, B, S, H, D, lens):
    k = _kernel()
    lens_t = ragged_lens(B, 0, S, 11 + S) if lens is None else torch.tensor(lens, dtype=torch.int32)
    lens_l = [int(v) for v in lens_t]
    hid = H * D
    announce("ft_*", dtype, B, S, H, D, lens_l)
    want_valid, want_off = eager.ft_build_padding_offsets(lens_l, B, S)
    T = int(want_valid[0])

    tmp_off = torch.full((B, S), -7, dtype=torch.int32).cuda()
    mask_off = torch.full((B, S), -9, dtype=torch.int32).cuda()
    valid = torch.zeros(1, dtype=torch.int32).cuda()
    k.ft_build_padding_offsets(lens_t.cuda(), B, S, valid, tmp_off)
    assert int(valid[0].item()) == T
    assert torch.equal(tmp_off.flatten()[:T].cpu(), want_off)
    assert bool((tmp_off.flatten()[T:] == -7).all()), "entries past the valid count must not be written"

    g = torch.Generator().manual_seed(17)
    hq, hk, hv = (torch.rand(B, S, hid, generator=g).to(dtype) for _ in range(3))
    q = k.ft_remove_padding(hq.cuda(), tmp_off, mask_off, valid[0].item(), hid)
    want_q, want_mask = eager.ft_remove_padding(hq, want_off, T, hid)
    assert torch.equal(q.cpu(), want_q)
    assert torch.equal(mask_off.flatten()[:T].cpu(), want_mask)
    kk = k.ft_remove_padding(hk.cuda(), tmp_off, mask_off, T, hid)
    v = k.ft_remove_padding(hv.cuda(), tmp_off, mask_off, T, hid)
    assert torch.equal(q.cpu(), eager.depad(hq, B, lens_l))

    qv, kv, vv = (t.view(T, H, D) for t in (q, kk, v))
    bufs = [torch.full((B, H, S, D), 3.0, dtype=dtype).cuda() for _ in range(3)]
    k.ft_transpose_rebuild_padding(qv, kv, vv, bufs[0], bufs[1], bufs[2], B, S, H, D, T, mask_off)
    want_bufs = [torch.full((B, H, S, D), 3.0, dtype=dtype) for _ in range(3)]
    eager.ft_transpose_rebuild_padding(qv.cpu(), kv.cpu(), vv.cpu(), *want_bufs, B, S, H, D, T, want_mask)
    for got, want in zip(bufs, want_bufs):
        assert torch.equal(got.cpu(), want)   # padding rows keep the caller's 3.0

    back = k.ft_transpose_remove_padding(bufs[2], T, B, S, H, D, mask_off)
    assert back.shape == (1, T, hid)
    assert torch.equal(back.cpu(), eager.ft_transpose_remove_padding(want_bufs[2], T, B, S, H, D, want_mask))
    assert torch.equal(back, v)

    rebuilt = k.ft_rebuild_padding(back, mask_off, T, hid, B, S)
    want_rebuilt = eager.ft_rebuild_padding(back.cpu(), want_mask, T, hid, B, S)
    assert rebuilt.shape == (B, S, hid)
    assert torch.equal(rebuilt.cpu(), want_rebuilt)
    # the reference caller passes a slice of the temporary offsets (examples/gpt/gpt.py:321-323)
    rebuilt2 = k.ft_rebuild_padding(back, tmp_off.flatten()[0:T], T, hid, B, S)
    assert torch.equal(rebuilt2, rebuilt)


def test_outputs_fully_written():
    """Outputs come from torch.empty: poison the allocator's cache and check nothing leaks through."""
    k = _kernel()
    B, S, H, D = 4, 96, 6, 64
    lens = [10, 96, 0, 50]
    T = sum(lens)
    announce("fully written", B, S, H, D)
    lens_t = torch.tensor(lens, dtype=torch.int32).cuda()
    src = packed_randn(T, H * D, torch.float16, 21).reshape(1, T, H, D).cuda()
    for _ in range(3):
        poison = torch.full((B, H, S, D), float("nan"), dtype=torch.float16, device="cuda")
        del poison
        out = k.transpose_pad(src, B, S, lens_t, H, D)
        assert not torch.isnan(out).any()
        del out


def test_argument_errors():
    k = _kernel()
    announce("argument errors")
    lens = torch.tensor([1, 2], dtype=torch.int32)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        k.transpose_pad(torch.zeros(1, 3, 2, 4), 2, 4, lens, 2, 4)
    with pytest.raises(RuntimeError, match="Datatype not implemented"):
        k.transpose_pad(torch.zeros(1, 3, 2, 4, dtype=torch.float64).cuda(), 2, 4, lens.cuda(), 2, 4)
    with pytest.raises(RuntimeError, match="int32"):
        k.ft_build_padding_offsets(lens.cuda(), 2, 4, torch.zeros(1, dtype=torch.int64).cuda(),
                                   torch.zeros(8, dtype=torch.int32).cuda())
