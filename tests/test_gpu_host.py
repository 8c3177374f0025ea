"""GPU tests of the host side of the boundary: the stand-ins for the reference's compiled extension modules
called exactly as the reference's Python wrappers call them, and the per-batch offset cache under the
conditions of the reference worker (inference mode, lengths given as lists, more than one stream)."""
import pytest
import torch

from gpu_util import announce, max_abs, packed_randn
from oracle import eager

pytestmark = pytest.mark.gpu


def _ref_shape(ref_test_shape):
    r = ref_test_shape
    return r["batch"], r["seq"], r["heads"], r["head_dim"], r["lens"]


@pytest.mark.parametrize("lens_dtype", [torch.int64, torch.int32])
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_transpose_pad_extension_stand_in(ref_test_shape, dtype, lens_dtype):
    """energonai_transpose_pad.*_wrapper with the argument pattern of
    energonai/kernel/cuda_native/transpose_pad.py:12-87 (contiguous inputs, positional arguments, 0-d tensor
    totals) on the shape of the reference's own kernel test."""
    import energonai_amd.ext.energonai_transpose_pad as ext
    B, S, H, D, lens = _ref_shape(ref_test_shape)
    T = sum(lens)
    announce("ext transpose_pad", dtype, lens_dtype)
    seq_len_list = torch.tensor(lens, dtype=lens_dtype).cuda()
    src = packed_randn(T, H * D, dtype, 3).reshape(1, T, H, D)
    # transpose_pad / transpose_depad
    dst = ext.transpose_pad_wrapper(src.cuda().contiguous(), B, S, seq_len_list, H, D)
    want = eager.transpose_pad(src, B, S, lens, H, D)
    assert dst.shape == (B, H, S, D) and torch.equal(dst.cpu(), want)
    back = ext.transpose_depad_wrapper(dst.contiguous(), B, T, S, seq_len_list, H, D)
    assert back.shape == (1, T, H, D) and torch.equal(back.cpu(), src)
    # the FasterTransformer family: build offsets -> remove -> rebuild; transpose_rebuild -> transpose_remove
    lens32 = torch.tensor(lens, dtype=torch.int32).cuda()
    valid_word_num = torch.zeros(1, dtype=torch.int32, device="cuda")
    tmp_mask_offset = torch.zeros(B * S, dtype=torch.int32, device="cuda")
    mask_offset = torch.zeros(B * S, dtype=torch.int32, device="cuda")
    ext.ft_build_padding_offsets_wrapper(lens32.contiguous(), B, S, valid_word_num, tmp_mask_offset)
    want_valid, want_off = eager.ft_build_padding_offsets(lens, B, S)
    assert int(valid_word_num[0].item()) == int(want_valid[0]) == T
    assert torch.equal(tmp_mask_offset[:T].cpu(), want_off[:T].to(torch.int32))
    hid = H * D
    padded = torch.zeros(B, S, hid, dtype=dtype)
    flat = src.reshape(T, hid)
    t = 0
    for b, n in enumerate(lens):
        padded[b, :n] = flat[t:t + n]
        t += n
    removed = ext.ft_remove_padding_wrapper(padded.cuda().contiguous(), tmp_mask_offset, mask_offset,
                                            valid_word_num[0].item(), hid)
    assert removed.shape == (1, T, hid) and torch.equal(removed.cpu().reshape(T, hid), flat)
    assert torch.equal(mask_offset[:T], tmp_mask_offset[:T])
    rebuilt = ext.ft_rebuild_padding_wrapper(removed.contiguous(), mask_offset, T, hid, B, S)
    assert torch.equal(rebuilt.cpu(), padded)
    q_buf = torch.zeros(B, H, S, D, dtype=dtype, device="cuda")
    k_buf, v_buf = torch.zeros_like(q_buf), torch.zeros_like(q_buf)
    Q = src.reshape(T, H, D).cuda().contiguous()
    ext.ft_transpose_rebuild_padding_wrapper(Q, (2 * Q).contiguous(), (3 * Q).contiguous(), q_buf, k_buf, v_buf, B, S,
                                             H, D, T, mask_offset)
    assert torch.equal(q_buf.cpu(), want) and torch.equal(k_buf.cpu(), 2 * want) and torch.equal(v_buf.cpu(), 3 * want)
    flat_back = ext.ft_transpose_remove_padding_wrapper(q_buf.contiguous(), T, B, S, H, D, mask_offset)
    assert flat_back.shape == (1, T, hid) and torch.equal(flat_back.cpu().reshape(T, hid), flat)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_scale_mask_extension_stand_in(ref_test_shape, dtype):
    """energonai_scale_mask.scale_mask_softmax_wrapper(batch, seq, heads, correlation, real_seq_len) as in
    energonai/kernel/cuda_native/scale_mask_softmax.py:10-13: in place, its input returned."""
    import energonai_amd.ext.energonai_scale_mask as ext
    B, S, H, _, lens = _ref_shape(ref_test_shape)
    announce("ext scale_mask", dtype)
    g = torch.Generator().manual_seed(4)
    src = (2.0 * torch.randn(B, H, S, S, generator=g)).to(dtype)
    x = src.cuda().contiguous()
    dst = ext.scale_mask_softmax_wrapper(B, S, H, x, torch.tensor(lens, dtype=torch.int32).cuda())
    assert dst.data_ptr() == x.data_ptr()
    want = eager.scale_mask_softmax(B, S, H, src.float(), lens, out_dtype=torch.float32)
    got = dst.cpu()
    for b, n in enumerate(lens):
        assert max_abs(got[b, :, :n].float(), want[b, :, :n]) <= (2e-3 if dtype == torch.float16 else 1e-5)
        assert torch.equal(got[b, :, n:], src[b, :, n:])


@pytest.mark.parametrize("in_dtype,out_dtype", [(torch.float32, torch.float32), (torch.float32, torch.float16),
                                                (torch.float16, torch.float16)])
def test_layer_norm_extension_stand_in(in_dtype, out_dtype):
    """energonai_layer_norm.forward_affine(input_, normalized_shape, weight_, bias_, eps) -> [output, mean,
    invvar] as FusedLayerNormAffineFunction.forward unpacks it (energonai/kernel/cuda_native/layer_norm.py:24-28;
    the reference casts the input to fp32 first, so (fp32 in, 16-bit gamma) is its mixed case)."""
    import energonai_amd.ext.energonai_layer_norm as ext
    n1, n2 = 96, 768
    announce("ext layer_norm", in_dtype, out_dtype)
    g = torch.Generator().manual_seed(5)
    x = (1.5 * torch.randn(4, n1 // 4, n2, generator=g) + 0.25).to(in_dtype)
    gamma = (1 + 0.02 * torch.randn(n2, generator=g)).to(out_dtype)
    beta = (0.02 * torch.randn(n2, generator=g)).to(out_dtype)
    output, mean, invvar = ext.forward_affine(x.cuda().contiguous(), torch.Size([n2]), gamma.cuda().contiguous(),
                                              beta.cuda().contiguous(), 1e-5)
    want, want_mean, want_invvar, _ = eager.layer_norm(x, gamma, beta, 1e-5, acc_dtype=torch.float64,
                                                       out_dtype=torch.float64)
    assert output.shape == x.shape and output.dtype == out_dtype
    assert mean.dtype == torch.float32 and mean.shape == (n1,) and invvar.shape == (n1,)
    bound = 1e-5 if out_dtype == torch.float32 else 2e-3 + float(want.abs().max()) * 2.0 ** -11
    assert max_abs(output.cpu(), want) <= bound
    assert max_abs(mean.cpu(), want_mean.reshape(-1)) <= 1e-5
    assert float(((invvar.cpu().double() - want_invvar.reshape(-1).double()).abs() / want_invvar.reshape(-1).double()).max()) <= 1e-5
    with pytest.raises(RuntimeError, match="inference-only"):
        ext.backward_affine()


def test_extension_names_resolve_to_the_stand_ins_after_install():
    import importlib
    import sys
    from energonai_amd import ext
    announce("ext install")
    names = ("energonai_transpose_pad", "energonai_scale_mask", "energonai_layer_norm", "energonai_linear_func")
    saved = {n: sys.modules.pop(n, None) for n in names}
    try:
        ext.install()
        # the lookup the reference wrappers perform (cuda_native/transpose_pad.py:4-7)
        mod = importlib.import_module("energonai_transpose_pad")
        x = torch.arange(2 * 3 * 4, dtype=torch.float32).reshape(1, 2, 3, 4).cuda()
        out = mod.transpose_pad_wrapper(x, 2, 2, torch.tensor([1, 1]).cuda(), 3, 4)
        assert out.shape == (2, 3, 2, 4) and torch.equal(out[:, :, 0].cpu(), x[0].cpu())
    finally:
        for n in names:
            sys.modules.pop(n, None)
            if saved[n] is not None:
                sys.modules[n] = saved[n]


def test_lengths_created_in_inference_mode():
    """The reference worker runs the whole forward under torch.inference_mode() (energonai/worker.py:79); lengths
    made there carry no version counter.  Every wrapper must still work, and an in-place edit of such a tensor
    must be seen by the next call (nothing is cached for it)."""
    from energonai_amd import kernel as K
    B, S, H, D = 3, 16, 2, 8
    announce("inference-mode lens")
    x = torch.randn(B, S, H * D, generator=torch.Generator().manual_seed(6))
    with torch.inference_mode():
        lens = torch.tensor([5, 16, 1]).cuda()
        assert torch.is_inference(lens)
        packed = K.depad(x.cuda(), B, lens)
        assert torch.equal(packed.cpu(), eager.depad(x, B, [5, 16, 1]))
        padded = K.transpose_pad(packed.view(1, -1, H, D), B, S, lens, H, D)
        assert torch.equal(padded.cpu(), eager.transpose_pad(packed.cpu().view(1, -1, H, D), B, S, [5, 16, 1], H, D))
        lens[0] = 7
        packed2 = K.depad(x.cuda(), B, lens)
        assert torch.equal(packed2.cpu(), eager.depad(x, B, [7, 16, 1]))


def test_query_lengths_given_as_a_list():
    """q_len_list as a Python list lives in a device tensor owned by the call alone; the output tensor allocated
    right after must not be handed its memory before the kernel has run."""
    from energonai_amd import kernel as K
    B, H, Sq, Sk, D = 4, 2, 8, 64, 32
    kl, ql = [64, 40, 9, 33], [8, 8, 3, 1]
    announce("q_len_list as list")
    g = torch.Generator().manual_seed(7)
    q = torch.randn(B, H, Sq, D, generator=g).half().cuda()
    k = torch.randn(B, H, Sk, D, generator=g).half().cuda()
    v = torch.randn(B, H, Sk, D, generator=g).half().cuda()
    kl_t, ql_t = torch.tensor(kl, dtype=torch.int32).cuda(), torch.tensor(ql, dtype=torch.int32).cuda()
    for _ in range(3):      # repeated so that freed blocks are there to be reused
        s_list = K.attn_qk(q, k, kl, q_len_list=ql)
        s_tens = K.attn_qk(q, k, kl_t, q_len_list=ql_t)
        p_list = K.scale_mask_softmax(B, Sq, H, s_list, kl, scale=D ** -0.5, k_seq_len=Sk, q_len_list=ql)
        p_tens = K.scale_mask_softmax(B, Sq, H, s_tens, kl_t, scale=D ** -0.5, k_seq_len=Sk, q_len_list=ql_t)
        c_list = K.attn_pv(p_list, v, kl, q_len_list=ql)
        c_tens = K.attn_pv(p_tens, v, kl_t, q_len_list=ql_t)
        f_list = K.attn_fused(q, k, v, kl, q_len_list=ql)
        f_tens = K.attn_fused(q, k, v, kl_t, q_len_list=ql_t)
        for b in range(B):
            assert torch.equal(c_list[b, :, :ql[b]], c_tens[b, :, :ql[b]])
            assert torch.equal(f_list[b, :, :ql[b]], f_tens[b, :, :ql[b]])
    want = eager.attn_pv(eager.scale_mask_softmax(B, Sq, H, eager.attn_qk(q.cpu(), k.cpu(), torch.float32), kl,
                                                  scale=D ** -0.5, k_seq_len=Sk, q_lens=ql), v.cpu(), torch.float32)
    for b in range(B):
        assert max_abs(c_list[b, :, :ql[b]].cpu(), want[b, :, :ql[b]]) <= 2e-3


def test_cached_offsets_used_on_another_stream():
    """The offsets of a batch are computed by a kernel on the stream of first use and cached; a later call on
    another stream must be ordered behind that kernel."""
    from energonai_amd import _lib
    from energonai_amd import kernel as K
    from energonai_amd.seqinfo import clear_cache, seq_info
    B, S, hid = 6, 64, 256
    lens = [64, 1, 30, 17, 0, 55]
    announce("offsets across streams")
    x = torch.randn(B, S, hid, generator=torch.Generator().manual_seed(8))
    xg = x.cuda()
    lens_t = torch.tensor(lens, dtype=torch.int32).cuda()
    want = eager.depad(x, B, lens)
    torch.cuda.synchronize()
    clear_cache()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        info = seq_info(lens_t, B, xg.device)                  # prefix kernel launched on `side`
        assert _lib.stream_of(xg) in info._ordered
    main_raw = _lib.stream_of(xg)
    assert main_raw not in info._ordered
    got = K.depad(xg, B, lens_t, sum_seq=sum(lens))          # cache hit on the main stream
    assert seq_info(lens_t, B, xg.device) is info and main_raw in info._ordered
    assert torch.equal(got.cpu(), want)
    off = info.row_offsets(S, True)                           # produced on the main stream ...
    with torch.cuda.stream(side):                             # ... and consumed on the other one
        y = K.layer_norm_forward(torch.zeros(1, sum(lens), hid, device="cuda"), torch.ones(hid, device="cuda"),
                                 torch.zeros(hid, device="cuda"), (hid,), 1e-5, residual=xg,
                                 residual_row_offsets=info.row_offsets(S, True))
    side.synchronize()
    left = torch.cat([x[b, S - n:] for b, n in enumerate(lens)])
    assert max_abs(y.cpu()[0], torch.nn.functional.layer_norm(left, (hid,))) <= 1e-5
    assert off.data_ptr() == info.row_offsets(S, True).data_ptr()


def test_yardstick_kernels_touch_exactly_their_pattern():
    """The bandwidth yardsticks are measuring sticks, but a stick that moved other bytes than it claims would
    mislead: the copy copies, the write-only pass writes its whole range, the prefix passes write the causal
    prefixes of the valid rows (whole 16-byte vectors) and nothing else."""
    import torch
    from energonai_amd import _lib
    from energonai_amd.kernel.attention import packed_scores_elems
    lib = _lib.load()
    stream = torch.cuda.current_stream().cuda_stream
    n = 1 << 20
    a = torch.randint(0, 255, (n,), dtype=torch.uint8, device="cuda")
    for nt in (0, 1):
        b = torch.zeros(n, dtype=torch.uint8, device="cuda")
        _lib.check(lib.en_stream_yardstick(a.data_ptr(), b.data_ptr(), n, 0, nt, stream), "copy")
        assert torch.equal(a, b)
        b.fill_(7)
        _lib.check(lib.en_stream_yardstick(None, b.data_ptr(), n, 2, nt, stream), "write")
        assert bool((b == 0).all())
        b.fill_(7)
        _lib.check(lib.en_stream_yardstick(a.data_ptr(), b.data_ptr(), n, 1, nt, stream), "read")
        assert bool((b == 7).all())
    B, H, S = 3, 2, 200
    lens = [200, 0, 77]
    lens_t = torch.tensor(lens, dtype=torch.int32, device="cuda")
    for packed in (0, 1):
        numel = packed_scores_elems(B, H, S, torch.float16) if packed else B * H * S * S
        src = torch.randn(numel, device="cuda").half()
        for mode in (0, 1, 2, 3, 4, 5, 6, 7):
            buf = src.clone()
            out = torch.full_like(src, 5.0)
            _lib.check(lib.en_prefix_yardstick(buf.data_ptr(), out.data_ptr(), lens_t.data_ptr(), B, H, S, packed, mode, 0, 2,
                                               stream), "prefix")
            touched = torch.zeros(numel, dtype=torch.bool)
            for b in range(B):
                for h in range(H):
                    unit = b * H + h
                    if packed:       # a unit's valid rows are one contiguous range: rows back to back, 128-byte groups
                        t = lens[b] // 64
                        end = 64 * (64 * t * (t + 1) // 2 + (lens[b] - 64 * t) * (t + 1))
                        touched[unit * (numel // (B * H)):unit * (numel // (B * H)) + end] = True
                        continue
                    for q in range(lens[b]):
                        start = (unit * S + q) * S
                        touched[start:start + -(-(q + 1) // 8) * 8] = True
            if mode in (0, 2, 4, 5, 6, 7):     # 4..7: read only, a 128-row tile at a time along the keys
                assert torch.equal(buf, src) and bool((out == 5.0).all())
            if mode == 1:
                assert bool((buf.cpu()[touched] == 0).all()) and torch.equal(buf.cpu()[~touched], src.cpu()[~touched])
            if mode == 3:
                assert torch.equal(out.cpu()[touched], src.cpu()[touched]) and bool((out.cpu()[~touched] == 5.0).all())
