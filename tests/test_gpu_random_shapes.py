"""Seeded random shapes through the packing ops, the row softmax and the LayerNorm.

The fixed cases elsewhere follow the reference's tests and the benchmark workloads; these draw batch sizes,
buckets, head counts, widths (including ones that force the 8-, 4- and 2-byte paths), empty and full
sequences, dtypes and padding sides from a seeded generator and compare with the oracle: bit-exact for the
packing ops, within the stated tolerances for softmax and LayerNorm.
"""
import pytest
import torch

from gpu_util import BASE, assert_ctx_close, assert_stored_close, announce, max_abs, packed_randn
from oracle import eager

pytestmark = pytest.mark.gpu


def _kernel():
    from energonai_amd import kernel
    return kernel


def _draw(seed):
    g = torch.Generator().manual_seed(seed)
    return lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))


def _lens(ri, B, S):
    lens = [ri(0, S) for _ in range(B)]
    lens[ri(0, B - 1)] = S                       # one full sequence
    if B > 1:
        lens[ri(0, B - 1)] = ri(0, 1)            # and an empty or one-token one (may replace the full one)
    return lens


@pytest.mark.parametrize("seed", list(range(16)))
def test_packing_ops_random_shapes(seed):
    k = _kernel()
    ri = _draw(7000 + seed)
    B, S, H = ri(1, 9), ri(1, 300), ri(1, 5)
    D = [1, 2, 3, 4, 6, 8, 20, 64, 96, 192][ri(0, 9)]
    dtype = [torch.float16, torch.float32, torch.bfloat16][ri(0, 2)]
    left = bool(ri(0, 1))
    lens = _lens(ri, B, S)
    T = sum(lens)
    announce("packing random", seed, B, S, H, D, dtype, left, lens)
    lens_t = torch.tensor(lens, dtype=torch.int64 if ri(0, 1) else torch.int32).cuda()
    # depad / repad on [B,S,hid] with hid = H*D
    hid = H * D
    x = packed_randn(B * S, hid, dtype, seed).reshape(B, S, hid)
    want = eager.depad(x, B, lens, left_padded=left)
    got = k.depad(x.cuda(), B, lens_t, left_padded=left)
    assert got.shape == (1, T, hid) and torch.equal(got.cpu(), want)
    back = k.repad(got, B, S, lens_t, left_padded=left).cpu()
    assert torch.equal(back, eager.repad(want, B, S, lens, left_padded=left))
    # transpose_pad / transpose_depad on [1,T,H,D]
    src = packed_randn(max(T, 1), hid, dtype, seed + 1)[:T].reshape(1, T, H, D)
    pad = k.transpose_pad(src.cuda(), B, S, lens_t, H, D)
    ref_pad = eager.transpose_pad(src, B, S, lens, H, D)
    assert torch.equal(pad.cpu(), ref_pad)
    part = k.transpose_pad(src.cuda(), B, S, lens_t, H, D, zero_padding=False).cpu()
    for b, n in enumerate(lens):
        assert torch.equal(part[b, :, :n], ref_pad[b, :, :n])
    assert torch.equal(k.transpose_depad(pad, B, T, S, lens_t, H, D).cpu(), src)


@pytest.mark.parametrize("seed", list(range(16)))
def test_softmax_random_shapes(seed):
    k = _kernel()
    ri = _draw(7100 + seed)
    B, H = ri(1, 5), ri(1, 4)
    rect = bool(ri(0, 1))
    Sk = ri(1, 130) * [1, 1, 8][ri(0, 2)]        # odd widths take the scalar kernel, multiples of 8 the row kernel
    Sq = ri(1, 40) if rect else Sk
    dtype = [torch.float16, torch.float32, torch.bfloat16][ri(0, 2)]
    causal = bool(ri(0, 1))
    tail = [0, 1, 32, 128][ri(0, 3)]
    scale = [1.0, 0.125, 0.37][ri(0, 2)]
    k_lens = _lens(ri, B, Sk)
    q_lens = [min(ri(0, Sq), n) for n in k_lens] if rect else None
    announce("softmax random", seed, B, H, Sq, Sk, dtype, causal, tail, scale, k_lens, q_lens)
    src = (2.0 * packed_randn(B * H * Sq, Sk, torch.float32, seed)).to(dtype).reshape(B, H, Sq, Sk)
    want = eager.scale_mask_softmax(B, Sq, H, src, k_lens, scale=scale, causal=causal, k_seq_len=Sk, q_lens=q_lens,
                                    acc_dtype=torch.float64, out_dtype=torch.float64)
    kw = dict(scale=scale, causal=causal, tail_rows=tail)
    if rect:
        kw.update(k_seq_len=Sk, q_len_list=torch.tensor(q_lens, dtype=torch.int32).cuda())
    got = k.scale_mask_softmax(B, Sq, H, src.clone().cuda(), torch.tensor(k_lens, dtype=torch.int32).cuda(), **kw).cpu()
    tol = {torch.float16: 1e-3, torch.bfloat16: 8e-3, torch.float32: 1e-6}[dtype]
    ql = [min(n, Sq) for n in k_lens] if q_lens is None else q_lens
    for b in range(B):
        # untouched rows stay bit-identical; on valid rows the visible prefix matches the oracle
        assert torch.equal(got[b, :, ql[b]:], src[b, :, ql[b]:])
        for q in range(ql[b]):
            n = eager.visible_keys(q, ql[b], k_lens[b], causal)
            assert max_abs(got[b, :, q, :n], want[b, :, q, :n]) <= tol
            if tail == 0:
                assert not got[b, :, q, n:].any()


@pytest.mark.parametrize("seed", list(range(16)))
def test_layernorm_random_shapes(seed):
    k = _kernel()
    ri = _draw(7200 + seed)
    n1 = ri(1, 70)
    n2 = [ri(1, 40), 8 * ri(1, 40), 64 * ri(1, 40), 768, 1000, 4096 + 8 * ri(0, 3)][ri(0, 5)]
    pair = [(torch.float16, torch.float16), (torch.bfloat16, torch.bfloat16), (torch.float32, torch.float32),
            (torch.float32, torch.float16), (torch.float32, torch.bfloat16)][ri(0, 4)]
    with_res = bool(ri(0, 1))
    announce("layernorm random", seed, n1, n2, pair, with_res)
    x = (1.5 * packed_randn(n1, n2, torch.float32, seed) + 0.5).to(pair[0])
    r = packed_randn(n1, n2, torch.float32, seed + 1).to(pair[0]) if with_res else None
    gamma = (1.0 + 0.1 * packed_randn(1, n2, torch.float32, seed + 2)).to(pair[1]).reshape(n2)
    beta = (0.1 * packed_randn(1, n2, torch.float32, seed + 3)).to(pair[1]).reshape(n2)
    y, mean, invvar = k.layer_norm_forward(x.cuda(), gamma.cuda(), beta.cuda(), (n2,), 1e-5,
                                           residual=None if r is None else r.cuda(), return_stats=True)
    wy, wmean, winv, _ = eager.layer_norm(x, gamma, beta, 1e-5, residual=r, acc_dtype=torch.float64,
                                          out_dtype=torch.float64)
    assert y.dtype == pair[1] and y.shape == x.shape
    # fp32 arithmetic error of the kernel (1e-5 relative to the row's largest value) on top of half an ulp of the
    # stored output
    assert_stored_close(y.cpu(), wy, pair[1], base=1e-5 * max(1.0, float(wy.abs().max())), what="LayerNorm output")
    assert max_abs(mean.cpu(), wmean) <= 1e-5 * max(1.0, float(wmean.abs().max()))
    assert max_abs(invvar.cpu(), winv) <= 2e-5 * max(1.0, float(winv.abs().max()))


@pytest.mark.parametrize("seed", list(range(10)))
def test_decode_random_shapes(seed):
    """Single-query QK^T -> softmax -> PV against a ragged cache whose unused rows hold NaN."""
    k = _kernel()
    ri = _draw(7300 + seed)
    B, H = ri(1, 7), ri(1, 6)
    D = [32, 64, 80, 96, 128][ri(0, 4)]
    S = 8 * ri(1, 150)
    dtype = [torch.float16, torch.bfloat16, torch.float32][ri(0, 2)]
    kv = [ri(1, S) for _ in range(B)]
    kv[ri(0, B - 1)] = S
    announce("decode random", seed, B, H, S, D, dtype, kv)
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, H, 1, D, generator=g).to(dtype)
    kc = torch.randn(B, H, S, D, generator=g).to(dtype)
    vc = torch.randn(B, H, S, D, generator=g).to(dtype)
    for b, n in enumerate(kv):
        kc[b, :, n:] = float("nan")
        vc[b, :, n:] = float("nan")
    kv_t = torch.tensor(kv, dtype=torch.int32).cuda()
    scale = D ** -0.5
    _, want_probs, want_ctx = eager.decode_attention(q, torch.nan_to_num(kc, nan=0.0), torch.nan_to_num(vc, nan=0.0),
                                                     kv, scale, acc_dtype=torch.float64)
    scores = k.decode_qk(q.cuda(), kc.cuda(), kv_t)
    probs = k.scale_mask_softmax(B, 1, H, scores, kv_t, scale=scale, k_seq_len=S,
                                 q_len_list=torch.ones(B, dtype=torch.int32).cuda())
    tol = {torch.float16: 2e-3, torch.bfloat16: 1.6e-2, torch.float32: 1e-5}[dtype]
    assert max_abs(probs.cpu(), want_probs) <= tol
    ctx = k.decode_pv(probs, vc.cuda(), kv_t).cpu()
    assert torch.isfinite(ctx).all()
    assert_ctx_close(ctx, want_ctx, dtype, "decode_pv")


@pytest.mark.parametrize("seed", list(range(10)))
def test_ft_family_random_shapes(seed):
    """The offset-based helpers: offsets, remove / rebuild, the three-tensor transposing pair; bit-exact."""
    k = _kernel()
    ri = _draw(7400 + seed)
    B, S, H = ri(1, 8), ri(1, 200), ri(1, 6)
    D = [2, 4, 8, 24, 64, 128][ri(0, 5)]
    dtype = [torch.float16, torch.float32][ri(0, 1)]
    lens = _lens(ri, B, S)
    lens[0] = max(lens[0], 1)                    # at least one token
    hid = H * D
    announce("ft random", seed, B, S, H, D, dtype, lens)
    want_valid, want_off = eager.ft_build_padding_offsets(lens, B, S)
    T = int(want_valid[0])
    tmp_off = torch.full((B, S), -7, dtype=torch.int32).cuda()
    mask_off = torch.full((B, S), -9, dtype=torch.int32).cuda()
    valid = torch.zeros(1, dtype=torch.int32).cuda()
    k.ft_build_padding_offsets(torch.tensor(lens, dtype=torch.int32).cuda(), B, S, valid, tmp_off)
    assert int(valid[0].item()) == T and torch.equal(tmp_off.flatten()[:T].cpu(), want_off)
    g = torch.Generator().manual_seed(seed)
    hq, hk, hv = (torch.rand(B, S, hid, generator=g).to(dtype) for _ in range(3))
    q = k.ft_remove_padding(hq.cuda(), tmp_off, mask_off, T, hid)
    want_q, want_mask = eager.ft_remove_padding(hq, want_off, T, hid)
    assert torch.equal(q.cpu(), want_q) and torch.equal(mask_off.flatten()[:T].cpu(), want_mask)
    kk = k.ft_remove_padding(hk.cuda(), tmp_off, mask_off, T, hid)
    v = k.ft_remove_padding(hv.cuda(), tmp_off, mask_off, T, hid)
    bufs = [torch.full((B, H, S, D), 3.0, dtype=dtype).cuda() for _ in range(3)]
    k.ft_transpose_rebuild_padding(q.view(T, H, D), kk.view(T, H, D), v.view(T, H, D), bufs[0], bufs[1], bufs[2],
                                   B, S, H, D, T, mask_off)
    want_bufs = [torch.full((B, H, S, D), 3.0, dtype=dtype) for _ in range(3)]
    eager.ft_transpose_rebuild_padding(q.cpu().view(T, H, D), kk.cpu().view(T, H, D), v.cpu().view(T, H, D),
                                       *want_bufs, B, S, H, D, T, want_mask)
    for got, want in zip(bufs, want_bufs):
        assert torch.equal(got.cpu(), want)
    back = k.ft_transpose_remove_padding(bufs[1], T, B, S, H, D, mask_off)
    assert torch.equal(back, kk)
    rebuilt = k.ft_rebuild_padding(back, mask_off, T, hid, B, S)
    assert torch.equal(rebuilt.cpu(), eager.ft_rebuild_padding(back.cpu(), want_mask, T, hid, B, S))


@pytest.mark.parametrize("seed", list(range(14)))
def test_layer_random_shapes(seed):
    """The whole step on drawn shapes (LayerNorm width equal to or different from heads x head size, either
    padding side, causal or not, every attention form, depad folded or not) against the oracle's layer."""
    from energonai_amd import layer
    ri = _draw(7500 + seed)
    B, S, H = ri(1, 6), 8 * ri(1, 40), ri(1, 4)
    D = [32, 64, 80, 128][ri(0, 3)]
    dtype = [torch.float16, torch.bfloat16, torch.float32][ri(0, 2)]
    wide = bool(ri(0, 1))                       # a dense projection between attention and LayerNorm
    hid = 8 * ri(4, 160) if wide else H * D
    causal, left = bool(ri(0, 1)), bool(ri(0, 1))
    lens = _lens(ri, B, S)
    if sum(lens) == 0:
        lens[0] = S
    T = sum(lens)
    announce("layer random", seed, B, S, H, D, hid, dtype, causal, left, lens)
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(B, S, hid, generator=g).to(dtype)
    qkv = torch.randn(1, T, H, 3 * D, generator=g).to(dtype)
    dense = torch.randn(1, T, hid, generator=g).to(dtype) if wide else None
    gamma = (1.0 + 0.05 * torch.randn(hid, generator=g)).to(dtype)
    beta = (0.05 * torch.randn(hid, generator=g)).to(dtype)
    scale = D ** -0.5
    want = eager.layer_unpadded(x, qkv, lens, H, D, gamma, beta, 1e-5, scale, causal, left, dense_out=dense,
                                acc_dtype=torch.float64)
    # the three-kernel path stores scores and probabilities in the activation dtype, as the reference does
    want_r = eager.layer_unpadded(x, qkv, lens, H, D, gamma, beta, 1e-5, scale, causal, left, dense_out=dense,
                                  acc_dtype=torch.float64, storage_dtype=dtype)
    args = (x.cuda(), qkv.cuda(), torch.tensor(lens, dtype=torch.int32).cuda(), H, D, gamma.cuda(), beta.cuda(),
            1e-5, scale, causal, left)
    dense_g = None if dense is None else dense.cuda()
    kept = layer.padding_removal_layer(*args, dense_out=dense_g, keep=True)
    assert torch.equal(kept["x"].cpu(), want["x"].to(dtype))
    # BASE[dtype] on top of half an ulp of the stored value; fp32: accumulation error grows with the values summed
    base_c = BASE[dtype] * (max(1.0, float(want["ctx_packed"].abs().max())) if dtype == torch.float32 else 1.0)
    assert_stored_close(kept["ctx_packed"].cpu(), want_r["ctx_packed"], dtype, base=base_c, what="context")
    # the LayerNorm hands the error of its input on scaled by gamma * invvar (nothing when a dense output stands
    # between attention and LayerNorm), and adds its own fp32 arithmetic and one rounding
    amp = 0.0 if wide else float(want["invvar"].max()) * float(gamma.float().abs().max())
    base_y = base_c * amp + 1e-5 * max(1.0, float(want["y"].abs().max()))
    forms = [(False, False), (False, True), ("varlen", False), ("varlen", True), (None, None)]
    if dtype != torch.float32:
        forms += [(True, False), ("packed", False), ("packed", True)]
        if causal:
            forms += [("varlen_packed", False), ("varlen_packed", True)]
    for form, fold in forms:
        y = layer.padding_removal_layer(*args, dense_out=dense_g, fused_attention=form, fold_depad=fold)
        assert y.shape == (1, T, hid)
        if form is None:        # the default: the fused kernel wherever it applies, else the three kernels
            three_kernels = layer.default_attention_form(causal, dtype, S, D, scale) != "packed"
        else:
            three_kernels = form in (False, "varlen", "varlen_packed")
        assert_stored_close(y.cpu(), (want_r if three_kernels else want)["y"], dtype, base=base_y, what=f"y {form} {fold}")
        if three_kernels:
            assert torch.equal(y, kept["y"]), (form, fold)      # the one-call step gives the op-by-op bits
