"""GPU parity: scale_mask_softmax and the fused LayerNorm against the fp32/fp64 oracle.

Tolerance (from the north-star statement): max-abs error <= 2e-3 against the
fp32 oracle for fp16 storage; fp32 storage must reach 1e-5.  bf16 storage is
held to its own rounding step (2^-8 relative).
"""
import pytest
import torch

from gpu_util import announce, assert_stored_close, max_abs, ragged_lens
from oracle import eager

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-5, torch.float16: 2e-3, torch.bfloat16: 3.2e-2}


def _kernel():
    from energonai_amd import kernel
    return kernel


def _valid_row_mask(B, H, Sq, Sk, q_lens):
    m = torch.zeros(B, H, Sq, Sk, dtype=torch.bool)
    for b, n in enumerate(q_lens):
        m[b, :, :n] = True
    return m


SOFTMAX_CASES = [
    # B, H, S, lens
    (8, 12, 128, [24, 127, 31, 65, 24, 127, 31, 65]),
    (2, 3, 8, [8, 1]),
    (3, 2, 40, [40, 0, 7]),
    (2, 2, 512, [300, 512]),
    (2, 1, 1024, [1024, 513]),
    (1, 2, 2048, [1500]),          # above the reference's 1024 limit
    (1, 1, 4096, [4096]),
    (2, 2, 37, [37, 5]),           # row length not a multiple of the vector: generic kernel
    (1, 1, 8200, [8200]),          # too long for registers (fp32): generic kernel
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("B,H,S,lens", SOFTMAX_CASES)
def test_softmax_reference_semantics(dtype, B, H, S, lens):
    """Five-argument call: causal, no scale, padded rows untouched, in place, same tensor returned."""
    k = _kernel()
    announce("softmax ref", dtype, B, H, S, lens)
    g = torch.Generator().manual_seed(S + B)
    src = (3.0 * torch.randn(B, H, S, S, generator=g)).to(dtype)
    want = eager.scale_mask_softmax(B, S, H, src.float(), lens, out_dtype=torch.float32)
    x = src.clone().cuda()
    out = k.scale_mask_softmax(B, S, H, x, torch.tensor(lens, dtype=torch.int32).cuda())
    assert out.data_ptr() == x.data_ptr(), "must be in place and return its input"
    got = out.cpu()
    valid = _valid_row_mask(B, H, S, S, lens)
    err = max_abs(got[valid].float(), want[valid])
    assert err <= TOL[dtype], err
    # padded query rows hold their raw scores, bit for bit (csrc/scale_mask_softmax_kernel.cu:14-17)
    assert torch.equal(got[~valid], src[~valid])
    # the zero tail is exact and valid rows sum to one
    for b, n in enumerate(lens):
        for q in (0, n // 2, n - 1):
            if 0 <= q < n:
                assert bool((got[b, :, q, q + 1:] == 0).all())
                assert abs(got[b, :, q].float().sum(-1) - 1).max() < 4 * TOL[dtype] + 1e-3 * (dtype != torch.float32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("causal", [True, False])
def test_softmax_scale_and_noncausal(dtype, causal):
    k = _kernel()
    B, H, S = 4, 3, 96
    lens = [96, 1, 50, 17]
    scale = 0.125
    announce("softmax scale", dtype, causal)
    g = torch.Generator().manual_seed(5)
    src = (8.0 * torch.randn(B, H, S, S, generator=g)).to(dtype)
    want = eager.scale_mask_softmax(B, S, H, src.float(), lens, scale=scale, causal=causal, out_dtype=torch.float32)
    got = k.scale_mask_softmax(B, S, H, src.clone().cuda(), torch.tensor(lens).cuda(), scale=scale,
                               causal=causal).cpu()
    valid = _valid_row_mask(B, H, S, S, lens)
    assert max_abs(got[valid].float(), want[valid]) <= TOL[dtype]
    if not causal:
        for b, n in enumerate(lens):
            assert bool((got[b, :, :n, n:] == 0).all())


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_softmax_rectangular_decode(dtype):
    """One query row per sequence against a longer ragged key axis."""
    k = _kernel()
    B, H, Sk = 5, 4, 640
    kv = [640, 1, 333, 64, 65]
    announce("softmax decode", dtype)
    g = torch.Generator().manual_seed(6)
    src = (4.0 * torch.randn(B, H, 1, Sk, generator=g)).to(dtype)
    want = eager.scale_mask_softmax(B, 1, H, src.float(), kv, scale=0.5, causal=True, k_seq_len=Sk,
                                    q_lens=[1] * B, out_dtype=torch.float32)
    got = k.scale_mask_softmax(B, 1, H, src.clone().cuda(), torch.tensor(kv, dtype=torch.int32).cuda(), scale=0.5,
                               k_seq_len=Sk, q_len_list=torch.ones(B, dtype=torch.int32).cuda()).cpu()
    assert max_abs(got.float(), want) <= TOL[dtype]
    # q_len_list omitted: defaults to min(k_len, Sq) = 1
    got2 = k.scale_mask_softmax(B, 1, H, src.clone().cuda(), torch.tensor(kv, dtype=torch.int32).cuda(), scale=0.5,
                                k_seq_len=Sk).cpu()
    assert torch.equal(got, got2)


def test_softmax_rectangular_chunked_prefill():
    """Sq < Sk with several query rows: queries are the last q_len positions."""
    k = _kernel()
    B, H, Sq, Sk = 3, 2, 16, 128
    kl, ql = [128, 40, 9], [16, 8, 9]
    announce("softmax chunk")
    g = torch.Generator().manual_seed(8)
    src = torch.randn(B, H, Sq, Sk, generator=g)
    want = eager.scale_mask_softmax(B, Sq, H, src, kl, causal=True, k_seq_len=Sk, q_lens=ql)
    got = k.scale_mask_softmax(B, Sq, H, src.clone().cuda(), torch.tensor(kl, dtype=torch.int32).cuda(),
                               k_seq_len=Sk, q_len_list=torch.tensor(ql, dtype=torch.int32).cuda()).cpu()
    valid = _valid_row_mask(B, H, Sq, Sk, ql)
    assert max_abs(got[valid], want[valid]) <= 1e-5
    assert torch.equal(got[~valid], src[~valid])


LN_CASES = [
    # n1, n2
    (698, 768), (64, 9216), (33, 7168), (20, 12288), (5, 1024), (7, 8), (3, 16384),
    (4, 40000),      # wide row: 1024-lane kernel
    (4100, 7168),    # 896 fp16 vectors and many rows: 512 lanes x 2 vectors (fp32: 1792 vectors, 512 x 4)
    (4097, 4000),    # fp32: 1000 vectors and many rows: 512 lanes x 2; fp16: 500 vectors on 256 lanes
    (3, 100),        # fp16: 100 % 8 != 0 -> generic kernel
    (2, 70001),      # too wide / odd: generic kernel
]
LN_DTYPES = [(torch.float32, torch.float32), (torch.float16, torch.float16), (torch.bfloat16, torch.bfloat16),
             (torch.float32, torch.float16), (torch.float32, torch.bfloat16)]


@pytest.mark.parametrize("in_dtype,out_dtype", LN_DTYPES)
@pytest.mark.parametrize("n1,n2", LN_CASES)
@pytest.mark.parametrize("with_residual", [False, True])
def test_layernorm(in_dtype, out_dtype, n1, n2, with_residual):
    k = _kernel()
    announce("layernorm", in_dtype, out_dtype, n1, n2, with_residual)
    g = torch.Generator().manual_seed(n2 % 1000 + n1)
    x = (torch.randn(1, n1, n2, generator=g) * 1.5 + 0.3).to(in_dtype)
    r = torch.randn(1, n1, n2, generator=g).to(in_dtype) if with_residual else None
    gamma = (1 + 0.02 * torch.randn(n2, generator=g)).to(out_dtype)
    beta = (0.02 * torch.randn(n2, generator=g)).to(out_dtype)
    want, mean, invvar, xsum = eager.layer_norm(x, gamma, beta, 1e-5, residual=r, acc_dtype=torch.float64,
                                                out_dtype=torch.float64)
    res = k.layer_norm_forward(x.cuda(), gamma.cuda(), beta.cuda(), (n2,), 1e-5,
                               residual=None if r is None else r.cuda(), return_stats=True, return_sum=True)
    y, m, iv, s = (t.cpu() for t in res)
    assert y.dtype == out_dtype and y.shape == x.shape
    assert m.dtype == torch.float32 and m.shape == (n1,)
    # fp32 arithmetic (1e-5 relative to the row's largest value) on top of the one rounding of the stored output
    assert_stored_close(y, want, out_dtype, base=1e-5 * max(1.0, float(want.abs().max())), what="LayerNorm output")
    assert max_abs(m, mean) <= 1e-5
    assert ((iv.double() - invvar.double()).abs() / invvar.double()).max() <= 1e-5
    # the emitted residual stream is the fp32 sum rounded once to the input dtype
    xsum32 = x.float() if r is None else x.float() + r.float()
    assert torch.equal(s, xsum32.to(in_dtype))
    assert max_abs(s, xsum) <= TOL[in_dtype] * max(1.0, float(xsum.abs().max()) / 2)


def test_layernorm_fp16_single_rounding():
    """fp16 output equals the fp64 result rounded once to fp16 in all but a sliver of entries."""
    k = _kernel()
    n1, n2 = 256, 12288
    announce("layernorm single rounding")
    g = torch.Generator().manual_seed(12)
    x = torch.randn(n1, n2, generator=g).half()
    gamma = (1 + 0.02 * torch.randn(n2, generator=g)).half()
    beta = (0.02 * torch.randn(n2, generator=g)).half()
    want64, _, _, _ = eager.layer_norm(x, gamma, beta, 1e-5, acc_dtype=torch.float64, out_dtype=torch.float64)
    y = k.layer_norm_forward(x.cuda(), gamma.cuda(), beta.cuda(), (n2,), 1e-5).cpu()
    assert_stored_close(y, want64, torch.float16, base=1e-5 * float(want64.abs().max()), what="LayerNorm output")
    frac_exact = (y == want64.half()).double().mean().item()
    assert frac_exact > 0.995, frac_exact


def test_layernorm_module_matches_reference_interface():
    from energonai_amd.kernel.cuda_native import LayerNorm
    announce("layernorm module")
    ln = LayerNorm(768, eps=1e-5, dtype=torch.float16).cuda()
    assert repr(ln) == "MixedFusedLayerNorm(normalized_shape=torch.Size([768]), eps=1e-05)"
    assert torch.equal(ln.weight.detach().cpu(), torch.ones(768, dtype=torch.float16))
    assert torch.equal(ln.bias.detach().cpu(), torch.zeros(768, dtype=torch.float16))
    x = torch.randn(2, 5, 768, generator=torch.Generator().manual_seed(1)).half()
    with torch.inference_mode():
        y = ln(x.cuda()).cpu()
    want = torch.nn.functional.layer_norm(x.float(), (768,), eps=1e-5)
    assert_stored_close(y, want, torch.float16, base=1e-5 * float(want.abs().max()), what="LayerNorm module")
    # constant row -> beta (here zero)
    with torch.inference_mode():
        z = ln(torch.full((3, 768), 2.5, dtype=torch.float16).cuda()).cpu()
    assert bool((z == 0).all())
    with pytest.raises(RuntimeError, match="expected input with shape"):
        ln(torch.zeros(2, 100, dtype=torch.float16).cuda())


@pytest.mark.parametrize("tile", [128, 32, 1])
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("scale", [0.5, -0.5])
def test_softmax_tiled_tail(dtype, causal, tile, scale):
    """tail_rows=t: valid entries identical to the full-tail result, zeros up to the extent of the row's
    t-row query tile (completed to a whole 16-byte vector), everything beyond left untouched.  t = 1 (the form
    in the step) writes no tail beyond that vector.  A negative scale takes the three-pass kernel, which must
    leave the same bytes."""
    k = _kernel()
    B, H, S = 3, 2, 512
    lens = [512, 130, 300]
    announce("softmax tiled tail", dtype, causal, tile, scale)
    g = torch.Generator().manual_seed(21)
    src = (3.0 * torch.randn(B, H, S, S, generator=g)).to(dtype)
    lens_t = torch.tensor(lens, dtype=torch.int32).cuda()
    epv = 16 // src.element_size()
    full = k.scale_mask_softmax(B, S, H, src.clone().cuda(), lens_t, scale=scale, causal=causal).cpu()
    tiled = k.scale_mask_softmax(B, S, H, src.clone().cuda(), lens_t, scale=scale, causal=causal, tail_rows=tile).cpu()
    want = eager.scale_mask_softmax(B, S, H, src.float(), lens, scale=scale, causal=causal, out_dtype=torch.float32)
    valid = _valid_row_mask(B, H, S, S, lens)
    assert max_abs(full[valid].float(), want[valid]) <= TOL[dtype]
    for b, n in enumerate(lens):
        for q0 in range(0, n, tile):
            rows = min(tile, n - q0)
            lim = min(n, q0 + rows) if causal else n
            lim_v = -(-lim // epv) * epv   # whole vectors are written
            assert torch.equal(tiled[b, :, q0:q0 + rows, :lim], full[b, :, q0:q0 + rows, :lim])
            assert bool((tiled[b, :, q0:q0 + rows, lim:lim_v] == 0).all())
            assert torch.equal(tiled[b, :, q0:q0 + rows, lim_v:], src[b, :, q0:q0 + rows, lim_v:])
        assert torch.equal(tiled[b, :, n:], src[b, :, n:])
