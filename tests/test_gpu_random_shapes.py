"""Seeded random shapes through the packing ops, the row softmax and the LayerNorm.

The fixed cases elsewhere follow the reference's tests and the benchmark workloads; these draw batch sizes,
buckets, head counts, widths (including ones that force the 8-, 4- and 2-byte paths), empty and full
sequences, dtypes and padding sides from a seeded generator and compare with the oracle: bit-exact for the
packing ops, within the stated tolerances for softmax and LayerNorm.
"""
import pytest
import torch

from gpu_util import announce, max_abs, packed_randn
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
    tol = {torch.float16: 4e-3, torch.bfloat16: 3e-2, torch.float32: 2e-5}[pair[1]]
    assert max_abs(y.cpu(), wy) <= tol * max(1.0, float(wy.abs().max()))
    assert max_abs(mean.cpu(), wmean) <= 1e-5 * max(1.0, float(wmean.abs().max()))
    assert max_abs(invvar.cpu(), winv) <= 2e-5 * max(1.0, float(winv.abs().max()))
