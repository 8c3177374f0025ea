"""Pins the oracle's floating-point functions (CPU only): softmax, LayerNorm,
the two contractions, the decode form and the whole-layer identity.

The reference has no test for scale_mask_softmax or its LayerNorm, so these are
pinned by library routines in float64, closed forms, brute-force replays of
the reference kernels' arithmetic (Python and C) and invariants.
"""
import math

import pytest
import torch

from oracle import brute, cref, eager


def _rand(shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g) * scale


@pytest.mark.parametrize("B,H,S,lens", [(2, 2, 5, [5, 2]), (3, 1, 4, [1, 0, 4]), (1, 3, 8, [8])])
def test_softmax_vs_kernel_replay(B, H, S, lens):
    src = _rand((B, H, S, S), seed=S, scale=3.0)
    got = eager.scale_mask_softmax(B, S, H, src, lens)
    flat = src.flatten().tolist()
    brute.softmax_reference_kernel(flat, lens, B, H, S)
    assert torch.allclose(got, torch.tensor(flat).view_as(src), atol=1e-6, rtol=1e-5)
    c = cref.softmax_f32(src, lens, B, H, S)
    assert torch.allclose(got, c, atol=1e-6, rtol=1e-5)
    for b, n in enumerate(lens):                       # padded query rows are untouched, bit for bit
        assert torch.equal(got[b, :, n:], src[b, :, n:])


def test_softmax_closed_forms():
    B, H, S = 2, 2, 6
    lens = [6, 1]
    const = torch.full((B, H, S, S), 2.5)
    out = eager.scale_mask_softmax(B, S, H, const, lens)
    for q in range(6):                                 # constant row -> uniform over the q+1 visible keys
        assert torch.allclose(out[0, :, q, :q + 1], torch.full((H, q + 1), 1.0 / (q + 1)))
        assert bool((out[0, :, q, q + 1:] == 0).all())
    assert out[1, 0, 0].tolist() == [1.0, 0, 0, 0, 0, 0]   # length 1 -> [1, 0, ...]
    x = _rand((B, H, S, S), seed=1)
    a = eager.scale_mask_softmax(B, S, H, x, lens)
    shifted = x + 7.0 * torch.arange(S).view(1, 1, S, 1)   # per-row constants do not change a softmax
    b = eager.scale_mask_softmax(B, S, H, shifted, lens)
    assert torch.allclose(a[0], b[0], atol=1e-6)
    assert torch.allclose(a[0].sum(-1), torch.ones(H, S), atol=1e-6)
    # scale k is the same as pre-multiplying the scores by k
    s1 = eager.scale_mask_softmax(B, S, H, x, lens, scale=0.125)
    s2 = eager.scale_mask_softmax(B, S, H, x * 0.125, lens)
    assert torch.allclose(s1[0], s2[0], atol=1e-7)
    # non-causal: every row of a sequence sees exactly its len keys
    nc = eager.scale_mask_softmax(B, S, H, x, [4, 2], causal=False)
    assert torch.allclose(nc[0, :, :4, :4], torch.softmax(x[0, :, :4, :4], -1), atol=1e-7)
    assert bool((nc[0, :, :4, 4:] == 0).all())


def test_softmax_hard_mask_matches_additive_mask_of_the_models():
    """The models mask with -1e4 added to the scores (energonai/model/attention.py:105-116);
    the kernel masks hard.  With scores of ordinary size the two agree to fp32 rounding."""
    B, H, S = 3, 2, 16
    lens = [16, 5, 9]
    x = _rand((B, H, S, S), seed=4, scale=4.0)
    hard = eager.scale_mask_softmax(B, S, H, x, lens, scale=0.25, causal=True)
    soft = eager.scale_mask_softmax_additive(x, lens, 0.25, True)
    for b, n in enumerate(lens):
        assert torch.allclose(hard[b, :, :n], soft[b, :, :n], atol=1e-6)


def test_softmax_rectangular_is_the_tail_of_the_square():
    """q_len < k_len: the queries are the last q_len positions (cached decode)."""
    B, H, Sk = 2, 2, 12
    kl, ql = [12, 7], [3, 2]
    full = _rand((B, H, Sk, Sk), seed=9)
    sq = eager.scale_mask_softmax(B, Sk, H, full, kl)
    Sq = 3
    rect = torch.zeros(B, H, Sq, Sk)
    for b in range(B):
        rect[b, :, :ql[b]] = full[b, :, kl[b] - ql[b]:kl[b]]
    out = eager.scale_mask_softmax(B, Sq, H, rect, kl, k_seq_len=Sk, q_lens=ql)
    for b in range(B):
        assert torch.allclose(out[b, :, :ql[b]], sq[b, :, kl[b] - ql[b]:kl[b]], atol=1e-7)


@pytest.mark.parametrize("n1,n2", [(3, 8), (2, 130), (5, 768)])
def test_layer_norm_pins(n1, n2):
    x = _rand((n1, n2), seed=n2, scale=2.0) + 0.5
    gamma = 1 + 0.1 * _rand((n2,), seed=1)
    beta = 0.1 * _rand((n2,), seed=2)
    y, mean, invvar, _ = eager.layer_norm(x, gamma, beta, 1e-5, acc_dtype=torch.float64, out_dtype=torch.float64)
    lib = torch.nn.functional.layer_norm(x.double(), (n2,), gamma.double(), beta.double(), 1e-5)
    assert torch.allclose(y, lib, atol=1e-12)
    assert torch.allclose(mean.double(), x.double().mean(-1), atol=1e-6)
    assert torch.allclose(invvar.double(), torch.rsqrt(x.double().var(-1, unbiased=False) + 1e-5), rtol=1e-6)
    # serial Welford replay of the reference kernel (Python floats)
    yb, mb, ib = brute.layer_norm_rows(x.flatten().tolist(), n1, n2, gamma.tolist(), beta.tolist(), 1e-5)
    assert torch.allclose(y.flatten(), torch.tensor(yb, dtype=torch.float64), atol=1e-6)
    # 128-lane Welford/Chan replay in fp32 (the reference's actual reduction tree)
    yc, mc, ic = cref.layer_norm_f32(x, gamma, beta, 1e-5)
    assert torch.allclose(yc.double(), y, atol=5e-6)
    assert torch.allclose(mc.double(), mean.double(), atol=1e-6)
    assert torch.allclose(ic.double(), invvar.double(), rtol=1e-5)


def test_layer_norm_closed_forms():
    n2 = 64
    gamma = 1 + 0.1 * _rand((n2,), seed=1)
    beta = 0.1 * _rand((n2,), seed=2)
    const = torch.full((2, n2), 3.25)
    y, _, _, _ = eager.layer_norm(const, gamma, beta, 1e-5)
    assert torch.allclose(y, beta.expand(2, n2), atol=1e-6)               # constant row -> beta
    x = _rand((4, n2), seed=3)
    y, _, _, _ = eager.layer_norm(x, torch.ones(n2), torch.zeros(n2), 0.0, acc_dtype=torch.float64,
                                  out_dtype=torch.float64)
    assert torch.allclose(y.mean(-1), torch.zeros(4, dtype=torch.float64), atol=1e-12)
    assert torch.allclose(y.var(-1, unbiased=False), torch.ones(4, dtype=torch.float64), atol=1e-12)
    r = _rand((4, n2), seed=5)
    a, _, _, s = eager.layer_norm(x, gamma, beta, 1e-5, residual=r)
    b, _, _, _ = eager.layer_norm(x + r, gamma, beta, 1e-5)
    assert torch.allclose(a, b, atol=1e-7) and torch.allclose(s, x + r)


def test_contractions_vs_loops():
    B, H, S, D = 1, 2, 3, 4
    q, k, v = (_rand((B, H, S, D), seed=i) for i in range(3))
    sc = eager.attn_qk(q, k, torch.float64)
    p = torch.softmax(sc, -1)
    ctx = eager.attn_pv(p, v, torch.float64)
    for h in range(H):
        for i in range(S):
            for j in range(S):
                assert math.isclose(sc[0, h, i, j].item(), sum(q[0, h, i, d].item() * k[0, h, j, d].item()
                                                               for d in range(D)), rel_tol=1e-12, abs_tol=1e-12)
            for d in range(D):
                assert math.isclose(ctx[0, h, i, d].item(), sum(p[0, h, i, j].item() * v[0, h, j, d].item()
                                                                for j in range(S)), rel_tol=1e-12, abs_tol=1e-12)


@pytest.mark.parametrize("causal,left", [(False, False), (True, False), (True, True)])
def test_unpadded_layer_equals_padded_layer(causal, left):
    """The property the padding-removal path rests on (examples/bert/bert.py:100-126):
    on valid tokens it gives what the ordinary padded layer gives."""
    B, S, H, D = 3, 10, 2, 4
    hid = H * D
    lens = [10, 3, 6]
    T = sum(lens)
    g = torch.Generator().manual_seed(11)
    x = torch.randn(T, hid, generator=g, dtype=torch.float64)
    qkv = torch.randn(T, H, 3 * D, generator=g, dtype=torch.float64)
    gamma = 1 + 0.1 * torch.randn(hid, generator=g, dtype=torch.float64)
    beta = 0.1 * torch.randn(hid, generator=g, dtype=torch.float64)
    hidden_padded = torch.zeros(B, S, hid, dtype=torch.float64)
    qkv_padded = torch.zeros(B, S, H, 3 * D, dtype=torch.float64)
    t = 0
    for b, n in enumerate(lens):
        sl = slice(S - n, S) if left else slice(0, n)
        hidden_padded[b, sl] = x[t:t + n]
        qkv_padded[b, sl] = qkv[t:t + n]
        t += n
    un = eager.layer_unpadded(hidden_padded, qkv.view(1, T, H, 3 * D), lens, H, D, gamma, beta, 1e-5, D ** -0.5,
                              causal, left_padded=left, acc_dtype=torch.float64)
    pad = eager.layer_padded(hidden_padded, qkv_padded, lens, H, D, gamma, beta, 1e-5, D ** -0.5, causal,
                             left_padded=left, acc_dtype=torch.float64)
    want = eager.depad(pad, B, lens, left_padded=left)
    assert torch.allclose(un["y"], want, atol=1e-9)


def test_decode_is_last_row_of_full_recompute():
    B, H, Smax, D = 2, 2, 9, 4
    kv = [9, 4]
    q, kc, vc = _rand((B, H, 1, D), 1), _rand((B, H, Smax, D), 2), _rand((B, H, Smax, D), 3)
    _, probs, ctx = eager.decode_attention(q, kc, vc, kv, 0.5, acc_dtype=torch.float64)
    for b, n in enumerate(kv):
        # full square recompute over the n cached positions with the new query as the last row
        qfull = torch.zeros(1, H, n, D, dtype=torch.float64)
        qfull[0, :, n - 1] = q[b, :, 0]
        sc = eager.attn_qk(qfull, kc[b:b + 1, :, :n], torch.float64)
        p = eager.scale_mask_softmax(1, n, H, sc, [n], scale=0.5, acc_dtype=torch.float64)
        c = eager.attn_pv(p, vc[b:b + 1, :, :n], torch.float64)
        assert torch.allclose(ctx[b, :, 0], c[0, :, n - 1], atol=1e-12)
        assert torch.allclose(probs[b, :, 0, :n], p[0, :, n - 1], atol=1e-12)
        assert bool((probs[b, :, 0, n:] == 0).all())
