"""Pins oracle/models.py against library routines (CPU only)."""
import pytest
import torch
import torch.nn.functional as F

from oracle import eager, models


def _params(hid, heads, g, fused=True, mlp_ratio=4):
    r = lambda *s: 0.2 * torch.randn(*s, generator=g)
    p = {"dense.weight": r(hid, hid), "dense.bias": r(hid)}
    if fused:
        p["query_key_value.weight"] = r(3 * hid, hid)
        p["query_key_value.bias"] = r(3 * hid)
    else:
        for n in ("query_", "key_", "value_"):
            p[n + ".weight"] = r(hid, hid)
            p[n + ".bias"] = r(hid)
    return p


@pytest.mark.parametrize("is_decoder", [True, False])
@pytest.mark.parametrize("fused", [True, False])
def test_mha_forward_equals_library_multi_head_attention(is_decoder, fused):
    g = torch.Generator().manual_seed(3)
    B, S, hid, heads = 3, 10, 32, 4
    p = _params(hid, heads, g, fused)
    x = torch.randn(B, S, hid, generator=g)
    lens = [10, 4, 7]
    valid = torch.zeros(B, S)
    for b, n in enumerate(lens):
        valid[b, S - n:] = 1          # left padded
    got = models.mha_forward(x, p, heads, is_decoder, models.additive_mask(valid), fused)
    if fused:
        w, bias = p["query_key_value.weight"], p["query_key_value.bias"]
        wk, wv, wq = w[:hid], w[hid:2 * hid], w[2 * hid:]
        bk, bv, bq = bias[:hid], bias[hid:2 * hid], bias[2 * hid:]
    else:
        wq, wk, wv = p["query_.weight"], p["key_.weight"], p["value_.weight"]
        bq, bk, bv = p["query_.bias"], p["key_.bias"], p["value_.bias"]
    attn_mask = torch.triu(torch.ones(S, S, dtype=torch.bool), 1) if is_decoder else None
    want, _ = F.multi_head_attention_forward(
        x.transpose(0, 1), x.transpose(0, 1), x.transpose(0, 1), hid, heads, torch.cat([wq, wk, wv]),
        torch.cat([bq, bk, bv]), None, None, False, 0.0, p["dense.weight"], p["dense.bias"], training=False,
        key_padding_mask=(valid == 0), need_weights=False, attn_mask=attn_mask)
    want = want.transpose(0, 1)
    for b, n in enumerate(lens):      # rows of padded queries are undefined in both
        assert torch.allclose(got[b, S - n:], want[b, S - n:], atol=2e-5, rtol=1e-5)


def test_mha_last_row_does_not_depend_on_later_rows_when_causal():
    """The cached decode of the reference returns the last row of the full recomputation; under
    the causal mask that row of position t is the same whether or not later positions exist."""
    g = torch.Generator().manual_seed(4)
    B, S, hid, heads = 2, 9, 16, 2
    p = _params(hid, heads, g)
    x = torch.randn(B, S, hid, generator=g)
    full = models.mha_forward(x, p, heads, True)
    part = models.mha_forward(x[:, :6], p, heads, True)
    assert torch.allclose(full[:, :6], part, atol=1e-5)


@pytest.mark.parametrize("post", [True, False])
def test_block_forward_equals_stepwise_library_composition(post):
    g = torch.Generator().manual_seed(5)
    B, S, hid, heads = 2, 8, 16, 2
    r = lambda *s: 0.2 * torch.randn(*s, generator=g)
    p = {"attn." + k: v for k, v in _params(hid, heads, g).items()}
    p.update({"norm1.weight": 1 + r(hid), "norm1.bias": r(hid), "norm2.weight": 1 + r(hid), "norm2.bias": r(hid),
              "mlp.dense_1.weight": r(4 * hid, hid), "mlp.dense_1.bias": r(4 * hid),
              "mlp.dense_2.weight": r(hid, 4 * hid), "mlp.dense_2.bias": r(hid)})
    x = torch.randn(B, S, hid, generator=g)
    got = models.block_forward(x, p, heads, 1e-5, post, True, None)
    # same block, written as the textbook pre-/post-LN formulas
    ln = lambda t, n: (t - t.mean(-1, keepdim=True)) / torch.sqrt(t.var(-1, unbiased=False, keepdim=True) + 1e-5) \
        * p[n + ".weight"] + p[n + ".bias"]
    attn = lambda t: models.mha_forward(t, {k[5:]: v for k, v in p.items() if k.startswith("attn.")}, heads, True)
    mlp = lambda t: F.gelu(t @ p["mlp.dense_1.weight"].T + p["mlp.dense_1.bias"]) @ p["mlp.dense_2.weight"].T \
        + p["mlp.dense_2.bias"]
    if post:
        a = ln(x, "norm1")
        b_ = ln(a + attn(a), "norm2")
        want = b_ + mlp(b_)
    else:
        a = x + attn(ln(x, "norm1"))
        want = a + mlp(ln(a, "norm2"))
    assert torch.allclose(got, want, atol=2e-5, rtol=1e-5)


@pytest.mark.parametrize("left", [True, False])
def test_repad_inverts_depad(left):
    g = torch.Generator().manual_seed(6)
    B, S, hid = 4, 7, 5
    lens = [7, 0, 3, 1]
    x = torch.randn(B, S, hid, generator=g)
    for b, n in enumerate(lens):
        if left:
            x[b, :S - n] = 0
        else:
            x[b, n:] = 0
    packed = eager.depad(x, B, lens, left_padded=left)
    assert torch.equal(eager.repad(packed, B, S, lens, left_padded=left), x)
