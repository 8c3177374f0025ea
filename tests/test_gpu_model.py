"""Model glue (attention / MLP / block modules, K/V cache, repad) against the padded eager oracle."""
import pytest
import torch
import torch.nn.functional as F

from gpu_util import announce, max_abs
from oracle import eager, models

pytestmark = pytest.mark.gpu


def _mods():
    import energonai_amd.kernel as K
    import energonai_amd.model as M
    return K, M


def _fp32_params(module):
    return {k: v.detach().float().cpu() for k, v in module.state_dict().items()}


def _padded_batch(B, S, hid, lens, left, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(B, S, hid, generator=g).to(dtype)
    valid = torch.zeros(B, S)
    for b, n in enumerate(lens):
        if left:
            valid[b, S - n:] = 1
        else:
            valid[b, :n] = 1
    return x * valid.unsqueeze(-1).to(dtype), valid


def _init(module, seed):
    g = torch.Generator().manual_seed(seed)
    with torch.no_grad():
        for name, prm in module.named_parameters():
            if name.endswith("weight") and prm.dim() == 1:
                prm.copy_(1.0 + 0.05 * torch.randn(prm.shape, generator=g))
            elif prm.dim() == 1:
                prm.copy_(0.05 * torch.randn(prm.shape, generator=g))
            else:
                prm.copy_(torch.randn(prm.shape, generator=g) / prm.shape[1] ** 0.5)


def _valid_rows(t, lens, left):
    S = t.shape[1]
    return torch.cat([t[b, S - n:] if left else t[b, :n] for b, n in enumerate(lens)])


@pytest.mark.parametrize("left", [True, False])
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_repad_is_inverse_of_depad(dtype, left):
    K, _ = _mods()
    B, S, hid = 5, 37, 96
    lens = [37, 1, 0, 20, 36]
    announce("repad", dtype, left)
    x, _ = _padded_batch(B, S, hid, lens, left, dtype, 11)
    lens_t = torch.tensor(lens, dtype=torch.int64).cuda()
    packed = K.depad(x.cuda(), B, lens_t, left_padded=left)
    back = K.repad(packed, B, S, lens_t, left_padded=left).cpu()
    assert torch.equal(back, x)
    assert torch.equal(back, eager.repad(packed.cpu(), B, S, lens, left_padded=left))


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_kv_cache_fill_and_append_bit_exact(dtype):
    K, M = _mods()
    B, H, D, Smax = 3, 4, 64, 50
    lens = [7, 30, 1]
    T = sum(lens)
    announce("kv cache", dtype)
    g = torch.Generator().manual_seed(12)
    kvq = torch.randn(T, 3 * H, D, generator=g).to(dtype)
    info_lens = torch.tensor(lens, dtype=torch.int32).cuda()
    cache = M.KVCache(B, H, Smax, D, dtype, "cuda")
    from energonai_amd.seqinfo import seq_info
    info = seq_info(info_lens, B, torch.device("cuda"))
    cache.fill(kvq.cuda(), kvq.cuda(), info, 0, H, longest=max(lens))
    want_k = torch.zeros(B, H, Smax, D, dtype=dtype)
    want_v = torch.zeros_like(want_k)
    start = 0
    for b, n in enumerate(lens):
        want_k[b, :, :n] = kvq[start:start + n, :H].permute(1, 0, 2)
        want_v[b, :, :n] = kvq[start:start + n, H:2 * H].permute(1, 0, 2)
        start += n
    assert torch.equal(cache.k.cpu(), want_k) and torch.equal(cache.v.cpu(), want_v)
    assert cache.lens.cpu().tolist() == lens
    for step in range(3):
        new = torch.randn(B, 3 * H, D, generator=g).to(dtype)
        new_g = new.cuda()
        cache.append(new_g[:, :H], new_g[:, H:2 * H])
        for b, n in enumerate(lens):
            want_k[b, :, n + step] = new[b, :H]
            want_v[b, :, n + step] = new[b, H:2 * H]
        assert torch.equal(cache.k.cpu(), want_k) and torch.equal(cache.v.cpu(), want_v)
        assert cache.lens.cpu().tolist() == [n + step + 1 for n in lens]
    # a cache that may be full refuses the next row instead of dropping it silently
    small = M.KVCache(B, H, max(lens) + 2, D, dtype, "cuda")
    small.fill(kvq.cuda(), kvq.cuda(), info, 0, H, longest=max(lens))
    new_g = torch.randn(B, 3 * H, D, generator=g).to(dtype).cuda()
    small.append(new_g[:, :H], new_g[:, H:2 * H])
    small.append(new_g[:, :H], new_g[:, H:2 * H])
    with pytest.raises(RuntimeError, match="max_seq_len"):
        small.append(new_g[:, :H], new_g[:, H:2 * H])
    assert small.lens.cpu().tolist() == [n + 2 for n in lens]
    # a caller of the C entry point itself (no host-side bound of the lengths) is told through a device counter:
    # sequence 1 is full now, the other two take the row
    overflow = torch.zeros(1, dtype=torch.int32, device="cuda")
    before_k = small.k.clone()
    K.kv_cache_append(new_g[:, :H], new_g[:, H:2 * H], small.k, small.v, small.info, overflow=overflow)
    assert overflow.item() == 1
    assert torch.equal(small.k[1], before_k[1])
    for b in (0, 2):
        assert torch.equal(small.k[b, :, lens[b] + 2], new_g[b, :H])
    K.kv_cache_append(new_g[:, :H], new_g[:, H:2 * H], small.k, small.v, small.info, overflow=overflow)
    assert overflow.item() == 2


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_kv_cache_fill_without_zero_fill_leaves_padding_untouched(dtype):
    """zero_padding=False: rows below each length are written, every other row keeps the bits it had
    (tiles that lie wholly in the padding are skipped, tiles that straddle a length are written in part)."""
    K, _ = _mods()
    B, H, D, Smax = 4, 3, 64, 700
    lens = [700, 0, 129, 64]
    T = sum(lens)
    announce("kv fill no zero", dtype)
    g = torch.Generator().manual_seed(31)
    src = torch.randn(T, 2 * H, D, generator=g).to(dtype)
    sentinel = torch.full((B, H, Smax, D), 123.0, dtype=dtype)
    lens_t = torch.tensor(lens, dtype=torch.int32).cuda()
    got = K.kv_cache_fill(src.cuda(), sentinel.clone().cuda(), B, lens_t, head_first=H, zero_padding=False).cpu()
    full = K.kv_cache_fill(src.cuda(), sentinel.clone().cuda(), B, lens_t, head_first=H).cpu()
    want = sentinel.clone()
    start = 0
    for b, n in enumerate(lens):
        want[b, :, :n] = src[start:start + n, H:].permute(1, 0, 2)
        start += n
    assert torch.equal(got, want)
    for b, n in enumerate(lens):
        assert torch.equal(full[b, :, :n], want[b, :, :n]) and not full[b, :, n:].any()


@pytest.mark.parametrize("fused_qkv", [True, False])
@pytest.mark.parametrize("is_decoder", [True, False])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_attention_module_prefill(dtype, is_decoder, fused_qkv):
    """MultiHeadAttention1D.forward on a padded batch equals the reference forward on valid positions."""
    _, M = _mods()
    B, S, hid, heads = 4, 160, 256, 4
    lens = [160, 33, 97, 128]
    left = is_decoder
    announce("mha prefill", dtype, is_decoder, fused_qkv)
    attn = M.MultiHeadAttention1D(hid, heads, dtype=dtype, max_seq_len=192, fused_qkv=fused_qkv,
                                  is_decoder=is_decoder, disable_past_cache=True).cuda()
    _init(attn, 21)
    x, valid = _padded_batch(B, S, hid, lens, left, dtype, 22)
    mask = models.additive_mask(valid)
    got = attn(x.cuda(), attention_mask=mask.to(dtype).cuda()).float().cpu()
    want = models.mha_forward(x, _fp32_params(attn), heads, is_decoder, mask, fused_qkv)
    tol = {torch.float16: 4e-3, torch.bfloat16: 3e-2, torch.float32: 2e-4}[dtype]
    assert max_abs(_valid_rows(got, lens, left), _valid_rows(want, lens, left)) <= tol
    pad = torch.cat([got[b, :S - n] if left else got[b, n:] for b, n in enumerate(lens)])
    assert bool((pad == 0).all())          # padding rows come back as zeros


@pytest.mark.parametrize("post", [True, False])
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_block_prefill_and_incremental_decode(dtype, post):
    """Block1D: prefill with first_cache=True, then three decode steps; the newest position of each
    step equals the reference block recomputed on the whole extended (left-padded) batch."""
    _, M = _mods()
    B, S, hid, heads = 3, 70, 128, 2
    lens = [70, 9, 41]
    announce("block decode", dtype, post)
    blk = M.Block1D(hid, heads, 4.0, dtype=dtype, apply_post_layernorm=post, max_seq_len=96).cuda()
    _init(blk, 31)
    p = _fp32_params(blk)
    x, valid = _padded_batch(B, S, hid, lens, True, dtype, 32)
    tol = {torch.float16: 1.5e-2, torch.float32: 5e-4}[dtype]
    mask = models.additive_mask(valid)
    got = blk(x.cuda(), attention_mask=mask.to(dtype).cuda(), first_cache=True).float().cpu()
    want = models.block_forward(x, p, heads, 1e-5, post, True, mask)
    assert max_abs(_valid_rows(got, lens, True), _valid_rows(want, lens, True)) <= tol
    g = torch.Generator().manual_seed(33)
    for step in range(3):
        x = torch.cat((x, torch.randn(B, 1, hid, generator=g).to(dtype)), 1)
        valid = torch.cat((valid, torch.ones(B, 1)), 1)
        mask = models.additive_mask(valid)
        got = blk(x.cuda(), attention_mask=mask.to(dtype).cuda(), first_cache=False).float().cpu()
        want = models.block_forward(x, p, heads, 1e-5, post, True, mask)
        assert got.shape == want.shape
        assert max_abs(got[:, -1], want[:, -1]) <= tol, step


def test_block_with_tuned_gemms_matches_the_reference_block():
    """set_gemm_tuning(True): every projection of the block runs on the fastest hipBLASLt candidate for its
    shape (prefill shapes and the skinny decode shapes are separate problems); same tolerances as untuned."""
    _, M = _mods()
    from energonai_amd.kernel.cuda_native import linear_func as lf
    B, S, hid, heads = 3, 70, 128, 2
    lens = [70, 9, 41]
    dtype = torch.float16
    announce("block tuned gemms")
    blk = M.Block1D(hid, heads, 4.0, activation=F.relu, dtype=dtype, max_seq_len=96).cuda()
    _init(blk, 35)
    p = _fp32_params(blk)
    x, valid = _padded_batch(B, S, hid, lens, True, dtype, 36)
    mask = models.additive_mask(valid)
    lf._tuned.clear()
    M.set_gemm_tuning(True)
    try:
        assert M.gemm_tuning()
        got = blk(x.cuda(), attention_mask=mask.to(dtype).cuda(), first_cache=True).float().cpu()
        n_prefill = len(lf._tuned)
        assert n_prefill == 4                 # qkv, dense, fc1 (+ReLU), fc2 at the packed row count
        want = models.block_forward(x, p, heads, 1e-5, False, True, mask, activation=F.relu)
        assert max_abs(_valid_rows(got, lens, True), _valid_rows(want, lens, True)) <= 1.5e-2
        g = torch.Generator().manual_seed(37)
        for step in range(2):
            x = torch.cat((x, torch.randn(B, 1, hid, generator=g).to(dtype)), 1)
            valid = torch.cat((valid, torch.ones(B, 1)), 1)
            mask = models.additive_mask(valid)
            got = blk(x.cuda(), attention_mask=mask.to(dtype).cuda(), first_cache=False).float().cpu()
            want = models.block_forward(x, p, heads, 1e-5, False, True, mask, activation=F.relu)
            assert max_abs(got[:, -1], want[:, -1]) <= 1.5e-2, step
        assert len(lf._tuned) == 2 * n_prefill        # the decode shapes were searched once, not per step
    finally:
        M.set_gemm_tuning(False)
    assert not M.gemm_tuning()


@pytest.mark.parametrize("act_name", ["relu", "gelu_tanh", "gelu"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_mlp_with_gemm_epilogues(dtype, act_name):
    """MLP1D: ReLU and tanh-GELU ride in the first GEMM's epilogue, erf-GELU stays a separate op; all
    three equal the reference MLP forward."""
    import functools
    _, M = _mods()
    hid, rows = 256, 77
    announce("mlp", dtype, act_name)
    act = {"relu": F.relu, "gelu_tanh": functools.partial(F.gelu, approximate="tanh"), "gelu": F.gelu}[act_name]
    mlp = M.MLP1D(hid, 4.0, act, dtype=dtype, disable_past_cache=True).cuda()
    assert (mlp._epilogue is None) == (act_name == "gelu")
    _init(mlp, 51)
    g = torch.Generator().manual_seed(52)
    x = torch.randn(1, rows, hid, generator=g).to(dtype)
    got = mlp(x.cuda()).float().cpu()
    want = models.mlp_forward(x, _fp32_params(mlp), act)
    tol = {torch.float16: 6e-3, torch.float32: 2e-4}[dtype]
    assert max_abs(got, want) <= tol * max(1.0, float(want.abs().max()))


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_packed_stack_prefill_and_decode(dtype):
    """Three blocks with the padding dropped once for all of them, then two decode steps, against the
    reference blocks chained on the padded batch."""
    _, M = _mods()
    B, S, hid, heads, L = 3, 48, 128, 2, 3
    lens = [48, 5, 30]
    announce("stack", dtype)
    blocks = [M.Block1D(hid, heads, 4.0, activation=F.relu, dtype=dtype, max_seq_len=64) for _ in range(L)]
    stack = M.PackedStack(blocks).cuda()
    for i, blk in enumerate(stack.blocks):
        _init(blk, 60 + i)
    ps = [_fp32_params(blk) for blk in stack.blocks]
    x, valid = _padded_batch(B, S, hid, lens, True, dtype, 70)
    tol = {torch.float16: 4e-2, torch.float32: 2e-3}[dtype]

    def reference(x, valid):
        h = x.float()
        for p in ps:
            h = models.block_forward(h, p, heads, 1e-5, False, True, models.additive_mask(valid), F.relu)
        return h

    mask = models.additive_mask(valid)
    got = stack(x.cuda(), attention_mask=mask.to(dtype).cuda(), first_cache=True).float().cpu()
    want = reference(x, valid)
    scale = max(1.0, float(_valid_rows(want, lens, True).abs().max()))
    assert max_abs(_valid_rows(got, lens, True), _valid_rows(want, lens, True)) <= tol * scale
    g = torch.Generator().manual_seed(71)
    for step in range(2):
        x = torch.cat((x, torch.randn(B, 1, hid, generator=g).to(dtype)), 1)
        valid = torch.cat((valid, torch.ones(B, 1)), 1)
        got = stack(x.cuda(), attention_mask=models.additive_mask(valid).to(dtype).cuda(), first_cache=False)
        want = reference(x, valid)
        assert got.shape == want.shape
        assert max_abs(got[:, -1].float().cpu(), want[:, -1]) <= tol * scale, step


@pytest.mark.parametrize("seed", list(range(10)))
def test_block_random_shapes(seed):
    """Block1D on drawn shapes (head sizes 32 / 64 / 80 / 128, pre- or post-LN, ReLU / tanh-GELU / erf-GELU,
    fused or separate projections): prefill, then two incremental steps, against the reference block."""
    import functools
    _, M = _mods()
    g = torch.Generator().manual_seed(9100 + seed)
    ri = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))
    heads, D = ri(1, 4), [32, 64, 80, 128][ri(0, 3)]
    hid = heads * D
    B, S = ri(1, 5), ri(2, 90)
    dtype = [torch.float16, torch.float32, torch.bfloat16][ri(0, 2)]
    post, fused_qkv = bool(ri(0, 1)), bool(ri(0, 1))
    act_name = ["relu", "gelu_tanh", "gelu"][ri(0, 2)]
    act = {"relu": F.relu, "gelu_tanh": functools.partial(F.gelu, approximate="tanh"), "gelu": F.gelu}[act_name]
    lens = [ri(1, S) for _ in range(B)]
    lens[ri(0, B - 1)] = S
    announce("block random", seed, B, S, heads, D, dtype, post, fused_qkv, act_name, lens)
    blk = M.Block1D(hid, heads, 4.0, activation=act, dtype=dtype, apply_post_layernorm=post, max_seq_len=S + 8,
                    fused_qkv=fused_qkv).cuda()
    _init(blk, 9200 + seed)
    p = _fp32_params(blk)
    x, valid = _padded_batch(B, S, hid, lens, True, dtype, 9300 + seed)
    tol = {torch.float16: 2e-2, torch.bfloat16: 1.5e-1, torch.float32: 1e-3}[dtype]
    mask = models.additive_mask(valid)
    got = blk(x.cuda(), attention_mask=mask.to(dtype).cuda(), first_cache=True).float().cpu()
    want = models.block_forward(x, p, heads, 1e-5, post, True, mask, activation=act, fused_qkv=fused_qkv)
    ref_scale = max(1.0, float(want.abs().max()))
    assert max_abs(_valid_rows(got, lens, True), _valid_rows(want, lens, True)) <= tol * ref_scale
    for step in range(2):
        x = torch.cat((x, torch.randn(B, 1, hid, generator=g).to(dtype)), 1)
        valid = torch.cat((valid, torch.ones(B, 1)), 1)
        mask = models.additive_mask(valid)
        got = blk(x.cuda(), attention_mask=mask.to(dtype).cuda(), first_cache=False).float().cpu()
        want = models.block_forward(x, p, heads, 1e-5, post, True, mask, activation=act, fused_qkv=fused_qkv)
        assert max_abs(got[:, -1], want[:, -1]) <= tol * ref_scale, step
