"""K/V caches kept in pages of a shared pool: prefill, append and the single-pass decode attention over the pages,
against the float64 oracle of the contiguous cache (the reference's recompute, energonai/model/attention.py:61-71,
106-118, restated in oracle.eager.decode_attention) and bit for bit against the contiguous-cache kernels."""
import pytest
import torch

from gpu_util import announce, assert_ctx_close, max_abs
from oracle import eager, models

pytestmark = pytest.mark.gpu


def _mods():
    import energonai_amd.kernel as K
    import energonai_amd.model as M
    return K, M


def _scatter(cache, lens, P, pool_pages, g):
    """Host-side paging of a contiguous [B,H,S,D] cache: random distinct page ids, NaN in every pool row that holds
    no cached position.  Returns (pool [pages,H,P,D], table [B, max_pages])."""
    B, H, S, D = cache.shape
    max_pages = (S + P - 1) // P
    need = sum((n + P - 1) // P for n in lens)
    assert need <= pool_pages
    ids = torch.randperm(pool_pages, generator=g)[:need].tolist()
    pool = torch.full((pool_pages, H, P, D), float("nan"), dtype=cache.dtype)
    table = torch.full((B, max_pages), -1, dtype=torch.int32)
    for b, n in enumerate(lens):
        for pi in range((n + P - 1) // P):
            pid = ids.pop()
            table[b, pi] = pid
            rows = min(P, n - pi * P)
            pool[pid, :, :rows] = cache[b, :, pi * P:pi * P + rows]
    return pool, table


PAGED_CASES = [
    # B, H, S (capacity), D, page, lengths
    (5, 4, 640, 128, 64, [640, 1, 63, 64, 65]),
    (9, 3, 2048, 128, 64, [3, 1989, 2048, 1, 0, 777, 1024, 65, 64]),    # keys shared between workgroups, an empty cache
    (2, 2, 320, 96, 16, [300, 131]),                                    # twelve vectors per key on sixteen lanes
    (3, 2, 256, 32, 16, [17, 256, 100]),                                # four lanes per key: a wave's 16 keys fill a page
    (1, 2, 5120, 64, 16, [4999]),                                       # 313 pages: the wave's page ids are refilled
    (40, 16, 512, 64, 256, None),                                       # 640 units: nothing is shared
    (2, 8, 4096, 128, 256, [4096, 2500]),
]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("B,H,S,D,P,kv", PAGED_CASES)
def test_decode_attn_paged(dtype, B, H, S, D, P, kv):
    K, _ = _mods()
    g = torch.Generator().manual_seed(3 * S + D + B + P)
    if kv is None:
        kv = torch.randint(0, S + 1, (B,), generator=g).tolist()
    announce("decode attn paged", dtype, B, H, S, D, P, kv[:12])
    q = torch.randn(B, H, 1, D, generator=g).to(dtype)
    kc = torch.randn(B, H, S, D, generator=g).to(dtype)
    vc = torch.randn(B, H, S, D, generator=g).to(dtype)
    for b, n in enumerate(kv):
        kc[b, :, n:] = float("nan")
        vc[b, :, n:] = float("nan")
    pool_pages = B * ((S + P - 1) // P) + 7
    k_pool, table = _scatter(kc, kv, P, pool_pages, torch.Generator().manual_seed(5))
    v_pool, table_v = _scatter(vc, kv, P, pool_pages, torch.Generator().manual_seed(5))
    assert torch.equal(table, table_v)
    kv_t = torch.tensor(kv, dtype=torch.int32).cuda()
    scale = D ** -0.5
    _, _, want = eager.decode_attention(q, torch.nan_to_num(kc, nan=0.0), torch.nan_to_num(vc, nan=0.0), kv, scale,
                                        acc_dtype=torch.float64)
    for b, n in enumerate(kv):
        if n == 0:
            want[b] = 0
    out = torch.full((B, H, 1, D), 777.0, dtype=dtype, device="cuda")
    got = K.decode_attn_paged(q.cuda(), k_pool.cuda(), v_pool.cuda(), kv_t, table.cuda(), scale=scale, out=out)
    assert got.data_ptr() == out.data_ptr()
    assert_ctx_close(got.cpu(), want, dtype, "decode_attn_paged")
    # the same kernel on the contiguous cache takes every key on the same lanes in the same order
    flat = K.decode_attn(q.cuda(), kc.cuda(), vc.cuda(), kv_t, scale=scale)
    assert torch.equal(got, flat)
    one_wg = K.decode_attn_paged(q.cuda(), k_pool.cuda(), v_pool.cuda(), kv_t, table.cuda(), scale=scale, split=False)
    assert_ctx_close(one_wg.cpu(), want, dtype, "decode_attn_paged, one workgroup per unit")
    # K and V as two halves of one pool [pages, 2, H, P, D]
    both = torch.stack([k_pool, v_pool], dim=1).cuda()
    got2 = K.decode_attn_paged(q.cuda(), both[:, 0], both[:, 1], kv_t, table.cuda(), scale=scale)
    assert torch.equal(got2, got)


def test_decode_attn_paged_treats_ids_outside_the_pool_as_zero_rows():
    """A table entry that names no page of the pool (-1, or past its end) must not be followed: the positions it
    covers read as zero keys and zero values."""
    K, _ = _mods()
    B, H, S, D, P = 3, 2, 256, 64, 32
    kv = [256, 100, 33]
    g = torch.Generator().manual_seed(9)
    q = torch.randn(B, H, 1, D, generator=g).half()
    kc = torch.randn(B, H, S, D, generator=g).half()
    vc = torch.randn(B, H, S, D, generator=g).half()
    pool_pages = 40
    k_pool, table = _scatter(kc, kv, P, pool_pages, torch.Generator().manual_seed(1))
    v_pool, _ = _scatter(vc, kv, P, pool_pages, torch.Generator().manual_seed(1))
    announce("decode attn paged, bad ids")
    table[0, 3] = -1
    table[1, 1] = pool_pages          # one past the last page
    table[2, 0] = 1 << 30
    for b, pi in ((0, 3), (1, 1), (2, 0)):
        kc[b, :, pi * P:(pi + 1) * P] = 0
        vc[b, :, pi * P:(pi + 1) * P] = 0
    _, _, want = eager.decode_attention(q, kc, vc, kv, D ** -0.5, acc_dtype=torch.float64)
    got = K.decode_attn_paged(q.cuda(), torch.nan_to_num(k_pool).cuda(), torch.nan_to_num(v_pool).cuda(),
                              torch.tensor(kv, dtype=torch.int32).cuda(), table.cuda())
    assert_ctx_close(got.cpu(), want, torch.float16, "decode_attn_paged with ids outside the pool")


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_pages_fill_and_append_bit_exact(dtype):
    """Prefill from the k and v thirds of a fused projection, then appends across a page boundary, against plain
    indexing; rows that belong to no position keep their bytes; a sequence without a page for its next position is
    counted and left alone."""
    K, _ = _mods()
    B, H, D, P, S = 4, 3, 64, 16, 80
    lens = [31, 16, 1, 48]
    T = sum(lens)
    g = torch.Generator().manual_seed(2)
    announce("pages fill/append", dtype)
    kvq = torch.randn(T, 3 * H, D, generator=g).to(dtype)
    max_pages = S // P
    pool_pages = 24
    table = torch.full((B, max_pages), -1, dtype=torch.int32)
    ids = torch.randperm(pool_pages, generator=g).tolist()
    for b, n in enumerate(lens):
        for pi in range(n // P + 1):                      # room for the next position as well
            table[b, pi] = ids.pop()
    table[2, 0] = -1                                      # sequence 2 has no page at all
    lens_t = torch.tensor(lens, dtype=torch.int32).cuda()
    sentinel = 3.0
    k_pool = torch.full((pool_pages, H, P, D), sentinel, dtype=dtype).cuda()
    v_pool = torch.full((pool_pages, H, P, D), sentinel, dtype=dtype).cuda()
    over = torch.zeros(1, dtype=torch.int32).cuda()
    K.kv_pages_fill(kvq.cuda(), k_pool, B, S, lens_t, table.cuda(), 0, overflow=over)
    K.kv_pages_fill(kvq.cuda(), v_pool, B, S, lens_t, table.cuda(), H, overflow=over)
    want_k = torch.full((pool_pages, H, P, D), sentinel, dtype=dtype)
    want_v = want_k.clone()
    t0 = 0
    for b, n in enumerate(lens):
        for s in range(n):
            pid = int(table[b, s // P])
            if pid >= 0:
                want_k[pid, :, s % P] = kvq[t0 + s, :H]
                want_v[pid, :, s % P] = kvq[t0 + s, H:2 * H]
        t0 += n
    assert torch.equal(k_pool.cpu(), want_k) and torch.equal(v_pool.cpu(), want_v)
    assert int(over.item()) == 2                          # the one row of sequence 2, once per fill
    cur = list(lens)
    for step in range(3):
        new = torch.randn(B, 3 * H, D, generator=g).to(dtype).cuda()
        over.zero_()
        K.kv_pages_append(new[:, :H], new[:, H:2 * H], k_pool, v_pool, torch.tensor(cur, dtype=torch.int32).cuda(),
                          table.cuda(), overflow=over)
        lost = 0
        for b, n in enumerate(cur):
            pid = int(table[b, n // P]) if n // P < max_pages else -1
            if pid >= 0:
                want_k[pid, :, n % P] = new[b, :H].cpu()
                want_v[pid, :, n % P] = new[b, H:2 * H].cpu()
            else:
                lost += 1
        assert torch.equal(k_pool.cpu(), want_k) and torch.equal(v_pool.cpu(), want_v), step
        assert int(over.item()) == lost, step
        cur = [n + 1 for n in cur]
    # in the last step: sequence 2 (never had a page) and sequence 0, which passed position 32 without a third page
    assert lost == 2


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_block_decodes_the_same_from_pages(dtype):
    """Block1D with its K/V cache in pages of 16 positions: prefill and five decode steps (sequences cross page
    boundaries) give the bits of the block that keeps [B,H,Smax,D] caches, and stay within the model tolerance of
    the float reference block."""
    _, M = _mods()
    B, S, hid, heads = 3, 70, 128, 2
    lens = [70, 9, 41]
    announce("block decode from pages", dtype)
    flat = M.Block1D(hid, heads, 4.0, dtype=dtype, max_seq_len=96).cuda()
    paged = M.Block1D(hid, heads, 4.0, dtype=dtype, max_seq_len=96, kv_page_size=16, kv_pool_pages=12).cuda()
    g = torch.Generator().manual_seed(31)
    with torch.no_grad():
        for name, prm in flat.named_parameters():
            if prm.dim() > 1:
                prm.copy_(torch.randn(prm.shape, generator=g) / prm.shape[1] ** 0.5)
            else:
                prm.copy_((1.0 if name.endswith("weight") else 0.0) + 0.05 * torch.randn(prm.shape, generator=g))
    paged.load_state_dict(flat.state_dict())
    p = {k: v.detach().float().cpu() for k, v in flat.state_dict().items()}
    x = torch.randn(B, S, hid, generator=g).to(dtype)
    valid = torch.zeros(B, S)
    for b, n in enumerate(lens):
        valid[b, S - n:] = 1
    x = x * valid.unsqueeze(-1).to(dtype)
    tol = {torch.float16: 1.5e-2, torch.float32: 5e-4}[dtype]
    mask = models.additive_mask(valid)
    a = flat(x.cuda(), attention_mask=mask.to(dtype).cuda(), first_cache=True)
    b_ = paged(x.cuda(), attention_mask=mask.to(dtype).cuda(), first_cache=True)
    assert torch.equal(a, b_)
    cache = paged.attn.kv_cache
    assert cache.pages_in_use() == sum((n + 15) // 16 for n in lens) == 9
    for step in range(5):
        x = torch.cat((x, torch.randn(B, 1, hid, generator=g).to(dtype)), 1)
        valid = torch.cat((valid, torch.ones(B, 1)), 1)
        mask = models.additive_mask(valid)
        a = flat(x.cuda(), attention_mask=mask.to(dtype).cuda(), first_cache=False)
        b_ = paged(x.cuda(), attention_mask=mask.to(dtype).cuda(), first_cache=False)
        assert torch.equal(a[:, -1], b_[:, -1]), step
        want = models.block_forward(x, p, heads, 1e-5, False, True, mask)
        assert max_abs(b_[:, -1].float().cpu(), want[:, -1]) <= tol, step
    # 70 -> 75, 9 -> 14, 41 -> 46: no new page; a sixth and seventh step take sequence 1 to 16 and need one
    assert cache.pages_in_use() == 9
    for step in range(3):
        x = torch.cat((x, torch.randn(B, 1, hid, generator=g).to(dtype)), 1)
        valid = torch.cat((valid, torch.ones(B, 1)), 1)
        mask = models.additive_mask(valid)
        a = flat(x.cuda(), attention_mask=mask.to(dtype).cuda(), first_cache=False)
        b_ = paged(x.cuda(), attention_mask=mask.to(dtype).cuda(), first_cache=False)
        assert torch.equal(a[:, -1], b_[:, -1]), step
    assert cache.pages_in_use() == 11                    # sequence 1 passed 16, sequence 2 passed 48
    cache.release(1)                                     # a finished sequence hands its two pages back
    assert cache.pages_in_use() == 9


@pytest.mark.parametrize("seed", list(range(12)))
def test_decode_attn_paged_random_shapes(seed):
    """Random batch, heads, head size, page size, capacity and lengths: pages against the float64 oracle and against
    the contiguous-cache kernel bit for bit."""
    K, _ = _mods()
    g = torch.Generator().manual_seed(1000 + seed)
    pick = lambda xs: xs[int(torch.randint(0, len(xs), (1,), generator=g))]
    dtype = pick([torch.float16, torch.bfloat16, torch.float32])
    D = pick([32, 64, 80, 96, 128] if dtype != torch.float32 else [32, 64, 96, 128])
    P = pick([16, 32, 64, 128])
    B = int(torch.randint(1, 20, (1,), generator=g))
    H = int(torch.randint(1, 9, (1,), generator=g))
    S = P * int(torch.randint(1, max(2, 3000 // P), (1,), generator=g))
    kv = torch.randint(0, S + 1, (B,), generator=g).tolist()
    announce("decode attn paged random", seed, dtype, B, H, S, D, P, kv[:8])
    q = torch.randn(B, H, 1, D, generator=g).to(dtype)
    kc = torch.randn(B, H, S, D, generator=g).to(dtype)
    vc = torch.randn(B, H, S, D, generator=g).to(dtype)
    for b, n in enumerate(kv):
        kc[b, :, n:] = float("nan")
        vc[b, :, n:] = float("nan")
    pool_pages = B * (S // P) + 3
    k_pool, table = _scatter(kc, kv, P, pool_pages, torch.Generator().manual_seed(seed))
    v_pool, _ = _scatter(vc, kv, P, pool_pages, torch.Generator().manual_seed(seed))
    kv_t = torch.tensor(kv, dtype=torch.int32).cuda()
    scale = D ** -0.5
    _, _, want = eager.decode_attention(q, torch.nan_to_num(kc, nan=0.0), torch.nan_to_num(vc, nan=0.0), kv, scale,
                                        acc_dtype=torch.float64)
    for b, n in enumerate(kv):
        if n == 0:
            want[b] = 0
    got = K.decode_attn_paged(q.cuda(), k_pool.cuda(), v_pool.cuda(), kv_t, table.cuda(), scale=scale)
    assert_ctx_close(got.cpu(), want, dtype, "decode_attn_paged")
    assert torch.equal(got, K.decode_attn(q.cuda(), kc.cuda(), vc.cuda(), kv_t, scale=scale))


def test_stack_of_blocks_on_pages():
    """Two blocks behind one depad, both with paged caches: the lengths are copied to the host once for both
    (SeqInfo.lens_host), and prefill plus four decode steps give the bits of the same stack on contiguous caches."""
    _, M = _mods()
    from energonai_amd.seqinfo import seq_info
    B, S, hid, heads = 4, 40, 128, 4
    lens = [40, 7, 16, 33]
    announce("stack on pages")
    dtype = torch.float16

    def stack(**kw):
        return M.PackedStack([M.Block1D(hid, heads, 4.0, dtype=dtype, max_seq_len=64, **kw) for _ in range(2)]).cuda()
    flat, paged = stack(), stack(kv_page_size=16)
    g = torch.Generator().manual_seed(77)
    with torch.no_grad():
        for name, prm in flat.named_parameters():
            if prm.dim() > 1:
                prm.copy_(torch.randn(prm.shape, generator=g) / prm.shape[1] ** 0.5)
            else:
                prm.copy_((1.0 if name.endswith("weight") else 0.0) + 0.05 * torch.randn(prm.shape, generator=g))
    paged.load_state_dict(flat.state_dict())
    x = torch.randn(B, S, hid, generator=g).to(dtype)
    valid = torch.zeros(B, S)
    for b, n in enumerate(lens):
        valid[b, S - n:] = 1
    x = x * valid.unsqueeze(-1).to(dtype)
    lens_t = torch.tensor(lens, dtype=torch.int32).cuda()
    a = flat(x.cuda(), first_cache=True, seq_lens=lens_t)
    b_ = paged(x.cuda(), first_cache=True, seq_lens=lens_t)
    assert torch.equal(a, b_)
    info = seq_info(lens_t, B, lens_t.device)
    assert info.lens_host() == lens and info._lens_host is not None
    for blk in paged.blocks:
        assert blk.attn.kv_cache.pages_in_use() == sum((n + 15) // 16 for n in lens)
    for step in range(4):
        x = torch.cat((x, torch.randn(B, 1, hid, generator=g).to(dtype)), 1)
        a = flat(x.cuda(), first_cache=False)
        b_ = paged(x.cuda(), first_cache=False)
        assert torch.equal(a[:, -1], b_[:, -1]), step
