"""GPU parity: QK^T, PV and their single-query decode forms against the fp32/fp64 oracle.

fp16: max-abs error <= 2e-3 on probabilities-weighted outputs (north-star
tolerance); raw scores are compared relative to their fp16 rounding step.
fp32: 1e-5 relative to the score scale.
"""
import pytest
import torch

from gpu_util import BASE, announce, assert_ctx_close, assert_stored_close, max_abs, pad_bhsd, packed_randn
from oracle import eager

pytestmark = pytest.mark.gpu


def _kernel():
    from energonai_amd import kernel
    return kernel


def _visible_mask(B, H, Sq, Sk, k_lens, q_lens, causal):
    m = torch.zeros(B, H, Sq, Sk, dtype=torch.bool)
    for b in range(B):
        for q in range(min(q_lens[b], Sq)):
            n = eager.visible_keys(q, q_lens[b], k_lens[b], causal)
            m[b, :, q, :n] = True
    return m


ATTN_CASES = [
    # B, H, S, D, lens
    (8, 12, 128, 64, [24, 127, 31, 65, 24, 127, 31, 65]),
    (2, 3, 256, 128, [256, 129]),
    (3, 2, 200, 64, [200, 0, 77]),       # S not a multiple of the tile, an empty sequence
    (2, 2, 384, 32, [300, 1]),           # head dim below the tile's 64
    (1, 2, 520, 80, [515]),              # OPT-2.7B head dim: padded to 128 inside the kernel
    (9, 1, 130, 128, [130, 5, 64, 65, 127, 128, 129, 1, 33]),   # more units than XCDs, odd split
    # head sizes between the two tile widths: the 16-byte chunks past the head must arrive as zeros, for every
    # remainder and in each of the swizzled slot positions
    (2, 1, 200, 72, [200, 131]),
    (1, 3, 136, 96, [133]),
    (2, 2, 264, 104, [264, 9]),
    (1, 1, 328, 120, [321]),
    (2, 2, 136, 40, [136, 70]),
    (1, 2, 72, 8, [65]),
]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("B,H,S,D,lens", ATTN_CASES)
def test_attn_qk_pv_fused_layout(dtype, causal, B, H, S, D, lens):
    """q/k/v are the strided chunk views of the fused [B,H,S,3D] buffer, as in the reference callers."""
    k = _kernel()
    announce("attn", dtype, causal, B, H, S, D, lens)
    T = sum(lens)
    qkv_packed = packed_randn(max(T, 1), H * 3 * D, dtype, 100 + S)[:T].reshape(T, H, 3 * D)
    qkv = pad_bhsd(qkv_packed, lens, S, H, 3 * D)
    q, kk, v = torch.chunk(qkv, 3, dim=-1)
    lens_t = torch.tensor(lens, dtype=torch.int32).cuda()
    qkv_g = qkv.cuda()
    qg, kg, vg = torch.chunk(qkv_g, 3, dim=-1)
    assert not qg.is_contiguous() or D * 3 == D

    # ---- QK^T
    sentinel = 777.0
    out = torch.full((B, H, S, S), sentinel, dtype=dtype, device="cuda")
    scores = k.attn_qk(qg, kg, lens_t, causal=causal, out=out).cpu()
    want_scores = eager.attn_qk(q, kk, torch.float64)
    vis = _visible_mask(B, H, S, S, lens, lens, causal)
    step = {torch.float16: 2.0 ** -11, torch.bfloat16: 2.0 ** -8, torch.float32: 2.0 ** -16}[dtype]
    if vis.any():
        rel = ((scores.double() - want_scores).abs() / (want_scores.abs() + 1.0))[vis].max().item()
        assert rel <= 1.5 * step, rel
    # rows of padded queries are never written
    rows_pad = torch.ones(B, H, S, dtype=torch.bool)
    for b, n in enumerate(lens):
        rows_pad[b, :, :n] = False
    assert bool((scores[rows_pad] == sentinel).all())

    # ---- PV on oracle probabilities (so the two kernels are checked independently)
    probs64 = eager.scale_mask_softmax(B, S, H, want_scores, lens, scale=D ** -0.5, causal=causal,
                                       acc_dtype=torch.float64, out_dtype=torch.float64)
    probs = probs64.to(dtype)
    for b, n in enumerate(lens):      # garbage in the rows of padded queries must not matter
        probs[b, :, n:, :] = float("nan")
    ctx_out = torch.full((B, H, S, D), sentinel, dtype=dtype, device="cuda")
    ctx = k.attn_pv(probs.cuda(), vg, lens_t, causal=causal, out=ctx_out).cpu()
    want_ctx = eager.attn_pv(torch.nan_to_num(probs, nan=0.0), v, torch.float64)
    rows_ok = ~rows_pad
    if rows_ok.any():
        assert_ctx_close(ctx[rows_ok], want_ctx[rows_ok], dtype, "attn_pv")
    assert bool((ctx[rows_pad] == sentinel).all())
    # zero_padding writes zeros there instead
    ctx0 = k.attn_pv(probs.cuda(), vg, lens_t, causal=causal, zero_padding=True).cpu()
    assert bool((ctx0[rows_pad] == 0).all())
    if rows_ok.any():
        assert torch.equal(ctx0[rows_ok], ctx[rows_ok])


def test_attn_nan_in_padding_of_v_is_ignored():
    """Cache rows past the valid length may hold anything (torch.empty caches)."""
    k = _kernel()
    B, H, S, D = 2, 2, 192, 64
    lens = [100, 192]
    announce("attn nan padding")
    g = torch.Generator().manual_seed(4)
    q = torch.randn(B, H, S, D, generator=g).half()
    kk = torch.randn(B, H, S, D, generator=g).half()
    v = torch.randn(B, H, S, D, generator=g).half()
    for b, n in enumerate(lens):
        kk[b, :, n:] = float("nan")
        v[b, :, n:] = float("nan")
    lens_t = torch.tensor(lens, dtype=torch.int32).cuda()
    scores = k.attn_qk(q.cuda(), kk.cuda(), lens_t, causal=True)
    probs = k.scale_mask_softmax(B, S, H, scores, lens_t, scale=0.125)
    ctx = k.attn_pv(probs, v.cuda(), lens_t, causal=True).cpu()
    for b, n in enumerate(lens):
        assert torch.isfinite(ctx[b, :, :n]).all()


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("causal", [True, False])
def test_attn_pv_reads_a_row_only_as_far_as_its_query_sees(dtype, causal):
    """The score buffer comes from torch.empty and the softmax with tail_rows=1 writes the visible prefix of a
    row only: NaNs parked everywhere else (past the last 16-byte vector with a visible key, and in the rows of
    padded queries) must not reach the context."""
    k = _kernel()
    B, H, S, D = 3, 2, 328, 64
    lens = [328, 131, 9]
    epv = 16 // torch.empty(0, dtype=dtype).element_size()
    announce("attn pv row extent", dtype, causal)
    g = torch.Generator().manual_seed(8)
    p = torch.rand(B, H, S, S, generator=g).to(dtype)
    v = torch.randn(B, H, S, D, generator=g).to(dtype)
    clean = torch.zeros_like(p)
    dirty = torch.full_like(p, float("nan"))
    for b, n in enumerate(lens):
        for q in range(n):
            vis = min(n, q + 1) if causal else n
            clean[b, :, q, :vis] = p[b, :, q, :vis]
            dirty[b, :, q, :vis] = p[b, :, q, :vis]
            dirty[b, :, q, vis:-(-vis // epv) * epv] = 0      # the softmax completes the last vector with zeros
    lens_t = torch.tensor(lens, dtype=torch.int32).cuda()
    want = k.attn_pv(clean.cuda(), v.cuda(), lens_t, causal=causal).cpu()
    got = k.attn_pv(dirty.cuda(), v.cuda(), lens_t, causal=causal).cpu()
    for b, n in enumerate(lens):
        assert torch.equal(got[b, :, :n], want[b, :, :n])


DECODE_CASES = [
    # B, H, Smax, D, kv lens
    (5, 4, 640, 128, [640, 1, 333, 64, 65]),
    (3, 2, 100, 64, [100, 17, 2]),
    (2, 3, 77, 32, [77, 40]),
    (3, 4, 200, 80, [200, 1, 77]),        # OPT-2.7B head size: ten vectors per key, run on sixteen lanes
    (4, 72, 2048, 128, [2048, 3, 1024, 1989]),
]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("B,H,S,D,kv", DECODE_CASES)
def test_decode_qk_pv(dtype, B, H, S, D, kv):
    k = _kernel()
    announce("decode", dtype, B, H, S, D, kv)
    g = torch.Generator().manual_seed(S + D)
    q = torch.randn(B, H, 1, D, generator=g).to(dtype)
    kc = torch.randn(B, H, S, D, generator=g).to(dtype)
    vc = torch.randn(B, H, S, D, generator=g).to(dtype)
    for b, n in enumerate(kv):           # unused cache rows hold garbage
        kc[b, :, n:] = float("nan")
        vc[b, :, n:] = float("nan")
    kv_t = torch.tensor(kv, dtype=torch.int32).cuda()
    scale = D ** -0.5
    want_scores, want_probs, want_ctx = eager.decode_attention(
        q, torch.nan_to_num(kc, nan=0.0), torch.nan_to_num(vc, nan=0.0), kv, scale, acc_dtype=torch.float64)
    scores = k.decode_qk(q.cuda(), kc.cuda(), kv_t)
    assert scores.shape == (B, H, 1, S)
    vis = torch.zeros(B, H, 1, S, dtype=torch.bool)
    for b, n in enumerate(kv):
        vis[b, :, :, :n] = True
    step = {torch.float16: 2.0 ** -11, torch.bfloat16: 2.0 ** -8, torch.float32: 2.0 ** -16}[dtype]
    rel = ((scores.cpu().double() - want_scores).abs() / (want_scores.abs() + 1.0))[vis].max().item()
    assert rel <= 1.5 * step, rel
    probs = k.scale_mask_softmax(B, 1, H, scores, kv_t, scale=scale, k_seq_len=S,
                                 q_len_list=torch.ones(B, dtype=torch.int32).cuda())
    tol = {torch.float16: 2e-3, torch.bfloat16: 1.6e-2, torch.float32: 1e-5}[dtype]
    assert max_abs(probs.cpu(), want_probs) <= tol
    ctx = k.decode_pv(probs, vc.cuda(), kv_t).cpu()
    assert ctx.shape == (B, H, 1, D)
    assert_ctx_close(ctx, want_ctx, dtype, "decode_pv")


DECODE_ATTN_CASES = DECODE_CASES + [
    (9, 3, 2048, 128, [3, 1989, 2048, 1, 0, 777, 1024, 65, 64]),   # an empty cache among full and short ones
    (2, 2, 300, 96, [300, 131]),                                     # twelve vectors per key on sixteen lanes
    (300, 1, 40, 64, None),                                          # more sequences than are ranked by length
    (1, 2, 5000, 64, [4999]),                                        # a single sequence (no ranking), a long cache
]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("B,H,S,D,kv", DECODE_ATTN_CASES)
def test_decode_attn_single_pass(dtype, B, H, S, D, kv):
    """QK^T, softmax and PV of the decode step in one kernel against the float64 oracle (the last row of the
    reference's recompute), NaN in every cache row past a sequence's length."""
    k = _kernel()
    g = torch.Generator().manual_seed(7 * S + D + B)
    if kv is None:
        kv = torch.randint(0, S + 1, (B,), generator=g).tolist()
    announce("decode attn", dtype, B, H, S, D, kv[:12])
    q = torch.randn(B, H, 1, D, generator=g).to(dtype)
    kc = torch.randn(B, H, S, D, generator=g).to(dtype)
    vc = torch.randn(B, H, S, D, generator=g).to(dtype)
    for b, n in enumerate(kv):
        kc[b, :, n:] = float("nan")
        vc[b, :, n:] = float("nan")
    kv_t = torch.tensor(kv, dtype=torch.int32).cuda()
    scale = D ** -0.5
    _, _, want = eager.decode_attention(q, torch.nan_to_num(kc, nan=0.0), torch.nan_to_num(vc, nan=0.0), kv, scale,
                                        acc_dtype=torch.float64)
    for b, n in enumerate(kv):
        if n == 0:
            want[b] = 0          # no key to attend to: a zero row (the oracle's softmax of nothing is NaN)
    out = torch.full((B, H, 1, D), 777.0, dtype=dtype, device="cuda")
    got = k.decode_attn(q.cuda(), kc.cuda(), vc.cuda(), kv_t, scale=scale, out=out)
    assert got.data_ptr() == out.data_ptr()
    assert_ctx_close(got.cpu(), want, dtype, "decode_attn")
    # the caches as strided views of one [B,H,S,2D] buffer, K and V interleaved per position
    both = torch.cat([kc, vc], dim=-1).cuda()
    got2 = k.decode_attn(q.cuda(), both[..., :D], both[..., D:], kv_t, scale=scale)
    assert torch.equal(got2, got)
    # small batches share a unit's keys between workgroups (partial results through a workspace, then a combine
    # kernel); with one workgroup per unit the result meets the same bound, and a caller's own workspace gives the
    # bits of the temporary one
    one_wg = k.decode_attn(q.cuda(), kc.cuda(), vc.cuda(), kv_t, scale=scale, split=False)
    assert_ctx_close(one_wg.cpu(), want, dtype, "decode_attn, one workgroup per unit")
    need = k.decode_attn_workspace_bytes(B, H, S, D)
    assert (need > 0) == (B * H < 512 and S >= 1024)
    if need:
        ws = torch.full((need + 64,), 0xFF, dtype=torch.uint8, device="cuda")
        got3 = k.decode_attn(q.cuda(), kc.cuda(), vc.cuda(), kv_t, scale=scale, workspace=ws)
        assert torch.equal(got3, got)
        assert bool((ws[need:] == 0xFF).all())


def test_decode_attn_agrees_with_the_three_launch_route():
    """decode_qk -> scale_mask_softmax -> decode_pv store scores and probabilities in fp16 on the way; the single
    pass keeps them in fp32.  Both meet the bound against the oracle, so they agree within twice that bound."""
    k = _kernel()
    B, H, S, D = 6, 8, 1024, 128
    kv = [1024, 5, 600, 77, 1, 333]
    announce("decode attn vs three launches")
    g = torch.Generator().manual_seed(4)
    q, kc, vc = (torch.randn(B, H, n, D, generator=g).half().cuda() for n in (1, S, S))
    kv_t = torch.tensor(kv, dtype=torch.int32).cuda()
    one = k.decode_attn(q, kc, vc, kv_t)
    scores = k.decode_qk(q, kc, kv_t)
    probs = k.scale_mask_softmax(B, 1, H, scores, kv_t, scale=D ** -0.5, k_seq_len=S,
                                 q_len_list=torch.ones(B, dtype=torch.int32).cuda())
    three = k.decode_pv(probs, vc, kv_t)
    assert_stored_close(one.cpu(), three.cpu().double(), torch.float16, base=2 * BASE[torch.float16],
                        what="single pass vs three launches")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("B,H,S,D,lens", ATTN_CASES)
def test_attn_fused(dtype, causal, B, H, S, D, lens):
    """One kernel for QK^T + mask/softmax + PV against the float64 oracle of the three steps."""
    k = _kernel()
    if dtype == torch.float32 and D > 64:
        with pytest.raises(RuntimeError, match="Datatype not implemented"):
            k.attn_fused(*(torch.zeros(B, H, S, D, device="cuda") for _ in range(3)), torch.tensor(lens).cuda())
        return
    announce("attn fused", dtype, causal, B, H, S, D, lens)
    T = sum(lens)
    qkv_packed = packed_randn(max(T, 1), H * 3 * D, dtype, 300 + S)[:T].reshape(T, H, 3 * D)
    qkv = pad_bhsd(qkv_packed, lens, S, H, 3 * D)
    for b, n in enumerate(lens):              # whatever sits in the padding must not matter
        qkv[b, :, n:] = float("nan")
    q, kk, v = torch.chunk(qkv, 3, dim=-1)
    lens_t = torch.tensor(lens, dtype=torch.int32).cuda()
    qg, kg, vg = torch.chunk(qkv.cuda(), 3, dim=-1)
    scale = D ** -0.5
    sentinel = 777.0
    out = torch.full((B, H, S, D), sentinel, dtype=dtype, device="cuda")
    ctx = k.attn_fused(qg, kg, vg, lens_t, scale=scale, causal=causal, out=out).cpu()
    qz, kz, vz = (torch.nan_to_num(t, nan=0.0) for t in (q, kk, v))
    scores = eager.attn_qk(qz, kz, torch.float64)
    probs = eager.scale_mask_softmax(B, S, H, scores, lens, scale=scale, causal=causal, acc_dtype=torch.float64,
                                     out_dtype=torch.float64)
    rows_pad = torch.ones(B, H, S, dtype=torch.bool)
    for b, n in enumerate(lens):
        rows_pad[b, :, :n] = False
        probs[b, :, n:] = 0
    want = eager.attn_pv(probs, vz, torch.float64)
    if (~rows_pad).any():
        assert_ctx_close(ctx[~rows_pad], want[~rows_pad], dtype, "attn_fused")
    assert bool((ctx[rows_pad] == sentinel).all())


@pytest.mark.parametrize("D", [64, 128, 40])
def test_attn_fused_and_pv_write_an_output_that_is_not_16_byte_aligned(D):
    """The whole-row output path needs 16-byte aligned rows; an output that is only 8-byte aligned (a view four
    elements into a wider tensor) takes the piecewise stores.  Both give the bits of the aligned call, and neither
    touches the columns beside the view or the rows of the padding."""
    k = _kernel()
    B, H, S = 3, 2, 200
    lens = [200, 77, 1]
    announce("unaligned ctx", D, lens)
    g = torch.Generator().manual_seed(31 + D)
    q, kk, v = (torch.randn(B, H, S, D, generator=g).half().cuda() for _ in range(3))
    lens_t = torch.tensor(lens, dtype=torch.int32).cuda()
    aligned = k.attn_fused(q, kk, v, lens_t, causal=True)
    wide = torch.full((B, H, S, D + 8), 5.0, dtype=torch.float16, device="cuda")
    view = wide[..., 4:4 + D]
    assert view.data_ptr() % 16 == 8
    k.attn_fused(q, kk, v, lens_t, causal=True, out=view)
    for b, n in enumerate(lens):
        assert torch.equal(view[b, :, :n], aligned[b, :, :n])
        assert bool((view[b, :, n:] == 5.0).all())
    assert bool((wide[..., :4] == 5.0).all()) and bool((wide[..., 4 + D:] == 5.0).all())
    # the same for PV on the probabilities of these scores
    scores = k.attn_qk(q, kk, lens_t, alpha=D ** -0.5, causal=True)
    probs = k.scale_mask_softmax(B, S, H, scores, lens_t)
    ctx_aligned = k.attn_pv(probs, v, lens_t, causal=True)
    wide.fill_(5.0)
    k.attn_pv(probs, v, lens_t, causal=True, out=view)
    for b, n in enumerate(lens):
        assert torch.equal(view[b, :, :n], ctx_aligned[b, :, :n])
    assert bool((wide[..., :4] == 5.0).all()) and bool((wide[..., 4 + D:] == 5.0).all())


# fp16 / bf16: every case; fp32: the cases with heads of up to 64 channels (what the fp32 fused kernel takes)
FUSED_PACKED_CASES = [(dt,) + c for dt in (torch.float16, torch.bfloat16) for c in ATTN_CASES] + \
                     [(torch.float32,) + c for c in ATTN_CASES if c[3] <= 64]


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("dtype,B,H,S,D,lens", FUSED_PACKED_CASES)
def test_attn_fused_packed(dtype, causal, B, H, S, D, lens):
    """The fused kernel addressing the packed [T,H,3D] projections and the packed [T,H*D] context
    directly: same result as pad -> attention -> depad, with no padded tensor in between."""
    k = _kernel()
    announce("attn fused packed", dtype, causal, B, H, S, D, lens)
    T = sum(lens)
    qkv_packed = packed_randn(max(T, 1), H * 3 * D, dtype, 400 + S)[:T].reshape(T, H, 3 * D)
    qkv = pad_bhsd(qkv_packed, lens, S, H, 3 * D)
    q, kk, v = torch.chunk(qkv, 3, dim=-1)
    scale = D ** -0.5
    scores = eager.attn_qk(q, kk, torch.float64)
    probs = eager.scale_mask_softmax(B, S, H, scores, lens, scale=scale, causal=causal, acc_dtype=torch.float64,
                                     out_dtype=torch.float64)
    for b, n in enumerate(lens):
        probs[b, :, n:] = 0
    ctx = eager.attn_pv(probs, v, torch.float64)
    want = torch.cat([ctx[b, :, :n].permute(1, 0, 2).reshape(n, H * D) for b, n in enumerate(lens)])
    sentinel = 555.0
    guard = torch.full((T + 2, H * D), sentinel, dtype=dtype, device="cuda")
    lens_t = torch.tensor(lens, dtype=torch.int64).cuda()
    got = k.attn_fused_packed(qkv_packed.reshape(1, T, H, 3 * D).cuda(), B, S, lens_t, H, D, scale=scale,
                              causal=causal, out=guard[1:T + 1])
    assert got.data_ptr() == guard[1:].data_ptr()
    g = guard.cpu()
    assert_ctx_close(g[1:T + 1], want, dtype, "attn_fused_packed")
    assert bool((g[0] == sentinel).all()) and bool((g[T + 1] == sentinel).all())


@pytest.mark.parametrize("slope", [0.002, 0.02, 0.3])
def test_attn_fused_growing_maximum(slope):
    """Scores that rise with the key index: the running maximum keeps moving, slowly (the kernel
    may keep an older maximum for a while) or by large steps (it must rescale every tile)."""
    k = _kernel()
    B, H, S, D = 2, 2, 512, 64
    lens = [512, 333]
    announce("attn fused growing max", slope)
    g = torch.Generator().manual_seed(5)
    q = (1.0 + 0.1 * torch.randn(B, H, S, D, generator=g)).half()
    ramp = (slope * torch.arange(S, dtype=torch.float32)).view(1, 1, S, 1)
    kk = (ramp * (1.0 + 0.05 * torch.randn(B, H, S, D, generator=g))).half()
    v = torch.randn(B, H, S, D, generator=g).half()
    lens_t = torch.tensor(lens, dtype=torch.int32).cuda()
    for causal in (True, False):
        ctx = k.attn_fused(q.cuda(), kk.cuda(), v.cuda(), lens_t, scale=D ** -0.5, causal=causal).cpu()
        scores = eager.attn_qk(q, kk, torch.float64)
        probs = eager.scale_mask_softmax(B, S, H, scores, lens, scale=D ** -0.5, causal=causal,
                                         acc_dtype=torch.float64, out_dtype=torch.float64)
        want = eager.attn_pv(probs, v, torch.float64)
        for b, n in enumerate(lens):
            assert_ctx_close(ctx[b, :, :n], want[b, :, :n], torch.float16, "attn_fused, rising scores")


def test_attn_fused_matches_unfused_pipeline_on_c2_shape():
    """Same inputs through the three separate kernels and through the fused one."""
    k = _kernel()
    B, H, S, D = 4, 12, 512, 64
    lens = [512, 64, 301, 97]
    announce("attn fused vs unfused")
    g = torch.Generator().manual_seed(77)
    qkv = torch.randn(B, H, S, 3 * D, generator=g).half().cuda()
    q, kk, v = torch.chunk(qkv, 3, dim=-1)
    lens_t = torch.tensor(lens, dtype=torch.int32).cuda()
    scores = k.attn_qk(q, kk, lens_t, causal=True)
    probs = k.scale_mask_softmax(B, S, H, scores, lens_t, scale=D ** -0.5, causal=True, tail_rows=128)
    ctx_a = k.attn_pv(probs, v, lens_t, causal=True).cpu()
    ctx_b = k.attn_fused(q, kk, v, lens_t, causal=True).cpu()
    # each against the oracle at 2e-3 (plus the rounding of the stored context): the fused kernel against the
    # oracle that rounds nothing in between, the three kernels against the one that stores fp16 scores and
    # probabilities as they do
    qc, kc, vc = q.cpu(), kk.cpu(), v.cpu()
    s32 = eager.attn_qk(qc, kc, torch.float32)
    for rounded, got in ((True, ctx_a), (False, ctx_b)):
        sc = s32.half().float() if rounded else s32
        pr = eager.scale_mask_softmax(B, S, H, sc, lens, scale=D ** -0.5, causal=True, out_dtype=torch.float32)
        want = eager.attn_pv(pr.half().float() if rounded else pr, vc, torch.float32)
        for b, n in enumerate(lens):
            assert_stored_close(got[b, :, :n], want[b, :, :n], torch.float16, what=f"rounded={rounded}")


@pytest.mark.parametrize("seed", list(range(12)))
def test_attention_random_shapes(seed):
    """Seeded random shapes (head sizes 32..128, buckets that are not multiples of the tiles, empty and
    full sequences) through QK^T -> softmax -> PV and through the fused kernel, against the float64 oracle."""
    k = _kernel()
    g = torch.Generator().manual_seed(9000 + seed)
    ri = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))
    B, H = ri(1, 5), ri(1, 4)
    D = [32, 64, 80, 96, 128][ri(0, 4)]
    S = 8 * ri(2, 60)
    lens = [ri(0, S) for _ in range(B)]
    lens[ri(0, B - 1)] = S
    causal = bool(ri(0, 1))
    dtype = [torch.float16, torch.bfloat16][ri(0, 1)]
    announce("attn random", seed, B, H, S, D, lens, causal, dtype)
    T = sum(lens)
    qkv_packed = packed_randn(T, H * 3 * D, dtype, 500 + seed).reshape(T, H, 3 * D)
    qkv = pad_bhsd(qkv_packed, lens, S, H, 3 * D)
    q, kk, v = torch.chunk(qkv, 3, dim=-1)
    lens_t = torch.tensor(lens, dtype=torch.int32).cuda()
    qg, kg, vg = torch.chunk(qkv.cuda(), 3, dim=-1)
    scale = D ** -0.5
    scores = eager.attn_qk(q, kk, torch.float64)

    def oracle_ctx(rounded):    # rounded: scores and probabilities pass through the storage dtype, as in the three-kernel path
        sc = scores.to(dtype).double() if rounded else scores
        probs = eager.scale_mask_softmax(B, S, H, sc, lens, scale=scale, causal=causal, acc_dtype=torch.float64,
                                         out_dtype=torch.float64)
        for b, n in enumerate(lens):
            probs[b, :, n:] = 0
        return eager.attn_pv(probs.to(dtype).double() if rounded else probs, v, torch.float64)
    want, want_r = oracle_ctx(False), oracle_ctx(True)
    s_gpu = k.attn_qk(qg, kg, lens_t, causal=causal)
    p_gpu = k.scale_mask_softmax(B, S, H, s_gpu, lens_t, scale=scale, causal=causal, tail_rows=128)
    ctx_a = k.attn_pv(p_gpu, vg, lens_t, causal=causal).cpu()
    ctx_b = k.attn_fused(qg, kg, vg, lens_t, scale=scale, causal=causal).cpu()
    ctx_c = k.attn_fused_packed(qkv_packed.reshape(1, T, H, 3 * D).cuda(), B, S, lens_t, H, D, scale=scale,
                                causal=causal).cpu().reshape(T, H, D)
    t0 = 0
    for b, n in enumerate(lens):
        if n:
            # BASE[dtype] on top of half an ulp of the stored context; the three-kernel path against the oracle
            # that stores scores and probabilities in the same dtype, the fused kernels against the exact one
            assert_stored_close(ctx_a[b, :, :n], want_r[b, :, :n], dtype, what="three kernels")
            assert_stored_close(ctx_b[b, :, :n], want[b, :, :n], dtype, what="fused")
            assert_stored_close(ctx_c[t0:t0 + n].permute(1, 0, 2), want[b, :, :n], dtype, what="fused, packed")
        t0 += n


@pytest.mark.parametrize("causal", [True, False])
def test_attention_long_bucket(causal):
    """A 4096-token bucket (32 query tiles, 64 key tiles, 8 KiB score rows): the three routes against the fp32
    oracle on one full-length and one short sequence."""
    k = _kernel()
    B, H, S, D = 2, 2, 4096, 128
    lens = [4096, 777]
    announce("attn long bucket", causal)
    T = sum(lens)
    qkv_packed = packed_randn(T, H * 3 * D, torch.float16, 4242).reshape(T, H, 3 * D)
    qkv = pad_bhsd(qkv_packed, lens, S, H, 3 * D)
    q, kk, v = torch.chunk(qkv, 3, dim=-1)
    scale = D ** -0.5
    scores = eager.attn_qk(q, kk, torch.float32)
    probs = eager.scale_mask_softmax(B, S, H, scores, lens, scale=scale, causal=causal, acc_dtype=torch.float32,
                                     out_dtype=torch.float32)
    for b, n in enumerate(lens):
        probs[b, :, n:] = 0
    want = eager.attn_pv(probs, v, torch.float32)
    lens_t = torch.tensor(lens, dtype=torch.int32).cuda()
    qg, kg, vg = torch.chunk(qkv.cuda(), 3, dim=-1)
    s_gpu = k.attn_qk(qg, kg, lens_t, causal=causal)
    p_gpu = k.scale_mask_softmax(B, S, H, s_gpu, lens_t, scale=scale, causal=causal, tail_rows=128)
    for b, n in enumerate(lens):      # rows of probabilities sum to one over the keys the row may see
        blk = p_gpu[b, :, :n, :n].float()      # what lies past a row's query tile is never written: mask it
        rows = (torch.tril(blk) if causal else blk).sum(-1)
        # up to 4096 probabilities, each rounded to fp16 (relative 2^-11, independent): the sum strays by
        # about 2^-11 / sqrt(number of comparable terms); 2e-3 per-entry tolerance is the cap used here
        assert float((rows - 1).abs().max()) <= 2e-3 + 2.0 ** -11
    ctx_a = k.attn_pv(p_gpu, vg, lens_t, causal=causal).cpu()
    ctx_b = k.attn_fused(qg, kg, vg, lens_t, scale=scale, causal=causal).cpu()
    ctx_c = k.attn_fused_packed(qkv_packed.reshape(1, T, H, 3 * D).cuda(), B, S, lens_t, H, D, scale=scale,
                                causal=causal).cpu().reshape(T, H, D)
    t0 = 0
    for b, n in enumerate(lens):
        ref = want[b, :, :n]
        assert max_abs(ctx_a[b, :, :n], ref) <= 2e-3
        assert max_abs(ctx_b[b, :, :n], ref) <= 2e-3
        assert max_abs(ctx_c[t0:t0 + n].permute(1, 0, 2), ref) <= 2e-3
        t0 += n


@pytest.mark.parametrize("tail_rows", [1, 128])
@pytest.mark.parametrize("dtype,S", [(torch.float32, 4104), (torch.float16, 8200)])
def test_attention_rows_past_the_register_limit(dtype, S, tail_rows):
    """Score rows too long for the register softmax (the three-pass kernel runs) whose length is a multiple of
    the 16-byte vector: QK^T stores whole vectors and PV loads whole vectors, so the softmax must clear the
    vector that straddles the end of a row's prefix.  Causal, one full-length and one short sequence, score
    buffer pre-filled with a large value that would wreck the context if it leaked."""
    k = _kernel()
    B, H, D = 2, 1, 64
    lens = [S, 1029]
    announce("attn past register limit", dtype, S, tail_rows)
    T = sum(lens)
    qkv_packed = packed_randn(T, H * 3 * D, dtype, 77 + S).reshape(T, H, 3 * D)
    qkv = pad_bhsd(qkv_packed, lens, S, H, 3 * D)
    q, kk, v = torch.chunk(qkv, 3, dim=-1)
    scale = D ** -0.5
    lens_t = torch.tensor(lens, dtype=torch.int32).cuda()
    qg, kg, vg = torch.chunk(qkv.cuda(), 3, dim=-1)
    out = torch.full((B, H, S, S), 1000.0, dtype=dtype, device="cuda")
    s_gpu = k.attn_qk(qg, kg, lens_t, causal=True, out=out)
    p_gpu = k.scale_mask_softmax(B, S, H, s_gpu, lens_t, scale=scale, causal=True, tail_rows=tail_rows)
    ctx = k.attn_pv(p_gpu, vg, lens_t, causal=True).cpu()
    del out, s_gpu, p_gpu
    tol = {torch.float16: 2e-3, torch.float32: 1e-5}[dtype]
    for b, n in enumerate(lens):
        # the oracle one sequence at a time keeps the float32 score tensor of the CPU side small
        sc = eager.attn_qk(q[b:b + 1, :, :n], kk[b:b + 1, :, :n], torch.float32)
        pr = eager.scale_mask_softmax(1, n, H, sc, [n], scale=scale, causal=True, acc_dtype=torch.float32,
                                      out_dtype=torch.float32)
        want = eager.attn_pv(pr, v[b:b + 1, :, :n], torch.float32)
        assert_ctx_close(ctx[b:b + 1, :, :n], want, dtype, "rows past the register limit")


VARLEN_CASES = [
    # B, H, S, D, lens
    (8, 12, 128, 64, [24, 127, 31, 65, 24, 127, 31, 65]),
    (3, 2, 200, 64, [200, 0, 77]),
    (2, 3, 256, 128, [256, 129]),
    (1, 2, 520, 80, [515]),
    (9, 1, 136, 128, [130, 5, 64, 65, 127, 128, 129, 1, 33]),
    (2, 2, 2048, 128, [2048, 700]),
]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("B,H,S,D,lens", VARLEN_CASES)
def test_contractions_on_packed_tokens_match_the_padded_route(dtype, causal, B, H, S, D, lens):
    """attn_qk_varlen / attn_pv_varlen read q, k, v where the projection left them ([T,H,3D], batch b at row
    cu_seqlens[b]) and write the packed context: bit for bit what transpose_pad -> attn_qk -> softmax -> attn_pv ->
    transpose_depad give.  With packed_scores (causal, 16-bit) the score tensor holds each row's visible prefix
    only, the same bits as the padded tensor's prefix."""
    k = _kernel()
    announce("attn varlen", dtype, causal, B, H, S, D, lens)
    T = sum(lens)
    qkv_packed = packed_randn(T, H * 3 * D, dtype, 900 + S).reshape(T, H, 3 * D)
    lens_t = torch.tensor(lens, dtype=torch.int32).cuda()
    qkv_g = qkv_packed.cuda()
    scale = D ** -0.5
    padded = k.transpose_pad(qkv_g.reshape(1, T, H, 3 * D), B, S, lens_t, H, 3 * D)
    qp, kp, vp = torch.chunk(padded, 3, dim=-1)
    s_pad = k.attn_qk(qp, kp, lens_t, causal=causal)
    scores_raw = s_pad.clone()
    p_pad = k.scale_mask_softmax(B, S, H, s_pad, lens_t, scale=scale, causal=causal, tail_rows=1)
    want = k.transpose_depad(k.attn_pv(p_pad, vp, lens_t, causal=causal), B, T, S, lens_t, H, D)

    q, kk, v = torch.chunk(qkv_g, 3, dim=-1)
    s_var = k.attn_qk_varlen(q, kk, B, S, lens_t, causal=causal)
    for b, n in enumerate(lens):
        for qi in (0, n // 2, n - 1):
            if 0 <= qi < n:
                vis = (qi + 1) if causal else n
                assert torch.equal(s_var[b, :, qi, :vis], scores_raw[b, :, qi, :vis])
    p_var = k.scale_mask_softmax(B, S, H, s_var, lens_t, scale=scale, causal=causal, tail_rows=1)
    sentinel = torch.full((1, T + 1, H, D), 9.0, dtype=dtype, device="cuda")
    got = k.attn_pv_varlen(p_var, v, B, S, lens_t, causal=causal, out=sentinel[:, :T])
    assert torch.equal(got, want)
    assert bool((sentinel[:, T] == 9.0).all())          # nothing is written past the last token
    if causal and dtype != torch.float32:
        epv, grp = 8, 64       # 16-byte vectors; rows of the packed layout are whole 128-byte groups
        flat = k.attn_qk_varlen(q, kk, B, S, lens_t, causal=True, packed_scores=True)
        assert flat.numel() == k.packed_scores_elems(B, H, S, dtype)

        def row_start(r):
            t = r // grp
            return grp * (grp * t * (t + 1) // 2 + (r - grp * t) * (t + 1))
        unit = row_start(S)
        for b, n in enumerate(lens):
            for qi in (0, n // 2, n - 1):
                if 0 <= qi < n:
                    for h in (0, H - 1):
                        o = (b * H + h) * unit + row_start(qi)
                        assert torch.equal(flat[o:o + qi + 1], scores_raw[b, h, qi, :qi + 1])
        probs = k.scale_mask_softmax_packed(B, S, H, flat, lens_t, scale=scale)
        assert probs.data_ptr() == flat.data_ptr()
        for b, n in enumerate(lens):
            for qi in (0, n // 2, n - 1):
                if 0 <= qi < n:
                    o = (b * H + (H - 1)) * unit + row_start(qi)
                    if S <= 1024:
                        assert torch.equal(probs[o:o + qi + 1], p_pad[b, H - 1, qi, :qi + 1])
                    else:
                        assert max_abs(probs[o:o + qi + 1], p_pad[b, H - 1, qi, :qi + 1]) <= 2.0 ** -11
                    assert not probs[o + qi + 1:o + (qi // epv + 1) * epv].any()
        got_p = k.attn_pv_varlen(probs, v, B, S, lens_t, causal=True, packed_scores=True)
        if S <= 1024:
            assert torch.equal(got_p, want)
        else:
            # rows of more than 1024 keys: the softmax on [B,H,S,S] gives every row 64 lanes, the one on packed
            # scores sizes the lane group by the row, so the row sums are added up in another order and a
            # probability may differ in its last bit
            assert max_abs(got_p, want) <= 2.0 ** -10 * max(1.0, float(want.abs().max()))
    elif dtype == torch.float32 or not causal:
        with pytest.raises(RuntimeError):
            k.attn_qk_varlen(q, kk, B, S, lens_t, causal=causal, packed_scores=True)


@pytest.mark.parametrize("tiles_first", [False, True])
@pytest.mark.parametrize("B,H,S,lens", [(16, 7, 1000, None), (3, 12, 130, [130, 0, 77]), (9, 1, 2048, None),
                                        (1, 1, 8, [5])])
def test_attn_tile_table_lists_every_real_query_tile_once_longest_sequence_first(B, H, S, lens, tiles_first):
    """en_attn_tile_table: workgroup w of a launch finds unit * ntq + query tile or -1.  Every 128-row query tile a
    sequence really has appears exactly once, tiles past a sequence's end never; a unit stays on one XCD (w % 8);
    its tiles run from the last to the first; sequences come in the order of decreasing length.  In the
    tiles-first order (units with little K and V) an XCD runs the last tiles of all its units, then the
    second-to-last ..., the longer sequence first within a tile index."""
    from energonai_amd import _lib
    from energonai_amd.seqinfo import build_seq_info
    if lens is None:
        g = torch.Generator().manual_seed(B * 31 + S)
        lens = torch.randint(0, S + 40, (B,), generator=g).tolist()      # some longer than the bucket
    announce("tile table", B, H, S, lens)
    info = build_seq_info(torch.tensor(lens, dtype=torch.int32), B)
    tab = info.tile_table(H, S, (64 << 10) if tiles_first else (1 << 20)).cpu().tolist()
    ntq = -(-S // 128)
    assert len(tab) == _lib.fn.en_attn_tile_table_elems(B, H, S, 128) == -(-B * H // 8) * 8 * ntq
    want = {(b * H + h) * ntq + qi for b in range(B) for h in range(H) for qi in range(-(-min(lens[b], S) // 128))}
    got = [c for c in tab if c >= 0]
    assert len(got) == len(set(got)) and set(got) == want
    assert all(c >= -1 for c in tab)
    where = {}
    for w, c in enumerate(tab):
        if c >= 0:
            where.setdefault(c // ntq, []).append((w, c % ntq))
    first = {}
    for unit, entries in where.items():
        assert len({w % 8 for w, _ in entries}) == 1                     # one XCD per unit
        assert [qi for _, qi in entries] == sorted((qi for _, qi in entries), reverse=True)
        first[unit] = entries[0][0]
    if tiles_first:
        # on an XCD the tile indices never grow along the launch, and within one index the longer sequence is first
        for x in range(8):
            seq = [(c % ntq, min(lens[(c // ntq) // H], S)) for w, c in enumerate(tab) if c >= 0 and w % 8 == x]
            assert seq == sorted(seq, key=lambda t: (-t[0], -t[1]))
    else:
        # of two units on the same XCD the one of the longer sequence starts earlier, and a unit's tiles are adjacent
        units = sorted(first, key=lambda u: first[u])
        for x in range(8):
            seq = [min(lens[u // H], S) for u in units if first[u] % 8 == x]
            assert seq == sorted(seq, reverse=True)
        for unit, entries in where.items():
            ws = [w for w, _ in entries]
            assert ws == list(range(ws[0], ws[0] + 8 * len(ws), 8))


@pytest.mark.parametrize("causal", [True, False])
def test_attention_kernels_give_the_same_bits_with_and_without_a_tile_table(causal):
    """The table only reorders the workgroups of a launch."""
    import ctypes
    from energonai_amd import _lib
    from energonai_amd.seqinfo import build_seq_info
    B, H, S, D = 5, 3, 520, 128
    lens = [520, 3, 0, 257, 128]
    announce("tile table on/off", causal)
    dtype = torch.float16
    g = torch.Generator().manual_seed(77)
    q, kk, v = (torch.randn(B, H, S, D, generator=g).to(dtype).cuda() for _ in range(3))
    info = build_seq_info(torch.tensor(lens, dtype=torch.int32), B)
    tab = info.tile_table(H, S)
    strides = (H * S * D, S * D, D)
    arr = (ctypes.c_int64 * 3)(*strides)
    stream = _lib.stream_of(q)
    outs = []
    for t in (None, tab.data_ptr()):
        scores = torch.zeros(B, H, S, S, dtype=dtype, device="cuda")
        ctx = torch.zeros(B, H, S, D, dtype=dtype, device="cuda")
        fused = torch.zeros(B, H, S, D, dtype=dtype, device="cuda")
        _lib.check(_lib.fn.en_attn_qk(q.data_ptr(), kk.data_ptr(), scores.data_ptr(), info.lens.data_ptr(), None, B, H, S,
                                      S, D, *strides, *strides, 1.0, int(causal), 1, None, None, 0, t, stream), "qk")
        probs = _kernel().scale_mask_softmax(B, S, H, scores, info, scale=D ** -0.5, causal=causal, tail_rows=1)
        _lib.check(_lib.fn.en_attn_pv(probs.data_ptr(), v.data_ptr(), ctx.data_ptr(), info.lens.data_ptr(), None, B, H, S,
                                      S, D, *strides, *strides, int(causal), 0, 1, None, None, 0, t, stream), "pv")
        _lib.check(_lib.fn.en_attn_fused(q.data_ptr(), kk.data_ptr(), v.data_ptr(), fused.data_ptr(), info.lens.data_ptr(),
                                         None, B, H, S, S, D, arr, arr, arr, arr, None, None, D ** -0.5, int(causal), 1,
                                         t, 128, stream), "fused")
        outs.append((probs.clone(), ctx, fused))
    for a, b in zip(*outs):
        assert torch.equal(a, b)
    assert bool(outs[0][2].any())


def test_attn_tile_table_of_a_batch_beyond_the_sort_limit_keeps_the_batch_order():
    """More than 1024 sequences: the table still lists every real tile once (in batch order)."""
    from energonai_amd.seqinfo import build_seq_info
    B, H, S = 1100, 1, 200
    g = torch.Generator().manual_seed(5)
    lens = torch.randint(0, S + 1, (B,), generator=g).tolist()
    announce("tile table, large batch", B)
    info = build_seq_info(torch.tensor(lens, dtype=torch.int32), B)
    tab = info.tile_table(H, S).cpu().tolist()
    ntq = 2
    want = {b * ntq + qi for b in range(B) for qi in range(-(-lens[b] // 128))}
    got = [c for c in tab if c >= 0]
    assert len(got) == len(set(got)) and set(got) == want
    # and the kernels run with it
    D = 32
    q, kk, v = (torch.randn(B, H, S, D, generator=g).half().cuda() for _ in range(3))
    ctx = _kernel().attn_fused(q, kk, v, info, causal=True).cpu().float()
    b = max(range(B), key=lambda i: lens[i])
    n = lens[b]
    ref = torch.nn.functional.scaled_dot_product_attention(q[b:b + 1, :, :n].float().cpu(), kk[b:b + 1, :, :n].float().cpu(),
                                                           v[b:b + 1, :, :n].float().cpu(), is_causal=True)
    assert_ctx_close(ctx[b:b + 1, :, :n], ref, torch.float16, "attn_fused with a large-batch table")


def test_tile_table_follows_lengths_that_change_in_place():
    """A SeqInfo built on a caller's own lengths tensor (the K/V cache's) keeps its workgroup order per version of
    that tensor: after an in-place edit the attention calls must schedule the query tiles of the new lengths."""
    from energonai_amd.seqinfo import SeqInfo
    k = _kernel()
    B, H, S, D = 2, 2, 512, 64
    announce("tile table after lens.add_")
    g = torch.Generator().manual_seed(91)
    q, kk, v = (torch.randn(B, H, S, D, generator=g).half().cuda() for _ in range(3))
    lens = torch.tensor([100, 60], dtype=torch.int32).cuda()
    info = SeqInfo(lens, None, B, None, lens)
    first = k.attn_fused(q, kk, v, info, causal=True)
    tab_before = info.tile_table(H, S, 2 * S * D * 2)
    lens.add_(300)
    tab_after = info.tile_table(H, S, 2 * S * D * 2)
    assert tab_after is not tab_before
    got = k.attn_fused(q, kk, v, info, causal=True, out=torch.full((B, H, S, D), 777.0, dtype=torch.float16, device="cuda"))
    want = k.attn_fused(q, kk, v, lens.clone(), causal=True)
    for b, n in enumerate([400, 360]):
        assert torch.equal(got[b, :, :n], want[b, :, :n])
        assert bool((got[b, :, n:] == 777.0).all())
    assert torch.equal(first[0, :, :100], got[0, :, :100])      # causal: the old rows see the same keys
    scores = k.attn_qk(q, kk, info, causal=True)
    want_s = k.attn_qk(q, kk, lens.clone(), causal=True)
    probs = k.scale_mask_softmax(B, S, H, scores, info, scale=D ** -0.5)
    want_p = k.scale_mask_softmax(B, S, H, want_s, lens.clone(), scale=D ** -0.5)
    ctx = k.attn_pv(probs, v, info, causal=True)
    want_c = k.attn_pv(want_p, v, lens.clone(), causal=True)
    for b, n in enumerate([400, 360]):
        assert torch.equal(ctx[b, :, :n], want_c[b, :, :n])


WIDE_CASES = [c for c in ATTN_CASES if c[3] > 64] + [
    (3, 2, 700, 128, [700, 257, 64]),       # three, two and one 256-row tiles; a wave whose second block is empty
    (2, 1, 1030, 128, [1030, 511]),         # a fifth tile of six rows
    (2, 2, 512, 96, [512, 300]),
]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("B,H,S,D,lens", WIDE_CASES)
def test_attn_fused_with_64_queries_per_wave(dtype, causal, B, H, S, D, lens):
    """The 256-row tile of the fused kernel (query_tile=256) against the float64 oracle of the three steps, NaN in
    every padding position, untouched rows checked; the packed form gives the same bits as the padded one."""
    k = _kernel()
    announce("attn fused, 64 queries per wave", dtype, causal, B, H, S, D, lens)
    T = sum(lens)
    qkv_packed = packed_randn(max(T, 1), H * 3 * D, dtype, 500 + S)[:T].reshape(T, H, 3 * D)
    qkv = pad_bhsd(qkv_packed, lens, S, H, 3 * D)
    for b, n in enumerate(lens):
        qkv[b, :, n:] = float("nan")
    q, kk, v = torch.chunk(qkv, 3, dim=-1)
    lens_t = torch.tensor(lens, dtype=torch.int32).cuda()
    qg, kg, vg = torch.chunk(qkv.cuda(), 3, dim=-1)
    scale = D ** -0.5
    sentinel = 777.0
    out = torch.full((B, H, S, D), sentinel, dtype=dtype, device="cuda")
    ctx = k.attn_fused(qg, kg, vg, lens_t, scale=scale, causal=causal, out=out, query_tile=256).cpu()
    qz, kz, vz = (torch.nan_to_num(t, nan=0.0) for t in (q, kk, v))
    scores = eager.attn_qk(qz, kz, torch.float64)
    probs = eager.scale_mask_softmax(B, S, H, scores, lens, scale=scale, causal=causal, acc_dtype=torch.float64,
                                     out_dtype=torch.float64)
    rows_pad = torch.ones(B, H, S, dtype=torch.bool)
    for b, n in enumerate(lens):
        rows_pad[b, :, :n] = False
        probs[b, :, n:] = 0
    want = eager.attn_pv(probs, vz, torch.float64)
    if (~rows_pad).any():
        assert_ctx_close(ctx[~rows_pad], want[~rows_pad], dtype, "attn_fused, query_tile 256")
    assert bool((ctx[rows_pad] == sentinel).all())
    if T:
        guard = torch.full((T + 2, H * D), sentinel, dtype=dtype, device="cuda")
        k.attn_fused_packed(qkv_packed.reshape(1, T, H, 3 * D).cuda(), B, S, lens_t, H, D, scale=scale, causal=causal,
                            out=guard[1:T + 1], query_tile=256)
        g = guard.cpu()
        t = 0
        for b, n in enumerate(lens):
            assert torch.equal(g[1 + t:1 + t + n].view(n, H, D).permute(1, 0, 2), ctx[b, :, :n])
            t += n
        assert bool((g[0] == sentinel).all()) and bool((g[T + 1] == sentinel).all())


def test_tile_table_of_256_row_tiles():
    """The workgroup order for the 64-queries-per-wave kernel lists every real 256-row tile once."""
    from energonai_amd.seqinfo import build_seq_info
    B, H, S = 7, 3, 1000
    lens = [1000, 1, 256, 257, 0, 513, 777]
    announce("tile table, 256-row tiles")
    info = build_seq_info(torch.tensor(lens, dtype=torch.int32), B)
    tab = info.tile_table(H, S, query_tile=256).cpu().tolist()
    ntq = 4
    want = {(b * H + h) * ntq + qi for b in range(B) for h in range(H) for qi in range(-(-lens[b] // 256))}
    got = [c for c in tab if c >= 0]
    assert len(got) == len(set(got)) and set(got) == want
    assert len(tab) == -(-B * H // 8) * 8 * ntq
