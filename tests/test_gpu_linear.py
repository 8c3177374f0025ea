"""The projection GEMM on hipBLASLt (linear / find_algo of the reference API) against torch in float64."""
import pytest
import torch
import torch.nn.functional as F

from gpu_util import announce, max_abs

pytestmark = pytest.mark.gpu


def _lf():
    from energonai_amd.kernel.cuda_native import linear_func
    return linear_func


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("activation", [None, "relu", "gelu_tanh"])
@pytest.mark.parametrize("with_bias", [False, True])
def test_linear_matches_float64(dtype, activation, with_bias):
    lf = _lf()
    B, S, din, dout = 3, 37, 256, 192
    announce("linear", dtype, activation, with_bias)
    g = torch.Generator().manual_seed(41)
    x = torch.randn(B, S, din, generator=g).to(dtype)
    w = (torch.randn(dout, din, generator=g) / din ** 0.5).to(dtype)
    b = torch.randn(dout, generator=g).to(dtype) if with_bias else None
    got = lf.linear(x.cuda(), w.cuda(), -1, bias=None if b is None else b.cuda(), activation=activation).cpu()
    want = x.double() @ w.double().T
    if b is not None:
        want = want + b.double()
    if activation == "relu":
        want = torch.relu(want)
    elif activation == "gelu_tanh":
        want = F.gelu(want, approximate="tanh")
    tol = {torch.float16: 4e-3, torch.bfloat16: 3e-2, torch.float32: 2e-4}[dtype]
    assert got.shape == (B, S, dout) and got.dtype == dtype
    assert max_abs(got, want) <= tol * max(1.0, float(want.abs().max()))


def test_every_candidate_gives_the_same_product_and_find_algo_returns_one_of_them():
    lf = _lf()
    B, S, din, dout = 4, 64, 512, 1024
    announce("linear candidates")
    g = torch.Generator().manual_seed(42)
    x = torch.randn(B, S, din, generator=g).half().cuda()
    w = (torch.randn(dout, din, generator=g) / din ** 0.5).half().cuda()
    n = lf.algo_count(B * S, din, dout)
    assert n >= 1
    want = (x.double() @ w.double().T).cpu()
    for algo in range(min(n, 8)):
        assert max_abs(lf.linear(x, w, algo).cpu(), want) <= 4e-3 * float(want.abs().max())
    with pytest.raises(RuntimeError):
        lf.linear(x, w, n + 1000)
    best = lf.find_algo(batch_size=B, seq_len=S, din=din, dout=dout, inner_loop=2)
    assert 0 <= best < n


def test_reference_extension_stand_in_uses_the_same_gemm():
    import energonai_amd.ext.energonai_linear_func as ext
    announce("linear ext")
    g = torch.Generator().manual_seed(43)
    x = torch.randn(2, 16, 128, generator=g).half().cuda()
    w = torch.randn(64, 128, generator=g).half().cuda()
    want = (x.double() @ w.double().T).cpu()
    for algo in (-1, 5, 99, 115):       # the reference's id ranges are accepted
        assert max_abs(ext.mlp_gemm(x, w, algo).cpu(), want) <= 4e-3 * float(want.abs().max())


def test_auto_algo_is_searched_once_per_problem_and_gives_the_same_product():
    lf = _lf()
    B, S, din, dout = 1, 48, 384, 640          # a skinny problem, as in a decode step
    announce("linear auto algo")
    g = torch.Generator().manual_seed(44)
    x = torch.randn(B, S, din, generator=g).half().cuda()
    w = (torch.randn(dout, din, generator=g) / din ** 0.5).half().cuda()
    b = torch.randn(dout, generator=g).half().cuda()
    lf._tuned.clear()
    best = lf.tuned_algo(x, w, bias=b, activation="relu", inner_loop=2)
    assert 0 <= best < lf.algo_count(B * S, din, dout, torch.float16, True, "relu")
    assert len(lf._tuned) == 1
    got = lf.linear(x, w, "auto", bias=b, activation="relu").cpu()
    assert len(lf._tuned) == 1 and lf.tuned_algo(x, w, bias=b, activation="relu") == best    # remembered
    want = torch.relu(x.double() @ w.double().T + b.double()).cpu()
    assert max_abs(got, want) <= 4e-3 * float(want.abs().max())
    lf.linear(x, w, "auto")                      # no bias, no activation: another problem
    assert len(lf._tuned) == 2
    with pytest.raises(RuntimeError):
        lf.linear(x, w, "fastest")
