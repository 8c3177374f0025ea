"""Helpers shared by the GPU parity tests."""
import sys

import torch


def announce(*parts):
    """Name the case before touching the GPU, flushed, so a fault can be traced to it."""
    print("[case]", *parts, flush=True)
    sys.stdout.flush()


def ragged_lens(batch, lo, hi, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(lo, hi + 1, (batch,), generator=g, dtype=torch.int32)


def packed_randn(T, width, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(T, width, generator=g).to(dtype)


def pad_bhsd(packed, lens, S, H, D):
    """[T,H,D] -> zero padded [B,H,S,D] on the CPU (plain indexing)."""
    B = len(lens)
    out = torch.zeros(B, H, S, D, dtype=packed.dtype)
    t = 0
    for b, n in enumerate(lens):
        out[b, :, :n] = packed[t:t + n].permute(1, 0, 2)
        t += n
    return out


def max_abs(a, b):
    return (a.double() - b.double()).abs().max().item()


# ---------------------------------------------------------------------------------------------------------------
# Tolerances, in one place.  The bar is: max-abs error <= BASE[dtype] against the float32 (or float64) oracle, on
# top of the rounding the result's own storage type forces on it (half a unit in the last place of the stored
# value: 9.8e-4 for an fp16 value in [2, 4), 1.95e-3 in [4, 8), which no kernel can avoid).  BASE is 2e-3 for
# fp16 and 1e-5 for fp32; bf16 carries 8 fewer mantissa bits than fp16, hence 8 x 2e-3.
# ---------------------------------------------------------------------------------------------------------------
BASE = {torch.float32: 1e-5, torch.float16: 2e-3, torch.bfloat16: 1.6e-2}
_MANT = {torch.float32: 23, torch.float16: 10, torch.bfloat16: 7}
_MIN_EXP = {torch.float32: -126, torch.float16: -14, torch.bfloat16: -126}


def half_ulp(ref, dtype):
    """Half the spacing of `dtype` at |ref|, elementwise, as float64."""
    a = ref.double().abs()
    e = torch.floor(torch.log2(a.clamp_min(2.0 ** _MIN_EXP[dtype]))).clamp_min(_MIN_EXP[dtype])
    return 0.5 * torch.pow(torch.tensor(2.0, dtype=torch.float64), e - _MANT[dtype])


def excess(got, want, dtype):
    """max(|got - want| - half_ulp(want)): the error left after the unavoidable rounding of the stored result."""
    if got.numel() == 0:
        return 0.0
    return float(((got.double() - want.double()).abs() - half_ulp(want, dtype)).max())


def assert_stored_close(got, want, dtype, base=None, what=""):
    """|got - want| <= base + half_ulp_dtype(|want|) elementwise; base defaults to BASE[dtype]."""
    base = BASE[dtype] if base is None else base
    ex = excess(got, want, dtype)
    assert ex <= base, f"{what}: error exceeds half an ulp of the stored value by {ex:.3e} > {base:.3e}"


def assert_ctx_close(got, want, dtype, what=""):
    """The bound for attention outputs.  16-bit storage: BASE[dtype] on top of half an ulp of the stored value,
    elementwise (assert_stored_close).  fp32: a relative bound, 1e-5 x max(1, largest reference magnitude),
    because fp32 results carry rounding in proportion to the values they add up."""
    if got.numel() == 0:
        return
    if dtype == torch.float32:
        err = max_abs(got, want)
        assert err <= BASE[dtype] * max(1.0, float(want.abs().max())), f"{what}: {err:.3e}"
    else:
        assert_stored_close(got, want, dtype, what=what)
