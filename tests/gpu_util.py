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
