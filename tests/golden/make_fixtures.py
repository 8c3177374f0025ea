#!/usr/bin/env python3
"""Writes tests/golden/*.json: small known-answer vectors for the packing ops,
the causal softmax and LayerNorm.

The reference repository holds no stored vectors for this path (its kernel test
draws unseeded random inputs, tests/test_kernel/test_transpose_pad_fusion_kernel.py:14-29),
and its Python package cannot be imported here (it needs colossalai and its own
compiled CUDA extensions).  The expected values below therefore come from
oracle/brute.py, the pure-Python replay of the reference CUDA kernels' index
arithmetic and formulas, on inputs small enough to check by hand; the fixed
shape and lengths of the reference test are recorded alongside.

    python tests/golden/make_fixtures.py
"""
import json
import os
import random
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import brute  # noqa: E402


def pack_cases():
    rnd = random.Random(20240)
    cases = []
    for B, S, H, D, lens in [(2, 3, 2, 2, [3, 1]), (3, 4, 1, 3, [0, 4, 2]), (2, 5, 3, 2, [5, 2])]:
        T = sum(lens)
        src = [float(rnd.randint(-50, 50)) / 4 for _ in range(T * H * D)]       # exact in fp16
        padded = brute.transpose_pad(src, B, S, lens, H, D)
        total, off = brute.build_offsets(lens, B, S)
        hidden = [float(rnd.randint(-50, 50)) / 4 for _ in range(B * S * H * D)]
        removed = brute.remove_padding(hidden, off, total, H * D)
        rebuilt = brute.rebuild_padding(removed, off, total, H * D, B * S)
        buf = [0.5] * (B * H * S * D)
        brute.transpose_rebuild_padding(removed, buf, S, H, D, off, total)
        cases.append(dict(B=B, S=S, H=H, D=D, lens=lens, packed=src, padded=padded,
                          depadded=brute.transpose_depad(padded, B, S, lens, H, D),
                          valid=total, offsets=off, hidden=hidden, removed=removed, rebuilt=rebuilt,
                          transposed_rebuilt=buf,
                          transposed_removed=brute.transpose_remove_padding(buf, S, H, D, off, total)))
    return cases


def math_cases():
    rnd = random.Random(20241)
    B, H, S = 2, 2, 6
    lens = [6, 3]
    scores = [float(rnd.randint(-24, 24)) / 8 for _ in range(B * H * S * S)]
    probs = list(scores)
    brute.softmax_reference_kernel(probs, lens, B, H, S)
    n1, n2 = 3, 16
    x = [float(rnd.randint(-40, 40)) / 8 for _ in range(n1 * n2)]
    gamma = [1.0 + float(rnd.randint(-8, 8)) / 64 for _ in range(n2)]
    beta = [float(rnd.randint(-8, 8)) / 64 for _ in range(n2)]
    y, mean, invvar = brute.layer_norm_rows(x, n1, n2, gamma, beta, 1e-5)
    return dict(softmax=dict(B=B, H=H, S=S, lens=lens, scores=scores, probs=probs),
                layernorm=dict(n1=n1, n2=n2, eps=1e-5, x=x, gamma=gamma, beta=beta, y=y, mean=mean, invvar=invvar))


def main():
    ref = dict(source="tests/test_kernel/test_transpose_pad_fusion_kernel.py:6-11 and test_ft_transpose_pad.py:6-11",
               batch_size=8, max_padding_size=128, head_size=64, head_num=12,
               seq_lens=[24, 127, 31, 65, 24, 127, 31, 65])
    with open(os.path.join(HERE, "pack_kat.json"), "w") as f:
        json.dump(dict(reference_test=ref, cases=pack_cases()), f)
    with open(os.path.join(HERE, "math_kat.json"), "w") as f:
        json.dump(math_cases(), f)
    print("wrote pack_kat.json, math_kat.json")


if __name__ == "__main__":
    main()
