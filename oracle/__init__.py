"""CPU oracle for the padding-removal hot path.  TEST INFRASTRUCTURE ONLY.

Nothing under this package is part of the shipped product: only the test
suite, the smoke check and the CPU-baseline leg of the benchmark may import
it, and only as the checker.  The product (`energonai_amd`) never imports it
and has no CPU fallback.

Contents
--------
eager.py      torch-eager restatement of every op on the path, written from the
              reference's Python wrappers, CUDA index formulas and its own test
              oracle (each function cites the reference file:line it follows).
models.py     the same for the reference's attention / MLP / block modules on padded
              batches (the callers either side of the path).
brute.py      pure-Python triple loops that replay the reference CUDA kernels'
              blockIdx/threadIdx arithmetic on tiny inputs; they pin eager.py.
kernels_ref.c plain-C replay of the same kernels (grid loops on the CPU) for
              medium sizes; built by oracle/Makefile into oracle/_build/.

Pinning status
--------------
transpose_pad / transpose_depad   pinned: reference test's permute/manual_depad
                                  oracle and its fixed shape, brute-force index
                                  replay, C replay, round trip, zero padding.
depad, ft_* family                pinned: closed forms, brute-force replay,
                                  C replay, inverse pairs.
scale_mask_softmax                the reference has no test for it: pinned by
                                  torch.softmax on the visible prefix, closed
                                  forms (len 1, constant rows, shift
                                  invariance) and the C replay of the kernel's
                                  arithmetic.  By the reference's own tests:
                                  PARITY UNPINNED.
LayerNorm forward                 the reference has no test for it: pinned by
                                  torch.nn.functional.layer_norm in float64,
                                  closed forms (constant row -> beta) and the C
                                  replay of its Welford/Chan arithmetic.  By
                                  the reference's own tests: PARITY UNPINNED.
QK^T / PV / per-layer pipeline    pinned by torch.matmul in float32/float64 and
                                  by the padded-vs-unpadded layer identity.
The reference's CUDA sources cannot be compiled in this image (they need nvcc,
cub, cuda_fp16 and ATen CUDA headers), so there is no oracle/_ref build.
"""
